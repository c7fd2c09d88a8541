// A model step as one call: the launch sequence of a decoder made of pre-norm attention and pre-norm
// feed-forward operations, run from a list that the parts filled once at load.
//
// The host side of a step that is not a graph replay used to be a few hundred calls from Python into
// this library (one per kernel, each with its checks and its output allocation). Here the parts
// describe themselves once (matrices, norms, head sizes, cache pools), and a step is: fill the step's
// metadata, hand over one workspace, call tm_program_run. Which kernel runs for which row count and
// type is decided here exactly as the Python parts decide it (tokenmill_amd/parts, hip/gemm.py,
// hip/attention.py), so both ways launch the same kernels in the same order and give the same bits.
// (The reference's step is its model's forward pass in torch: src/infer/engine/model_runner.py:76-97,
// src/infer/model/qwen2.py:43-52.)
#include "common.h"
#include "api.h"
#include "step_program.h"

#include <stdint.h>
#include <vector>

namespace {

constexpr int SKINNY_ROWS = 16;         // most rows the skinny and norm-fused kernels are preferred for
constexpr int PANEL_ROWS = 48;          // most rows the products that keep the normed input in LDS are preferred for
constexpr int SKINNY_MAX_ROWS = 64;
constexpr int DECODE_CHUNK = 256;       // keys per block of the split decode attention
constexpr int DECODE_SPLIT_PAIRS = 192; // below this many (request, kv head) pairs the split kernels run

struct Op {
    int kind;                           // 0 attention, 1 feed-forward
    TmAttentionOp att;
    TmFfnOp ffn;
};

inline size_t align_up(size_t n) { return (n + 255) & ~(size_t)255; }
inline bool is_pow2(int x) { return x > 0 && (x & (x - 1)) == 0; }
inline bool aligned(const void* p, int to) { return ((uintptr_t)p % to) == 0; }
inline int elem_size(int dtype) { return dtype == TM_BF16 ? 2 : 4; }

}  // namespace

struct TmProgram {
    int dtype = TM_BF16;
    int hidden = 0;
    TmEmbedOp embed{};
    TmFinalOp final_op{};
    bool has_embed = false, has_final = false;
    std::vector<Op> ops;
    // the widest of each kind of activation over all operations
    int max_qkv = 0, max_q = 0, max_gu = 0, max_act = 0, max_heads_d = 0;
    // how often each way of computing q|k|v and the activation was taken (for tests and curiosity)
    mutable long long taken[TM_PROGRAM_COUNTERS] = {};
};

namespace {

// Does the normed input of M tokens fit a block's LDS in the norm-fused decode products?
bool fused_lds_fits(int M, int K) {
    const int rows = M <= 4 ? 4 : (M <= 8 ? 8 : 16);
    const int waves = K >= 2048 ? 8 : 4;
    return (size_t)rows * (K + 8) * 2 + (size_t)4 * waves * 2 * 64 * 5 + 1024 <= 160 * 1024;
}

bool fused_decode_ok(const float* resid, const TmLinear& L, int M) {
    return L.packed && M > 0 && M <= SKINNY_ROWS && L.K % 8 == 0 && fused_lds_fits(M, L.K) && aligned(resid, 16);
}

bool packed_ok(const TmLinear& L, const void* x, int ldx, int M, int dtype) {
    return L.packed && M > 0 && M <= SKINNY_ROWS && dtype == TM_BF16 && L.K % 8 == 0 && ldx % 8 == 0 && aligned(x, 16);
}

bool skinny_ok(const TmLinear& L, const void* x, int ldx, int dtype) {
    return dtype == TM_BF16 && L.dtype == TM_BF16 && L.K % 8 == 0 && ldx % 8 == 0 && aligned(x, 16) && aligned(L.w, 16);
}

bool panel_ok(const TmLinear& L, const void* x, int ldx, int M, int dtype) {
    return L.packed && M > SKINNY_ROWS && M <= PANEL_ROWS && dtype == TM_BF16 && ldx % 8 == 0 && aligned(x, 16) &&
           tm_gemm_panel_fits(M, L.K);
}

struct Run {
    const TmProgram* p;
    const TmStep* s;
    hipStream_t stream;
    void* lib_ws;
    size_t lib_ws_bytes;
    int dtype;
    // workspace
    float* resid;
    void *x, *qkv, *attn, *gu, *act, *delta_buf, *hnorm;
    float *part_o, *part_ml;
    const void* delta = nullptr;        // product output still to be added to the residual stream

    int linear(const TmLinear& L, const void* x_, int ldx, int M, void* out, int ldc, int out_dtype) {
        if (M == 0) return TM_OK;
        if (L.packed && L.packed_parts == 1 && packed_ok(L, x_, ldx, M, dtype) && !L.library_first)
            return tm_gemm_skinny_packed(x_, ldx, L.packed, L.packed_rows, L.bias, L.bias_dtype, out, ldc, M, L.N, L.K,
                                         out_dtype, 0, nullptr, 0, stream);
        if (dtype != TM_BF16) {
            const bool gemv = L.dtype == TM_F32 && out_dtype == TM_F32 && (L.bias_dtype == TM_NONE || L.bias_dtype == TM_F32) &&
                              M <= 16 && L.K % 4 == 0 && ldx % 4 == 0 && aligned(x_, 16) && aligned(L.w, 16);
            if (gemv) return tm_gemv_f32((const float*)x_, ldx, (const float*)L.w, (const float*)L.bias, (float*)out, ldc, M, L.N, L.K, stream);
            if (L.dtype == TM_F32 && out_dtype == TM_F32 && (L.bias_dtype == TM_NONE || L.bias_dtype == TM_F32) &&
                tm_gemm_f32_mfma_fits(x_, ldx, L.w, L.bias, out, ldc, M, L.N, L.K))
                return tm_gemm_f32_mfma((const float*)x_, ldx, (const float*)L.w, (const float*)L.bias, (float*)out, ldc, M, L.N, L.K, stream);
            return tm_gemm_nt_tiled(x_, ldx, L.w, L.bias, L.bias_dtype, out, ldc, M, L.N, L.K, dtype, out_dtype, stream);
        }
        const bool skinny = skinny_ok(L, x_, ldx, dtype);
        const bool library = L.dtype == TM_BF16;
        if (library && L.library_first) {
            const int rc = tm_gemm_library(x_, ldx, L.w, L.K, L.bias, L.bias_dtype, out, ldc, out_dtype == TM_F32, M, L.N, L.K,
                                           lib_ws, lib_ws_bytes, stream);
            if (rc != TM_ERR_UNSUPPORTED) return rc;
        }
        if (skinny && M <= SKINNY_ROWS)
            return tm_gemm_skinny(x_, ldx, L.w, L.bias, L.bias_dtype, out, ldc, M, L.N, L.K, out_dtype, 0, nullptr, 0, stream);
        if (library) {
            const int rc = tm_gemm_library(x_, ldx, L.w, L.K, L.bias, L.bias_dtype, out, ldc, out_dtype == TM_F32, M, L.N, L.K,
                                           lib_ws, lib_ws_bytes, stream);
            if (rc != TM_ERR_UNSUPPORTED) return rc;
        }
        if (skinny) {
            const int es = elem_size(dtype), eo = elem_size(out_dtype);
            for (int r0 = 0; r0 < M; r0 += SKINNY_MAX_ROWS) {
                const int m = M - r0 < SKINNY_MAX_ROWS ? M - r0 : SKINNY_MAX_ROWS;
                const int rc = tm_gemm_skinny((const char*)x_ + (size_t)r0 * ldx * es, ldx, L.w, L.bias, L.bias_dtype,
                                              (char*)out + (size_t)r0 * ldc * eo, ldc, m, L.N, L.K, out_dtype, 0, nullptr, 0, stream);
                if (rc) return rc;
            }
            return TM_OK;
        }
        return tm_gemm_nt_tiled(x_, ldx, L.w, L.bias, L.bias_dtype, out, ldc, M, L.N, L.K, dtype, out_dtype, stream);
    }

    // resid += round(x W^T + b) in the product's epilogue where a kernel does that; else the product goes to
    // delta_buf and is added by the next norm.
    int project_into_residual(const TmLinear& L, const void* x_, int ldx, int M) {
        if (L.dtype == dtype) {
            if (L.packed_parts == 1 && packed_ok(L, x_, ldx, M, dtype)) {
                delta = nullptr;
                return tm_gemm_skinny_packed(x_, ldx, L.packed, L.packed_rows, L.bias, L.bias_dtype, nullptr, L.N, M, L.N, L.K,
                                             TM_BF16, 0, resid, L.N, stream);
            }
            if (M > 0 && M <= SKINNY_ROWS && skinny_ok(L, x_, ldx, dtype)) {
                delta = nullptr;
                return tm_gemm_skinny(x_, ldx, L.w, L.bias, L.bias_dtype, nullptr, L.N, M, L.N, L.K, TM_BF16, 0, resid, L.N, stream);
            }
        }
        delta = delta_buf;
        return linear(L, x_, ldx, M, delta_buf, L.N, dtype);
    }

    // x = norm(resid + delta), resid updated
    int normed(const TmNorm& n) {
        const int rc = tm_add_rmsnorm(resid, delta, nullptr, n.w, n.w_dtype, x, dtype, s->T, p->hidden, n.eps, stream);
        delta = nullptr;
        return rc;
    }

    int attention(const TmAttentionOp& a) {
        const int T = s->T, S = s->S, nd = s->num_decode, tp = T - nd, hidden = p->hidden;
        const int HD = a.H * a.D, QKV = (a.H + 2 * a.KVH) * a.D;
        if (a.group < 0 || a.group >= s->num_groups) return TM_ERR_ARG;
        const int* tables = s->block_tables[a.group];
        const int W = s->table_width[a.group];
        const int* slots = a.write ? s->slot_mapping[a.group] : nullptr;
        void* kp = a.write ? a.k_pool : nullptr;
        void* vp = a.write ? a.v_pool : nullptr;
        if (a.rot > 0 && s->max_context_len > a.max_positions) return TM_ERR_ARG;       // beyond the rotary table
        if (!tables || W <= 0 || (long long)W * a.page < s->max_context_len) return TM_ERR_ARG;   // a table that does not reach the newest position
        const bool tables_fusable = a.rot == a.D && a.cos_t && a.sin_t;
        const bool bias_ok = !a.qkv.bias || aligned(a.qkv.bias, 16);
        const void* q = nullptr;
        int q_stride = 0;
        int rc = TM_OK;
        // 1. the kernel that starts at the norm (at most 16 tokens)
        if (dtype == TM_BF16 && a.D % 32 == 0 && delta == nullptr && a.norm.w && tables_fusable &&
            fused_decode_ok(resid, a.qkv, T) && is_pow2(a.page) && bias_ok) {
            rc = tm_fused_norm_qkv_rope(resid, a.norm.w, a.norm.w_dtype, a.norm.eps, T, hidden, a.qkv.packed, a.qkv.bias,
                                        a.qkv.bias_dtype, qkv, a.H, a.KVH, a.D, a.cos_t, a.sin_t, s->positions, slots, kp, vp,
                                        a.page, stream);
            q = qkv;
            q_stride = HD;
            ++p->taken[TM_QKV_FROM_NORM];
        } else {
            if ((rc = normed(a.norm))) return rc;
            // 2. the normed input kept in LDS (17 to 48 tokens)
            if (tables_fusable && a.D % 32 == 0 && panel_ok(a.qkv, x, hidden, T, dtype) && is_pow2(a.page) && bias_ok) {
                rc = tm_panel_qkv_rope(x, hidden, T, hidden, a.qkv.packed, a.qkv.bias, a.qkv.bias_dtype, qkv, a.H, a.KVH, a.D,
                                       a.cos_t, a.sin_t, s->positions, slots, kp, vp, a.page, stream);
                q = qkv;
                q_stride = HD;
                ++p->taken[TM_QKV_PANEL];
            } else {
                // 3. product, then rotation and cache write
                if ((rc = linear(a.qkv, x, hidden, T, qkv, QKV, dtype))) return rc;
                if (a.rot > 0 || a.write)
                    rc = tm_rope_kv_write(qkv, dtype, T, a.H, a.KVH, a.D, a.rot, a.rot > 0 ? a.cos_t : nullptr,
                                          a.rot > 0 ? a.sin_t : nullptr, a.rot > 0 ? s->positions : nullptr, slots, kp, vp,
                                          a.write ? a.page : 0, a.write ? 1 : 0, stream);
                q = qkv;
                q_stride = QKV;
                ++p->taken[TM_QKV_PLAIN];
            }
        }
        if (rc) return rc;
        // attention over the cache
        const int es = elem_size(dtype);
        const bool page_ok = a.page >= 16 && is_pow2(a.page);
        const bool head_mfma = a.D == 32 || a.D == 64 || a.D == 96 || a.D == 128;
        bool done_prefill = false, done_decode = false;
        if (tp && s->n_tiles > 0 && dtype == TM_BF16 && head_mfma && page_ok) {
            rc = tm_attn_prefill_mfma(q, q_stride, attn, HD, a.k_pool, a.v_pool, tables, W, s->prefill_tiles, s->n_tiles, a.H,
                                      a.KVH, a.D, a.page, a.scale, a.window, stream);
            done_prefill = true;
        } else if (tp && s->n_tiles > 0 && dtype == TM_F32 && a.D % 16 == 0 && a.D >= 16 && a.D <= 128 && page_ok &&
                   q_stride % 4 == 0) {
            rc = tm_attn_prefill_f32(q, q_stride, attn, HD, a.k_pool, a.v_pool, tables, W, s->prefill_tiles, s->n_tiles, a.H,
                                     a.KVH, a.D, a.page, a.scale, a.window, stream);
            done_prefill = true;
        }
        if (rc) return rc;
        const char* q_dec = (const char*)q + (size_t)tp * q_stride * es;
        char* out_dec = (char*)attn + (size_t)tp * HD * es;
        if (nd && dtype == TM_BF16 && head_mfma && page_ok && a.H / a.KVH <= 16) {
            const int chunks = (s->max_decode_context + DECODE_CHUNK - 1) / DECODE_CHUNK;
            const bool split = nd * a.KVH < DECODE_SPLIT_PAIRS && chunks > 1;
            rc = tm_attn_decode_mfma(q_dec, q_stride, out_dec, HD, a.k_pool, a.v_pool, tables + (size_t)(S - nd) * W, W,
                                     s->context_lens + (S - nd), split ? part_o : nullptr, split ? part_ml : nullptr, chunks, nd,
                                     a.H, a.KVH, a.D, a.page, a.scale, a.window, stream);
            done_decode = true;
        }
        if (rc) return rc;
        if (tp && !done_prefill && nd && !done_decode) {
            rc = tm_attn_paged_generic(q, q_stride, attn, HD, a.k_pool, a.v_pool, tables, W, s->seq_of_token, s->positions, T,
                                       a.H, a.KVH, a.D, a.page, a.scale, a.window, dtype, stream);
        } else {
            if (tp && !done_prefill)
                rc = tm_attn_paged_generic(q, q_stride, attn, HD, a.k_pool, a.v_pool, tables, W, s->seq_of_token, s->positions, tp,
                                           a.H, a.KVH, a.D, a.page, a.scale, a.window, dtype, stream);
            if (!rc && nd && !done_decode)
                rc = tm_attn_paged_generic(q_dec, q_stride, out_dec, HD, a.k_pool, a.v_pool, tables, W, s->seq_of_token + tp,
                                           s->positions + tp, nd, a.H, a.KVH, a.D, a.page, a.scale, a.window, dtype, stream);
        }
        if (rc) return rc;
        return project_into_residual(a.o, attn, HD, T);
    }

    int feed_forward(const TmFfnOp& f) {
        const int T = s->T, hidden = p->hidden;
        int rc = TM_OK;
        const bool plain = f.gate_up.dtype == dtype && f.gate_up.bias == nullptr;
        if (dtype == TM_BF16 && f.gate_up.bias == nullptr && f.I % 4 == 0 && delta == nullptr && f.norm.w &&
            f.gate_up.packed_parts == 2 && f.gate_up.packed_rows == 16 && fused_decode_ok(resid, f.gate_up, T)) {
            rc = tm_fused_norm_gate_up_silu(resid, f.norm.w, f.norm.w_dtype, f.norm.eps, T, hidden, f.gate_up.packed, act, f.I, stream);
            ++p->taken[TM_GATE_UP_FROM_NORM];
        } else {
            if ((rc = normed(f.norm))) return rc;
            if (plain && f.gate_up.packed_parts == 2 && f.gate_up.packed_rows == 16 && packed_ok(f.gate_up, x, hidden, T, dtype)) {
                rc = tm_gemm_skinny_packed(x, hidden, f.gate_up.packed, 16, nullptr, TM_NONE, act, f.I, T, f.I, hidden, TM_BF16, 1,
                                           nullptr, 0, stream);
            } else if (plain && T <= SKINNY_ROWS && skinny_ok(f.gate_up, x, hidden, dtype)) {
                rc = tm_gemm_skinny(x, hidden, f.gate_up.w, nullptr, TM_NONE, act, f.I, T, f.I, hidden, TM_BF16, 1, nullptr, 0, stream);
            } else if (plain && f.gate_up.packed_parts == 2 && f.gate_up.packed_rows == 16 && f.I % 4 == 0 &&
                       panel_ok(f.gate_up, x, hidden, T, dtype)) {
                rc = tm_panel_gate_up_silu(x, hidden, T, hidden, f.gate_up.packed, act, f.I, stream);
                ++p->taken[TM_GATE_UP_PANEL];
            } else {
                if ((rc = linear(f.gate_up, x, hidden, T, gu, 2 * f.I, dtype))) return rc;
                rc = tm_silu_mul(gu, act, dtype, T, f.I, stream);
                ++p->taken[TM_GATE_UP_PLAIN];
            }
        }
        if (rc) return rc;
        return project_into_residual(f.down, act, f.I, T);
    }
};

}  // namespace

extern "C" {

TmProgram* tm_program_create(int dtype, int hidden) {
    if ((dtype != TM_F32 && dtype != TM_BF16) || hidden <= 0) return nullptr;
    TmProgram* p = new TmProgram();
    p->dtype = dtype;
    p->hidden = hidden;
    return p;
}

void tm_program_destroy(TmProgram* p) { delete p; }

static bool linear_valid(const TmLinear& L, int dtype) {
    return L.w && L.N > 0 && L.K > 0 && L.dtype == dtype && (L.packed == nullptr || (L.packed_rows > 0 && L.packed_parts > 0));
}

int tm_program_set_embedding(TmProgram* p, const TmEmbedOp* e) {
    if (!p || !e || !e->table || e->hidden != p->hidden || e->V <= 0) return TM_ERR_ARG;
    p->embed = *e;
    p->has_embed = true;
    return TM_OK;
}

int tm_program_add_attention(TmProgram* p, const TmAttentionOp* a) {
    if (!p || !a || a->H <= 0 || a->KVH <= 0 || a->H % a->KVH || a->D <= 0 || !a->k_pool || !a->v_pool || a->page <= 0 ||
        !a->norm.w || !linear_valid(a->qkv, p->dtype) || !linear_valid(a->o, p->dtype) || a->qkv.K != p->hidden ||
        a->qkv.N != (a->H + 2 * a->KVH) * a->D || a->o.K != a->H * a->D || a->o.N != p->hidden || a->window < 0 ||
        a->rot < 0 || a->rot > a->D || (a->rot > 0 && (!a->cos_t || !a->sin_t)))
        return TM_ERR_ARG;
    Op op{};
    op.kind = 0;
    op.att = *a;
    p->ops.push_back(op);
    if (a->qkv.N > p->max_qkv) p->max_qkv = a->qkv.N;
    if (a->H * a->D > p->max_heads_d) p->max_heads_d = a->H * a->D;
    return TM_OK;
}

int tm_program_add_feed_forward(TmProgram* p, const TmFfnOp* f) {
    if (!p || !f || f->I <= 0 || !f->norm.w || !linear_valid(f->gate_up, p->dtype) || !linear_valid(f->down, p->dtype) ||
        f->gate_up.K != p->hidden || f->gate_up.N != 2 * f->I || f->down.K != f->I || f->down.N != p->hidden)
        return TM_ERR_ARG;
    Op op{};
    op.kind = 1;
    op.ffn = *f;
    p->ops.push_back(op);
    if (2 * f->I > p->max_gu) p->max_gu = 2 * f->I;
    if (f->I > p->max_act) p->max_act = f->I;
    return TM_OK;
}

int tm_program_set_final(TmProgram* p, const TmFinalOp* f) {
    if (!p || !f || !f->norm.w || !linear_valid(f->head, p->dtype) || f->head.K != p->hidden) return TM_ERR_ARG;
    p->final_op = *f;
    p->has_final = true;
    return TM_OK;
}

void tm_program_counters(const TmProgram* p, long long* out) {
    for (int i = 0; i < TM_PROGRAM_COUNTERS; ++i) out[i] = p ? p->taken[i] : 0;
}

// Bytes of workspace a step of T tokens with R logit rows needs, of which ``num_decode`` are single tokens
// whose contexts reach ``max_decode_context``.
size_t tm_program_workspace_bytes(const TmProgram* p, int T, int R, int num_decode, int max_decode_context) {
    if (!p || T <= 0) return 0;
    const size_t es = elem_size(p->dtype);
    size_t n = 0;
    n += align_up((size_t)T * p->hidden * 4);                        // residual stream
    n += align_up((size_t)T * p->hidden * es);                       // normed input
    n += align_up((size_t)T * p->max_qkv * es);                      // q|k|v
    n += align_up((size_t)T * p->max_heads_d * es);                  // attention output
    n += align_up((size_t)T * p->max_gu * es);                       // gate|up
    n += align_up((size_t)T * p->max_act * es);                      // silu(gate) * up
    n += align_up((size_t)T * p->hidden * es);                       // a product's output still to be added
    n += align_up((size_t)(R > 0 ? R : 1) * p->hidden * es);         // normed rows for the head
    size_t heads = 0, heads_d = 0;
    for (const Op& op : p->ops)
        if (op.kind == 0) {
            if ((size_t)op.att.H > heads) heads = op.att.H;
            if ((size_t)op.att.H * op.att.D > heads_d) heads_d = (size_t)op.att.H * op.att.D;
        }
    const size_t chunks = (size_t)(max_decode_context + DECODE_CHUNK - 1) / DECODE_CHUNK;
    n += align_up((size_t)num_decode * heads_d * chunks * 4);        // split decode attention: partial values
    n += align_up((size_t)num_decode * heads * chunks * 2 * 4);      // ... and their (max, sum)
    return n;
}

int tm_program_run(const TmProgram* p, const TmStep* s, void* workspace, size_t workspace_bytes, void* library_workspace,
                   size_t library_workspace_bytes, float* logits, hipStream_t stream) {
    if (!p || !s || !p->has_embed || !p->has_final || s->T <= 0 || s->S <= 0 || s->num_decode < 0 || s->num_decode > s->S ||
        s->R < 0 || !workspace || !aligned(workspace, 256) || s->num_groups < 0 || s->num_groups > TM_MAX_GROUPS)
        return TM_ERR_ARG;
    if (workspace_bytes < tm_program_workspace_bytes(p, s->T, s->R, s->num_decode, s->max_decode_context)) return TM_ERR_ARG;
    if (s->R > 0 && !logits) return TM_ERR_ARG;
    const size_t es = elem_size(p->dtype);
    const int T = s->T, R = s->R;
    char* w = (char*)workspace;
    auto take = [&](size_t bytes) {
        char* at = w;
        w += align_up(bytes);
        return (void*)at;
    };
    Run r{};
    r.p = p; r.s = s; r.stream = stream; r.lib_ws = library_workspace; r.lib_ws_bytes = library_workspace_bytes; r.dtype = p->dtype;
    r.resid = (float*)take((size_t)T * p->hidden * 4);
    r.x = take((size_t)T * p->hidden * es);
    r.qkv = take((size_t)T * p->max_qkv * es);
    r.attn = take((size_t)T * p->max_heads_d * es);
    r.gu = take((size_t)T * p->max_gu * es);
    r.act = take((size_t)T * p->max_act * es);
    r.delta_buf = take((size_t)T * p->hidden * es);
    r.hnorm = take((size_t)(R > 0 ? R : 1) * p->hidden * es);
    size_t heads = 0, heads_d = 0;
    for (const Op& op : p->ops)
        if (op.kind == 0) {
            if ((size_t)op.att.H > heads) heads = op.att.H;
            if ((size_t)op.att.H * op.att.D > heads_d) heads_d = (size_t)op.att.H * op.att.D;
        }
    const size_t chunks = (size_t)(s->max_decode_context + DECODE_CHUNK - 1) / DECODE_CHUNK;
    r.part_o = (float*)take((size_t)s->num_decode * heads_d * chunks * 4);
    r.part_ml = (float*)take((size_t)s->num_decode * heads * chunks * 2 * 4);

    int rc = tm_embed_gather(p->embed.table, p->embed.dtype, s->token_ids, r.resid, T, p->hidden, p->embed.V, stream);
    if (rc) return rc;
    for (const Op& op : p->ops) {
        rc = op.kind == 0 ? r.attention(op.att) : r.feed_forward(op.ffn);
        if (rc) return rc;
    }
    if (R == 0) return TM_OK;
    const TmFinalOp& f = p->final_op;
    rc = tm_add_rmsnorm(r.resid, r.delta, s->logit_rows, f.norm.w, f.norm.w_dtype, r.hnorm, p->dtype, R, p->hidden, f.norm.eps, stream);
    if (rc) return rc;
    return r.linear(f.head, r.hnorm, p->hidden, R, logits, f.head.N, TM_F32);
}

}  // extern "C"
