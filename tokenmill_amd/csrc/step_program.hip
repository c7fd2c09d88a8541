// A model step as a few calls: the launch sequence of a decoder, run from a list of operations that the
// model's parts described once at load (embedding, pre-norm attention, pre-norm feed-forward, final norm and
// output head).
//
// This file is the one place where a step's kernels are chosen: which product kernel for which row count
// and type, which attention kernel for which head size, page and batch (the thresholds stand in choose.h).
// The Python parts hold no such rule: the engine runs consecutive operations with one tm_program_run call,
// a part that the library has no operation for runs between two such calls through its own code, and a part
// that is called by itself (from such code, or a test) runs its own one-operation program through the same
// entry. tm_linear_run is the product rule alone, for a matrix used outside an operation.
// (The reference's step is its model's forward pass in torch: src/infer/engine/model_runner.py:76-97,
// src/infer/model/qwen2.py:43-52.)
#include "common.h"
#include "api.h"
#include "choose.h"
#include "step_program.h"

#include <stdint.h>
#include <string.h>
#include <vector>

namespace {

enum { OP_EMBED = 0, OP_ATTENTION, OP_FEED_FORWARD, OP_HEAD };
constexpr int TM_MAX_SUMS = 8;          // most groups of blocks a product's K is split over (tm_stream_linear_parts)

struct Op {
    int kind;
    TmEmbedOp embed;
    TmAttentionOp att;
    TmFfnOp ffn;
    TmFinalOp head;
};

inline size_t align_up(size_t n) { return (n + 255) & ~(size_t)255; }
inline bool is_pow2(int x) { return x > 0 && (x & (x - 1)) == 0; }
inline bool aligned(const void* p, int to) { return ((uintptr_t)p % to) == 0; }
inline int elem_size(int dtype) { return dtype == TM_BF16 ? 2 : 4; }

}  // namespace

struct TmProgram {
    int dtype = TM_BF16;
    int hidden = 0;
    std::vector<Op> ops;
    // the widest of each kind of activation over all operations
    int max_qkv = 0, max_gu = 0, max_act = 0, max_heads = 0, max_heads_d = 0;
    // a matrix the checkpoint stores in 32-bit stays 32-bit in a bfloat16 model: its product runs in 32-bit on a
    // widened copy of the activations; the widest input and output of such products
    int max_wide_in = 0, max_wide_out = 0;
    TmHook hook = nullptr;
    void* hook_user = nullptr;
    TmTune tune{0, 3, 0};
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

// `most`: the most rows the family is preferred for at this model's width (tm_skinny_rows, tm_from_norm_rows)
bool fused_decode_ok(const float* resid, const TmLinear& L, int M, int most) {
    return resid && L.packed && M > 0 && M <= most && L.K % 8 == 0 && fused_lds_fits(M, L.K) && aligned(resid, 16);
}

bool packed_ok(const TmLinear& L, const void* x, int ldx, int M, int dtype, int most) {
    return L.packed && M > 0 && M <= most && dtype == TM_BF16 && L.dtype == TM_BF16 && L.K % 8 == 0 && ldx % 8 == 0 &&
           aligned(x, 16);
}

bool skinny_ok(const TmLinear& L, const void* x, int ldx, int dtype) {
    return dtype == TM_BF16 && L.dtype == TM_BF16 && L.K % 8 == 0 && ldx % 8 == 0 && aligned(x, 16) && aligned(L.w, 16);
}

// `beyond`: the rows up to which the kernels for at most 16 rows are preferred
bool panel_ok(const TmLinear& L, const void* x, int ldx, int M, int dtype, int beyond, int most_rows) {
    return L.packed && M > beyond && M <= most_rows && dtype == TM_BF16 && ldx % 8 == 0 && aligned(x, 16) &&
           tm_gemm_panel_fits(M, L.K);
}

// the products that stream a packed matrix once for up to 64 tokens (gemm_stream.hip)
bool stream_ok(const TmLinear& L, const void* x, int ldx, int M, int dtype, int beyond) {
    return L.packed && M > beyond && M <= TM_STREAM_ROWS && dtype == TM_BF16 && L.dtype == TM_BF16 && ldx % 8 == 0 &&
           aligned(x, 16) && tm_gemm_stream_fits(M, L.K);
}

// The product rule. x_dtype: type of x (the model's activations); the matrix has its own (L.dtype).
struct Products {
    hipStream_t stream;
    void* lib_ws;
    size_t lib_ws_bytes;
    TmTune tune;
    float* wide_in = nullptr;           // room for a product's input and output in 32-bit (see TmProgram::max_wide_in)
    float* wide_out = nullptr;
    int skinny_rows = TM_SKINNY_ROWS;   // rows up to which the packed products for at most 16 rows are preferred (tm_skinny_rows)

    int library(const TmLinear& L, const void* x, int ldx, int M, void* out, int ldc, int out_dtype) const {
        return tm_gemm_library(x, ldx, L.w, L.K, L.bias, L.bias_dtype, out, ldc, out_dtype == TM_F32, M, L.N, L.K, lib_ws,
                               lib_ws_bytes, &tune, stream);
    }

    int linear(const TmLinear& L, int dtype, const void* x, int ldx, int M, void* out, int ldc, int out_dtype) const {
        if (M == 0) return TM_OK;
        if (L.dtype != dtype) {
            // a 32-bit matrix under bfloat16 activations: the activations are widened, the product runs in 32-bit,
            // and the result is rounded to the type asked for
            if (L.dtype != TM_F32 || dtype != TM_BF16 || !wide_in || !wide_out || ldx != L.K) return TM_ERR_ARG;
            int rc = tm_convert(x, TM_BF16, wide_in, TM_F32, (long long)M * L.K, stream);
            if (rc) return rc;
            if (out_dtype == TM_F32) return linear(L, TM_F32, wide_in, L.K, M, out, ldc, TM_F32);
            if (ldc != L.N) return TM_ERR_ARG;
            if ((rc = linear(L, TM_F32, wide_in, L.K, M, wide_out, L.N, TM_F32))) return rc;
            return tm_convert(wide_out, TM_F32, out, TM_BF16, (long long)M * L.N, stream);
        }
        if (L.packed_parts == 1 && packed_ok(L, x, ldx, M, dtype, skinny_rows) && !L.library_first)
            return tm_gemm_skinny_packed(x, ldx, L.packed, L.packed_rows, L.bias, L.bias_dtype, out, ldc, M, L.N, L.K,
                                         out_dtype, 0, nullptr, 0, stream);
        if (dtype != TM_BF16) {
            const bool plain32 = out_dtype == TM_F32 && (L.bias_dtype == TM_NONE || L.bias_dtype == TM_F32);
            if (plain32 && M <= TM_GEMV_F32_ROWS && L.K % 4 == 0 && ldx % 4 == 0 && aligned(x, 16) && aligned(L.w, 16))
                return tm_gemv_f32((const float*)x, ldx, (const float*)L.w, (const float*)L.bias, (float*)out, ldc, M, L.N, L.K, stream);
            if (plain32 && tm_gemm_f32_mfma_fits(x, ldx, L.w, L.bias, out, ldc, M, L.N, L.K))
                return tm_gemm_f32_mfma((const float*)x, ldx, (const float*)L.w, (const float*)L.bias, (float*)out, ldc, M, L.N, L.K, stream);
            return tm_gemm_nt_tiled(x, ldx, L.w, L.bias, L.bias_dtype, out, ldc, M, L.N, L.K, dtype, out_dtype, stream);
        }
        const bool skinny = skinny_ok(L, x, ldx, dtype);
        if (L.library_first) {
            const int rc = library(L, x, ldx, M, out, ldc, out_dtype);
            if (rc != TM_ERR_UNSUPPORTED) return rc;
        }
        if (skinny && M <= TM_SKINNY_ROWS)
            return tm_gemm_skinny(x, ldx, L.w, L.bias, L.bias_dtype, out, ldc, M, L.N, L.K, out_dtype, 0, nullptr, 0, stream);
        {
            const int rc = library(L, x, ldx, M, out, ldc, out_dtype);
            if (rc != TM_ERR_UNSUPPORTED) return rc;
        }
        if (skinny) {
            const int es = elem_size(dtype), eo = elem_size(out_dtype);
            for (int r0 = 0; r0 < M; r0 += TM_SKINNY_MAX_ROWS) {
                const int m = M - r0 < TM_SKINNY_MAX_ROWS ? M - r0 : TM_SKINNY_MAX_ROWS;
                const int rc = tm_gemm_skinny((const char*)x + (size_t)r0 * ldx * es, ldx, L.w, L.bias, L.bias_dtype,
                                              (char*)out + (size_t)r0 * ldc * eo, ldc, m, L.N, L.K, out_dtype, 0, nullptr, 0, stream);
                if (rc) return rc;
            }
            return TM_OK;
        }
        return tm_gemm_nt_tiled(x, ldx, L.w, L.bias, L.bias_dtype, out, ldc, M, L.N, L.K, dtype, out_dtype, stream);
    }

    // Is there a kernel that adds round(x W^T + b) into a 32-bit accumulator in its epilogue?
    bool accumulates(const TmLinear& L, int dtype, const void* x, int ldx, int M) const {
        if (L.dtype != dtype || M <= 0) return false;
        return (L.packed_parts == 1 && packed_ok(L, x, ldx, M, dtype, skinny_rows)) ||
               (M <= TM_SKINNY_ROWS && skinny_ok(L, x, ldx, dtype));
    }

    int accumulate(const TmLinear& L, int dtype, const void* x, int ldx, int M, float* accum, int ldacc) const {
        if (L.packed_parts == 1 && packed_ok(L, x, ldx, M, dtype, skinny_rows))
            return tm_gemm_skinny_packed(x, ldx, L.packed, L.packed_rows, L.bias, L.bias_dtype, nullptr, L.N, M, L.N, L.K, TM_BF16,
                                         0, accum, ldacc, stream);
        return tm_gemm_skinny(x, ldx, L.w, L.bias, L.bias_dtype, nullptr, L.N, M, L.N, L.K, TM_BF16, 0, accum, ldacc, stream);
    }
};

struct Run {
    const TmProgram* p;
    const TmStep* s;
    hipStream_t stream;
    Products products;
    int dtype;
    int from_norm_rows;                 // rows up to which q|k|v and gate|up start at the norm (tm_from_norm_rows)
    bool labels;
    // what crosses between operations
    float* resid;
    const void* delta;                  // product output still to be added to the residual stream
    const void* x_in;                   // the next operation's input, already normed
    const void* qkv_in;                 // the next (attention) operation's q|k|v, already encoded and stored
    bool accumulate;
    // workspace
    void *x, *qkv, *attn, *gu, *act, *delta_buf, *hnorm;
    float *part_o, *part_ml;
    float* sums;                        // room for the partial sums of a product whose K is split over blocks, or null
    int pending_sums = 0;               // that many partial sums [T, hidden] in `sums` are still to be added to the residual

    struct Label {
        const Run* r;
        int op, label;
        Label(const Run* r_, int op_, int label_) : r(r_), op(op_), label(label_) {
            if (r->labels && r->p->hook) r->p->hook(r->p->hook_user, op, label, 1);
        }
        ~Label() {
            if (r->labels && r->p->hook) r->p->hook(r->p->hook_user, op, label, 0);
        }
    };

    int linear(const TmLinear& L, const void* x_, int ldx, int M, void* out, int ldc, int out_dtype) {
        return products.linear(L, dtype, x_, ldx, M, out, ldc, out_dtype);
    }

    // resid += round(x W^T + b) in the product's epilogue where a kernel does that and the caller lets it; else the
    // product goes to delta_buf and is added by the next norm (or handed back).
    int project(const TmLinear& L, const void* x_, int ldx, int M) {
        // 17 to 64 rows over a matrix with few rows of output: K split over groups of blocks, whose partial sums the
        // next norm adds up (or, where the caller wants the result itself, a small kernel)
        const int groups = (sums && L.N == p->hidden && L.packed_parts == 1 && stream_ok(L, x_, ldx, M, dtype, products.skinny_rows))
                               ? tm_stream_linear_parts(L.N, L.K) : 1;
        if (groups >= 2 && groups <= TM_MAX_SUMS) {
            const int rc = tm_stream_linear_split(x_, ldx, M, L.K, L.packed, L.packed_rows, L.N, L.bias, L.bias_dtype, sums, stream);
            if (rc) return rc;
            delta = nullptr;
            pending_sums = groups;
            return accumulate && resid ? TM_OK : settle();
        }
        if (accumulate && resid && products.accumulates(L, dtype, x_, ldx, M)) {
            delta = nullptr;
            return products.accumulate(L, dtype, x_, ldx, M, resid, L.N);
        }
        delta = delta_buf;
        return linear(L, x_, ldx, M, delta_buf, L.N, dtype);
    }

    // The partial sums become the tensor the product would have stored: delta.
    int settle() {
        if (!pending_sums) return TM_OK;
        const size_t n = (size_t)s->T * p->hidden;
        const int rc = tm_sum_parts(sums, pending_sums, n, delta_buf, dtype, n, stream);
        pending_sums = 0;
        delta = delta_buf;
        return rc;
    }

    // out = norm(resid + what is pending), for all rows (resid updated) or the rows named
    int add_norm(const TmNorm& n, const int* rows, void* out, int R) {
        if (!n.w || !resid) return TM_ERR_ARG;
        int rc;
        if (pending_sums)
            rc = tm_add_rmsnorm_parts(resid, sums, pending_sums, (size_t)s->T * p->hidden, rows, n.w, n.w_dtype, out, dtype, R,
                                      p->hidden, n.eps, stream);
        else
            rc = tm_add_rmsnorm(resid, delta, rows, n.w, n.w_dtype, out, dtype, R, p->hidden, n.eps, stream);
        delta = nullptr;
        pending_sums = 0;
        return rc;
    }

    // x = norm(resid + delta), resid updated
    int normed(const TmNorm& n) { return add_norm(n, nullptr, x, s->T); }

    int embedding(int op, const TmEmbedOp& e) {
        Label l(this, op, TM_LABEL_EMBED);
        if (!resid) return TM_ERR_ARG;
        delta = nullptr;
        pending_sums = 0;
        return tm_embed_gather(e.table, e.dtype, s->token_ids, resid, s->T, p->hidden, e.V, stream);
    }

    int attention(int op, const TmAttentionOp& a) {
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
        if (a.write && !slots) return TM_ERR_ARG;
        if (!s->positions || !s->context_lens || !s->seq_of_token) return TM_ERR_ARG;
        const bool tables_fusable = a.rot == a.D && a.cos_t && a.sin_t;
        const bool bias_ok = !a.qkv.bias || aligned(a.qkv.bias, 16);
        const void* q = nullptr;
        int q_stride = 0;
        int rc = TM_OK;
        if (qkv_in) {                       // projected, encoded and stored by the caller
            q = qkv_in;
            q_stride = QKV;
            qkv_in = nullptr;
        } else {
            Label l(this, op, TM_LABEL_QKV);
            const bool own_norm = x_in == nullptr;
            // 1. the kernel that starts at the norm (at most 16 tokens)
            if (own_norm && dtype == TM_BF16 && a.qkv.dtype == TM_BF16 && a.D % 32 == 0 && delta == nullptr && !pending_sums && a.norm.w &&
                tables_fusable && fused_decode_ok(resid, a.qkv, T, from_norm_rows) && is_pow2(a.page) && bias_ok) {
                rc = tm_fused_norm_qkv_rope(resid, a.norm.w, a.norm.w_dtype, a.norm.eps, T, hidden, a.qkv.packed, a.qkv.bias,
                                            a.qkv.bias_dtype, qkv, a.H, a.KVH, a.D, a.cos_t, a.sin_t, s->positions, slots, kp, vp,
                                            a.page, stream);
                q = qkv;
                q_stride = HD;
                ++p->taken[TM_QKV_FROM_NORM];
            } else {
                const void* xn = x_in;
                x_in = nullptr;
                if (own_norm) {
                    if ((rc = normed(a.norm))) return rc;
                    xn = x;
                }
                // 2. the normed input kept in LDS (17 to 48 tokens)
                if (tables_fusable && a.D % 32 == 0 && a.qkv.dtype == TM_BF16 && panel_ok(a.qkv, xn, hidden, T, dtype, from_norm_rows, TM_PANEL_QKV_ROWS) &&
                    is_pow2(a.page) && bias_ok) {
                    rc = tm_panel_qkv_rope(xn, hidden, T, hidden, a.qkv.packed, a.qkv.bias, a.qkv.bias_dtype, qkv, a.H, a.KVH, a.D,
                                           a.cos_t, a.sin_t, s->positions, slots, kp, vp, a.page, stream);
                    q = qkv;
                    q_stride = HD;
                    ++p->taken[TM_QKV_PANEL];
                } else if (tables_fusable && a.D % 32 == 0 && a.qkv.packed_parts == 1 && stream_ok(a.qkv, xn, hidden, T, dtype, from_norm_rows) &&
                           is_pow2(a.page)) {
                    // 3. the packed matrix streamed once for up to 64 tokens
                    rc = tm_stream_qkv_rope(xn, hidden, T, hidden, a.qkv.packed, a.qkv.packed_rows, a.qkv.bias, a.qkv.bias_dtype,
                                            qkv, a.H, a.KVH, a.D, a.cos_t, a.sin_t, s->positions, slots, kp, vp, a.page, stream);
                    q = qkv;
                    q_stride = HD;
                    ++p->taken[TM_QKV_STREAM];
                } else {
                    // 4. product, then rotation and cache write
                    if ((rc = linear(a.qkv, xn, hidden, T, qkv, QKV, dtype))) return rc;
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
        }
        {
            Label l(this, op, TM_LABEL_ATTENTION);
            const int es = elem_size(dtype);
            const bool page_ok = a.page >= 16 && is_pow2(a.page);
            const bool head_mfma = a.D == 32 || a.D == 64 || a.D == 96 || a.D == 128;
            const bool q_ok = aligned(q, 16) && q_stride % 8 == 0;
            bool done_prefill = false, done_decode = false;
            if (tp && s->n_tiles > 0 && s->prefill_tiles && dtype == TM_BF16 && head_mfma && page_ok && q_ok) {
                if (tm_prefill_shares_keys(a.D, a.H, a.KVH, s->n_tiles) && tm_attn_prefill_shared_takes(a.H, a.KVH, a.D) &&
                    HD % 4 == 0 && aligned(attn, 8)) {
                    ++p->taken[TM_PREFILL_SHARED_KEYS];
                    rc = tm_attn_prefill_shared(q, q_stride, attn, HD, a.k_pool, a.v_pool, tables, W, s->prefill_tiles,
                                                s->n_tiles, a.H, a.KVH, a.D, a.page, a.scale, a.window, stream);
                } else {
                    ++p->taken[TM_PREFILL_SPLIT_KEYS];
                    rc = tm_attn_prefill_mfma(q, q_stride, attn, HD, a.k_pool, a.v_pool, tables, W, s->prefill_tiles,
                                              s->n_tiles, a.H, a.KVH, a.D, a.page, a.scale, a.window, stream);
                }
                done_prefill = true;
            } else if (tp && s->n_tiles > 0 && s->prefill_tiles && dtype == TM_F32 && a.D % 16 == 0 && a.D >= 16 &&
                       a.D <= 128 && page_ok && q_stride % 4 == 0 && aligned(q, 16)) {
                rc = tm_attn_prefill_f32(q, q_stride, attn, HD, a.k_pool, a.v_pool, tables, W, s->prefill_tiles, s->n_tiles, a.H,
                                         a.KVH, a.D, a.page, a.scale, a.window, stream);
                done_prefill = true;
            }
            if (rc) return rc;
            const char* q_dec = (const char*)q + (size_t)tp * q_stride * es;
            char* out_dec = (char*)attn + (size_t)tp * HD * es;
            if (nd && dtype == TM_BF16 && head_mfma && page_ok && a.H / a.KVH <= 16 && q_ok) {
                const bool split = tm_decode_splits(nd, a.KVH, s->max_decode_context);
                rc = tm_attn_decode_mfma(q_dec, q_stride, out_dec, HD, a.k_pool, a.v_pool, tables + (size_t)(S - nd) * W, W,
                                         s->context_lens + (S - nd), split ? part_o : nullptr, split ? part_ml : nullptr,
                                         tm_decode_chunks(s->max_decode_context), nd, a.H, a.KVH, a.D, a.page, a.scale, a.window,
                                         stream);
                done_decode = true;
            }
            if (rc) return rc;
            if (tp && !done_prefill && nd && !done_decode) {
                rc = tm_attn_paged_generic(q, q_stride, attn, HD, a.k_pool, a.v_pool, tables, W, s->seq_of_token, s->positions, T,
                                           a.H, a.KVH, a.D, a.page, a.scale, a.window, dtype, stream);
            } else {
                if (tp && !done_prefill)
                    rc = tm_attn_paged_generic(q, q_stride, attn, HD, a.k_pool, a.v_pool, tables, W, s->seq_of_token, s->positions,
                                               tp, a.H, a.KVH, a.D, a.page, a.scale, a.window, dtype, stream);
                if (!rc && nd && !done_decode)
                    rc = tm_attn_paged_generic(q_dec, q_stride, out_dec, HD, a.k_pool, a.v_pool, tables, W, s->seq_of_token + tp,
                                               s->positions + tp, nd, a.H, a.KVH, a.D, a.page, a.scale, a.window, dtype, stream);
            }
            if (rc) return rc;
        }
        Label l(this, op, TM_LABEL_O_PROJ);
        return project(a.o, attn, HD, T);
    }

    int feed_forward(int op, const TmFfnOp& f) {
        const int T = s->T, hidden = p->hidden;
        int rc = TM_OK;
        {
            Label l(this, op, TM_LABEL_GATE_UP);
            const bool own_norm = x_in == nullptr;
            const bool plain = f.gate_up.dtype == dtype && f.gate_up.bias == nullptr;
            const bool two_parts = f.gate_up.packed_parts == 2 && f.gate_up.packed_rows == 16;
            if (own_norm && dtype == TM_BF16 && plain && f.I % 4 == 0 && delta == nullptr && !pending_sums && f.norm.w && two_parts &&
                fused_decode_ok(resid, f.gate_up, T, from_norm_rows)) {
                rc = tm_fused_norm_gate_up_silu(resid, f.norm.w, f.norm.w_dtype, f.norm.eps, T, hidden, f.gate_up.packed, act, f.I, stream);
                ++p->taken[TM_GATE_UP_FROM_NORM];
            } else {
                const void* xn = x_in;
                x_in = nullptr;
                if (own_norm) {
                    if ((rc = normed(f.norm))) return rc;
                    xn = x;
                }
                if (plain && two_parts && packed_ok(f.gate_up, xn, hidden, T, dtype, from_norm_rows)) {
                    rc = tm_gemm_skinny_packed(xn, hidden, f.gate_up.packed, 16, nullptr, TM_NONE, act, f.I, T, f.I, hidden, TM_BF16, 1,
                                               nullptr, 0, stream);
                    ++p->taken[TM_GATE_UP_PLAIN];
                } else if (plain && two_parts && f.I % 4 == 0 && stream_ok(f.gate_up, xn, hidden, T, dtype, from_norm_rows)) {
                    rc = tm_stream_gate_up_silu(xn, hidden, T, hidden, f.gate_up.packed, act, f.I, stream);
                    ++p->taken[TM_GATE_UP_STREAM];
                } else if (plain && T <= TM_SKINNY_ROWS && skinny_ok(f.gate_up, xn, hidden, dtype)) {   // (a matrix without a packed copy)
                    rc = tm_gemm_skinny(xn, hidden, f.gate_up.w, nullptr, TM_NONE, act, f.I, T, f.I, hidden, TM_BF16, 1, nullptr, 0, stream);
                    ++p->taken[TM_GATE_UP_PLAIN];
                } else {
                    if ((rc = linear(f.gate_up, xn, hidden, T, gu, 2 * f.I, dtype))) return rc;
                    rc = tm_silu_mul(gu, act, dtype, T, f.I, stream);
                    ++p->taken[TM_GATE_UP_PLAIN];
                }
            }
            if (rc) return rc;
        }
        Label l(this, op, TM_LABEL_DOWN);
        return project(f.down, act, f.I, T);
    }

    int head(int op, const TmFinalOp& f, float* logits) {
        const int R = s->R;
        if (R == 0) return TM_OK;
        if (!logits || !s->logit_rows) return TM_ERR_ARG;
        const void* h = x_in;                   // rows already normed (R of them), or the residual's rows to norm
        x_in = nullptr;
        if (!h) {
            Label l(this, op, TM_LABEL_NORM);
            const int rc = add_norm(f.norm, s->logit_rows, hnorm, R);
            if (rc) return rc;
            h = hnorm;
        }
        delta = nullptr;
        pending_sums = 0;
        Label l(this, op, TM_LABEL_HEAD);
        return linear(f.head, h, p->hidden, R, logits, f.head.N, TM_F32);
    }
};

bool linear_valid(const TmLinear& L) {
    return L.w && L.N > 0 && L.K > 0 && (L.dtype == TM_F32 || L.dtype == TM_BF16) &&
           (L.packed == nullptr || (L.packed_rows > 0 && L.packed_parts > 0 && L.dtype == TM_BF16));
}

// A matrix a program of type `dtype` can multiply by: of that type, or 32-bit under bfloat16 activations.
bool linear_fits(TmProgram* p, const TmLinear& L) {
    if (!linear_valid(L)) return false;
    if (L.dtype == p->dtype) return true;
    if (L.dtype != TM_F32 || p->dtype != TM_BF16) return false;
    if (L.K > p->max_wide_in) p->max_wide_in = L.K;
    if (L.N > p->max_wide_out) p->max_wide_out = L.N;
    return true;
}

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

void tm_program_set_hook(TmProgram* p, TmHook hook, void* user) {
    if (!p) return;
    p->hook = hook;
    p->hook_user = user;
}

int tm_program_set_tune(TmProgram* p, int candidates, int every) {
    if (!p || candidates < 0 || candidates > 32 || (every && candidates < 2)) return TM_ERR_ARG;
    p->tune = TmTune{candidates, 3, every ? 1 : 0};
    return TM_OK;
}

int tm_program_add_embedding(TmProgram* p, const TmEmbedOp* e) {
    if (!p || !e || !e->table || e->hidden != p->hidden || e->V <= 0) return -1;
    Op op{};
    op.kind = OP_EMBED;
    op.embed = *e;
    p->ops.push_back(op);
    return (int)p->ops.size() - 1;
}

int tm_program_add_attention(TmProgram* p, const TmAttentionOp* a) {
    if (!p || !a || a->H <= 0 || a->KVH <= 0 || a->H % a->KVH || a->D <= 0 || !a->k_pool || !a->v_pool || a->page <= 0 ||
        !linear_fits(p, a->qkv) || !linear_fits(p, a->o) || a->qkv.K != p->hidden || a->qkv.N != (a->H + 2 * a->KVH) * a->D || a->o.K != a->H * a->D || a->o.N != p->hidden ||
        a->window < 0 || a->rot < 0 || a->rot > a->D || (a->rot > 0 && (!a->cos_t || !a->sin_t)))
        return -1;
    Op op{};
    op.kind = OP_ATTENTION;
    op.att = *a;
    p->ops.push_back(op);
    if (a->qkv.N > p->max_qkv) p->max_qkv = a->qkv.N;
    if (a->H > p->max_heads) p->max_heads = a->H;
    if (a->H * a->D > p->max_heads_d) p->max_heads_d = a->H * a->D;
    return (int)p->ops.size() - 1;
}

int tm_program_add_feed_forward(TmProgram* p, const TmFfnOp* f) {
    if (!p || !f || f->I <= 0 || !linear_fits(p, f->gate_up) || !linear_fits(p, f->down) || f->gate_up.K != p->hidden || f->gate_up.N != 2 * f->I || f->down.K != f->I ||
        f->down.N != p->hidden)
        return -1;
    Op op{};
    op.kind = OP_FEED_FORWARD;
    op.ffn = *f;
    p->ops.push_back(op);
    if (2 * f->I > p->max_gu) p->max_gu = 2 * f->I;
    if (f->I > p->max_act) p->max_act = f->I;
    return (int)p->ops.size() - 1;
}

int tm_program_add_head(TmProgram* p, const TmFinalOp* f) {
    if (!p || !f || !linear_fits(p, f->head) || f->head.K != p->hidden) return -1;
    Op op{};
    op.kind = OP_HEAD;
    op.head = *f;
    p->ops.push_back(op);
    return (int)p->ops.size() - 1;
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
    n += align_up((size_t)T * p->hidden * es);                       // normed input
    n += align_up((size_t)T * p->max_qkv * es);                      // q|k|v
    n += align_up((size_t)T * p->max_heads_d * es);                  // attention output
    n += align_up((size_t)T * p->max_gu * es);                       // gate|up
    n += align_up((size_t)T * p->max_act * es);                      // silu(gate) * up
    n += align_up((size_t)T * p->hidden * es);                       // a product's output still to be added
    n += align_up((size_t)(R > 0 ? R : 1) * p->hidden * es);         // normed rows for the head
    const size_t chunks = (size_t)tm_decode_chunks(max_decode_context > 0 ? max_decode_context : 1);
    n += align_up((size_t)num_decode * p->max_heads_d * chunks * 4); // split decode attention: partial values
    n += align_up((size_t)num_decode * p->max_heads * chunks * 2 * 4);   // ... and their (max, sum)
    if (T <= TM_STREAM_ROWS && p->dtype == TM_BF16)
        n += align_up((size_t)TM_MAX_SUMS * T * p->hidden * 4);      // partial sums of a product whose K is split over blocks
    const size_t rows = (size_t)(T > R ? T : R);
    n += align_up(rows * p->max_wide_in * 4);                        // 32-bit copies around the product of a 32-bit matrix
    n += align_up(rows * p->max_wide_out * 4);
    return n;
}

int tm_program_run(const TmProgram* p, int first, int count, const TmStep* s, TmStream* io, void* workspace,
                   size_t workspace_bytes, void* library_workspace, size_t library_workspace_bytes, float* logits,
                   int flags, hipStream_t stream) {
    if (!p || !s || !io || first < 0 || count <= 0 || (size_t)first + (size_t)count > p->ops.size() || s->T <= 0 || s->S < 0 ||
        s->num_decode < 0 || s->num_decode > s->S || s->num_decode > s->T || s->R < 0 || !workspace || !aligned(workspace, 256) ||
        s->num_groups < 0 || s->num_groups > TM_MAX_GROUPS)
        return TM_ERR_ARG;
    if (workspace_bytes < tm_program_workspace_bytes(p, s->T, s->R, s->num_decode, s->max_decode_context)) return TM_ERR_ARG;
    if (!io->resid && (io->accumulate || count != 1 || (!io->x && !io->qkv))) return TM_ERR_ARG;
    if (io->qkv && p->ops[first].kind != OP_ATTENTION) return TM_ERR_ARG;
    const size_t es = elem_size(p->dtype);
    const int T = s->T, R = s->R;
    char* w = (char*)workspace;
    auto take = [&](size_t bytes) {
        char* at = w;
        w += align_up(bytes);
        return (void*)at;
    };
    Run r{};
    r.p = p; r.s = s; r.stream = stream; r.dtype = p->dtype;
    r.products.stream = stream; r.products.lib_ws = library_workspace; r.products.lib_ws_bytes = library_workspace_bytes;
    r.products.tune = p->tune;
    if (flags & TM_RUN_TUNE_AT_ONCE) r.products.tune.after = 1;
    r.products.skinny_rows = tm_skinny_rows(p->hidden);
    r.from_norm_rows = tm_from_norm_rows(p->hidden);
    r.labels = (flags & TM_RUN_LABELS) != 0;
    r.resid = io->resid; r.delta = io->delta; r.x_in = io->x; r.qkv_in = io->qkv; r.accumulate = io->accumulate != 0;
    r.x = take((size_t)T * p->hidden * es);
    r.qkv = take((size_t)T * p->max_qkv * es);
    r.attn = take((size_t)T * p->max_heads_d * es);
    r.gu = take((size_t)T * p->max_gu * es);
    r.act = take((size_t)T * p->max_act * es);
    r.delta_buf = take((size_t)T * p->hidden * es);
    r.hnorm = take((size_t)(R > 0 ? R : 1) * p->hidden * es);
    const size_t chunks = (size_t)tm_decode_chunks(s->max_decode_context > 0 ? s->max_decode_context : 1);
    r.part_o = (float*)take((size_t)s->num_decode * p->max_heads_d * chunks * 4);
    r.part_ml = (float*)take((size_t)s->num_decode * p->max_heads * chunks * 2 * 4);
    r.sums = (T <= TM_STREAM_ROWS && p->dtype == TM_BF16) ? (float*)take((size_t)TM_MAX_SUMS * T * p->hidden * 4) : nullptr;
    const size_t rows = (size_t)(T > R ? T : R);
    if (p->max_wide_in) r.products.wide_in = (float*)take(rows * p->max_wide_in * 4);
    if (p->max_wide_out) r.products.wide_out = (float*)take(rows * p->max_wide_out * 4);
    int rc = TM_OK;
    for (int i = first; i < first + count && !rc; ++i) {
        const Op& op = p->ops[i];
        switch (op.kind) {
            case OP_EMBED: rc = r.embedding(i, op.embed); break;
            case OP_ATTENTION: rc = r.attention(i, op.att); break;
            case OP_FEED_FORWARD: rc = r.feed_forward(i, op.ffn); break;
            default: rc = r.head(i, op.head, logits); break;
        }
    }
    if (!rc) rc = r.settle();                   // partial sums do not cross to the caller: it gets the tensor
    io->delta = r.delta;
    io->x = nullptr;
    io->qkv = nullptr;
    return rc;
}

int tm_linear_accumulates(const TmLinear* L, int x_dtype, const void* x, int ldx, int M) {
    if (!L || !linear_valid(*L)) return 0;
    Products pr{};
    return pr.accumulates(*L, x_dtype, x, ldx, M) ? 1 : 0;
}

int tm_linear_run(const TmLinear* L, int x_dtype, const void* x, int ldx, int M, void* out, int ldc, int out_dtype,
                  float* accum, int ldacc, void* library_workspace, size_t library_workspace_bytes, const TmTune* tune,
                  hipStream_t stream) {
    if (!L || !linear_valid(*L) || !x || M < 0 || ldx < L->K || (x_dtype != TM_F32 && x_dtype != TM_BF16)) return TM_ERR_ARG;
    Products pr{};
    pr.stream = stream; pr.lib_ws = library_workspace; pr.lib_ws_bytes = library_workspace_bytes;
    pr.tune = tune ? *tune : TmTune{0, 3, 0};
    if (accum) {
        if (ldacc < L->N || !pr.accumulates(*L, x_dtype, x, ldx, M)) return TM_ERR_ARG;
        return pr.accumulate(*L, x_dtype, x, ldx, M, accum, ldacc);
    }
    if (!out || ldc < L->N || (out_dtype != TM_F32 && out_dtype != TM_BF16) || (x_dtype == TM_F32 && out_dtype != TM_F32))
        return TM_ERR_ARG;
    return pr.linear(*L, x_dtype, x, ldx, M, out, ldc, out_dtype);
}

int tm_rule(const char* name) {
    if (!name) return -1;
    if (!strcmp(name, "skinny_rows")) return TM_SKINNY_ROWS;
    if (!strcmp(name, "panel_qkv_rows")) return TM_PANEL_QKV_ROWS;
    if (!strcmp(name, "stream_rows")) return TM_STREAM_ROWS;
    if (!strcmp(name, "skinny_max_rows")) return TM_SKINNY_MAX_ROWS;
    if (!strcmp(name, "gemv_f32_rows")) return TM_GEMV_F32_ROWS;
    if (!strcmp(name, "decode_chunk")) return TM_DECODE_CHUNK;
    if (!strcmp(name, "decode_split_pairs")) return TM_DECODE_SPLIT_PAIRS;
    return -1;
}

int tm_decode_split_chunks(int requests, int kv_heads, int max_context) {
    return tm_decode_splits(requests, kv_heads, max_context) ? tm_decode_chunks(max_context) : 0;
}

}  // extern "C"
