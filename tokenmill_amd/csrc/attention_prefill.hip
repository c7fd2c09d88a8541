// Paged attention for portions of prompts on MFMA (bfloat16), flash style: online softmax over
// blocks of 32 keys, nothing but registers between the two products.
//
//   A wavefront takes 16 consecutive query tokens of one request (a "tile"), one kv head and up to
//   four of the query heads that share it, so that every key and value fragment it loads feeds up
//   to four heads. Keys and values are read in place through the block table, this step's own
//   tokens included (they were stored before this kernel runs). A query at position p sees keys
//   lo..p, lo = 0 or p - window + 1                (reference src/infer/kv/context.py:70-75,
//                                                   src/infer/model/layers.py:100-107).
//   Key blocks are aligned to absolute positions (multiples of 32) and visited in ascending order,
//   so a token's result does not depend on how its prompt was cut into portions nor on the rest of
//   the batch.
//
//   S^T = K Q^T      A = keys  [16 keys x 32 d]   from K[page][slot][kvh][d]
//                    B = Q^T   [32 d x 16 tokens]
//   O^T = V^T P^T    A = V^T   [16 d x 32 keys]   from V[page][kvh][d][slot]
//                    B = P^T   [32 keys x 16 tokens] straight from the S^T accumulators
#include "common.h"
#include "api.h"

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));

union PFrag {
    u32x4_t u;
    bf16x8_t b;
};

__device__ __forceinline__ uint32_t pf_pack(float a, float b) {
    return (uint32_t)f32_to_bf16(a) | ((uint32_t)f32_to_bf16(b) << 16);
}

#define AP_HPW 4            // query heads per wavefront

template <int D>
struct KVBlock {
    PFrag k[2][D / 32];     // [16-key tile][d chunk]
    u32x2_t v[D / 16][2];   // [d tile][16-key tile]: 4 keys each
};

template <int D>
__device__ __forceinline__ void load_kv_block(KVBlock<D>& blk, int kb, int first_key, int last_key,
                                              const int* __restrict__ table,
                                              const bf16_t* __restrict__ k_pool, const bf16_t* __restrict__ v_pool,
                                              int kvh, int KVH, int page, int r, int g) {
#pragma unroll
    for (int t = 0; t < 2; ++t) {
        const int tile0 = kb * 32 + 16 * t;
        if (tile0 <= last_key && tile0 + 15 >= first_key) {         // wave-uniform: the tile holds a visible key
            const int pg = table[tile0 / page];
            const int in_page = tile0 % page;
            const bf16_t* kr = k_pool + (((size_t)pg * page + in_page + r) * KVH + kvh) * D + 8 * g;
#pragma unroll
            for (int c = 0; c < D / 32; ++c) blk.k[t][c].u = *(const u32x4_t*)(kr + 32 * c);
            const bf16_t* vr = v_pool + (((size_t)pg * KVH + kvh) * D + r) * page + in_page + 4 * g;
#pragma unroll
            for (int dt = 0; dt < D / 16; ++dt) blk.v[dt][t] = *(const u32x2_t*)(vr + (size_t)16 * dt * page);
        } else {
#pragma unroll
            for (int c = 0; c < D / 32; ++c) blk.k[t][c].u = u32x4_t{0, 0, 0, 0};
#pragma unroll
            for (int dt = 0; dt < D / 16; ++dt) blk.v[dt][t] = u32x2_t{0, 0};
        }
    }
}

// tiles: int32 [n_tiles][4] = (request index in the step, first row of the tile in the flat batch,
//                              tokens in the tile (1..16), position of its first token)
template <int D>
__global__ __launch_bounds__(64) void attn_prefill_mfma_kernel(
    const bf16_t* __restrict__ q, int q_stride, bf16_t* __restrict__ out, int out_stride,
    const bf16_t* __restrict__ k_pool, const bf16_t* __restrict__ v_pool, const int* __restrict__ block_tables,
    int table_width, const int* __restrict__ tiles, int H, int KVH, int page, float scale, int window) {
    constexpr int NDC = D / 32, NDT = D / 16;
    const int lane = threadIdx.x, r = lane % 16, g = lane / 16;
    const int G = H / KVH;
    const int splits = (G + AP_HPW - 1) / AP_HPW;
    const int kvh = blockIdx.y / splits, split = blockIdx.y % splits;
    const int h0 = kvh * G + split * AP_HPW;
    const int nh = (G - split * AP_HPW) < AP_HPW ? (G - split * AP_HPW) : AP_HPW;
    const int* tl = tiles + (size_t)blockIdx.x * 4;
    const int s = tl[0], row0 = tl[1], valid = tl[2], pos0 = tl[3];
    const int* table = block_tables + (size_t)s * table_width;
    const int last_key = pos0 + valid - 1;                           // newest key any query of the tile sees
    const int my_pos = pos0 + r < last_key ? pos0 + r : last_key;    // position of this lane's query column
    const int my_lo = (window > 0 && my_pos - window + 1 > 0) ? my_pos - window + 1 : 0;
    const int first_key = (window > 0 && pos0 - window + 1 > 0) ? pos0 - window + 1 : 0;
    const int kb0 = first_key / 32, kb1 = last_key / 32;

    PFrag qf[AP_HPW][NDC];
#pragma unroll
    for (int hh = 0; hh < AP_HPW; ++hh)
#pragma unroll
        for (int c = 0; c < NDC; ++c) {
            if (hh < nh && r < valid)
                qf[hh][c].u = *(const u32x4_t*)(q + (size_t)(row0 + r) * q_stride + (size_t)(h0 + hh) * D + 32 * c + 8 * g);
            else
                qf[hh][c].u = u32x4_t{0, 0, 0, 0};
        }
    float m[AP_HPW], l[AP_HPW];
    f32x4_t o[AP_HPW][NDT];
#pragma unroll
    for (int hh = 0; hh < AP_HPW; ++hh) {
        m[hh] = -INFINITY;
        l[hh] = 0.f;
#pragma unroll
        for (int dt = 0; dt < NDT; ++dt) o[hh][dt] = f32x4_t{0.f, 0.f, 0.f, 0.f};
    }

    KVBlock<D> cur, nxt;
    load_kv_block<D>(cur, kb0, first_key, last_key, table, k_pool, v_pool, kvh, KVH, page, r, g);
    for (int kb = kb0; kb <= kb1; ++kb) {
        if (kb < kb1) load_kv_block<D>(nxt, kb + 1, first_key, last_key, table, k_pool, v_pool, kvh, KVH, page, r, g);
        const int key0 = kb * 32;
        // values of keys nobody may see (beyond the newest key) can hold anything: clear them
        if (key0 + 31 > last_key) {
#pragma unroll
            for (int t = 0; t < 2; ++t) {
                const int k0 = key0 + 16 * t + 4 * g;
                const uint32_t keep0 = ((k0 <= last_key) ? 0x0000ffffu : 0u) | ((k0 + 1 <= last_key) ? 0xffff0000u : 0u);
                const uint32_t keep1 = ((k0 + 2 <= last_key) ? 0x0000ffffu : 0u) | ((k0 + 3 <= last_key) ? 0xffff0000u : 0u);
#pragma unroll
                for (int dt = 0; dt < NDT; ++dt) {
                    cur.v[dt][t][0] &= keep0;
                    cur.v[dt][t][1] &= keep1;
                }
            }
        }
#pragma unroll
        for (int hh = 0; hh < AP_HPW; ++hh) {
            if (hh >= nh) continue;                                  // wave-uniform
            float sc[2][4];
            float bm = -INFINITY;
#pragma unroll
            for (int t = 0; t < 2; ++t) {
                f32x4_t acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int c = 0; c < NDC; ++c)
                    acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(cur.k[t][c].b, qf[hh][c].b, acc, 0, 0, 0);
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const int kj = key0 + 16 * t + 4 * g + i;
                    sc[t][i] = (kj <= my_pos && kj >= my_lo) ? acc[i] * scale : -INFINITY;
                    bm = fmaxf(bm, sc[t][i]);
                }
            }
            bm = fmaxf(bm, __shfl_xor(bm, 16, TM_WAVE));
            bm = fmaxf(bm, __shfl_xor(bm, 32, TM_WAVE));
            const float m_new = fmaxf(m[hh], bm);
            // a column that has seen no key yet (m_new = -inf) keeps zeros
            const float corr = (m_new == -INFINITY) ? 1.f : expf(m[hh] - m_new);
            float ps = 0.f;
            float pr[2][4];
#pragma unroll
            for (int t = 0; t < 2; ++t)
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    pr[t][i] = (sc[t][i] == -INFINITY) ? 0.f : expf(sc[t][i] - m_new);
                    ps += pr[t][i];
                }
            ps += __shfl_xor(ps, 16, TM_WAVE);
            ps += __shfl_xor(ps, 32, TM_WAVE);
            l[hh] = l[hh] * corr + ps;
            m[hh] = m_new;
            PFrag pt;
            pt.u = u32x4_t{pf_pack(pr[0][0], pr[0][1]), pf_pack(pr[0][2], pr[0][3]), pf_pack(pr[1][0], pr[1][1]),
                           pf_pack(pr[1][2], pr[1][3])};
#pragma unroll
            for (int dt = 0; dt < NDT; ++dt) {
                PFrag vf;
                vf.u = u32x4_t{cur.v[dt][0][0], cur.v[dt][0][1], cur.v[dt][1][0], cur.v[dt][1][1]};
#pragma unroll
                for (int i = 0; i < 4; ++i) o[hh][dt][i] *= corr;
                o[hh][dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf.b, pt.b, o[hh][dt], 0, 0, 0);
            }
        }
        if (kb < kb1) cur = nxt;
    }
    // lane: d = 16 dt + 4 g + i of token r
    if (r < valid) {
#pragma unroll
        for (int hh = 0; hh < AP_HPW; ++hh) {
            if (hh >= nh) continue;
            const float inv = 1.f / l[hh];
            bf16_t* orow = out + (size_t)(row0 + r) * out_stride + (size_t)(h0 + hh) * D + 4 * g;
#pragma unroll
            for (int dt = 0; dt < NDT; ++dt) {
                uint2 pk;
                pk.x = pf_pack(o[hh][dt][0] * inv, o[hh][dt][1] * inv);
                pk.y = pf_pack(o[hh][dt][2] * inv, o[hh][dt][3] * inv);
                *(uint2*)(orow + 16 * dt) = pk;
            }
        }
    }
}

extern "C" int tm_attn_prefill_mfma(const void* q, int q_stride, void* out, int out_stride, const void* k_pool,
                                    const void* v_pool, const int* block_tables, int table_width, const int* tiles,
                                    int n_tiles, int H, int KVH, int D, int page, float scale, int window,
                                    hipStream_t stream) {
    if (n_tiles <= 0) return TM_OK;
    if (H <= 0 || KVH <= 0 || H % KVH || page <= 0 || page % 16 || window < 0 || table_width <= 0 ||
        (q_stride % 8) || ((uintptr_t)q % 16) || (out_stride % 4) || ((uintptr_t)out % 8) || q_stride < H * D ||
        out_stride < H * D)
        return TM_ERR_ARG;
    const int G = H / KVH;
    const int splits = (G + AP_HPW - 1) / AP_HPW;
    if ((long long)KVH * splits > 65535) return TM_ERR_ARG;
    dim3 grid(n_tiles, KVH * splits);
#define TM_PREFILL_CASE(DD)                                                                                       \
    case DD:                                                                                                      \
        attn_prefill_mfma_kernel<DD><<<grid, 64, 0, stream>>>((const bf16_t*)q, q_stride, (bf16_t*)out, out_stride, \
                                                              (const bf16_t*)k_pool, (const bf16_t*)v_pool,       \
                                                              block_tables, table_width, tiles, H, KVH, page,     \
                                                              scale, window);                                     \
        break
    switch (D) {
        TM_PREFILL_CASE(32);
        TM_PREFILL_CASE(64);
        TM_PREFILL_CASE(96);
        TM_PREFILL_CASE(128);
        default:
            return TM_ERR_ARG;
    }
#undef TM_PREFILL_CASE
    TM_CHECK_LAUNCH();
    return TM_OK;
}
