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

#define AP_HPW 2            // query heads per wavefront
#define AP_KSPLIT 4         // wavefronts of a block, each taking every fourth block of 32 keys

typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef float f32x2_t __attribute__((ext_vector_type(2)));

// two floats -> packed bfloat16 (round to nearest even, one instruction on gfx950)
__device__ __forceinline__ uint32_t pk_bf16(float a, float b) {
    const bf16x2_t v = __builtin_convertvector(f32x2_t{a, b}, bf16x2_t);
    return *(const uint32_t*)&v;
}

template <int D>
struct KVBlock {
    PFrag k[2][D / 32];     // [16-key tile][d chunk]
    u32x2_t v[D / 16][2];   // [d tile][16-key tile]: 4 keys each
};

template <int D>
__device__ __forceinline__ void load_kv_block(KVBlock<D>& blk, int kb, int first_key, int last_key,
                                              const int* __restrict__ table,
                                              const bf16_t* __restrict__ k_pool, const bf16_t* __restrict__ v_pool,
                                              int kvh, int KVH, int page_shift, int r, int g) {
    const int page = 1 << page_shift;
#pragma unroll
    for (int t = 0; t < 2; ++t) {
        const int tile0 = kb * 32 + 16 * t;
        if (tile0 <= last_key && tile0 + 15 >= first_key) {         // wave-uniform: the tile holds a visible key
            const int pg = table[tile0 >> page_shift];
            const int in_page = tile0 & (page - 1);
            const bf16_t* kr = k_pool + ((((size_t)pg << page_shift) + in_page + r) * KVH + kvh) * D + 8 * g;
#pragma unroll
            for (int c = 0; c < D / 32; ++c) blk.k[t][c].u = *(const u32x4_t*)(kr + 32 * c);
            const bf16_t* vr = v_pool + ((((size_t)pg * KVH + kvh) * D + r) << page_shift) + in_page + 4 * g;
#pragma unroll
            for (int dt = 0; dt < D / 16; ++dt) blk.v[dt][t] = *(const u32x2_t*)(vr + ((size_t)(16 * dt) << page_shift));
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
// A block is AP_KSPLIT wavefronts on the same tile and heads; wavefront j takes the key blocks kb
// with kb % AP_KSPLIT == j and the partial results are merged through LDS in wavefront order.
// Which blocks a wavefront takes depends on absolute positions only, and a block in which a token
// sees no key changes nothing for it, so a token's bits do not depend on the tile it falls into.
// (two blocks per CU where the head size leaves room: a second wavefront per SIMD hides the first one's loads)
template <int D>
__global__ __launch_bounds__(64 * AP_KSPLIT, D <= 64 ? 3 : 1) void attn_prefill_mfma_kernel(
    const bf16_t* __restrict__ q, int q_stride, bf16_t* __restrict__ out, int out_stride,
    const bf16_t* __restrict__ k_pool, const bf16_t* __restrict__ v_pool, const int* __restrict__ block_tables,
    int table_width, const int* __restrict__ tiles, int H, int KVH, int page_shift, float scale_log2, int window) {
    constexpr int NDC = D / 32, NDT = D / 16;
    __shared__ float s_m[AP_KSPLIT][16], s_l[AP_KSPLIT][16];
    __shared__ float s_o[AP_KSPLIT][16][D + 1];
    const int wave = threadIdx.x / TM_WAVE, lane = threadIdx.x % TM_WAVE, r = lane % 16, g = lane / 16;
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
    const int last_lo = (window > 0 && last_key - window + 1 > 0) ? last_key - window + 1 : 0;
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
    // m: running maximum of (score * scale * log2 e) of this lane's column; l: this lane's share of
    // the running sum (its 8 keys of every block), reduced over the lanes of a column at the end
    float m[AP_HPW], l[AP_HPW];
    f32x4_t o[AP_HPW][NDT];
#pragma unroll
    for (int hh = 0; hh < AP_HPW; ++hh) {
        m[hh] = -INFINITY;
        l[hh] = 0.f;
#pragma unroll
        for (int dt = 0; dt < NDT; ++dt) o[hh][dt] = f32x4_t{0.f, 0.f, 0.f, 0.f};
    }

    int kb = kb0 + ((wave - kb0) & (AP_KSPLIT - 1));                 // first block >= kb0 of this wavefront
    KVBlock<D> cur, nxt;
    if (kb <= kb1) load_kv_block<D>(cur, kb, first_key, last_key, table, k_pool, v_pool, kvh, KVH, page_shift, r, g);
    for (; kb <= kb1; kb += AP_KSPLIT) {
        const bool more = kb + AP_KSPLIT <= kb1;
        if (more)
            load_kv_block<D>(nxt, kb + AP_KSPLIT, first_key, last_key, table, k_pool, v_pool, kvh, KVH, page_shift, r, g);
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
        // does any (query, key) pair of this block fall outside the causal / window limits?
        const bool edge = (key0 + 31 > pos0) || (key0 < last_lo);
#pragma unroll
        for (int hh = 0; hh < AP_HPW; ++hh) {
            if (hh >= nh) continue;                                  // wave-uniform
            float sc[2][4];
#pragma unroll
            for (int t = 0; t < 2; ++t) {
                f32x4_t acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int c = 0; c < NDC; ++c)
                    acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(cur.k[t][c].b, qf[hh][c].b, acc, 0, 0, 0);
#pragma unroll
                for (int i = 0; i < 4; ++i) sc[t][i] = acc[i];
            }
            if (edge) {
#pragma unroll
                for (int t = 0; t < 2; ++t)
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        const int kj = key0 + 16 * t + 4 * g + i;
                        if (kj > my_pos || kj < my_lo) sc[t][i] = -INFINITY;
                    }
            }
            float bm = fmaxf(fmaxf(fmaxf(sc[0][0], sc[0][1]), fmaxf(sc[0][2], sc[0][3])),
                             fmaxf(fmaxf(sc[1][0], sc[1][1]), fmaxf(sc[1][2], sc[1][3])));
            bm = fmaxf(bm, __shfl_xor(bm, 16, TM_WAVE));
            bm = fmaxf(bm, __shfl_xor(bm, 32, TM_WAVE));
            bm *= scale_log2;                                        // scale > 0: the maximum commutes with it
            if (__any(bm > m[hh])) {                                 // some column's maximum grew: rescale
                const float m_new = fmaxf(m[hh], bm);
                const float corr = (m_new == -INFINITY) ? 1.f : __builtin_amdgcn_exp2f(m[hh] - m_new);
                m[hh] = m_new;
                l[hh] *= corr;
#pragma unroll
                for (int dt = 0; dt < NDT; ++dt)
#pragma unroll
                    for (int i = 0; i < 4; ++i) o[hh][dt][i] *= corr;
            }
            // a column that has seen no key yet (m = -inf) gets zeros: exp2(-inf - 0)
            const float neg_m = (m[hh] == -INFINITY) ? 0.f : -m[hh];
            float pr[2][4];
#pragma unroll
            for (int t = 0; t < 2; ++t)
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    pr[t][i] = __builtin_amdgcn_exp2f(fmaf(sc[t][i], scale_log2, neg_m));
                    l[hh] += pr[t][i];
                }
            PFrag pt;
            pt.u = u32x4_t{pk_bf16(pr[0][0], pr[0][1]), pk_bf16(pr[0][2], pr[0][3]), pk_bf16(pr[1][0], pr[1][1]),
                           pk_bf16(pr[1][2], pr[1][3])};
#pragma unroll
            for (int dt = 0; dt < NDT; ++dt) {
                PFrag vf;
                vf.u = u32x4_t{cur.v[dt][0][0], cur.v[dt][0][1], cur.v[dt][1][0], cur.v[dt][1][1]};
                o[hh][dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf.b, pt.b, o[hh][dt], 0, 0, 0);
            }
        }
        if (more) cur = nxt;
    }

    // merge the wavefronts' partials head by head, in wavefront order; lane: d = 16 dt + 4 g + i of token r
#pragma unroll
    for (int hh = 0; hh < AP_HPW; ++hh) {
        if (hh >= nh) continue;                                      // block-uniform
        float lsum = l[hh];
        lsum += __shfl_xor(lsum, 16, TM_WAVE);
        lsum += __shfl_xor(lsum, 32, TM_WAVE);
        if (g == 0) {
            s_m[wave][r] = m[hh];
            s_l[wave][r] = lsum;
        }
#pragma unroll
        for (int dt = 0; dt < NDT; ++dt)
#pragma unroll
            for (int i = 0; i < 4; ++i) s_o[wave][r][16 * dt + 4 * g + i] = o[hh][dt][i];
        __syncthreads();
        for (int idx = threadIdx.x; idx < 16 * (D / 2); idx += 64 * AP_KSPLIT) {
            const int col = idx / (D / 2), d = 2 * (idx % (D / 2));
            if (col >= valid) continue;
            float mm = s_m[0][col];
#pragma unroll
            for (int w = 1; w < AP_KSPLIT; ++w) mm = fmaxf(mm, s_m[w][col]);
            float ll = 0.f, o0 = 0.f, o1 = 0.f;
#pragma unroll
            for (int w = 0; w < AP_KSPLIT; ++w) {
                const float f = (s_m[w][col] == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f(s_m[w][col] - mm);
                ll = fmaf(s_l[w][col], f, ll);
                o0 = fmaf(s_o[w][col][d], f, o0);
                o1 = fmaf(s_o[w][col][d + 1], f, o1);
            }
            const float inv = 1.f / ll;
            *(uint32_t*)(out + (size_t)(row0 + col) * out_stride + (size_t)(h0 + hh) * D + d) = pk_bf16(o0 * inv, o1 * inv);
        }
        __syncthreads();
    }
}

extern "C" int tm_attn_prefill_mfma(const void* q, int q_stride, void* out, int out_stride, const void* k_pool,
                                    const void* v_pool, const int* block_tables, int table_width, const int* tiles,
                                    int n_tiles, int H, int KVH, int D, int page, float scale, int window,
                                    hipStream_t stream) {
    if (n_tiles <= 0) return TM_OK;
    if (H <= 0 || KVH <= 0 || H % KVH || page < 16 || (page & (page - 1)) || window < 0 || table_width <= 0 ||
        (q_stride % 8) || ((uintptr_t)q % 16) || (out_stride % 2) || ((uintptr_t)out % 4) || q_stride < H * D ||
        out_stride < H * D || !(scale > 0.f))
        return TM_ERR_ARG;
    const int G = H / KVH;
    const int splits = (G + AP_HPW - 1) / AP_HPW;
    if ((long long)KVH * splits > 65535) return TM_ERR_ARG;
    int page_shift = 0;
    while ((1 << page_shift) < page) ++page_shift;
    const float scale_log2 = scale * 1.4426950408889634f;
    dim3 grid(n_tiles, KVH * splits);
#define TM_PREFILL_CASE(DD)                                                                                       \
    case DD:                                                                                                      \
        attn_prefill_mfma_kernel<DD><<<grid, 64 * AP_KSPLIT, 0, stream>>>(                                        \
            (const bf16_t*)q, q_stride, (bf16_t*)out, out_stride, (const bf16_t*)k_pool, (const bf16_t*)v_pool,   \
            block_tables, table_width, tiles, H, KVH, page_shift, scale_log2, window);                            \
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
