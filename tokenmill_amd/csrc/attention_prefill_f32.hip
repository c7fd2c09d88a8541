// Paged attention for portions of prompts in true 32-bit, flash style on the 32-bit MFMA
// (v_mfma_f32_16x16x4_f32: 32-bit inputs, 32-bit products and sums; no reduced-precision mode).
//
//   A block takes 16 consecutive query tokens of one request (a "tile") and one query head. The keys
//   the tile may see are cut into blocks of 16 at absolute positions; the block's four wavefronts take
//   every fourth key block each (key block kb goes to wavefront kb % 4), in ascending position with an
//   online softmax of their own, and their four partial results are merged through LDS in the order of
//   the wavefronts: a query at position p sees keys lo..p, lo = 0 or p - window + 1
//                               (reference src/infer/kv/context.py:70-75, src/infer/model/layers.py:100-107).
//   Which wavefront takes a key block hangs on the key's position only, so a token's result depends
//   on its request only. The longest tile of a 2,048-token prompt walks 32 key blocks a wavefront
//   instead of 128; the heads of a kv head run in blocks of their own and share its keys through the
//   second-level cache.
//
//   S^T = K Q^T   A = keys  [16 keys x 4 d]   B = Q^T [4 d x 16 tokens]   (D / 4 steps; which d a step
//                 multiplies is free as long as keys and queries agree: the lanes of group g = lane / 16
//                 hold d = 16 c + 4 g .. + 3 for c = 0 .. D/16 - 1 of their key / token, so one 16-byte
//                 load of the four groups of a key is one run of 64 bytes)
//   O^T = V^T P^T A = V^T   [16 d x 4 keys]   B = P^T [4 keys x 16 tokens]: in step i the lanes of
//                 group g hold key 4 g + i, which is where the S^T accumulators already have it
//                 (register i of the same lane) and what one 16-byte load of V[d][4 g .. 4 g + 3] gives.
#include "common.h"
#include "api.h"

typedef float f32x4_t __attribute__((ext_vector_type(4)));

#define AF_SPLIT 4          // wavefronts of a block; each takes every fourth key block

template <int D>
__global__ __launch_bounds__(64 * AF_SPLIT) void attn_prefill_f32_kernel(
    const float* __restrict__ q, int q_stride, float* __restrict__ out, int out_stride,
    const float* __restrict__ k_pool, const float* __restrict__ v_pool, const int* __restrict__ block_tables,
    int table_width, const int* __restrict__ tiles, int H, int KVH, int page_shift, float scale, int window) {
    constexpr int DQ = D / 4;           // values of a key (or query) a lane holds
    constexpr int NDT = D / 16;         // 16-row tiles of d
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / TM_WAVE);
    const int lane = threadIdx.x % TM_WAVE, r = lane % 16, g = lane / 16;
    const int h = blockIdx.y;
    const int kvh = h / (H / KVH);
    const int* tl = tiles + (size_t)blockIdx.x * 4;
    const int s = tl[0], row0 = tl[1], valid = tl[2], pos0 = tl[3];
    const int* table = block_tables + (size_t)s * table_width;
    const int page = 1 << page_shift;
    const int last_key = pos0 + valid - 1;
    const int my_pos = pos0 + r < last_key ? pos0 + r : last_key;       // position of this lane's query column
    const int my_lo = (window > 0 && my_pos - window + 1 > 0) ? my_pos - window + 1 : 0;
    const int first_key = (window > 0 && pos0 - window + 1 > 0) ? pos0 - window + 1 : 0;
    const int last_lo = (window > 0 && last_key - window + 1 > 0) ? last_key - window + 1 : 0;

    float qf[DQ];
#pragma unroll
    for (int c = 0; c < DQ; c += 4) {
        f32x4_t t = {0.f, 0.f, 0.f, 0.f};
        if (r < valid) t = *(const f32x4_t*)(q + (size_t)(row0 + r) * q_stride + (size_t)h * D + 4 * c + 4 * g);
        qf[c] = t[0]; qf[c + 1] = t[1]; qf[c + 2] = t[2]; qf[c + 3] = t[3];
    }
    float m = -INFINITY, l = 0.f;       // running maximum of the scaled scores of this lane's column; this lane's share of the sum
    f32x4_t o[NDT];
#pragma unroll
    for (int dt = 0; dt < NDT; ++dt) o[dt] = f32x4_t{0.f, 0.f, 0.f, 0.f};

    const int kb_first = first_key >> 4, kb_last = last_key >> 4;
    int kb = kb_first + ((wave - kb_first) & (AF_SPLIT - 1));
    // a key block's page id is asked for one block ahead (always at an entry this tile may see)
    int pg_next = table[((kb <= kb_last ? kb : kb_last) << 4) >> page_shift];
    for (; kb <= kb_last; kb += AF_SPLIT) {
        const int key0 = kb << 4;
        const int pg = pg_next;
        pg_next = table[((kb + AF_SPLIT <= kb_last ? kb + AF_SPLIT : kb) << 4) >> page_shift];
        const int in_page = key0 & (page - 1);
        // keys: lane (r, g) holds K[key0 + r][16 c + 4 g .. + 3], c = 0 .. D/16 - 1
        const float* kr = k_pool + ((((size_t)pg << page_shift) + in_page + r) * KVH + kvh) * D + 4 * g;
        float kf[DQ];
#pragma unroll
        for (int c = 0; c < DQ; c += 4) {
            const f32x4_t t = *(const f32x4_t*)(kr + 4 * c);
            kf[c] = t[0]; kf[c + 1] = t[1]; kf[c + 2] = t[2]; kf[c + 3] = t[3];
        }
        // values: lane (r, g) holds V[d = 16 dt + r][key0 + 4 g .. + 3]
        const float* vr = v_pool + ((((size_t)pg * KVH + kvh) * D + r) << page_shift) + in_page + 4 * g;
        f32x4_t vf[NDT];
#pragma unroll
        for (int dt = 0; dt < NDT; ++dt) vf[dt] = *(const f32x4_t*)(vr + ((size_t)(16 * dt) << page_shift));
        // values of keys nobody may see yet (beyond the newest key) can hold anything: clear them
        if (key0 + 15 > last_key) {
#pragma unroll
            for (int dt = 0; dt < NDT; ++dt)
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    if (key0 + 4 * g + i > last_key) vf[dt][i] = 0.f;
        }
        f32x4_t sc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int c = 0; c < DQ; ++c) sc = __builtin_amdgcn_mfma_f32_16x16x4f32(kf[c], qf[c], sc, 0, 0, 0);
        // sc[i] = score of key key0 + 4 g + i for this lane's token
        const bool edge = (key0 + 15 > pos0) || (key0 < last_lo);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            sc[i] *= scale;
            if (edge) {
                const int kj = key0 + 4 * g + i;
                if (kj > my_pos || kj < my_lo) sc[i] = -INFINITY;
            }
        }
        float bm = fmaxf(fmaxf(sc[0], sc[1]), fmaxf(sc[2], sc[3]));
        bm = fmaxf(bm, __shfl_xor(bm, 16, TM_WAVE));
        bm = fmaxf(bm, __shfl_xor(bm, 32, TM_WAVE));
        const float m_new = fmaxf(m, bm);
        // a column that has seen no key yet keeps m = -inf; its weights and its correction are zeros
        // (every lane stays in step: the matrix instructions below are wave-wide)
        const float m_ref = (m_new == -INFINITY) ? 0.f : m_new;
        const float corr = expf(m - m_ref);                 // exp(-inf) = 0 on the column's first visible block
        m = m_new;
        l *= corr;
        f32x4_t pr;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            pr[i] = expf(sc[i] - m_ref);
            l += pr[i];
        }
#pragma unroll
        for (int dt = 0; dt < NDT; ++dt) {
#pragma unroll
            for (int i = 0; i < 4; ++i) o[dt][i] *= corr;
#pragma unroll
            for (int i = 0; i < 4; ++i) o[dt] = __builtin_amdgcn_mfma_f32_16x16x4f32(vf[dt][i], pr[i], o[dt], 0, 0, 0);
        }
    }
    // o[dt][i] = sum for d = 16 dt + 4 g + i of token r; the column's sum is spread over its four lanes
    l += __shfl_xor(l, 16, TM_WAVE);
    l += __shfl_xor(l, 32, TM_WAVE);
    // the four wavefronts' partial results meet in LDS; a wavefront that had no key block brings m = -inf, l = 0, o = 0
    __shared__ float m_s[AF_SPLIT][16], l_s[AF_SPLIT][16];
    __shared__ __attribute__((aligned(16))) float o_s[AF_SPLIT][16][D + 4];
    if (g == 0) {
        m_s[wave][r] = m;
        l_s[wave][r] = l;
    }
#pragma unroll
    for (int dt = 0; dt < NDT; ++dt) *(f32x4_t*)&o_s[wave][r][16 * dt + 4 * g] = o[dt];
    __syncthreads();
    const int tok = threadIdx.x >> 4;
    if (tok < valid) {
        float mw[AF_SPLIT], sw[AF_SPLIT], top = -INFINITY, sum = 0.f;
#pragma unroll
        for (int w = 0; w < AF_SPLIT; ++w) {
            mw[w] = m_s[w][tok];
            top = fmaxf(top, mw[w]);
        }
#pragma unroll
        for (int w = 0; w < AF_SPLIT; ++w) {
            sw[w] = (mw[w] == -INFINITY) ? 0.f : expf(mw[w] - top);     // a token always sees its own key: top is finite
            sum += l_s[w][tok] * sw[w];
        }
        const float inv = 1.f / sum;
        float* orow = out + (size_t)(row0 + tok) * out_stride + (size_t)h * D;
        for (int d = (threadIdx.x & 15) * 4; d < D; d += 64) {
            f32x4_t acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int w = 0; w < AF_SPLIT; ++w) {
                const f32x4_t part = *(const f32x4_t*)&o_s[w][tok][d];
#pragma unroll
                for (int i = 0; i < 4; ++i) acc[i] += part[i] * sw[w];
            }
            *(f32x4_t*)(orow + d) = f32x4_t{acc[0] * inv, acc[1] * inv, acc[2] * inv, acc[3] * inv};
        }
    }
}

// q float32 [T, >= H*D] rows, out float32 [T, >= H*D]; pools float32, K [pages, page, KVH, D], V [pages, KVH, D, page];
// tiles int32 [n_tiles][4] = (request index, first row, tokens (1..16), position of the first token).
// Needs D % 16 == 0 (at most 128), page a power of two >= 16, 16-byte aligned q, out and pools, strides % 4 == 0.
extern "C" int tm_attn_prefill_f32(const void* q, int q_stride, void* out, int out_stride, const void* k_pool,
                                   const void* v_pool, const int* block_tables, int table_width, const int* tiles,
                                   int n_tiles, int H, int KVH, int D, int page, float scale, int window,
                                   hipStream_t stream) {
    if (n_tiles <= 0) return TM_OK;
    if (H <= 0 || KVH <= 0 || H % KVH || page < 16 || (page & (page - 1)) || window < 0 || table_width <= 0 ||
        (q_stride % 4) || (out_stride % 4) || ((uintptr_t)q % 16) || ((uintptr_t)out % 16) || ((uintptr_t)k_pool % 16) ||
        ((uintptr_t)v_pool % 16) || q_stride < H * D || out_stride < H * D || !(scale > 0.f))
        return TM_ERR_ARG;
    if (H > 65535) return TM_ERR_ARG;
    int page_shift = 0;
    while ((1 << page_shift) < page) ++page_shift;
    dim3 grid(n_tiles, H);
#define TM_PREFILL_F32_CASE(DD)                                                                                   \
    case DD:                                                                                                      \
        attn_prefill_f32_kernel<DD><<<grid, 64 * AF_SPLIT, 0, stream>>>(                                          \
            (const float*)q, q_stride, (float*)out, out_stride, (const float*)k_pool, (const float*)v_pool,       \
            block_tables, table_width, tiles, H, KVH, page_shift, scale, window);                                 \
        break
    switch (D) {
        TM_PREFILL_F32_CASE(16);
        TM_PREFILL_F32_CASE(32);
        TM_PREFILL_F32_CASE(48);
        TM_PREFILL_F32_CASE(64);
        TM_PREFILL_F32_CASE(80);
        TM_PREFILL_F32_CASE(96);
        TM_PREFILL_F32_CASE(112);
        TM_PREFILL_F32_CASE(128);
        default:
            return TM_ERR_ARG;
    }
#undef TM_PREFILL_F32_CASE
    TM_CHECK_LAUNCH();
    return TM_OK;
}
