// Paged attention for single decoded tokens on MFMA (bfloat16), split over the context.
//
//   One token per request; its G = H / KVH query heads that share a kv head are the 16 columns of
//   one MFMA tile, so the keys and values of a kv head are read once for all of them
//   (the reference folds the group into query rows the same way: src/infer/model/layers.py:110-124).
//   The context is cut into chunks of 256 positions, fixed by position alone; each block of four
//   wavefronts takes one chunk of one (request, kv head), each wavefront 64 keys of it, and writes
//   an unnormalised partial (max, sum, weighted values) in 32-bit. The block that finishes last for
//   a (request, kv head) (a counter tells it) adds the partials in ascending chunk order and writes
//   the result; the order of the sum is fixed, whichever block happens to do it. What a request
//   gets therefore does not depend on which other requests are in the batch.
//
//   Operand layouts need no LDS: keys K[page][slot][kvh][d] give the A operand of S^T = K Q^T
//   (16 keys x 32 d per instruction), values V[page][kvh][d][slot] give the A operand of
//   O^T = V^T P^T (16 d x 32 keys), and P^T comes straight from the S^T accumulators.
#include "common.h"
#include "api.h"

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4_t __attribute__((ext_vector_type(4)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));

#define AD_CHUNK 256        // keys per block
#define AD_WKEYS 64         // keys per wavefront

typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef float f32x2_t __attribute__((ext_vector_type(2)));

// two floats -> packed bfloat16 (round to nearest even, one instruction on gfx950)
__device__ __forceinline__ uint32_t pack_bf16(float a, float b) {
    const bf16x2_t v = __builtin_convertvector(f32x2_t{a, b}, bf16x2_t);
    return *(const uint32_t*)&v;
}

union Bf16x8Bits {
    u32x4_t u;
    bf16x8_t b;
};

// D = head size (multiple of 32, at most 128); page a power of two >= 16; G <= 16.
// Scores are kept as score * scale * log2(e) so that the exponentials are single exp2 instructions.
template <int D>
__global__ __launch_bounds__(256) void attn_decode_mfma_kernel(
    const bf16_t* __restrict__ q, int q_stride, const bf16_t* __restrict__ k_pool,
    const bf16_t* __restrict__ v_pool, const int* __restrict__ block_tables, int table_width,
    const int* __restrict__ context_lens, float* __restrict__ part_o, float* __restrict__ part_ml,
    int* __restrict__ counters, bf16_t* __restrict__ out, int out_stride, int max_chunks, int H, int KVH,
    int page_shift, float scale_log2, int window) {
    constexpr int NDC = D / 32;          // 32-wide d chunks of the q.k product
    constexpr int NDT = D / 16;          // 16-wide d tiles of the output
    __shared__ float s_m[4][16], s_l[4][16];
    __shared__ float s_o[4][16][D + 1];

    const int s = blockIdx.x, kvh = blockIdx.y, chunk = blockIdx.z;
    const int G = H / KVH;
    const int ctx = context_lens[s];
    const int p = ctx - 1;
    const int lo = (window > 0 && p - window + 1 > 0) ? p - window + 1 : 0;
    const int chunk_lo = chunk * AD_CHUNK;
    if (chunk_lo >= ctx || chunk_lo + AD_CHUNK <= lo) return;       // nothing of this chunk is visible

    const int wave = threadIdx.x / TM_WAVE, lane = threadIdx.x % TM_WAVE;
    const int r = lane % 16, g = lane / 16;
    const int* table = block_tables + (size_t)s * table_width;
    const int page_mask = (1 << page_shift) - 1;
    const int wbase = chunk_lo + wave * AD_WKEYS;                   // first key of this wavefront

    // every load of the wavefront is issued before the first product
    int tile_page[4];
#pragma unroll
    for (int t = 0; t < 4; ++t) {
        const int tile0 = wbase + 16 * t;
        tile_page[t] = (tile0 < ctx && tile0 + 16 > lo) ? table[tile0 >> page_shift] : -1;      // wave-uniform
    }
    // Q^T operand: column r = query head kvh*G + r, rows d = 32c + 8g .. +7
    Bf16x8Bits qreg[NDC];
#pragma unroll
    for (int c = 0; c < NDC; ++c) {
        if (r < G)
            qreg[c].u = *(const u32x4_t*)(q + (size_t)s * q_stride + (size_t)(kvh * G + r) * D + 32 * c + 8 * g);
        else
            qreg[c].u = u32x4_t{0, 0, 0, 0};
    }
    Bf16x8Bits kreg[4][NDC];
    u32x2_t vreg[NDT][4];
#pragma unroll
    for (int t = 0; t < 4; ++t) {
        const int tile0 = wbase + 16 * t;
        const int in_page = tile0 & page_mask;
        const bool have = tile_page[t] >= 0;
        const size_t pg = have ? (size_t)tile_page[t] : 0;
        const bf16_t* kr = k_pool + (((pg << page_shift) + in_page + r) * KVH + kvh) * D + 8 * g;
        const bf16_t* vr = v_pool + (((pg * KVH + kvh) * D + r) << page_shift) + in_page + 4 * g;
#pragma unroll
        for (int c = 0; c < NDC; ++c)
            kreg[t][c].u = (have && tile0 + r < ctx) ? *(const u32x4_t*)(kr + 32 * c) : u32x4_t{0, 0, 0, 0};
#pragma unroll
        for (int dt = 0; dt < NDT; ++dt)
            vreg[dt][t] = have ? *(const u32x2_t*)(vr + ((size_t)(16 * dt) << page_shift)) : u32x2_t{0, 0};
    }

    float sc[4][4];                                                 // [16-key tile][key 4g+i] for head r
#pragma unroll
    for (int t = 0; t < 4; ++t) {
        f32x4_t acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int c = 0; c < NDC; ++c)
            acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kreg[t][c].b, qreg[c].b, acc, 0, 0, 0);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int kj = wbase + 16 * t + 4 * g + i;
            sc[t][i] = (kj < ctx && kj >= lo) ? acc[i] * scale_log2 : -INFINITY;
        }
    }
    // softmax pieces of this wavefront's 64 keys, per head r: combine the four key groups g
    float m = -INFINITY;
#pragma unroll
    for (int t = 0; t < 4; ++t)
#pragma unroll
        for (int i = 0; i < 4; ++i) m = fmaxf(m, sc[t][i]);
    m = fmaxf(m, __shfl_xor(m, 16, TM_WAVE));
    m = fmaxf(m, __shfl_xor(m, 32, TM_WAVE));
    const float neg_m = (m == -INFINITY) ? 0.f : -m;
    float l = 0.f;
    float pr[4][4];
#pragma unroll
    for (int t = 0; t < 4; ++t)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            pr[t][i] = __builtin_amdgcn_exp2f(sc[t][i] + neg_m);
            l += pr[t][i];
        }
    l += __shfl_xor(l, 16, TM_WAVE);
    l += __shfl_xor(l, 32, TM_WAVE);

    // O^T[d][head] += V^T[d][keys] P^T[keys][head], 32 keys (tiles 2b, 2b+1) per instruction
    f32x4_t o[NDT];
#pragma unroll
    for (int dt = 0; dt < NDT; ++dt) o[dt] = f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int b = 0; b < 2; ++b) {
        if (tile_page[2 * b] < 0 && tile_page[2 * b + 1] < 0) continue;
        Bf16x8Bits pt;
        pt.u = u32x4_t{pack_bf16(pr[2 * b][0], pr[2 * b][1]), pack_bf16(pr[2 * b][2], pr[2 * b][3]),
                       pack_bf16(pr[2 * b + 1][0], pr[2 * b + 1][1]), pack_bf16(pr[2 * b + 1][2], pr[2 * b + 1][3])};
        // which of this lane's 4 + 4 keys exist (a value beyond the context may hold anything)
        uint32_t keep[4];
#pragma unroll
        for (int half = 0; half < 2; ++half) {
            const int k0 = wbase + 16 * (2 * b + half) + 4 * g;
#pragma unroll
            for (int w2 = 0; w2 < 2; ++w2) {
                const int ka = k0 + 2 * w2, kb = ka + 1;
                keep[half * 2 + w2] = ((ka < ctx && ka >= lo) ? 0x0000ffffu : 0u) | ((kb < ctx && kb >= lo) ? 0xffff0000u : 0u);
            }
        }
#pragma unroll
        for (int dt = 0; dt < NDT; ++dt) {
            Bf16x8Bits vf;
            vf.u = u32x4_t{vreg[dt][2 * b][0] & keep[0], vreg[dt][2 * b][1] & keep[1],
                           vreg[dt][2 * b + 1][0] & keep[2], vreg[dt][2 * b + 1][1] & keep[3]};
            o[dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf.b, pt.b, o[dt], 0, 0, 0);
        }
    }

    // the four wavefronts of the block -> one partial, added in wavefront order
    if (g == 0) {
        s_m[wave][r] = m;
        s_l[wave][r] = l;
    }
#pragma unroll
    for (int dt = 0; dt < NDT; ++dt)
#pragma unroll
        for (int i = 0; i < 4; ++i) s_o[wave][r][16 * dt + 4 * g + i] = o[dt][i];
    __syncthreads();
    for (int idx = threadIdx.x; idx < G * D; idx += 256) {
        const int n = idx / D, d = idx % D;
        float mm = -INFINITY;
#pragma unroll
        for (int w = 0; w < 4; ++w) mm = fmaxf(mm, s_m[w][n]);
        float ll = 0.f, oo = 0.f;
#pragma unroll
        for (int w = 0; w < 4; ++w) {
            const float f = (s_m[w][n] == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f(s_m[w][n] - mm);
            ll += s_l[w][n] * f;
            oo += s_o[w][n][d] * f;
        }
        const size_t slot = ((size_t)s * H + kvh * G + n) * max_chunks + chunk;
        part_o[slot * D + d] = oo;
        if (d == 0) {
            part_ml[slot * 2 + 0] = mm;
            part_ml[slot * 2 + 1] = ll;
        }
    }
    // Is this the last block of its (request, kv head)? Its partial is published first (release),
    // the counter is bumped, and the one that sees the full count reads the others' (acquire).
    __shared__ int s_last;
    const int c0 = lo / AD_CHUNK, c1 = (ctx - 1) / AD_CHUNK;
    __threadfence();
    __syncthreads();
    if (threadIdx.x == 0) {
        int* cnt = counters + (size_t)s * KVH + kvh;
        const int old = __hip_atomic_fetch_add(cnt, 1, __ATOMIC_ACQ_REL, __HIP_MEMORY_SCOPE_AGENT);
        s_last = (old == c1 - c0);
        if (s_last) __hip_atomic_store(cnt, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);   // ready for the next call
    }
    __syncthreads();
    if (!s_last) return;
    __threadfence();
    for (int idx = threadIdx.x; idx < G * D; idx += 256) {
        const int n = idx / D, d = idx % D;
        const size_t base = ((size_t)s * H + kvh * G + n) * max_chunks;
        float mm = -INFINITY;
        for (int c = c0; c <= c1; ++c)
            mm = fmaxf(mm, __hip_atomic_load(part_ml + (base + c) * 2, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT));
        float ll = 0.f, oo = 0.f;
        for (int c = c0; c <= c1; ++c) {
            const float mc = __hip_atomic_load(part_ml + (base + c) * 2, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            const float f = (mc == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f(mc - mm);
            ll += __hip_atomic_load(part_ml + (base + c) * 2 + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) * f;
            oo += __hip_atomic_load(part_o + (base + c) * D + d, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) * f;
        }
        out[(size_t)s * out_stride + (size_t)(kvh * G + n) * D + d] = f32_to_bf16(oo / ll);
    }
}

template <int D>
static int launch_decode(const void* q, int q_stride, void* out, int out_stride, const void* k_pool,
                         const void* v_pool, const int* block_tables, int table_width, const int* context_lens,
                         float* part_o, float* part_ml, int* counters, int max_chunks, int S, int H, int KVH,
                         int page, float scale, int window, hipStream_t stream) {
    int page_shift = 0;
    while ((1 << page_shift) < page) ++page_shift;
    const float scale_log2 = scale * 1.4426950408889634f;
    dim3 grid(S, KVH, max_chunks);
    attn_decode_mfma_kernel<D><<<grid, 256, 0, stream>>>((const bf16_t*)q, q_stride, (const bf16_t*)k_pool,
                                                         (const bf16_t*)v_pool, block_tables, table_width,
                                                         context_lens, part_o, part_ml, counters, (bf16_t*)out,
                                                         out_stride, max_chunks, H, KVH, page_shift, scale_log2,
                                                         window);
    TM_CHECK_LAUNCH();
    return TM_OK;
}

// q: first decode row (one row per request, rows q_stride apart); out likewise; block_tables and
// context_lens: first decode request. part_o: float [S, H, max_chunks, D]; part_ml: [S, H, max_chunks, 2];
// counters: int [S * KVH], all zero on entry (and again on exit). Calls that share counters must not overlap.
extern "C" int tm_attn_decode_mfma(const void* q, int q_stride, void* out, int out_stride, const void* k_pool,
                                   const void* v_pool, const int* block_tables, int table_width,
                                   const int* context_lens, float* part_o, float* part_ml, int* counters,
                                   int max_chunks, int S, int H, int KVH, int D, int page, float scale, int window,
                                   hipStream_t stream) {
    if (S <= 0) return TM_OK;
    if (!counters) return TM_ERR_ARG;
    if (H <= 0 || KVH <= 0 || H % KVH || H / KVH > 16 || page < 16 || (page & (page - 1)) || max_chunks <= 0 ||
        !(scale > 0.f) ||
        max_chunks > 65535 || KVH > 65535 || window < 0 || table_width <= 0 || (q_stride % 8) ||
        ((uintptr_t)q % 16) || q_stride < H * D || out_stride < H * D)
        return TM_ERR_ARG;
#define TM_DECODE_CASE(DD)                                                                                        \
    case DD:                                                                                                      \
        return launch_decode<DD>(q, q_stride, out, out_stride, k_pool, v_pool, block_tables, table_width,         \
                                 context_lens, part_o, part_ml, counters, max_chunks, S, H, KVH, page, scale, window, stream)
    switch (D) {
        TM_DECODE_CASE(32);
        TM_DECODE_CASE(64);
        TM_DECODE_CASE(96);
        TM_DECODE_CASE(128);
        default:
            return TM_ERR_ARG;
    }
#undef TM_DECODE_CASE
}
