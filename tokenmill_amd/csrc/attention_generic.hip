// Paged attention over the cache, generic form: one wavefront per (query token, query head).
//
//   scores = (q . k) * scale ; a query at position p of its request sees the keys of that request
//   at positions lo..p, lo = 0 or p - window + 1 ; softmax in 32-bit ; out = weights . v
//                               (reference src/infer/model/layers.py:72-124, mask rules
//                                src/infer/kv/context.py:73-74 and src/infer/model/layers.py:122)
//   query head h reads kv head h / (H / KVH)         (reference src/infer/model/layers.py:86-87,119)
//   keys and values are read in place through the request's block table
//                               (flat slot of position p = table[p / page] * page + p % page,
//                                reference src/infer/kv/paged_cache.py:4-5,90-91)
//   K pool [pages, page, KVH, D]; V pool [pages, KVH, D, page] (key-contiguous per head and d)
//
// It takes every head size that is a multiple of 4 up to 256 and any q length and start position,
// in 32-bit and in bfloat16; it is the attention of the true 32-bit path, and the bfloat16 path
// uses it for shapes its MFMA kernels refuse. Keys are visited in ascending position in groups of
// 64 starting at lo, whatever else the batch holds, so a token's result depends on nothing but its
// own request.
#include "common.h"
#include "api.h"

#define AG_WAVES 4
#define AG_MAXD 256

template <typename T>
__global__ __launch_bounds__(AG_WAVES * TM_WAVE) void attn_paged_generic_kernel(
    const T* __restrict__ q, int q_stride, T* __restrict__ out, int out_stride,
    const T* __restrict__ k_pool, const T* __restrict__ v_pool, const int* __restrict__ block_tables,
    int table_width, const int* __restrict__ seq_of_token, const int* __restrict__ positions, int T_tokens,
    int H, int KVH, int D, int page, float scale, int window) {
    __shared__ float q_s[AG_WAVES][AG_MAXD];
    const int wave = threadIdx.x / TM_WAVE, lane = threadIdx.x % TM_WAVE;
    const long long w = (long long)blockIdx.x * AG_WAVES + wave;
    const bool active = w < (long long)T_tokens * H;
    const int t = active ? (int)(w / H) : 0, h = active ? (int)(w % H) : 0;
    const int kvh = h / (H / KVH);
    const int s = seq_of_token[t];
    const int p = positions[t];
    const int lo = (window > 0 && p - window + 1 > 0) ? p - window + 1 : 0;
    const int* table = block_tables + (size_t)s * table_width;

    const T* qrow = q + (size_t)t * q_stride + (size_t)h * D;
    for (int d = lane; d < D; d += TM_WAVE) q_s[wave][d] = Elem<T>::load(qrow + d);
    __syncthreads();
    if (!active) return;

    float m = -INFINITY, l = 0.f;
    float acc[AG_MAXD / TM_WAVE];
#pragma unroll
    for (int i = 0; i < AG_MAXD / TM_WAVE; ++i) acc[i] = 0.f;

    for (int j0 = lo; j0 <= p; j0 += TM_WAVE) {
        const int j = j0 + lane;
        const bool valid = j <= p;
        long long row = 0;
        float sc = -INFINITY;
        if (valid) {
            row = (long long)table[j / page] * page + (j % page);
            const T* kr = k_pool + ((size_t)row * KVH + kvh) * D;
            float dot = 0.f;
            for (int d = 0; d < D; d += 4) {
                dot = fmaf(q_s[wave][d + 0], Elem<T>::load(kr + d + 0), dot);
                dot = fmaf(q_s[wave][d + 1], Elem<T>::load(kr + d + 1), dot);
                dot = fmaf(q_s[wave][d + 2], Elem<T>::load(kr + d + 2), dot);
                dot = fmaf(q_s[wave][d + 3], Elem<T>::load(kr + d + 3), dot);
            }
            sc = dot * scale;
        }
        const float m_new = fmaxf(m, wave_max(sc));     // finite: lane 0 of every group is valid
        const float corr = expf(m - m_new);             // exp(-inf) = 0 on the first group
        const float pr = valid ? expf(sc - m_new) : 0.f;
        l = l * corr + wave_sum(pr);
        m = m_new;
        const float pr_v = Elem<T>::round(pr);          // weights are stored-type values when they meet v
#pragma unroll
        for (int i = 0; i < AG_MAXD / TM_WAVE; ++i) acc[i] *= corr;
        const int n = (p - j0 + 1) < TM_WAVE ? (p - j0 + 1) : TM_WAVE;
        for (int jj = 0; jj < n; ++jj) {
            const float pj = __shfl(pr_v, jj, TM_WAVE);
            const long long rj = __shfl(row, jj, TM_WAVE);
            const T* vr = v_pool + ((size_t)(rj / page) * KVH + kvh) * D * page + (rj % page);
#pragma unroll
            for (int i = 0; i < AG_MAXD / TM_WAVE; ++i) {
                const int d = lane + i * TM_WAVE;
                if (d < D) acc[i] = fmaf(pj, Elem<T>::load(vr + (size_t)d * page), acc[i]);
            }
        }
    }
    T* orow = out + (size_t)t * out_stride + (size_t)h * D;
    const float inv = 1.f / l;
#pragma unroll
    for (int i = 0; i < AG_MAXD / TM_WAVE; ++i) {
        const int d = lane + i * TM_WAVE;
        if (d < D) Elem<T>::store(orow + d, acc[i] * inv);
    }
}

extern "C" int tm_attn_paged_generic(const void* q, int q_stride, void* out, int out_stride, const void* k_pool,
                                     const void* v_pool, const int* block_tables, int table_width,
                                     const int* seq_of_token, const int* positions, int T, int H, int KVH, int D,
                                     int page, float scale, int window, int dtype, hipStream_t stream) {
    if (T <= 0) return TM_OK;
    if (H <= 0 || KVH <= 0 || H % KVH || D <= 0 || D > AG_MAXD || D % 4 || page <= 0 || table_width <= 0 ||
        window < 0 || q_stride < H * D || out_stride < H * D)
        return TM_ERR_ARG;
    const long long waves = (long long)T * H;
    const long long blocks = (waves + AG_WAVES - 1) / AG_WAVES;
    if (blocks > 0x7fffffffLL) return TM_ERR_ARG;
    if (dtype == TM_F32)
        attn_paged_generic_kernel<float><<<(unsigned)blocks, AG_WAVES * TM_WAVE, 0, stream>>>(
            (const float*)q, q_stride, (float*)out, out_stride, (const float*)k_pool, (const float*)v_pool,
            block_tables, table_width, seq_of_token, positions, T, H, KVH, D, page, scale, window);
    else if (dtype == TM_BF16)
        attn_paged_generic_kernel<bf16_t><<<(unsigned)blocks, AG_WAVES * TM_WAVE, 0, stream>>>(
            (const bf16_t*)q, q_stride, (bf16_t*)out, out_stride, (const bf16_t*)k_pool, (const bf16_t*)v_pool,
            block_tables, table_width, seq_of_token, positions, T, H, KVH, D, page, scale, window);
    else
        return TM_ERR_ARG;
    TM_CHECK_LAUNCH();
    return TM_OK;
}
