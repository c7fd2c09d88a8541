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
// 64 starting at lo, so a token's result depends on its own request only (and, in the last bits, on
// whether the step was small enough for the wavefronts of a block to share a token's keys).
#include "common.h"
#include "api.h"

#define AG_WAVES 4
#define AG_SPLIT_WAVES 8
#define AG_MAXD 256
#define AG_KCHUNK 16        // floats of every key staged at a time
#define AG_KSTRIDE 20       // floats between two keys of the staged tile (rows 16 bytes aligned, no bank conflicts)

// four consecutive elements as 32-bit floats
__device__ __forceinline__ void ag_load4(const float* p, float (&v)[4]) {
    const float4 t = *(const float4*)p;
    v[0] = t.x; v[1] = t.y; v[2] = t.z; v[3] = t.w;
}
__device__ __forceinline__ void ag_load4(const bf16_t* p, float (&v)[4]) {
    const uint2 t = *(const uint2*)p;
    v[0] = __uint_as_float(t.x << 16);
    v[1] = __uint_as_float(t.x & 0xffff0000u);
    v[2] = __uint_as_float(t.y << 16);
    v[3] = __uint_as_float(t.y & 0xffff0000u);
}

// SPLIT = false: a block is AG_WAVES (token, head) pairs, one per wavefront (steps with many tokens).
// SPLIT = true : a block is one (token, head) pair; its AG_SPLIT_WAVES wavefronts take the groups of 64
//                keys in turn (group i goes to wavefront i % AG_SPLIT_WAVES) and their partial results
//                are merged through LDS in wavefront order (steps with few tokens, where the pairs
//                alone would leave most of the chip idle). Which keys a wavefront takes depends on
//                the token's own position and window only.
// DMAX > 0 (head sizes up to 128): the weights meet the values with a lane still holding its own key, so
//                that a load of one d reads runs of consecutive keys; every lane keeps partial sums for
//                all d over its keys and the lanes are added once, at the end. DMAX = 0: a lane holds
//                d = lane, lane + 64, ... and the keys of a group are visited one after the other.
template <typename T, bool SPLIT, int DMAX>
__global__ __launch_bounds__((SPLIT ? AG_SPLIT_WAVES : AG_WAVES) * TM_WAVE) void attn_paged_generic_kernel(
    const T* __restrict__ q, int q_stride, T* __restrict__ out, int out_stride,
    const T* __restrict__ k_pool, const T* __restrict__ v_pool, const int* __restrict__ block_tables,
    int table_width, const int* __restrict__ seq_of_token, const int* __restrict__ positions, int T_tokens,
    int H, int KVH, int D, int page, float scale, int window) {
    constexpr int WAVES = SPLIT ? AG_SPLIT_WAVES : AG_WAVES;
    constexpr bool STAGED = DMAX > 0 && sizeof(T) == 4;         // 32-bit keys through LDS (see the key loop)
    __shared__ __align__(16) float k_tile[STAGED ? WAVES : 1][STAGED ? TM_WAVE * AG_KSTRIDE : 4];
    __shared__ float q_s[SPLIT ? 1 : AG_WAVES][AG_MAXD];
    __shared__ float s_m[SPLIT ? AG_SPLIT_WAVES : 1], s_l[SPLIT ? AG_SPLIT_WAVES : 1];
    __shared__ float s_acc[SPLIT ? AG_SPLIT_WAVES : 1][SPLIT ? AG_MAXD : 1];
    const int wave = threadIdx.x / TM_WAVE, lane = threadIdx.x % TM_WAVE;
    const long long w = SPLIT ? (long long)blockIdx.x : (long long)blockIdx.x * AG_WAVES + wave;
    const bool active = w < (long long)T_tokens * H;
    const int t = active ? (int)(w / H) : 0, h = active ? (int)(w % H) : 0;
    const int kvh = h / (H / KVH);
    const int s = seq_of_token[t];
    const int p = positions[t];
    const int lo = (window > 0 && p - window + 1 > 0) ? p - window + 1 : 0;
    const int* table = block_tables + (size_t)s * table_width;
    float* qs = q_s[SPLIT ? 0 : wave];

    const T* qrow = q + (size_t)t * q_stride + (size_t)h * D;
    if (SPLIT) {
        for (int d = threadIdx.x; d < D; d += WAVES * TM_WAVE) qs[d] = Elem<T>::load(qrow + d);
    } else {
        for (int d = lane; d < D; d += TM_WAVE) qs[d] = Elem<T>::load(qrow + d);
    }
    __syncthreads();
    if (!active) return;

    float m = -INFINITY, l = 0.f;
    float acc[AG_MAXD / TM_WAVE];
#pragma unroll
    for (int i = 0; i < AG_MAXD / TM_WAVE; ++i) acc[i] = 0.f;
    float part[DMAX > 0 ? DMAX : 1];            // DMAX > 0: this lane's sums over its own keys, every d
#pragma unroll
    for (int d = 0; d < (DMAX > 0 ? DMAX : 1); ++d) part[d] = 0.f;

    const int first = SPLIT ? lo + wave * TM_WAVE : lo;
    const int stride = SPLIT ? WAVES * TM_WAVE : TM_WAVE;
    for (int j0 = first; j0 <= p; j0 += stride) {
        const int j = j0 + lane;
        const bool valid = j <= p;
        long long row = 0;
        float sc = -INFINITY;
        if constexpr (STAGED) {
            // The group's key rows come through LDS, 16 floats of every key at a time: a load takes 64
            // bytes of each of 16 keys (whole runs of memory), where a lane reading its own key's row
            // 16 bytes at a time touches 64 cache lines a load and keeps coming back to them.
            // A lane beyond the newest key stands for the newest key (finite values, score masked).
            const int jc = valid ? j : p;
            row = (long long)table[jc / page] * page + (jc % page);
            long long row_of[4];
#pragma unroll
            for (int c = 0; c < 4; ++c) row_of[c] = __shfl(row, 16 * c + lane / 4, TM_WAVE);
            float* tile = k_tile[wave];
            float dot = 0.f;
            for (int dc = 0; dc < D; dc += AG_KCHUNK) {
                const int dp = dc + 4 * (lane % 4);
                // no test around the loads (a tested load is waited for by itself): beyond D they read
                // the row's first floats again, which the products below never use
                float4 piece[4];
#pragma unroll
                for (int c = 0; c < 4; ++c)
                    piece[c] = *(const float4*)(k_pool + ((size_t)row_of[c] * KVH + kvh) * D + (dp < D ? dp : 0));
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int c = 0; c < 4; ++c)
                    *(float4*)(tile + (16 * c + lane / 4) * AG_KSTRIDE + 4 * (lane % 4)) = piece[c];
#pragma unroll
                for (int dd = 0; dd < AG_KCHUNK; dd += 4) {
                    const float4 kv = *(const float4*)(tile + lane * AG_KSTRIDE + dd);
                    if (dc + dd < D) {
                        dot = fmaf(qs[dc + dd + 0], kv.x, dot);
                        dot = fmaf(qs[dc + dd + 1], kv.y, dot);
                        dot = fmaf(qs[dc + dd + 2], kv.z, dot);
                        dot = fmaf(qs[dc + dd + 3], kv.w, dot);
                    }
                }
            }
            if (valid) sc = dot * scale;
        } else if (valid) {
            row = (long long)table[j / page] * page + (j % page);
            const T* kr = k_pool + ((size_t)row * KVH + kvh) * D;
            float dot = 0.f;
            for (int d = 0; d < D; d += 4) {
                float kv[4];
                ag_load4(kr + d, kv);
                dot = fmaf(qs[d + 0], kv[0], dot);
                dot = fmaf(qs[d + 1], kv[1], dot);
                dot = fmaf(qs[d + 2], kv[2], dot);
                dot = fmaf(qs[d + 3], kv[3], dot);
            }
            sc = dot * scale;
        }
        const float m_new = fmaxf(m, wave_max(sc));     // finite: lane 0 of every group is valid
        const float corr = expf(m - m_new);             // exp(-inf) = 0 on the first group
        const float pr = valid ? expf(sc - m_new) : 0.f;
        l = l * corr + wave_sum(pr);
        m = m_new;
        const float pr_v = Elem<T>::round(pr);          // weights are stored-type values when they meet v
        if constexpr (DMAX > 0) {
            // a lane beyond the newest key reads the newest key's values (finite) with weight 0
            const long long rv = (valid || STAGED) ? row : (long long)table[p / page] * page + (p % page);
            const T* vr = v_pool + ((size_t)(rv / page) * KVH + kvh) * D * page + (rv % page);
            // every load without a test, all of a group in flight at once: beyond D a lane reads d = 0
            // again and the sum it feeds is never looked at
#pragma unroll
            for (int d0 = 0; d0 < DMAX; d0 += 64) {     // 64 loads in flight at a time
                float vals[64];
#pragma unroll
                for (int d = 0; d < 64; ++d) vals[d] = Elem<T>::load(vr + (size_t)(d0 + d < D ? d0 + d : 0) * page);
                __builtin_amdgcn_sched_barrier(0);      // (else the compiler asks for them one by one, to save registers)
#pragma unroll
                for (int d = 0; d < 64; ++d) part[d0 + d] = fmaf(pr_v, vals[d], part[d0 + d] * corr);
                __builtin_amdgcn_sched_barrier(0);
            }
            continue;
        }
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
    if constexpr (DMAX > 0) {                   // the lanes' sums added, lane d % 64 keeps d
#pragma unroll
        for (int d = 0; d < DMAX; ++d) {
            if (d < D) {
                const float total = wave_sum(part[d]);
                if (lane == d % TM_WAVE) acc[d / TM_WAVE] = total;
            }
        }
    }
    T* orow = out + (size_t)t * out_stride + (size_t)h * D;
    if (!SPLIT) {
        const float inv = 1.f / l;
#pragma unroll
        for (int i = 0; i < AG_MAXD / TM_WAVE; ++i) {
            const int d = lane + i * TM_WAVE;
            if (d < D) Elem<T>::store(orow + d, acc[i] * inv);
        }
        return;
    }
    // the wavefronts' partial results, merged in wavefront order (one that saw no key has m = -inf, l = 0)
    if (lane == 0) {
        s_m[wave] = m;
        s_l[wave] = l;
    }
#pragma unroll
    for (int i = 0; i < AG_MAXD / TM_WAVE; ++i) {
        const int d = lane + i * TM_WAVE;
        if (d < D) s_acc[wave][d] = acc[i];
    }
    __syncthreads();
    float mm = s_m[0];
#pragma unroll
    for (int ww = 1; ww < WAVES; ++ww) mm = fmaxf(mm, s_m[ww]);
    float ll = 0.f;
#pragma unroll
    for (int ww = 0; ww < WAVES; ++ww) ll += (s_m[ww] == -INFINITY) ? 0.f : s_l[ww] * expf(s_m[ww] - mm);
    for (int d = threadIdx.x; d < D; d += WAVES * TM_WAVE) {
        float oo = 0.f;
#pragma unroll
        for (int ww = 0; ww < WAVES; ++ww) oo += (s_m[ww] == -INFINITY) ? 0.f : s_acc[ww][d] * expf(s_m[ww] - mm);
        Elem<T>::store(orow + d, oo / ll);
    }
}

template <typename T, int DMAX>
static void launch_generic_d(const void* q, int q_stride, void* out, int out_stride, const void* k_pool,
                             const void* v_pool, const int* block_tables, int table_width, const int* seq_of_token,
                             const int* positions, int T_tokens, int H, int KVH, int D, int page, float scale,
                             int window, hipStream_t stream) {
    const long long pairs = (long long)T_tokens * H;
    if (pairs < 1024)           // too few (token, head) pairs to fill the chip: the wavefronts of a block split the keys
        attn_paged_generic_kernel<T, true, DMAX><<<(unsigned)pairs, AG_SPLIT_WAVES * TM_WAVE, 0, stream>>>(
            (const T*)q, q_stride, (T*)out, out_stride, (const T*)k_pool, (const T*)v_pool, block_tables,
            table_width, seq_of_token, positions, T_tokens, H, KVH, D, page, scale, window);
    else
        attn_paged_generic_kernel<T, false, DMAX><<<(unsigned)((pairs + AG_WAVES - 1) / AG_WAVES),
                                                    AG_WAVES * TM_WAVE, 0, stream>>>(
            (const T*)q, q_stride, (T*)out, out_stride, (const T*)k_pool, (const T*)v_pool, block_tables,
            table_width, seq_of_token, positions, T_tokens, H, KVH, D, page, scale, window);
}

template <typename T>
static void launch_generic(const void* q, int q_stride, void* out, int out_stride, const void* k_pool,
                           const void* v_pool, const int* block_tables, int table_width, const int* seq_of_token,
                           const int* positions, int T_tokens, int H, int KVH, int D, int page, float scale,
                           int window, hipStream_t stream) {
#define TM_GENERIC(DMAX)                                                                                       \
    launch_generic_d<T, DMAX>(q, q_stride, out, out_stride, k_pool, v_pool, block_tables, table_width,         \
                              seq_of_token, positions, T_tokens, H, KVH, D, page, scale, window, stream)
    if (D <= 64) TM_GENERIC(64);
    else if (D <= 128) TM_GENERIC(128);
    else TM_GENERIC(0);
#undef TM_GENERIC
}

extern "C" int tm_attn_paged_generic(const void* q, int q_stride, void* out, int out_stride, const void* k_pool,
                                     const void* v_pool, const int* block_tables, int table_width,
                                     const int* seq_of_token, const int* positions, int T, int H, int KVH, int D,
                                     int page, float scale, int window, int dtype, hipStream_t stream) {
    if (T <= 0) return TM_OK;
    if (H <= 0 || KVH <= 0 || H % KVH || D <= 0 || D > AG_MAXD || D % 4 || page <= 0 || table_width <= 0 ||
        window < 0 || q_stride < H * D || out_stride < H * D)
        return TM_ERR_ARG;
    if (((long long)T * H + AG_WAVES - 1) / AG_WAVES > 0x7fffffffLL) return TM_ERR_ARG;
    if (dtype == TM_F32) {
        if (((uintptr_t)k_pool % 16)) return TM_ERR_ARG;
        launch_generic<float>(q, q_stride, out, out_stride, k_pool, v_pool, block_tables, table_width, seq_of_token,
                              positions, T, H, KVH, D, page, scale, window, stream);
    } else if (dtype == TM_BF16) {
        if (((uintptr_t)k_pool % 8)) return TM_ERR_ARG;
        launch_generic<bf16_t>(q, q_stride, out, out_stride, k_pool, v_pool, block_tables, table_width, seq_of_token,
                               positions, T, H, KVH, D, page, scale, window, stream);
    } else {
        return TM_ERR_ARG;
    }
    TM_CHECK_LAUNCH();
    return TM_OK;
}
