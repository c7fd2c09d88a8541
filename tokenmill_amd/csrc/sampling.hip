// Sampling over rows of 32-bit logits: argmax, and temperature sampling with optional top-k and
// top-p filters, one token per row                    (reference src/infer/sampling.py:12-46).
//
// The random number of a row is given by the caller (u in [0, 1), drawn from the request's own
// counter-based stream), so a request's tokens do not depend on its batch-mates. The token is the
// inverse CDF of the filtered softmax in vocabulary order. Filters are found by a radix descent
// over the bit patterns of the logits with integer histograms, so no sort is needed and the
// result does not depend on the order in which threads add.
#include "common.h"
#include "api.h"

#define SM_NT 1024

// monotonic map float -> uint32 (larger float, larger key)
__device__ __forceinline__ uint32_t order_key(float f) {
    uint32_t u = __float_as_uint(f);
    return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}

struct ArgMax {
    float v;
    int i;
};

__device__ __forceinline__ ArgMax better(ArgMax a, ArgMax b) {
    // larger value wins; equal values: the lower index (the first maximum); NaN never wins
    if (b.i >= 0 && (a.i < 0 || b.v > a.v || (b.v == a.v && b.i < a.i))) return b;
    return a;
}

__device__ ArgMax block_argmax(const float* __restrict__ row, int V, ArgMax* smem /* SM_NT/64 */) {
    ArgMax best{-INFINITY, -1};
    for (int i = threadIdx.x; i < V; i += SM_NT) {
        const float v = row[i];
        if (v == v) best = better(best, ArgMax{v, i});
    }
#pragma unroll
    for (int off = TM_WAVE / 2; off > 0; off >>= 1) {
        ArgMax o{__shfl_xor(best.v, off, TM_WAVE), __shfl_xor(best.i, off, TM_WAVE)};
        best = better(best, o);
    }
    const int wave = threadIdx.x / TM_WAVE, lane = threadIdx.x % TM_WAVE;
    __syncthreads();
    if (lane == 0) smem[wave] = best;
    __syncthreads();
    ArgMax r = smem[0];
    for (int w = 1; w < SM_NT / TM_WAVE; ++w) r = better(r, smem[w]);
    if (r.i < 0) r.i = 0;
    return r;
}

__global__ __launch_bounds__(SM_NT) void argmax_rows_kernel(const float* __restrict__ logits, int V,
                                                            int* __restrict__ out) {
    __shared__ ArgMax smem[SM_NT / TM_WAVE];
    const ArgMax r = block_argmax(logits + (size_t)blockIdx.x * V, V, smem);
    if (threadIdx.x == 0) out[blockIdx.x] = r.i;
}

// Two stages for wide vocabularies: a row is cut into NB chunks, one block each, then the NB
// candidates are reduced. Ties go to the lower index in both stages (the first maximum).
#define AM_NT 256
__global__ __launch_bounds__(AM_NT) void argmax_partial_kernel(const float* __restrict__ logits, int V, int chunk,
                                                               float* __restrict__ part_v, int* __restrict__ part_i) {
    __shared__ ArgMax smem[AM_NT / TM_WAVE];
    const int row = blockIdx.x, c = blockIdx.y, NB = gridDim.y;
    const int lo = c * chunk, hi = lo + chunk < V ? lo + chunk : V;
    const float* src = logits + (size_t)row * V;
    ArgMax best{-INFINITY, -1};
    for (int i = lo + threadIdx.x; i < hi; i += AM_NT) {
        const float v = src[i];
        if (v == v) best = better(best, ArgMax{v, i});
    }
#pragma unroll
    for (int off = TM_WAVE / 2; off > 0; off >>= 1) {
        ArgMax o{__shfl_xor(best.v, off, TM_WAVE), __shfl_xor(best.i, off, TM_WAVE)};
        best = better(best, o);
    }
    const int wave = threadIdx.x / TM_WAVE, lane = threadIdx.x % TM_WAVE;
    if (lane == 0) smem[wave] = best;
    __syncthreads();
    if (threadIdx.x == 0) {
        ArgMax r = smem[0];
        for (int w = 1; w < AM_NT / TM_WAVE; ++w) r = better(r, smem[w]);
        part_v[(size_t)row * NB + c] = r.v;
        part_i[(size_t)row * NB + c] = r.i;
    }
}

__global__ __launch_bounds__(TM_WAVE) void argmax_final_kernel(const float* __restrict__ part_v,
                                                               const int* __restrict__ part_i, int NB,
                                                               int* __restrict__ out) {
    const int row = blockIdx.x;
    ArgMax best{-INFINITY, -1};
    for (int c = threadIdx.x; c < NB; c += TM_WAVE)
        best = better(best, ArgMax{part_v[(size_t)row * NB + c], part_i[(size_t)row * NB + c]});
#pragma unroll
    for (int off = TM_WAVE / 2; off > 0; off >>= 1) {
        ArgMax o{__shfl_xor(best.v, off, TM_WAVE), __shfl_xor(best.i, off, TM_WAVE)};
        best = better(best, o);
    }
    if (threadIdx.x == 0) out[row] = best.i < 0 ? 0 : best.i;
}

// work: at least R * tm_argmax_work_chunks(V) floats and as many ints (may be null when that is 1 chunk)
extern "C" int tm_argmax_work_chunks(int V) {
    int nb = (V + 4095) / 4096;
    return nb < 1 ? 1 : (nb > 256 ? 256 : nb);
}

extern "C" int tm_argmax_rows(const float* logits, int R, int V, int* out, float* work_v, int* work_i,
                              hipStream_t stream) {
    if (R <= 0) return TM_OK;
    if (V <= 0) return TM_ERR_ARG;
    const int NB = tm_argmax_work_chunks(V);
    if (NB == 1 || !work_v || !work_i) {
        argmax_rows_kernel<<<R, SM_NT, 0, stream>>>(logits, V, out);
        TM_CHECK_LAUNCH();
        return TM_OK;
    }
    const int chunk = (V + NB - 1) / NB;
    argmax_partial_kernel<<<dim3(R, NB), AM_NT, 0, stream>>>(logits, V, chunk, work_v, work_i);
    TM_CHECK_LAUNCH();
    argmax_final_kernel<<<R, TM_WAVE, 0, stream>>>(work_v, work_i, NB, out);
    TM_CHECK_LAUNCH();
    return TM_OK;
}

// Fixed-point weight of exp(z - zmax) in (0, 1]: integer sums are exact and order-free.
#define SM_FIX 4294967296.0f   // 2^32

__device__ __forceinline__ unsigned long long fix_weight(float e) {
    return (unsigned long long)(e * SM_FIX);
}

// One radix descent over the keys >= floor_key, eight bits a level, largest bucket first.
//   by_mass == 0: the key of the limit-th largest entry (weights are counts).
//   by_mass == 1: the smallest key whose entries have a weight <= limit ranked strictly before them
//                 (weights are fixed-point exp(z - zmax)).
// above_out[0] receives the weight of the entries whose key is larger than the returned key.
__device__ uint32_t radix_descend(const float* __restrict__ row, int V, float inv_t, float zmax, int by_mass,
                                  unsigned long long limit, uint32_t floor_key,
                                  unsigned long long* hist /* 256 */, uint32_t* pick /* 2 */,
                                  unsigned long long* above_out) {
    uint32_t prefix = 0, mask = 0;
    unsigned long long above = 0;            // weight of entries with key > every key matching prefix
    for (int shift = 24; shift >= 0; shift -= 8) {
        for (int b = threadIdx.x; b < 256; b += SM_NT) hist[b] = 0;
        __syncthreads();
        for (int i = threadIdx.x; i < V; i += SM_NT) {
            const float z = row[i] * inv_t;
            const uint32_t key = order_key(z);
            if (key < floor_key || (key & mask) != prefix) continue;
            const unsigned long long wgt = by_mass ? fix_weight(expf(z - zmax)) : 1ull;
            atomicAdd(&hist[(key >> shift) & 0xffu], wgt);
        }
        __syncthreads();
        if (threadIdx.x == 0) {
            unsigned long long run = above;
            int b = 255;
            // by count: the bucket where the running count first reaches the limit
            // by mass : the bucket where the weight before it is still <= limit but not after it
            for (; b > 0; --b) {
                const unsigned long long next = run + hist[b];
                if (by_mass ? (next > limit) : (next >= limit)) break;
                run = next;
            }
            pick[0] = (uint32_t)b;
            above_out[0] = run;
        }
        __syncthreads();
        above = above_out[0];
        prefix |= pick[0] << shift;
        mask |= 0xffu << shift;
        __syncthreads();
    }
    return prefix;
}

__global__ __launch_bounds__(SM_NT) void sample_rows_kernel(const float* __restrict__ logits, int V,
                                                            const float* __restrict__ temperature,
                                                            const int* __restrict__ top_k,
                                                            const float* __restrict__ top_p,
                                                            const float* __restrict__ u, int* __restrict__ out) {
    __shared__ ArgMax amax[SM_NT / TM_WAVE];
    __shared__ unsigned long long hist[256];
    __shared__ uint32_t pick[2];
    __shared__ unsigned long long above_s[1];
    __shared__ float part[SM_NT];
    __shared__ int found;

    const int r = blockIdx.x;
    const float* row = logits + (size_t)r * V;
    const float temp = temperature[r];
    const int k_raw = top_k[r];
    const ArgMax best = block_argmax(row, V, amax);
    if (temp <= 1e-5f || k_raw == 1) {                  // greedy (reference src/infer/engine/sequence.py:29-31)
        if (threadIdx.x == 0) out[r] = best.i;
        return;
    }
    const float inv_t = 1.f / temp;
    const float zmax = best.v * inv_t;
    const int k = (k_raw <= 0 || k_raw >= V) ? V : k_raw;
    const float p = top_p[r];

    // --- top-k: the key of the k-th largest entry; entries above it stay, ties at it stay in
    //     vocabulary order until k are kept.
    uint32_t k_key = 0;
    unsigned long long k_above = 0;
    if (k < V) {
        k_key = radix_descend(row, V, inv_t, zmax, 0, (unsigned long long)k, 0u, hist, pick, above_s);
        k_above = above_s[0];                            // entries strictly above k_key
    }
    __syncthreads();
    // --- top-p over what top-k kept: total weight Z of the kept set first
    uint32_t p_key = k_key;
    if (p < 1.f) {
        // Z = weight of entries with key >= k_key (ties at k_key beyond the k-th are few and are
        // dropped below; their weight is left out of Z by counting them in order)
        unsigned long long zsum = 0;
        {
            for (int b = threadIdx.x; b < 256; b += SM_NT) hist[b] = 0;
            __syncthreads();
            unsigned long long local = 0;
            for (int i = threadIdx.x; i < V; i += SM_NT) {
                const float z = row[i] * inv_t;
                if (order_key(z) >= k_key) local += fix_weight(expf(z - zmax));
            }
            atomicAdd(&hist[0], local);
            __syncthreads();
            zsum = hist[0];
            __syncthreads();
        }
        const unsigned long long limit = (unsigned long long)((double)zsum * (double)p);
        p_key = radix_descend(row, V, inv_t, zmax, 1, limit, k_key, hist, pick, above_s);
        if (p_key < k_key) p_key = k_key;
    }
    __syncthreads();

    // --- inverse CDF in vocabulary order over the kept entries.
    // Each thread owns a contiguous range; ties at k_key are kept first-come until k are kept.
    const int chunk = (V + SM_NT - 1) / SM_NT;
    const int begin = threadIdx.x * chunk;
    const int end = begin + chunk < V ? begin + chunk : V;
    const bool ties_matter = (k < V) && (p_key == k_key);
    // number of entries equal to k_key before this thread's range (only if ties matter)
    __shared__ int tie_cnt[SM_NT];
    int my_ties = 0;
    if (ties_matter)
        for (int i = begin; i < end; ++i) my_ties += order_key(row[i] * inv_t) == k_key;
    tie_cnt[threadIdx.x] = my_ties;
    __syncthreads();
    int ties_before = 0;
    if (ties_matter)
        for (int tix = 0; tix < (int)threadIdx.x; ++tix) ties_before += tie_cnt[tix];
    const long long tie_budget = (long long)k - (long long)k_above;   // ties that may stay

    float mine = 0.f;
    {
        int seen = ties_before;
        for (int i = begin; i < end; ++i) {
            const float z = row[i] * inv_t;
            const uint32_t key = order_key(z);
            bool keep = key >= p_key && z == z;
            if (keep && ties_matter && key == k_key) keep = (seen++) < tie_budget;
            if (keep) mine += expf(z - zmax);
        }
    }
    part[threadIdx.x] = mine;
    if (threadIdx.x == 0) found = -1;
    __syncthreads();
    // exclusive prefix over threads, in thread order (every thread computes the same sums)
    float before = 0.f, total = 0.f;
    for (int tix = 0; tix < SM_NT; ++tix) {
        if (tix == (int)threadIdx.x) before = total;
        total += part[tix];
    }
    const float target = u[r] * total;
    if (mine > 0.f && target >= before && (target < before + mine)) {
        float run = before;
        int seen = ties_before, tok = -1, last_kept = -1;
        for (int i = begin; i < end; ++i) {
            const float z = row[i] * inv_t;
            const uint32_t key = order_key(z);
            bool keep = key >= p_key && z == z;
            if (keep && ties_matter && key == k_key) keep = (seen++) < tie_budget;
            if (!keep) continue;
            last_kept = i;
            run += expf(z - zmax);
            if (target < run) { tok = i; break; }
        }
        if (tok < 0) tok = last_kept;
        atomicMax(&found, tok);
    }
    __syncthreads();
    if (threadIdx.x == 0) out[r] = found >= 0 ? found : best.i;   // rounding left target at the very end
}

extern "C" int tm_sample_rows(const float* logits, int R, int V, const float* temperature, const int* top_k,
                              const float* top_p, const float* u, int* out, hipStream_t stream) {
    if (R <= 0) return TM_OK;
    if (V <= 0) return TM_ERR_ARG;
    sample_rows_kernel<<<R, SM_NT, 0, stream>>>(logits, V, temperature, top_k, top_p, u, out);
    TM_CHECK_LAUNCH();
    return TM_OK;
}
