// Sampling over rows of 32-bit logits: argmax, and temperature sampling with optional top-k and
// top-p filters, one token per row                    (reference src/infer/sampling.py:12-46).
//
// The random number of a row is given by the caller (u in [0, 1), drawn from the request's own
// counter-based stream), so a request's tokens do not depend on its batch-mates. The token is the
// inverse CDF of the filtered softmax in vocabulary order. Filters are found by a radix descent
// over the bit patterns of the logits with integer histograms, so no sort is needed and the
// result does not depend on the order in which threads or blocks add.
#include "common.h"
#include "api.h"

#include <mutex>

#define SM_NT 1024

// monotonic map float -> uint32 (larger float, larger key)
__device__ __forceinline__ uint32_t order_key(float f) {
    uint32_t u = f == 0.f ? 0u : __float_as_uint(f);        // -0 and +0 are one value: one key
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
// clear (may be null): clear_per_row 64-bit words per row that the row's blocks set to zero between them
// (the sampler's histograms: no launch of its own for that).
__global__ __launch_bounds__(AM_NT) void argmax_partial_kernel(const float* __restrict__ logits, int V, int chunk,
                                                               float* __restrict__ part_v, int* __restrict__ part_i,
                                                               unsigned long long* __restrict__ clear,
                                                               int clear_per_row) {
    __shared__ ArgMax smem[AM_NT / TM_WAVE];
    const int row = blockIdx.x, c = blockIdx.y, NB = gridDim.y;
    if (clear) {
        const int share = (clear_per_row + NB - 1) / NB;
        const int first = c * share, last = first + share < clear_per_row ? first + share : clear_per_row;
        for (int i = first + threadIdx.x; i < last; i += AM_NT) clear[(size_t)row * clear_per_row + i] = 0ull;
    }
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
    argmax_partial_kernel<<<dim3(R, NB), AM_NT, 0, stream>>>(logits, V, chunk, work_v, work_i, nullptr, 0);
    TM_CHECK_LAUNCH();
    argmax_final_kernel<<<R, TM_WAVE, 0, stream>>>(work_v, work_i, NB, out);
    TM_CHECK_LAUNCH();
    return TM_OK;
}

// ---------------------------------------------------------------------------------------------------------
// The same argmax for callers that cannot allocate: the chunk candidates of the two-stage path live in
// a fixed array in device memory that is part of this library's image on every GPU it runs on.
//
// `argmax_scratch` names that array. In host code the name is only a handle for the runtime (not a
// device address): its address on the current device is asked for once per device
// (hipGetSymbolAddress) and kept; the kernels get that address as an argument, exactly as they get
// the caller's work buffers in tm_argmax_rows.
#define AM_STATIC_PAIRS (64 * 1024)                       // most (row, chunk) candidates: 512 KiB per GPU
#define AM_STATIC_DEVICES 64
static __device__ __align__(256) unsigned char argmax_scratch[AM_STATIC_PAIRS * (sizeof(float) + sizeof(int))];

static void* g_argmax_scratch[AM_STATIC_DEVICES];         // device address of the array, per device
static std::mutex g_argmax_scratch_mutex;

// The array's address on the device that is current now; null if the runtime cannot give it.
static void* argmax_scratch_here() {
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= AM_STATIC_DEVICES) return nullptr;
    std::lock_guard<std::mutex> lock(g_argmax_scratch_mutex);
    if (!g_argmax_scratch[dev]) {
        void* p = nullptr;
        if (hipGetSymbolAddress(&p, HIP_SYMBOL(argmax_scratch)) != hipSuccess) {
            (void)hipGetLastError();
            return nullptr;
        }
        g_argmax_scratch[dev] = p;
    }
    return g_argmax_scratch[dev];
}

extern "C" int tm_argmax_rows_static_max_pairs(void) { return AM_STATIC_PAIRS; }

extern "C" int tm_argmax_rows_static(const float* logits, int R, int V, int* out, hipStream_t stream) {
    if (R <= 0) return TM_OK;
    if (V <= 0 || !logits || !out) return TM_ERR_ARG;
    const int NB = tm_argmax_work_chunks(V);
    if (NB == 1) {                                         // a narrow row: one block, no scratch at all
        argmax_rows_kernel<<<R, SM_NT, 0, stream>>>(logits, V, out);
        TM_CHECK_LAUNCH();
        return TM_OK;
    }
    if ((long long)R * NB > AM_STATIC_PAIRS) return TM_ERR_ARG;      // beyond the fixed array: refused, nothing launched
    unsigned char* base = (unsigned char*)argmax_scratch_here();
    if (!base) return TM_ERR_LAUNCH;
    float* part_v = (float*)base;                                      // [R, NB]
    int* part_i = (int*)(base + (size_t)AM_STATIC_PAIRS * sizeof(float));   // [R, NB]
    // Nothing has to start at zero: the first kernel writes every (row, chunk) entry that the second reads.
    const int chunk = (V + NB - 1) / NB;
    argmax_partial_kernel<<<dim3(R, NB), AM_NT, 0, stream>>>(logits, V, chunk, part_v, part_i, nullptr, 0);
    TM_CHECK_LAUNCH();
    argmax_final_kernel<<<R, TM_WAVE, 0, stream>>>(part_v, part_i, NB, out);
    TM_CHECK_LAUNCH();
    return TM_OK;
}

// ---------------------------------------------------------------------------------------------------------
// Temperature sampling with top-k and top-p.
//
// A row of a wide vocabulary is cut into the chunks of the two-stage argmax (one block each), so a
// step's few rows still fill the chip; every stage is a launch over (row, chunk):
//   1. the chunk maxima (argmax_partial_kernel, which also clears the row's histograms) and the row
//      maximum (sample_rowmax_kernel): zmax for the softmax, and the token of a greedy row;
//   2. top-k, if some row asks for it: three launches, one per level of a radix descent (11, 11 and
//      10 bits of the order-preserving key of logit / temperature) that add the chunk's counts to
//      the row's histogram of that level; the blocks of the next level find the bucket that holds
//      the k-th largest entry from the histograms before it;
//   3. top-p over what top-k kept, if some row asks for it: the same descent with fixed-point
//      weights exp(z - zmax) * 2^32 instead of counts (the first level's histogram sums to the
//      kept mass Z, so the limit p * Z needs no pass of its own);
//   4. the kept mass of every chunk (sample_chunk_mass_kernel), then one block per row that walks
//      the chunks in vocabulary order to the one holding u * total and finds the token in it
//      (sample_pick_kernel).
// All histogram sums are integers, so they do not depend on the order in which blocks add; the
// float sums are taken in a fixed order that depends on V alone. A row's token depends on nothing
// but the row, its parameters and u.
// Ties at the k-th largest value are kept in vocabulary order until k entries are kept, and ties at the
// smallest value the nucleus reaches while the mass before them is at most p of the kept mass: the reference
// keeps entries by their rank in a descending sort (reference src/infer/sampling.py:15-23), which leaves the
// order of equal entries open; here, as in a stable sort, it is vocabulary order. -0 and +0 are equal.

#define SR_NT 256
#define SR_BINS 2048
#define SR_HIST_PER_ROW (6 * SR_BINS)        // three levels of the top-k descent, three of the top-p descent
#define SM_FIX 4294967296.0f                 // 2^32: fixed-point weight of exp(z - zmax) in (0, 1]

__device__ __forceinline__ unsigned long long fix_weight(float e) { return (unsigned long long)(e * SM_FIX); }
__device__ __forceinline__ int level_shift(int level) { return level == 0 ? 21 : (level == 1 ? 10 : 0); }
__device__ __forceinline__ int level_bins(int level) { return level == 2 ? 1024 : 2048; }
__device__ __forceinline__ float key_value(uint32_t key) {
    return __uint_as_float((key & 0x80000000u) ? (key ^ 0x80000000u) : ~key);
}

struct RowParams {
    bool greedy, need_k, need_p;
    int k;
    float p, inv_t, zmax;
};

__device__ __forceinline__ RowParams row_params(int r, int V, const float* temperature, const int* top_k,
                                                const float* top_p, const float* rowmax) {
    RowParams rp;
    const float temp = temperature[r];
    const int k_raw = top_k[r];
    rp.greedy = temp <= 1e-5f || k_raw == 1;           // reference src/infer/engine/sequence.py:29-31
    rp.inv_t = rp.greedy ? 1.f : 1.f / temp;
    rp.k = (k_raw <= 0 || k_raw >= V) ? V : k_raw;
    rp.need_k = !rp.greedy && rp.k < V;
    rp.p = top_p[r];
    rp.need_p = !rp.greedy && rp.p < 1.f;
    rp.zmax = rowmax[r] * rp.inv_t;
    return rp;
}

// Block-wide (SR_NT threads, all of them call): the bucket of one level's histogram, walking from
// the largest bucket down, in which
//   by count: the running count first reaches `limit`;
//   by mass : the running weight would first exceed `limit`
// (bucket 0 if that never happens), and the weight of the buckets above it added to `above`.
// frac >= 0: limit = frac * (the histogram's total - drop), returned through `limit` (first level by mass;
// drop: weight in the histogram that belongs to entries top-k does not keep after all, ties beyond its budget).
__device__ void pick_bucket(const unsigned long long* __restrict__ hist, int bins, bool by_mass, double frac,
                            unsigned long long drop, unsigned long long& limit, unsigned long long& above,
                            uint32_t& bucket, unsigned long long* s_scan /* SR_NT */, unsigned long long* s_res /* 2 */) {
    const int t = threadIdx.x, per = bins / SR_NT;
    unsigned long long local[SR_BINS / SR_NT];
    unsigned long long sum = 0;
#pragma unroll
    for (int j = 0; j < SR_BINS / SR_NT; ++j) {
        local[j] = j < per ? hist[bins - 1 - (t * per + j)] : 0ull;
        sum += local[j];
    }
    __syncthreads();                                     // s_scan and s_res may still be read from the call before
    s_scan[t] = sum;
    __syncthreads();
    for (int off = 1; off < SR_NT; off <<= 1) {          // inclusive scan over the threads
        const unsigned long long add = t >= off ? s_scan[t - off] : 0ull;
        __syncthreads();
        s_scan[t] += add;
        __syncthreads();
    }
    const unsigned long long incl = s_scan[t], excl = incl - sum, total = s_scan[SR_NT - 1];
    if (frac >= 0.0) limit = (unsigned long long)((double)(total > drop ? total - drop : 0ull) * frac);
    auto reached = [&](unsigned long long run) { return by_mass ? run > limit : run >= limit; };
    if (t == SR_NT - 1 && !reached(above + total)) {     // never: bucket 0, everything above it counts
        s_res[0] = 0ull;
        s_res[1] = above + total - hist[0];
    }
    if (reached(above + incl) && !reached(above + excl)) {
        unsigned long long run = above + excl;
        int pick = per - 1;                              // the last of the thread's buckets if no earlier one
        bool open = true;
#pragma unroll
        for (int j = 0; j < SR_BINS / SR_NT; ++j) {
            if (open && j < per - 1) {
                if (reached(run + local[j])) {
                    pick = j;
                    open = false;
                } else {
                    run += local[j];
                }
            }
        }
        s_res[0] = (unsigned long long)(bins - 1 - (t * per + pick));
        s_res[1] = run;
    }
    __syncthreads();
    bucket = (uint32_t)s_res[0];
    above = s_res[1];
}

// The key of the k-th largest entry (by count) or the smallest key the nucleus keeps (by mass) from a
// row's three finished histograms; `above` = count / weight of the entries with a larger key.
__device__ uint32_t descend(const unsigned long long* __restrict__ hist3, int levels, bool by_mass, double frac,
                            unsigned long long& limit, unsigned long long& above, uint32_t& mask,
                            unsigned long long* s_scan, unsigned long long* s_res, unsigned long long drop = 0ull) {
    uint32_t prefix = 0;
    mask = 0;
    above = 0;
    for (int level = 0; level < levels; ++level) {
        uint32_t bucket;
        pick_bucket(hist3 + (size_t)level * SR_BINS, level_bins(level), by_mass, level == 0 ? frac : -1.0, drop, limit,
                    above, bucket, s_scan, s_res);
        prefix |= bucket << level_shift(level);
        mask |= (uint32_t)(level_bins(level) - 1) << level_shift(level);
    }
    return prefix;
}

// Where top-k ends in a row (block-wide, all threads call; the row's three count histograms are finished):
// the key of the k-th largest entry, how many of the entries with that key stay (the first `budget` in
// vocabulary order: the entries with a larger key are fewer than k, the ties fill up to k), and the weight
// of the ties that do not stay (they are in the top-p histograms, which take every entry from that key up).
struct KEdge {
    uint32_t key;
    int budget;
    unsigned long long dropped;
};
__device__ KEdge k_edge(const unsigned long long* __restrict__ hist_k, const RowParams& rp,
                        unsigned long long* s_scan, unsigned long long* s_res) {
    unsigned long long limit = (unsigned long long)rp.k, above = 0;
    uint32_t mask;
    KEdge e;
    e.key = descend(hist_k, 3, false, -1.0, limit, above, mask, s_scan, s_res);
    const long long budget = (long long)rp.k - (long long)above;         // above: entries strictly larger
    e.budget = budget > 0x7fffffffLL ? 0x7fffffff : (budget < 0 ? 0 : (int)budget);
    const unsigned long long ties = hist_k[2 * SR_BINS + (e.key & (uint32_t)(level_bins(2) - 1))];
    const unsigned long long cut = ties > (unsigned long long)e.budget ? ties - (unsigned long long)e.budget : 0ull;
    e.dropped = cut * fix_weight(expf(key_value(e.key) - rp.zmax));
    return e;
}

__global__ __launch_bounds__(TM_WAVE) void sample_rowmax_kernel(const float* __restrict__ part_v,
                                                                const int* __restrict__ part_i, int NB,
                                                                float* __restrict__ rowmax, int* __restrict__ rowarg) {
    const int row = blockIdx.x;
    ArgMax best{-INFINITY, -1};
    for (int c = threadIdx.x; c < NB; c += TM_WAVE)
        best = better(best, ArgMax{part_v[(size_t)row * NB + c], part_i[(size_t)row * NB + c]});
#pragma unroll
    for (int off = TM_WAVE / 2; off > 0; off >>= 1) {
        ArgMax o{__shfl_xor(best.v, off, TM_WAVE), __shfl_xor(best.i, off, TM_WAVE)};
        best = better(best, o);
    }
    if (threadIdx.x == 0) {
        rowmax[row] = best.i < 0 ? 0.f : best.v;
        rowarg[row] = best.i < 0 ? 0 : best.i;
    }
}

// One level of a descent: the chunk's entries that match the buckets picked so far, into the row's
// histogram of this level. BY_MASS: the top-p descent (weights, over what top-k kept).
template <bool BY_MASS>
__global__ __launch_bounds__(SR_NT) void sample_hist_kernel(const float* __restrict__ logits, int V, int chunk,
                                                            const float* __restrict__ temperature,
                                                            const int* __restrict__ top_k,
                                                            const float* __restrict__ top_p,
                                                            const float* __restrict__ rowmax,
                                                            unsigned long long* __restrict__ hist_all, int level) {
    __shared__ unsigned long long s_hist[SR_BINS];
    __shared__ unsigned long long s_scan[SR_NT];
    __shared__ unsigned long long s_res[2];
    const int r = blockIdx.x, c = blockIdx.y;
    const RowParams rp = row_params(r, V, temperature, top_k, top_p, rowmax);
    if (BY_MASS ? !rp.need_p : !rp.need_k) return;       // block-uniform
    unsigned long long* hist_k = hist_all + (size_t)r * SR_HIST_PER_ROW;
    unsigned long long* hist_p = hist_k + 3 * SR_BINS;
    uint32_t floor_key = 0, prefix = 0, mask = 0;
    unsigned long long limit = 0, above = 0;
    if (BY_MASS) {
        unsigned long long dropped = 0;
        if (rp.need_k) {
            const KEdge e = k_edge(hist_k, rp, s_scan, s_res);
            floor_key = e.key;
            dropped = e.dropped;
        }
        prefix = descend(hist_p, level, true, (double)rp.p, limit, above, mask, s_scan, s_res, dropped);
    } else {
        limit = (unsigned long long)rp.k;
        prefix = descend(hist_k, level, false, -1.0, limit, above, mask, s_scan, s_res);
    }
    for (int b = threadIdx.x; b < SR_BINS; b += SR_NT) s_hist[b] = 0ull;
    __syncthreads();
    const float* row = logits + (size_t)r * V;
    const int lo = c * chunk, hi = lo + chunk < V ? lo + chunk : V;
    const int shift = level_shift(level);
    const uint32_t digit_mask = (uint32_t)(level_bins(level) - 1);
    for (int i = lo + threadIdx.x; i < hi; i += SR_NT) {
        const float z = row[i] * rp.inv_t;
        if (!(z == z)) continue;
        const uint32_t key = order_key(z);
        if (key < floor_key || (key & mask) != prefix) continue;
        atomicAdd(&s_hist[(key >> shift) & digit_mask], BY_MASS ? fix_weight(expf(z - rp.zmax)) : 1ull);
    }
    __syncthreads();
    unsigned long long* dst = (BY_MASS ? hist_p : hist_k) + (size_t)level * SR_BINS;
    for (int b = threadIdx.x; b < SR_BINS; b += SR_NT)
        if (s_hist[b]) atomicAdd(&dst[b], s_hist[b]);
}

// What a row keeps, as the last two stages need it.
struct RowKeep {
    uint32_t p_key;             // entries with a larger key stay, entries with a smaller one go
    int ties_matter;            // entries equal to p_key stay only until tie_budget of them are kept, in
    int tie_budget;             // vocabulary order (top-k: until k entries stay; top-p: while the mass before
};                              // the entry is at most p; both: the smaller of the two)

// The kept weight of one entry without the ties at p_key (0 if it is dropped or such a tie), and whether
// it is such a tie.
__device__ __forceinline__ float entry_weight(float logit, const RowParams& rp, const RowKeep& keep, bool& tie) {
    const float z = logit * rp.inv_t;
    tie = false;
    if (!(z == z)) return 0.f;
    const uint32_t key = order_key(z);
    if (key < keep.p_key) return 0.f;
    if (keep.ties_matter && key == keep.p_key) {
        tie = true;
        return 0.f;
    }
    return expf(z - rp.zmax);
}

// Block-wide sums in a fixed order: lanes by a butterfly, wavefronts one after the other.
__device__ __forceinline__ void block_sums(float& w, int& n, float* s_w /* SR_NT / 64 */, int* s_n) {
#pragma unroll
    for (int off = TM_WAVE / 2; off > 0; off >>= 1) {
        w += __shfl_xor(w, off, TM_WAVE);
        n += __shfl_xor(n, off, TM_WAVE);
    }
    const int wave = threadIdx.x / TM_WAVE, lane = threadIdx.x % TM_WAVE;
    __syncthreads();
    if (lane == 0) {
        s_w[wave] = w;
        s_n[wave] = n;
    }
    __syncthreads();
    w = s_w[0];
    n = s_n[0];
    for (int i = 1; i < SR_NT / TM_WAVE; ++i) {
        w += s_w[i];
        n += s_n[i];
    }
}

__global__ __launch_bounds__(SR_NT) void sample_chunk_mass_kernel(const float* __restrict__ logits, int V, int chunk,
                                                                  const float* __restrict__ temperature,
                                                                  const int* __restrict__ top_k,
                                                                  const float* __restrict__ top_p,
                                                                  const float* __restrict__ rowmax,
                                                                  const unsigned long long* __restrict__ hist_all,
                                                                  float* __restrict__ chunk_weight,
                                                                  int* __restrict__ chunk_ties,
                                                                  RowKeep* __restrict__ row_keep) {
    __shared__ unsigned long long s_scan[SR_NT];
    __shared__ unsigned long long s_res[2];
    __shared__ float s_w[SR_NT / TM_WAVE];
    __shared__ int s_n[SR_NT / TM_WAVE];
    const int r = blockIdx.x, c = blockIdx.y, NB = gridDim.y;
    const RowParams rp = row_params(r, V, temperature, top_k, top_p, rowmax);
    if (rp.greedy) return;                               // block-uniform
    const unsigned long long* hist_k = hist_all + (size_t)r * SR_HIST_PER_ROW;
    const unsigned long long* hist_p = hist_k + 3 * SR_BINS;
    RowKeep keep{0u, 0, 0};
    unsigned long long dropped = 0;
    if (rp.need_k) {
        const KEdge e = k_edge(hist_k, rp, s_scan, s_res);
        keep.p_key = e.key;
        keep.ties_matter = 1;
        keep.tie_budget = e.budget;
        dropped = e.dropped;
    }
    if (rp.need_p) {
        // the smallest key the nucleus reaches; the entries with that key stay while the mass before them
        // is at most p of the kept mass (reference src/infer/sampling.py:20-23: ties in sorted order, which
        // here is vocabulary order; the first always stays): limit = p * mass, above = mass of larger keys
        unsigned long long limit = 0, above = 0;
        uint32_t mask;
        const uint32_t pk = descend(hist_p, 3, true, (double)rp.p, limit, above, mask, s_scan, s_res, dropped);
        if (!rp.need_k || pk >= keep.p_key) {
            const unsigned long long w = fix_weight(expf(key_value(pk) - rp.zmax));
            const unsigned long long room = limit > above ? limit - above : 0ull;
            const unsigned long long fit = w ? room / w + 1ull : 0x7fffffffull;
            const int by_mass = fit > 0x7fffffffull ? 0x7fffffff : (int)fit;
            const bool same = rp.need_k && pk == keep.p_key;
            keep.tie_budget = same && keep.tie_budget < by_mass ? keep.tie_budget : by_mass;
            keep.p_key = pk;
            keep.ties_matter = 1;
        }
    }
    if (c == 0 && threadIdx.x == 0) row_keep[r] = keep;
    const float* row = logits + (size_t)r * V;
    const int lo = c * chunk, hi = lo + chunk < V ? lo + chunk : V;
    float w = 0.f;
    int ties = 0;
    for (int i = lo + threadIdx.x; i < hi; i += SR_NT) {
        bool tie;
        w += entry_weight(row[i], rp, keep, tie);
        ties += tie;
    }
    block_sums(w, ties, s_w, s_n);
    if (threadIdx.x == 0) {
        chunk_weight[(size_t)r * NB + c] = w;
        chunk_ties[(size_t)r * NB + c] = ties;
    }
}

// Of `ties` ties that follow `seen` earlier ones, how many stay.
__device__ __forceinline__ int kept_ties(const RowKeep& keep, int seen, int ties) {
    const int room = keep.tie_budget - seen;
    return room <= 0 ? 0 : (room < ties ? room : ties);
}

// Walks n masses (weight[i] + kept ties of ties[i] * w_tie) in order to the one that holds `target`
// (the last one with any mass if rounding left the target beyond the end); one thread calls it.
struct Walk {
    int pick, seen;             // -1 if nothing has mass; ties before the picked one
    float before;               // mass before the picked one
};
__device__ __forceinline__ Walk walk_to(const float* weight, const int* ties, int n, const RowKeep& keep, float w_tie,
                                        float target, float run, int seen) {
    Walk last{-1, 0, 0.f};
    for (int i = 0; i < n; ++i) {
        const float mass = weight[i] + (float)kept_ties(keep, seen, ties[i]) * w_tie;
        if (mass > 0.f) {
            last = Walk{i, seen, run};
            if (target < run + mass) return last;
        }
        run += mass;
        seen += ties[i];
    }
    return last;
}

#define SR_MAX_CHUNKS 256
#define SR_MAX_ROWS 16          // a chunk has at most 4096 entries: 16 lines of SR_NT

__global__ __launch_bounds__(SR_NT) void sample_pick_kernel(const float* __restrict__ logits, int V, int chunk, int NB,
                                                            const float* __restrict__ temperature,
                                                            const int* __restrict__ top_k,
                                                            const float* __restrict__ top_p,
                                                            const float* __restrict__ rowmax,
                                                            const int* __restrict__ rowarg,
                                                            const float* __restrict__ chunk_weight,
                                                            const int* __restrict__ chunk_ties,
                                                            const RowKeep* __restrict__ row_keep,
                                                            const float* __restrict__ u, int* __restrict__ out) {
    __shared__ float s_cw[SR_MAX_CHUNKS];
    __shared__ int s_ct[SR_MAX_CHUNKS];
    __shared__ float s_lw[SR_MAX_ROWS];
    __shared__ int s_lt[SR_MAX_ROWS];
    __shared__ float s_w[SR_NT / TM_WAVE];
    __shared__ int s_n[SR_NT / TM_WAVE];
    __shared__ float s_pw[SR_NT / TM_WAVE][SR_MAX_ROWS];
    __shared__ int s_pn[SR_NT / TM_WAVE][SR_MAX_ROWS];
    __shared__ Walk s_walk;
    __shared__ float s_target;
    __shared__ int s_first, s_last;
    const int r = blockIdx.x;
    const RowParams rp = row_params(r, V, temperature, top_k, top_p, rowmax);
    if (rp.greedy) {
        if (threadIdx.x == 0) out[r] = rowarg[r];
        return;
    }
    const RowKeep keep = row_keep[r];
    const float u_row = u[r];
    const float w_tie = keep.ties_matter ? expf(key_value(keep.p_key) - rp.zmax) : 0.f;
    // 1. the chunk that holds u * total, walking the chunks in vocabulary order
    for (int c = threadIdx.x; c < NB; c += SR_NT) {
        s_cw[c] = chunk_weight[(size_t)r * NB + c];
        s_ct[c] = chunk_ties[(size_t)r * NB + c];
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        float total = 0.f;
        int seen = 0;
        for (int c = 0; c < NB; ++c) {
            total += s_cw[c] + (float)kept_ties(keep, seen, s_ct[c]) * w_tie;
            seen += s_ct[c];
        }
        s_target = u_row * total;
        s_walk = walk_to(s_cw, s_ct, NB, keep, w_tie, s_target, 0.f, 0);
        s_first = 0x7fffffff;
        s_last = -1;
    }
    __syncthreads();
    const Walk at_chunk = s_walk;
    const float target = s_target;
    if (at_chunk.pick < 0) {                             // nothing kept (every entry NaN): the first maximum
        if (threadIdx.x == 0) out[r] = rowarg[r];
        return;
    }
    // 2. the line of SR_NT consecutive entries of that chunk: a thread holds one entry of every line (all
    //    loads in flight at once), the lines are summed lanes first, wavefronts one after the other
    const float* row = logits + (size_t)r * V;
    const int lo = at_chunk.pick * chunk, hi = lo + chunk < V ? lo + chunk : V;
    const int lines = (hi - lo + SR_NT - 1) / SR_NT;
    const int wave = threadIdx.x / TM_WAVE, lane = threadIdx.x % TM_WAVE;
    float raw[SR_MAX_ROWS];
#pragma unroll
    for (int j = 0; j < SR_MAX_ROWS; ++j) {
        const int i = lo + j * SR_NT + (int)threadIdx.x;
        raw[j] = row[i < hi ? i : hi - 1];
    }
    float wj[SR_MAX_ROWS];
    uint32_t tie_bits = 0;
#pragma unroll
    for (int j = 0; j < SR_MAX_ROWS; ++j) {
        const int i = lo + j * SR_NT + (int)threadIdx.x;
        bool tie = false;
        wj[j] = i < hi ? entry_weight(raw[j], rp, keep, tie) : 0.f;
        tie_bits |= (tie ? 1u : 0u) << j;
        float w = wj[j];
        int n = tie;
#pragma unroll
        for (int off = TM_WAVE / 2; off > 0; off >>= 1) {
            w += __shfl_xor(w, off, TM_WAVE);
            n += __shfl_xor(n, off, TM_WAVE);
        }
        if (lane == 0) {
            s_pw[wave][j] = w;
            s_pn[wave][j] = n;
        }
    }
    __syncthreads();
    if (threadIdx.x < SR_MAX_ROWS) {
        float w = s_pw[0][threadIdx.x];
        int n = s_pn[0][threadIdx.x];
        for (int v = 1; v < SR_NT / TM_WAVE; ++v) {
            w += s_pw[v][threadIdx.x];
            n += s_pn[v][threadIdx.x];
        }
        s_lw[threadIdx.x] = w;
        s_lt[threadIdx.x] = n;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        const Walk in_chunk = walk_to(s_lw, s_lt, lines, keep, w_tie, target, at_chunk.before, at_chunk.seen);
        s_walk = in_chunk;
    }
    __syncthreads();
    const Walk at_line = s_walk;
    if (at_line.pick < 0) {                              // (sums of another order saw mass here: take the maximum)
        if (threadIdx.x == 0) out[r] = rowarg[r];
        return;
    }
    // 3. the entry of that line: each thread its entry of it, a running sum over the threads in order
    const int i = lo + at_line.pick * SR_NT + (int)threadIdx.x;
    float w = 0.f;
#pragma unroll
    for (int j = 0; j < SR_MAX_ROWS; ++j) w = j == at_line.pick ? wj[j] : w;
    const bool tie = (tie_bits >> at_line.pick) & 1u;
    if (keep.ties_matter) {                              // a tie stays if fewer than the budget came before it
        const unsigned long long ballot = __ballot(tie);
        int rank = __popcll(ballot & ((1ull << lane) - 1ull));
        __syncthreads();
        if (lane == 0) s_n[wave] = __popcll(ballot);
        __syncthreads();
        for (int v = 0; v < wave; ++v) rank += s_n[v];
        if (tie && at_line.seen + rank < keep.tie_budget) w = w_tie;
    }
    float incl = w;
#pragma unroll
    for (int off = 1; off < TM_WAVE; off <<= 1) {
        const float up = __shfl_up(incl, off, TM_WAVE);
        if (lane >= off) incl += up;
    }
    __syncthreads();
    if (lane == TM_WAVE - 1) s_w[wave] = incl;
    __syncthreads();
    float base = at_line.before;
    for (int v = 0; v < wave; ++v) base += s_w[v];
    incl += base;
    // the first entry with mass whose running sum passes the target; else the last entry with mass
    if (w > 0.f) {
        if (target < incl) atomicMin(&s_first, i);
        atomicMax(&s_last, i);
    }
    __syncthreads();
    if (threadIdx.x == 0) out[r] = s_first != 0x7fffffff ? s_first : (s_last >= 0 ? s_last : rowarg[r]);
}

// Bytes of device memory tm_sample_rows needs for R rows of V logits (16-byte aligned start).
static size_t sample_hist_bytes(int R) { return (size_t)R * SR_HIST_PER_ROW * sizeof(unsigned long long); }
extern "C" size_t tm_sample_work_bytes(int R, int V) {
    const size_t NB = (size_t)tm_argmax_work_chunks(V);
    const size_t per_chunk = (size_t)R * NB * 4;         // part_v, part_i, chunk_weight, chunk_ties
    return sample_hist_bytes(R) + 4 * per_chunk + (size_t)R * (sizeof(RowKeep) + 8);
}

// stages: bit 0 = some row may use top-k, bit 1 = some row may use top-p (3 if the caller does not
// know: rows that use neither skip those launches' work). Calls on one `work` must not overlap.
extern "C" int tm_sample_rows(const float* logits, int R, int V, const float* temperature, const int* top_k,
                              const float* top_p, const float* u, int* out, void* work, size_t work_bytes,
                              int stages, hipStream_t stream) {
    if (R <= 0) return TM_OK;
    if (V <= 0 || !work || ((uintptr_t)work % 16) || work_bytes < tm_sample_work_bytes(R, V)) return TM_ERR_ARG;
    const int NB = tm_argmax_work_chunks(V);
    const int chunk = (V + NB - 1) / NB;
    if (chunk > SR_MAX_ROWS * SR_NT || NB > SR_MAX_CHUNKS) return TM_ERR_ARG;      // more than 2^20 logits a row
    unsigned char* w = (unsigned char*)work;
    unsigned long long* hist = (unsigned long long*)w;
    w += sample_hist_bytes(R);
    float* part_v = (float*)w;          w += (size_t)R * NB * 4;
    int* part_i = (int*)w;              w += (size_t)R * NB * 4;
    float* chunk_weight = (float*)w;    w += (size_t)R * NB * 4;
    int* chunk_ties = (int*)w;          w += (size_t)R * NB * 4;
    RowKeep* row_keep = (RowKeep*)w;    w += (size_t)R * sizeof(RowKeep);
    float* rowmax = (float*)w;          w += (size_t)R * 4;
    int* rowarg = (int*)w;
    const dim3 grid(R, NB);
    argmax_partial_kernel<<<grid, AM_NT, 0, stream>>>(logits, V, chunk, part_v, part_i, hist, SR_HIST_PER_ROW);
    TM_CHECK_LAUNCH();
    sample_rowmax_kernel<<<R, TM_WAVE, 0, stream>>>(part_v, part_i, NB, rowmax, rowarg);
    TM_CHECK_LAUNCH();
    if (stages & 1)
        for (int level = 0; level < 3; ++level) {
            sample_hist_kernel<false><<<grid, SR_NT, 0, stream>>>(logits, V, chunk, temperature, top_k, top_p, rowmax,
                                                                 hist, level);
            TM_CHECK_LAUNCH();
        }
    if (stages & 2)
        for (int level = 0; level < 3; ++level) {
            sample_hist_kernel<true><<<grid, SR_NT, 0, stream>>>(logits, V, chunk, temperature, top_k, top_p, rowmax,
                                                                hist, level);
            TM_CHECK_LAUNCH();
        }
    sample_chunk_mass_kernel<<<grid, SR_NT, 0, stream>>>(logits, V, chunk, temperature, top_k, top_p, rowmax, hist,
                                                         chunk_weight, chunk_ties, row_keep);
    TM_CHECK_LAUNCH();
    sample_pick_kernel<<<R, SR_NT, 0, stream>>>(logits, V, chunk, NB, temperature, top_k, top_p, rowmax, rowarg,
                                                chunk_weight, chunk_ties, row_keep, u, out);
    TM_CHECK_LAUNCH();
    return TM_OK;
}
