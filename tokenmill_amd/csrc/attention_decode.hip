// Paged attention for single decoded tokens on MFMA (bfloat16), split over the context.
//
//   One token per request; its G = H / KVH query heads that share a kv head are the 16 columns of
//   one MFMA tile, so the keys and values of a kv head are read once for all of them
//   (the reference folds the group into query rows the same way: src/infer/model/layers.py:110-124).
//   A wavefront always takes 64 consecutive keys, aligned to a multiple of 64 positions, and gets
//   their unnormalised partial (max, sum, weighted values) in 32-bit. Two ways to cover a context:
//
//   block kernel : one block of 8 (16 for head size 32) wavefronts per (request, kv head); wavefront
//                  w takes keys [64 (i W + w), +64) for i = 0, 1, ...; the partials are merged
//                  through LDS in wavefront order. One launch, no scratch memory: the way for large
//                  batches.
//   split kernels: with few requests more blocks than (request, kv head) pairs are needed to pull
//                  the cache at speed: blocks of four wavefronts take chunks of 256 positions and
//                  write partials to scratch memory; a second kernel adds the partials of a request
//                  in ascending chunk order.
//
//   Which keys meet in which partial and in which order partials are added depends on positions
//   only, so within either way what a request gets does not depend on which other requests are in
//   the batch (which way runs depends on how many there are: the two differ by rounding).
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

// The keys and values of 64 positions [wbase, wbase + 64) of one kv head as a wavefront holds them
// between asking for them and using them: four tiles of 16 keys as MFMA operands.
//
// Which 16 keys make a tile is chosen for the loads of the values. A lane of the second product needs, for
// 32 keys at a time, 8 keys of one row d of V^T, and it must be the 8 keys whose probabilities the lane got
// from the first product's accumulators: 4 from each tile of a pair. With tiles of consecutive keys those are
// 4 + 4 keys 16 apart: two 8-byte loads, and an instruction of the wavefront touches 32 bytes of each of 16
// rows, which reads the pool at 3.9 TB/s at best. So the tiles of a pair (2b, 2b + 1) split their 32 keys in
// runs of four: row rho of tile t is key 32 (t / 2) + 8 (rho / 4) + 4 (t % 2) + rho % 4. The lane that holds
// rows 4g..4g+3 of both tiles then has the keys 32b + 8g .. + 7: one 16-byte load, 64 bytes of a row an
// instruction (4.7 TB/s), and half as many loads. The keys are whole rows of the pool either way.
__device__ __forceinline__ int tile_key(int t, int rho) { return 32 * (t / 2) + 8 * (rho / 4) + 4 * (t % 2) + rho % 4; }

template <int D>
struct Keys64 {
    int group_page[4];                      // page of the 16 positions [wbase + 16 q, + 16), -1 if no query may see them (wave-uniform)
    Bf16x8Bits k[4][D / 32];                // [tile][32 d]
    u32x4_t v[D / 16][2];                   // [16 d][32 keys]: keys 32 b + 8 g .. + 7 of row d = 16 dt + r
};

// The block-table entries of the four 16-key tiles of [wbase, wbase + 64), read without a test at an
// index inside the row (what lies beyond the context is dropped by load_keys64): they depend on
// nothing but the request, so a kernel can ask for them before it knows the context length.
__device__ __forceinline__ void load_table_entries(int (&entry)[4], const int* __restrict__ table, int table_width,
                                                   int wbase, int page_shift) {
#pragma unroll
    for (int t = 0; t < 4; ++t) {
        const int at = (wbase + 16 * t) >> page_shift;
        entry[t] = table[at < table_width ? at : table_width - 1];
    }
}

// Ask for the keys and values of [wbase, wbase + 64): every load is issued, nothing is waited for.
template <int D>
__device__ __forceinline__ void load_keys64(Keys64<D>& kv, const bf16_t* __restrict__ k_pool,
                                            const bf16_t* __restrict__ v_pool, const int (&entry)[4], int wbase,
                                            int ctx, int lo, int kvh, int KVH, int page_shift, int r, int g) {
    constexpr int NDC = D / 32, NDT = D / 16;
    const int page_mask = (1 << page_shift) - 1;
#pragma unroll
    for (int q = 0; q < 4; ++q) {
        const int first = wbase + 16 * q;
        kv.group_page[q] = (first < ctx && first + 16 > lo) ? entry[q] : -1;                        // wave-uniform
    }
    // Every load is unconditional, so that none of them has to be waited for before the next is
    // issued: positions nobody may see read page 0 instead, and keys beyond the context read the rest of
    // their page. What such loads bring is never used: their scores are replaced by -inf and their
    // values are masked bit by bit.
#pragma unroll
    for (int t = 0; t < 4; ++t) {
        // the 16 positions of a row's key: the pair's first 16 for rows 0..7, its second 16 for rows 8..15
        const int key = wbase + tile_key(t, r);
        const int page = r < 8 ? kv.group_page[2 * (t / 2)] : kv.group_page[2 * (t / 2) + 1];
        const size_t pg = page >= 0 ? (size_t)page : 0;
        const bf16_t* kr = k_pool + (((pg << page_shift) + (key & page_mask)) * KVH + kvh) * D + 8 * g;
#pragma unroll
        for (int c = 0; c < NDC; ++c) kv.k[t][c].u = *(const u32x4_t*)(kr + 32 * c);
    }
#pragma unroll
    for (int b = 0; b < 2; ++b) {
        const int key = wbase + 32 * b + 8 * g;                      // this lane's 8 keys of the pair
        const int page = g < 2 ? kv.group_page[2 * b] : kv.group_page[2 * b + 1];
        const size_t pg = page >= 0 ? (size_t)page : 0;
        const bf16_t* vr = v_pool + (((pg * KVH + kvh) * D + r) << page_shift) + (key & page_mask);
#pragma unroll
        for (int dt = 0; dt < NDT; ++dt) kv.v[dt][b] = *(const u32x4_t*)(vr + ((size_t)(16 * dt) << page_shift));
    }
    // nothing that uses the keys may be scheduled above the loads of the values: both are on their
    // way before the first wait
    __builtin_amdgcn_sched_barrier(0);
}

// The partial of the 64 keys in kv for the (up to 16) query heads of one kv head.
// m is in units of score * scale * log2(e).
template <int D>
__device__ __forceinline__ void attend_keys64(const Keys64<D>& kv, const Bf16x8Bits (&qreg)[D / 32], int wbase, int ctx,
                                              int lo, float scale_log2, int g, float& m, float& l,
                                              f32x4_t (&o)[D / 16]) {
    constexpr int NDC = D / 32, NDT = D / 16;
    float sc[4][4];                                                 // [tile][row 4g+i of the tile] for head r
#pragma unroll
    for (int t = 0; t < 4; ++t) {
        f32x4_t acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int c = 0; c < NDC; ++c)
            acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kv.k[t][c].b, qreg[c].b, acc, 0, 0, 0);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int kj = wbase + tile_key(t, 4 * g + i);
            sc[t][i] = (kj < ctx && kj >= lo) ? acc[i] * scale_log2 : -INFINITY;
        }
    }
    m = -INFINITY;
#pragma unroll
    for (int t = 0; t < 4; ++t)
#pragma unroll
        for (int i = 0; i < 4; ++i) m = fmaxf(m, sc[t][i]);
    m = fmaxf(m, __shfl_xor(m, 16, TM_WAVE));
    m = fmaxf(m, __shfl_xor(m, 32, TM_WAVE));
    const float neg_m = (m == -INFINITY) ? 0.f : -m;
    l = 0.f;
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
    // O^T[d][head] = V^T[d][keys] P^T[keys][head], 32 keys (tiles 2b, 2b+1) per instruction
#pragma unroll
    for (int dt = 0; dt < NDT; ++dt) o[dt] = f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int b = 0; b < 2; ++b) {
        Bf16x8Bits pt;
        pt.u = u32x4_t{pack_bf16(pr[2 * b][0], pr[2 * b][1]), pack_bf16(pr[2 * b][2], pr[2 * b][3]),
                       pack_bf16(pr[2 * b + 1][0], pr[2 * b + 1][1]), pack_bf16(pr[2 * b + 1][2], pr[2 * b + 1][3])};
        // which of this lane's 8 keys exist (a value beyond the context may hold anything)
        uint32_t keep[4];
#pragma unroll
        for (int w2 = 0; w2 < 4; ++w2) {
            const int ka = wbase + 32 * b + 8 * g + 2 * w2, kb = ka + 1;
            keep[w2] = ((ka < ctx && ka >= lo) ? 0x0000ffffu : 0u) | ((kb < ctx && kb >= lo) ? 0xffff0000u : 0u);
        }
#pragma unroll
        for (int dt = 0; dt < NDT; ++dt) {
            Bf16x8Bits vf;
            vf.u = u32x4_t{kv.v[dt][b][0] & keep[0], kv.v[dt][b][1] & keep[1], kv.v[dt][b][2] & keep[2],
                           kv.v[dt][b][3] & keep[3]};
            o[dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf.b, pt.b, o[dt], 0, 0, 0);
        }
    }
}

// Load, then attend: the partial of 64 keys [wbase, wbase + 64).
template <int D>
__device__ __forceinline__ void wave_keys64(const Bf16x8Bits (&qreg)[D / 32], const bf16_t* __restrict__ k_pool,
                                            const bf16_t* __restrict__ v_pool, const int* __restrict__ table,
                                            int table_width, int wbase, int ctx, int lo, int kvh, int KVH,
                                            int page_shift, float scale_log2, int r, int g, float& m, float& l,
                                            f32x4_t (&o)[D / 16]) {
    int entry[4];
    load_table_entries(entry, table, table_width, wbase, page_shift);
    Keys64<D> kv;
    load_keys64<D>(kv, k_pool, v_pool, entry, wbase, ctx, lo, kvh, KVH, page_shift, r, g);
    attend_keys64<D>(kv, qreg, wbase, ctx, lo, scale_log2, g, m, l, o);
}

template <int D>
__device__ __forceinline__ void load_q_operand(Bf16x8Bits (&qreg)[D / 32], const bf16_t* __restrict__ q, int G,
                                               int kvh, int r, int g) {
    // Q^T operand: column r = query head kvh*G + r, rows d = 32c + 8g .. +7
#pragma unroll
    for (int c = 0; c < D / 32; ++c) {
        if (r < G)
            qreg[c].u = *(const u32x4_t*)(q + (size_t)(kvh * G + r) * D + 32 * c + 8 * g);
        else
            qreg[c].u = u32x4_t{0, 0, 0, 0};
    }
}

// ------------------------------------------------------------------------------------------------
// block kernel: grid (S, KVH), WAVES wavefronts
// ------------------------------------------------------------------------------------------------
template <int D, int WAVES>
__global__ __launch_bounds__(64 * WAVES) void attn_decode_block_kernel(
    const bf16_t* __restrict__ q, int q_stride, bf16_t* __restrict__ out, int out_stride,
    const bf16_t* __restrict__ k_pool, const bf16_t* __restrict__ v_pool, const int* __restrict__ block_tables,
    int table_width, const int* __restrict__ context_lens, int H, int KVH, int page_shift, float scale_log2,
    int window) {
    constexpr int NDT = D / 16;
    __shared__ float s_m[WAVES][16], s_l[WAVES][16];
    __shared__ float s_o[WAVES][16][16 + 1];                         // one 16-wide d tile at a time
    const int s = blockIdx.x, kvh = blockIdx.y;
    const int G = H / KVH;
    const int ctx = context_lens[s];
    const int p = ctx - 1;
    const int lo = (window > 0 && p - window + 1 > 0) ? p - window + 1 : 0;
    const int wave = threadIdx.x / TM_WAVE, lane = threadIdx.x % TM_WAVE;
    const int r = lane % 16, g = lane / 16;
    const int* table = block_tables + (size_t)s * table_width;

    Bf16x8Bits qreg[D / 32];
    load_q_operand<D>(qreg, q + (size_t)s * q_stride, G, kvh, r, g);

    float m = -INFINITY, l = 0.f;
    f32x4_t o[NDT];
#pragma unroll
    for (int dt = 0; dt < NDT; ++dt) o[dt] = f32x4_t{0.f, 0.f, 0.f, 0.f};
    const int first = (lo / AD_WKEYS) * AD_WKEYS;                   // aligned to 64 positions
    auto fold = [&](float mi, float li, const f32x4_t (&oi)[NDT]) {  // add a partial to the running one
        const float mn = fmaxf(m, mi);
        const float f0 = (m == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f(m - mn);
        const float f1 = (mi == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f(mi - mn);
        l = l * f0 + li * f1;
#pragma unroll
        for (int dt = 0; dt < NDT; ++dt)
#pragma unroll
            for (int i = 0; i < 4; ++i) o[dt][i] = o[dt][i] * f0 + oi[dt][i] * f1;
        m = mn;
    };
    for (int wbase = first + wave * AD_WKEYS; wbase < ctx; wbase += WAVES * AD_WKEYS) {
        float mi, li;
        f32x4_t oi[NDT];
        wave_keys64<D>(qreg, k_pool, v_pool, table, table_width, wbase, ctx, lo, kvh, KVH, page_shift, scale_log2, r, g, mi, li, oi);
        fold(mi, li, oi);
    }
    // merge the wavefronts in wavefront order; lane: head r, d = 16 dt + 4 g + i
    if (g == 0) {
        s_m[wave][r] = m;
        s_l[wave][r] = l;
    }
    __syncthreads();
    float mm = -INFINITY;
#pragma unroll
    for (int w = 0; w < WAVES; ++w) mm = fmaxf(mm, s_m[w][r]);
    float ll = 0.f;
#pragma unroll
    for (int w = 0; w < WAVES; ++w)
        ll += s_l[w][r] * ((s_m[w][r] == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f(s_m[w][r] - mm));
    const float inv = 1.f / ll;
#pragma unroll
    for (int dt = 0; dt < NDT; ++dt) {
#pragma unroll
        for (int i = 0; i < 4; ++i) s_o[wave][r][4 * g + i] = o[dt][i];
        __syncthreads();
        // wavefront dt % WAVES writes this tile: thread -> (head n, 4 consecutive d)
        if (wave == dt % WAVES) {
            const int n = lane / 4, d4 = (lane % 4) * 4;
            if (n < G) {
                float mx = -INFINITY;
#pragma unroll
                for (int w = 0; w < WAVES; ++w) mx = fmaxf(mx, s_m[w][n]);
                float lsum = 0.f, acc[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int w = 0; w < WAVES; ++w) {
                    const float f = (s_m[w][n] == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f(s_m[w][n] - mx);
                    lsum += s_l[w][n] * f;
#pragma unroll
                    for (int i = 0; i < 4; ++i) acc[i] += s_o[w][n][d4 + i] * f;
                }
                const float iv = 1.f / lsum;
                uint2 pk;
                pk.x = pack_bf16(acc[0] * iv, acc[1] * iv);
                pk.y = pack_bf16(acc[2] * iv, acc[3] * iv);
                *(uint2*)(out + (size_t)s * out_stride + (size_t)(kvh * G + n) * D + 16 * dt + d4) = pk;
            }
        }
        __syncthreads();
    }
    (void)inv;
}

// ------------------------------------------------------------------------------------------------
// split kernels: grid (S, KVH, chunks) with four wavefronts, then the merge
// ------------------------------------------------------------------------------------------------
template <int D>
__global__ __launch_bounds__(256) void attn_decode_split_kernel(
    const bf16_t* __restrict__ q, int q_stride, const bf16_t* __restrict__ k_pool,
    const bf16_t* __restrict__ v_pool, const int* __restrict__ block_tables, int table_width,
    const int* __restrict__ context_lens, float* __restrict__ part_o, float* __restrict__ part_ml,
    int max_chunks, int H, int KVH, int page_shift, float scale_log2, int window) {
    constexpr int NDT = D / 16;
    __shared__ float s_m[4][16], s_l[4][16];
    __shared__ float s_o[4][16][D + 1];
    const int s = blockIdx.x, kvh = blockIdx.y, chunk = blockIdx.z;
    const int G = H / KVH;
    const int wave = threadIdx.x / TM_WAVE, lane = threadIdx.x % TM_WAVE;
    const int r = lane % 16, g = lane / 16;
    const int chunk_lo = chunk * AD_CHUNK, wbase = chunk_lo + wave * AD_WKEYS;
    // the context length, the block-table entries and the query are asked for together: one trip to
    // memory before the keys, not two
    const int ctx = context_lens[s];
    int entry[4];
    load_table_entries(entry, block_tables + (size_t)s * table_width, table_width, wbase, page_shift);
    Bf16x8Bits qreg[D / 32];
    load_q_operand<D>(qreg, q + (size_t)s * q_stride, G, kvh, r, g);
    const int p = ctx - 1;
    const int lo = (window > 0 && p - window + 1 > 0) ? p - window + 1 : 0;
    if (chunk_lo >= ctx || chunk_lo + AD_CHUNK <= lo) return;       // nothing of this chunk is visible
    float m, l;
    f32x4_t o[NDT];
    {
        Keys64<D> kv;
        load_keys64<D>(kv, k_pool, v_pool, entry, wbase, ctx, lo, kvh, KVH, page_shift, r, g);
        attend_keys64<D>(kv, qreg, wbase, ctx, lo, scale_log2, g, m, l, o);
    }
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
}

// out[s, h, :] = the partial values of the visible chunks, weighted and normalised. Four wavefronts
// share a (request, head): wavefront w adds the chunks w, w + 4, ... in ascending order and the four
// sums are added in wavefront order, so the order of additions depends on the context length and
// the window only. A lane holds elements d = lane and lane + 64 of the head.
// For up to 64 chunks: lane c of every wavefront holds (max, sum) of chunk c, and those and the
// values of the first 16 chunks are asked for together with the context length, before it is known
// which of them count (scratch memory beyond the context holds anything: it is dropped by selects,
// never multiplied): one trip to memory for contexts up to 4,096.
#define AD_MERGE_WAVES 4
__global__ __launch_bounds__(64 * AD_MERGE_WAVES) void attn_decode_merge_kernel(
    const float* __restrict__ part_o, const float* __restrict__ part_ml, const int* __restrict__ context_lens,
    bf16_t* __restrict__ out, int out_stride, int max_chunks, int H, int D, int window) {
    __shared__ float s_l[AD_MERGE_WAVES], s_o[AD_MERGE_WAVES][128];
    const int s = blockIdx.x, h = blockIdx.y;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / TM_WAVE), lane = threadIdx.x % TM_WAVE;
    const size_t base = ((size_t)s * H + h) * max_chunks;
    const int last = max_chunks - 1;
    const int ctx = context_lens[s];
    const f32x2_t ml = *(const f32x2_t*)(part_ml + (base + (lane < last ? lane : last)) * 2);
    const int d0 = lane < D ? lane : D - 1, d1 = lane + 64 < D ? lane + 64 : D - 1;
    float a0[4], a1[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int c = wave + AD_MERGE_WAVES * i;
        const float* src = part_o + (base + (c < last ? c : last)) * D;
        a0[i] = src[d0];
        a1[i] = src[d1];
    }
    const int p = ctx - 1;
    const int lo = (window > 0 && p - window + 1 > 0) ? p - window + 1 : 0;
    const int c0 = lo / AD_CHUNK, c1 = (ctx - 1) / AD_CHUNK;
    const float mm = wave_max((lane >= c0 && lane <= c1) ? ml[0] : -INFINITY);
    float ll = 0.f, o0 = 0.f, o1 = 0.f;
    auto add_chunk = [&](int c, float v0, float v1) {               // c is the same in every lane
        const float mc = __shfl(ml[0], c, TM_WAVE), lc = __shfl(ml[1], c, TM_WAVE);
        const bool in = c >= c0 && c <= c1 && mc != -INFINITY;
        const float f = in ? __builtin_amdgcn_exp2f(mc - mm) : 0.f;
        ll = fmaf(in ? lc : 0.f, f, ll);
        o0 = fmaf(in ? v0 : 0.f, f, o0);
        o1 = fmaf(in ? v1 : 0.f, f, o1);
    };
#pragma unroll
    for (int i = 0; i < 4; ++i) add_chunk(wave + AD_MERGE_WAVES * i, a0[i], a1[i]);
    // chunks from 16 on (contexts beyond 4,096), four to a wavefront at a time
    for (int cb = 4 * AD_MERGE_WAVES; cb <= c1; cb += 4 * AD_MERGE_WAVES) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int c = cb + wave + AD_MERGE_WAVES * i;
            const float* src = part_o + (base + (c < last ? c : last)) * D;
            a0[i] = src[d0];
            a1[i] = src[d1];
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) add_chunk(cb + wave + AD_MERGE_WAVES * i, a0[i], a1[i]);
    }
    if (lane == 0) s_l[wave] = ll;
    s_o[wave][lane] = o0;
    s_o[wave][lane + 64] = o1;
    __syncthreads();
    if (wave != 0) return;
    ll = s_l[0];
    o0 = s_o[0][lane];
    o1 = s_o[0][lane + 64];
#pragma unroll
    for (int w = 1; w < AD_MERGE_WAVES; ++w) {
        ll += s_l[w];
        o0 += s_o[w][lane];
        o1 += s_o[w][lane + 64];
    }
    bf16_t* orow = out + (size_t)s * out_stride + (size_t)h * D;
    if (lane < D) orow[lane] = f32_to_bf16(o0 / ll);
    if (lane + 64 < D) orow[lane + 64] = f32_to_bf16(o1 / ll);
}

// The same for any number of chunks (contexts beyond 64 chunks): the maxima are found in a pass of
// their own, and wavefront w adds the chunks c0 + w, c0 + w + 4, ...
__global__ __launch_bounds__(64 * AD_MERGE_WAVES) void attn_decode_merge_long_kernel(
    const float* __restrict__ part_o, const float* __restrict__ part_ml, const int* __restrict__ context_lens,
    bf16_t* __restrict__ out, int out_stride, int max_chunks, int H, int D, int window) {
    __shared__ float s_m[AD_MERGE_WAVES], s_l[AD_MERGE_WAVES], s_o[AD_MERGE_WAVES][128];
    const int s = blockIdx.x, h = blockIdx.y;
    const int wave = threadIdx.x / TM_WAVE, lane = threadIdx.x % TM_WAVE;
    const int ctx = context_lens[s];
    const int p = ctx - 1;
    const int lo = (window > 0 && p - window + 1 > 0) ? p - window + 1 : 0;
    const int c0 = lo / AD_CHUNK, c1 = (ctx - 1) / AD_CHUNK;
    const size_t base = ((size_t)s * H + h) * max_chunks;
    float mm = -INFINITY;
    for (int c = c0 + (int)threadIdx.x; c <= c1; c += 64 * AD_MERGE_WAVES) mm = fmaxf(mm, part_ml[(base + c) * 2]);
    mm = wave_max(mm);
    if (lane == 0) s_m[wave] = mm;
    __syncthreads();
    mm = s_m[0];
#pragma unroll
    for (int w = 1; w < AD_MERGE_WAVES; ++w) mm = fmaxf(mm, s_m[w]);
    const bool two = lane + 64 < D;
    float ll = 0.f, o0 = 0.f, o1 = 0.f;
#pragma unroll 4
    for (int c = c0 + wave; c <= c1; c += AD_MERGE_WAVES) {
        const float mc = part_ml[(base + c) * 2];
        const float lc = part_ml[(base + c) * 2 + 1];
        const float a0 = lane < D ? part_o[(base + c) * D + lane] : 0.f;
        const float a1 = two ? part_o[(base + c) * D + lane + 64] : 0.f;
        const float f = (mc == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f(mc - mm);
        ll = fmaf(lc, f, ll);
        o0 = fmaf(a0, f, o0);
        o1 = fmaf(a1, f, o1);
    }
    if (lane == 0) s_l[wave] = ll;
    s_o[wave][lane] = o0;
    s_o[wave][lane + 64] = o1;
    __syncthreads();
    if (wave != 0) return;
    ll = s_l[0];
    o0 = s_o[0][lane];
    o1 = s_o[0][lane + 64];
#pragma unroll
    for (int w = 1; w < AD_MERGE_WAVES; ++w) {
        ll += s_l[w];
        o0 += s_o[w][lane];
        o1 += s_o[w][lane + 64];
    }
    bf16_t* orow = out + (size_t)s * out_stride + (size_t)h * D;
    if (lane < D) orow[lane] = f32_to_bf16(o0 / ll);
    if (two) orow[lane + 64] = f32_to_bf16(o1 / ll);
}

template <int D>
static int launch_decode(const void* q, int q_stride, void* out, int out_stride, const void* k_pool,
                         const void* v_pool, const int* block_tables, int table_width, const int* context_lens,
                         float* part_o, float* part_ml, int max_chunks, int S, int H, int KVH, int page,
                         float scale, int window, hipStream_t stream) {
    int page_shift = 0;
    while ((1 << page_shift) < page) ++page_shift;
    const float scale_log2 = scale * 1.4426950408889634f;
    constexpr int WAVES = D <= 32 ? 16 : 8;       // 16 wavefronts leave 128 registers each: enough for D = 32 only
    // few (request, kv head) pairs: more blocks than pairs are needed to pull the cache at speed; the caller
    // asks for that by bringing the scratch memory
    const bool split = part_o && part_ml && max_chunks > 1;
    if (!split) {
        attn_decode_block_kernel<D, WAVES><<<dim3(S, KVH), 64 * WAVES, 0, stream>>>(
            (const bf16_t*)q, q_stride, (bf16_t*)out, out_stride, (const bf16_t*)k_pool, (const bf16_t*)v_pool,
            block_tables, table_width, context_lens, H, KVH, page_shift, scale_log2, window);
        TM_CHECK_LAUNCH();
        return TM_OK;
    }
    attn_decode_split_kernel<D><<<dim3(S, KVH, max_chunks), 256, 0, stream>>>(
        (const bf16_t*)q, q_stride, (const bf16_t*)k_pool, (const bf16_t*)v_pool, block_tables, table_width,
        context_lens, part_o, part_ml, max_chunks, H, KVH, page_shift, scale_log2, window);
    TM_CHECK_LAUNCH();
    if (max_chunks <= TM_WAVE)
        attn_decode_merge_kernel<<<dim3(S, H), 64 * AD_MERGE_WAVES, 0, stream>>>(
            part_o, part_ml, context_lens, (bf16_t*)out, out_stride, max_chunks, H, D, window);
    else
        attn_decode_merge_long_kernel<<<dim3(S, H), 64 * AD_MERGE_WAVES, 0, stream>>>(
            part_o, part_ml, context_lens, (bf16_t*)out, out_stride, max_chunks, H, D, window);
    TM_CHECK_LAUNCH();
    return TM_OK;
}

// q: first decode row (one row per request, rows q_stride apart); out likewise; block_tables and
// context_lens: first decode request. part_o: float [S, H, max_chunks, D] and part_ml: [S, H, max_chunks, 2]
// are scratch for the split kernels, which run when both are given (the caller gives them when the
// (request, kv head) pairs alone are too few blocks for the chip); without them the block kernel runs.
extern "C" int tm_attn_decode_mfma(const void* q, int q_stride, void* out, int out_stride, const void* k_pool,
                                   const void* v_pool, const int* block_tables, int table_width,
                                   const int* context_lens, float* part_o, float* part_ml, int max_chunks, int S,
                                   int H, int KVH, int D, int page, float scale, int window, hipStream_t stream) {
    if (S <= 0) return TM_OK;
    if (H <= 0 || KVH <= 0 || H % KVH || H / KVH > 16 || page < 16 || (page & (page - 1)) || max_chunks <= 0 ||
        !(scale > 0.f) || max_chunks > 65535 || KVH > 65535 || window < 0 || table_width <= 0 || (q_stride % 8) ||
        ((uintptr_t)q % 16) || (out_stride % 4) || ((uintptr_t)out % 8) || q_stride < H * D || out_stride < H * D)
        return TM_ERR_ARG;
#define TM_DECODE_CASE(DD)                                                                                        \
    case DD:                                                                                                      \
        return launch_decode<DD>(q, q_stride, out, out_stride, k_pool, v_pool, block_tables, table_width,         \
                                 context_lens, part_o, part_ml, max_chunks, S, H, KVH, page, scale, window, stream)
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
