// Paged attention for portions of prompts on MFMA (bfloat16), the keys and values shared through LDS.
//
//   A block takes 16 consecutive query tokens of one request (a "tile") and one kv head; its wavefronts
//   take the query heads that share that kv head, two each. The keys and values of the tile's request are
//   staged through LDS 64 positions at a time, once for all of the block's heads, so a byte that comes
//   from the second-level cache feeds 16 tokens x G heads; in attention_prefill.hip, where every
//   wavefront loads its own key blocks straight into registers, it feeds 16 tokens x 2..4 heads, and both
//   head sizes stand at the same 9-10 TB/s out of that cache whatever else is changed.
//
//   Every wavefront visits all key blocks of its tokens in ascending order, in stages aligned to absolute
//   positions (multiples of 64), so a token's result does not depend on how its prompt was cut into
//   portions nor on the rest of the batch. (It differs by rounding from the other kernel's, whose
//   wavefronts split the key blocks among them: which kernel runs depends on the model's shape only.)
//
//   S^T = K Q^T      A = keys  [16 keys x 32 d]   from LDS, rows in tile order (see stage_row)
//                    B = Q^T   [32 d x 16 tokens] in registers
//   O^T = V^T P^T    A = V^T   [16 d x 32 keys]   from LDS
//                    B = P^T   [32 keys x 16 tokens] straight from the S^T accumulators
//   (reference src/infer/kv/context.py:70-75, src/infer/model/layers.py:100-107 for what a query sees)
#include "common.h"
#include "api.h"
#include "attention_prefill_common.h"

#define PS_KEYS 64          // positions per stage
#ifndef TM_SHARED_HPW64
#define TM_SHARED_HPW64 2
#define TM_SHARED_OCC64 3
#endif

// Where the stage's key at offset kk (0..63) lies in LDS. A lane of the second product needs the weights
// of 8 consecutive keys, and gets from the first product's accumulators rows 4g..4g+3 of two 16-key tiles:
// so the tiles of a pair (2a, 2a + 1) split their 32 keys in runs of four, and the rows are stored in tile
// order, where the operand loads of a tile are 16 consecutive rows.
__device__ __forceinline__ int stage_row(int kk) {
    const int a = kk >> 5, b = (kk >> 3) & 3, h = (kk >> 2) & 1, i = kk & 3;
    return 16 * (2 * a + h) + 4 * b + i;
}

template <int D>
struct SharedShape {
    // Rows padded by 32 bytes. An operand load has lane (r, g) read 16 bytes at row r, piece g; measured with the
    // bank-conflict counter, such loads are free of conflicts when the row stride is 32 bytes more than a multiple of
    // 64 (288, 160, 224, 96 bytes here) and take twice as long with a stride 16 bytes more than a multiple of 32 (272,
    // 144), the usual padding. The stores (whole key rows; value rows two lanes a row) are free of conflicts with these
    // strides too.
    static constexpr int K_STRIDE = D * 2 + 32, V_STRIDE = PS_KEYS * 2 + 32;
    static constexpr int K_BYTES = PS_KEYS * K_STRIDE, V_BYTES = D * V_STRIDE, STAGE = K_BYTES + V_BYTES;
    static constexpr int PIECES = PS_KEYS * D / 8;               // 16-byte pieces of a stage's keys; as many of its values
};

// Where the 16-key tiles of the next 16 stages lie in the pools: lane l holds tile 4 * base_stage + l
// (byte offsets of the tile's first key row of this kv head, and of its first value row). A tile that holds
// no key any query of the block may see is replaced by the nearest tile that does: its table entry may
// name no page; every score of such a tile is masked by the key's real position and its values are cleared.
struct TilePlaces {
    uint64_t k, v;
};

__device__ __forceinline__ TilePlaces lane_places(int base_stage, int lane, int first_tile, int last_tile,
                                                  const int* __restrict__ table, int page_shift, int kvh, int KVH, int D) {
    int tile = 4 * base_stage + lane;
    tile = tile < first_tile ? first_tile : (tile > last_tile ? last_tile : tile);
    const int tile0 = 16 * tile;
    const size_t pg = (size_t)table[tile0 >> page_shift];
    const int in_page = tile0 & ((1 << page_shift) - 1);
    TilePlaces p;
    p.k = ((((pg << page_shift) + in_page) * KVH + kvh) * D) * sizeof(bf16_t);
    p.v = ((((pg * KVH + kvh) * D) << page_shift) + in_page) * sizeof(bf16_t);
    return p;
}

__device__ __forceinline__ uint64_t lane_value(uint64_t v, int src_lane) {
    const uint32_t lo = __shfl((uint32_t)v, src_lane, TM_WAVE), hi = __shfl((uint32_t)(v >> 32), src_lane, TM_WAVE);
    return ((uint64_t)hi << 32) | lo;
}

template <int D, int THREADS>
struct StageCopy {
    static constexpr int PIECES = SharedShape<D>::PIECES, ITERS = (PIECES + THREADS - 1) / THREADS;
    static constexpr bool EXACT = PIECES % THREADS == 0;
    u32x4_t k[ITERS], v[ITERS];

    // Ask for the keys and values of stage `rel` of the stages `places` covers; nothing is waited for.
    __device__ __forceinline__ void load(const TilePlaces& places, int rel, const unsigned char* __restrict__ k_pool,
                                         const unsigned char* __restrict__ v_pool, int KVH, int page_shift, int tid) {
#pragma unroll
        for (int i = 0; i < ITERS; ++i) {
            int idx = tid + i * THREADS;
            if (!EXACT) idx = idx < PIECES ? idx : PIECES - 1;
            {   // keys: piece pc of the key at offset kk
                const int kk = idx / (D / 8), pc = idx % (D / 8);
                const uint64_t at = lane_value(places.k, 4 * rel + (kk >> 4));
                k[i] = *(const u32x4_t*)(k_pool + at + ((size_t)(kk & 15) * KVH * D + pc * 8) * sizeof(bf16_t));
            }
            {   // values: half `half` of the 16 keys of tile j in row d (two lanes a row: with rows 160 bytes apart the 16
                // pieces of 8 rows go to 16 different places of LDS's banks)
                const int j = idx / (2 * D), d = (idx % (2 * D)) / 2, half = idx & 1;
                const uint64_t at = lane_value(places.v, 4 * rel + j);
                v[i] = *(const u32x4_t*)(v_pool + at + (((size_t)d << page_shift) + half * 8) * sizeof(bf16_t));
            }
        }
    }

    // Store what was loaded into a stage of LDS. `keys` of the stage's 64 positions exist: the values of the
    // others (beyond the newest key; they can hold anything) are cleared here, once for all wavefronts, so that
    // the products need no mask (their weights are zero, but zero times anything is not).
    __device__ __forceinline__ void store(unsigned char* stage, int tid, int keys) const {
#pragma unroll
        for (int i = 0; i < ITERS; ++i) {
            const int idx = tid + i * THREADS;
            if (!EXACT && idx >= PIECES) continue;
            const int kk = idx / (D / 8), pc = idx % (D / 8);
            *(u32x4_t*)(stage + stage_row(kk) * SharedShape<D>::K_STRIDE + pc * 16) = k[i];
            const int j = idx / (2 * D), d = (idx % (2 * D)) / 2, half = idx & 1;
            u32x4_t val = v[i];
            if (keys < PS_KEYS) {                                    // block-uniform: a tile's last stage only
                const int first = 16 * j + 8 * half;
#pragma unroll
                for (int w = 0; w < 4; ++w)
                    val[w] &= ((first + 2 * w < keys) ? 0x0000ffffu : 0u) | ((first + 2 * w + 1 < keys) ? 0xffff0000u : 0u);
            }
            *(u32x4_t*)(stage + SharedShape<D>::K_BYTES + d * SharedShape<D>::V_STRIDE + j * 32 + half * 16) = val;
        }
    }
};

// 32 keys [key0, key0 + 32) of the stage in LDS against the wavefront's heads.
template <int D, int HPW>
__device__ __forceinline__ void attend_shared(const unsigned char* stage, int sub, HeadState<D, HPW>& st,
                                              const PFrag (&qf)[HPW][D / 32], int key0, const TileView& tv,
                                              int r, int g, float scale_log2) {
    constexpr int NDC = D / 32, NDT = D / 16;
    constexpr int KS = SharedShape<D>::K_STRIDE, VS = SharedShape<D>::V_STRIDE;
    // does any (query, key) pair of this block fall outside the causal / window limits?
    const bool edge = (key0 + 31 > tv.pos0) || (key0 < tv.last_lo);
    PFrag kf[2][NDC];
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int c = 0; c < NDC; ++c)
            kf[t][c].u = *(const u32x4_t*)(stage + (16 * (2 * sub + t) + r) * KS + 64 * c + 16 * g);
    PFrag pt[HPW];
#pragma unroll
    for (int hh = 0; hh < HPW; ++hh) {
        f32x4_t sc[2];
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            f32x4_t acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int c = 0; c < NDC; ++c)
                acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf[t][c].b, qf[hh][c].b, acc, 0, 0, 0);
            sc[t] = acc;
        }
        if (edge) {
#pragma unroll
            for (int t = 0; t < 2; ++t)
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const int kj = key0 + 8 * g + 4 * t + i;        // row 4g+i of tile t of the pair
                    if (kj > tv.my_pos || kj < tv.my_lo) sc[t][i] = -INFINITY;
                }
        }
        // this lane's largest score of the block (scale > 0: the maximum commutes with it)
        float lm = max3(-INFINITY, sc[0][0], sc[0][1]);
        lm = max3(lm, sc[0][2], sc[0][3]);
        lm = max3(lm, sc[1][0], sc[1][1]);
        lm = max3(lm, sc[1][2], sc[1][3]);
        // The running reference m of a column moves only when the block's maximum exceeds it by more than
        // PF_SLACK (in units of log2): until then the weights are exp2(s - m) <= 2^PF_SLACK instead of <= 1,
        // which changes nothing but their common scale. Each column decides for itself, so a query's result
        // does not depend on the other queries of its tile; whether any column moves is asked of the lanes'
        // own maxima first (a column's maximum exceeds the limit exactly when one of its four lanes' does).
        if (__any(lm * scale_log2 > st.m[hh] + PF_SLACK)) {          // (true for a column that has seen no key: m = -inf)
            const float bm = column_max(lm) * scale_log2;
            const bool grow = bm > st.m[hh] + PF_SLACK;
            const float m_new = grow ? bm : st.m[hh];
            const float corr = (m_new == -INFINITY) ? 1.f : __builtin_amdgcn_exp2f(st.m[hh] - m_new);
            st.m[hh] = m_new;
            st.l[hh] *= corr;
#pragma unroll
            for (int dt = 0; dt < NDT; ++dt)
#pragma unroll
                for (int i = 0; i < 4; ++i) st.o[hh][dt][i] *= corr;
        }
        // a column that has seen no key yet (m = -inf) gets zeros: exp2(-inf - 0)
        const float neg_m = (st.m[hh] == -INFINITY) ? 0.f : -st.m[hh];
        float pr[2][4];
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                pr[t][i] = __builtin_amdgcn_exp2f(fmaf(sc[t][i], scale_log2, neg_m));
                st.l[hh] += pr[t][i];
            }
        // keys 8g .. 8g+7 of the block, in order
        pt[hh].u = u32x4_t{pk_bf16(pr[0][0], pr[0][1]), pk_bf16(pr[0][2], pr[0][3]), pk_bf16(pr[1][0], pr[1][1]),
                           pk_bf16(pr[1][2], pr[1][3])};
    }
#pragma unroll
    for (int dt = 0; dt < NDT; ++dt) {
        PFrag vf;
        vf.u = *(const u32x4_t*)(stage + SharedShape<D>::K_BYTES + (16 * dt + r) * VS + 64 * sub + 16 * g);
#pragma unroll
        for (int hh = 0; hh < HPW; ++hh) {
            st.o[hh][dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf.b, pt[hh].b, st.o[hh][dt], 0, 0, 0);
        }
    }
}

// tiles: int32 [n_tiles][4] = (request index in the step, first row of the tile in the flat batch,
//                              tokens in the tile (1..16), position of its first token)
// With pair != 0 a block takes tile b and then tile n_tiles - 1 - b: in a table sorted by the number of
// keys a tile sees, the longest goes with the shortest and every block has the same work.
// query heads a wavefront takes, and wavefronts a SIMD the registers are limited for, by head size
template <int D> struct SharedPlan { static constexpr int HPW = D <= 64 ? TM_SHARED_HPW64 : 2, WAVES_PER_SIMD = D <= 64 ? TM_SHARED_OCC64 : 2; };

template <int D, int WAVES>
__global__ __launch_bounds__(64 * WAVES, SharedPlan<D>::WAVES_PER_SIMD) void attn_prefill_shared_kernel(
    const bf16_t* __restrict__ q, int q_stride, bf16_t* __restrict__ out, int out_stride,
    const bf16_t* __restrict__ k_pool, const bf16_t* __restrict__ v_pool, const int* __restrict__ block_tables,
    int table_width, const int* __restrict__ tiles, int n_tiles, int pair, int H, int KVH, int page_shift,
    float scale_log2, int window) {
    constexpr int NDC = D / 32, NDT = D / 16, THREADS = 64 * WAVES, STAGE = SharedShape<D>::STAGE, HPW = SharedPlan<D>::HPW;
    extern __shared__ __align__(16) unsigned char stages[];          // two stages
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / TM_WAVE);
    const int tid = threadIdx.x, lane = tid % TM_WAVE, r = lane % 16, g = lane / 16;
    const int G = H / KVH, kvh = blockIdx.y;
    const int h0 = kvh * G + wave * HPW;
    const int nh = G - wave * HPW < 0 ? 0 : (G - wave * HPW < HPW ? G - wave * HPW : HPW);
    const int other = n_tiles - 1 - (int)blockIdx.x;
    const int n_mine = (pair && other > (int)blockIdx.x) ? 2 : 1;
    const unsigned char* kp = (const unsigned char*)k_pool;
    const unsigned char* vp = (const unsigned char*)v_pool;

#pragma unroll 1
    for (int which = 0; which < n_mine; ++which) {
        const int* tl = tiles + (size_t)(which ? other : (int)blockIdx.x) * 4;
        const int s = tl[0], row0 = tl[1], valid = tl[2], pos0 = tl[3];
        const int* table = block_tables + (size_t)s * table_width;
        TileView tv;
        tv.pos0 = pos0;
        tv.last_key = pos0 + valid - 1;
        tv.my_pos = pos0 + r < tv.last_key ? pos0 + r : tv.last_key;
        tv.my_lo = (window > 0 && tv.my_pos - window + 1 > 0) ? tv.my_pos - window + 1 : 0;
        tv.last_lo = (window > 0 && tv.last_key - window + 1 > 0) ? tv.last_key - window + 1 : 0;
        const int first_key = (window > 0 && pos0 - window + 1 > 0) ? pos0 - window + 1 : 0;
        const int sb0 = first_key / PS_KEYS, sb1 = tv.last_key / PS_KEYS;
        const int first_tile = first_key / 16, last_tile = tv.last_key / 16;

        PFrag qf[HPW][NDC];
#pragma unroll
        for (int hh = 0; hh < HPW; ++hh)
#pragma unroll
            for (int c = 0; c < NDC; ++c) {
                if (hh < nh && r < valid)
                    qf[hh][c].u = *(const u32x4_t*)(q + (size_t)(row0 + r) * q_stride + (size_t)(h0 + hh) * D + 32 * c + 8 * g);
                else
                    qf[hh][c].u = u32x4_t{0, 0, 0, 0};
            }
        HeadState<D, HPW> st;
#pragma unroll
        for (int hh = 0; hh < HPW; ++hh) {
            st.m[hh] = -INFINITY;
            st.l[hh] = 0.f;
#pragma unroll
            for (int dt = 0; dt < NDT; ++dt) st.o[hh][dt] = f32x4_t{0.f, 0.f, 0.f, 0.f};
        }

        // The stages take turns in the two halves of LDS: while one is worked on, the next one's keys and values
        // are on their way into registers, and are stored when the work is done. The load after the last stage
        // repeats it, unused, so that no load hides behind a branch.
        int base = sb0;                                              // `places` covers stages base .. base + 15
        TilePlaces places = lane_places(base, lane, first_tile, last_tile, table, page_shift, kvh, KVH, D);
        StageCopy<D, THREADS> copy;
        copy.load(places, 0, kp, vp, KVH, page_shift, tid);
        copy.store(stages, tid, tv.last_key + 1 - sb0 * PS_KEYS);
        __syncthreads();
        for (int sb = sb0; sb <= sb1; ++sb) {
            const int cur = (sb - sb0) & 1;
            int next = sb + 1 <= sb1 ? sb + 1 : sb1;
            if (next - base == 16) {
                base = next;
                places = lane_places(base, lane, first_tile, last_tile, table, page_shift, kvh, KVH, D);
            }
            copy.load(places, next - base, kp, vp, KVH, page_shift, tid);
            if (nh > 0) {                                            // wave-uniform
#pragma unroll
                for (int sub = 0; sub < 2; ++sub) {
                    const int key0 = sb * PS_KEYS + 32 * sub;
                    if (key0 > tv.last_key || key0 + 31 < first_key) continue;     // block-uniform: nothing of it is visible
                    attend_shared<D, HPW>(stages + cur * STAGE, sub, st, qf, key0, tv, r, g, scale_log2);
                }
            }
            copy.store(stages + (cur ^ 1) * STAGE, tid, tv.last_key + 1 - next * PS_KEYS);
            __syncthreads();
        }

        // every wavefront has its heads' whole result; lane: d = 16 dt + 4 g + i of token r
#pragma unroll
        for (int hh = 0; hh < HPW; ++hh) {
            if (hh >= nh) continue;                                  // wave-uniform
            float lsum = st.l[hh];
            lsum += __shfl_xor(lsum, 16, TM_WAVE);
            lsum += __shfl_xor(lsum, 32, TM_WAVE);
            if (r >= valid) continue;
            const float inv = 1.f / lsum;
            bf16_t* orow = out + (size_t)(row0 + r) * out_stride + (size_t)(h0 + hh) * D + 4 * g;
#pragma unroll
            for (int dt = 0; dt < NDT; ++dt) {
                uint2 pk;
                pk.x = pk_bf16(st.o[hh][dt][0] * inv, st.o[hh][dt][1] * inv);
                pk.y = pk_bf16(st.o[hh][dt][2] * inv, st.o[hh][dt][3] * inv);
                *(uint2*)(orow + 16 * dt) = pk;
            }
        }
    }
}

template <int D, int WAVES>
static int launch_shared(const void* q, int q_stride, void* out, int out_stride, const void* k_pool, const void* v_pool,
                         const int* block_tables, int table_width, const int* tiles, int n_tiles, int H, int KVH,
                         int page_shift, float scale_log2, int window, hipStream_t stream) {
    constexpr int lds = 2 * SharedShape<D>::STAGE;
    static bool raised = false;
    if (lds > 48 * 1024 && !raised) {
        if (hipFuncSetAttribute((const void*)attn_prefill_shared_kernel<D, WAVES>, hipFuncAttributeMaxDynamicSharedMemorySize,
                                lds) != hipSuccess)
            return TM_ERR_LAUNCH;
        raised = true;
    }
    // fold the table in two once the folded launch still gives every CU a block
    const int pair = (long long)(n_tiles / 2) * KVH >= 256 ? 1 : 0;
    dim3 grid(pair ? (n_tiles + 1) / 2 : n_tiles, KVH);
    attn_prefill_shared_kernel<D, WAVES><<<grid, 64 * WAVES, lds, stream>>>(
        (const bf16_t*)q, q_stride, (bf16_t*)out, out_stride, (const bf16_t*)k_pool, (const bf16_t*)v_pool, block_tables,
        table_width, tiles, n_tiles, pair, H, KVH, page_shift, scale_log2, window);
    TM_CHECK_LAUNCH();
    return TM_OK;
}

// Does this kernel take the shape? Groups of up to 16 query heads a kv head; out rows 8-byte aligned.
extern "C" int tm_attn_prefill_shared_takes(int H, int KVH, int D) {
    if (H <= 0 || KVH <= 0 || H % KVH) return 0;
    const int G = H / KVH;
    if (!(D == 32 || D == 64 || D == 96 || D == 128) || KVH > 65535) return 0;
    return G <= 8 * (D <= 64 ? SharedPlan<64>::HPW : SharedPlan<128>::HPW);
}

extern "C" int tm_attn_prefill_shared(const void* q, int q_stride, void* out, int out_stride, const void* k_pool,
                                      const void* v_pool, const int* block_tables, int table_width, const int* tiles,
                                      int n_tiles, int H, int KVH, int D, int page, float scale, int window,
                                      hipStream_t stream) {
    if (n_tiles <= 0) return TM_OK;
    if (!tm_attn_prefill_shared_takes(H, KVH, D) || page < 16 || (page & (page - 1)) || window < 0 || table_width <= 0 ||
        (q_stride % 8) || ((uintptr_t)q % 16) || (out_stride % 4) || ((uintptr_t)out % 8) || q_stride < H * D ||
        out_stride < H * D || !(scale > 0.f))
        return TM_ERR_ARG;
    const int hpw = D <= 64 ? SharedPlan<64>::HPW : SharedPlan<128>::HPW;
    const int G = H / KVH, need = (G + hpw - 1) / hpw;
    int page_shift = 0;
    while ((1 << page_shift) < page) ++page_shift;
    const float scale_log2 = scale * 1.4426950408889634f;
#define TM_SHARED_ARGS q, q_stride, out, out_stride, k_pool, v_pool, block_tables, table_width, tiles, n_tiles, H, KVH, \
                       page_shift, scale_log2, window, stream
#define TM_SHARED_CASE(DD)                                                          \
    case DD:                                                                        \
        if (need <= 2) return launch_shared<DD, 2>(TM_SHARED_ARGS);                 \
        /* three wavefronts of work get a fourth, idle one: with two blocks a CU every working wavefront then */ \
        /* shares its SIMD with another, which is worth more than the SIMD the idle ones hold */                  \
        if (need <= 4) return launch_shared<DD, 4>(TM_SHARED_ARGS);                 \
        return launch_shared<DD, 8>(TM_SHARED_ARGS);
    switch (D) {
        TM_SHARED_CASE(32)
        TM_SHARED_CASE(64)
        TM_SHARED_CASE(96)
        TM_SHARED_CASE(128)
        default:
            return TM_ERR_ARG;
    }
#undef TM_SHARED_CASE
#undef TM_SHARED_ARGS
}
