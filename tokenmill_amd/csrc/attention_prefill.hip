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
#include "attention_prefill_common.h"
#include "choose.h"

template <int D>
struct KVBlock {
    PFrag k[2][D / 32];     // [16-key tile][d chunk]
    u32x2_t v[D / 16][2];   // [d tile][16-key tile]: 4 keys each
};

// What a lane adds to a tile's (wave-uniform) base address: constant for the whole kernel.
struct LaneOffsets {
    uint32_t k;             // bytes: key r of the tile, d = 8 g
    uint32_t v;             // bytes: d = r, keys 4 g .. 4 g + 3 of the tile
};

// A raw buffer descriptor over memory that starts at a wave-uniform address: loads through it take
// the base from scalar registers and a 32-bit offset per lane, so no lane computes a 64-bit address.
__device__ __forceinline__ __amdgpu_buffer_rsrc_t uniform_buffer(const void* base) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, 0x7fffffff, 0x00020000);
}

// The pages of the next 32 key blocks of a wavefront (blocks kb, kb + KS, ...), one 16-key tile per
// lane: lane 2 i + t holds the page of tile t of block kb + i * KS. A tile that holds no key any
// query of this wavefront may see (beyond the newest key, or wholly behind the window) is replaced
// by the nearest tile that does: its table entry may name no page. The caller masks every score of
// such a tile by the key's real position, so what is loaded in its place only has to be finite.
template <int KS>
__device__ __forceinline__ int2 lane_pages(int kb, int lane, int first_tile, int last_tile,
                                           const int* __restrict__ table, int page_shift) {
    int tile = 2 * (kb + (lane >> 1) * KS) + (lane & 1);
    tile = tile < first_tile ? first_tile : (tile > last_tile ? last_tile : tile);
    const int tile0 = 16 * tile;
    return int2{table[tile0 >> page_shift], tile0 & ((1 << page_shift) - 1)};
}

// Loads one block of 32 keys (two tiles of 16); slot = which of the 32 blocks held in `pages`.
template <int D>
__device__ __forceinline__ void load_kv_block(KVBlock<D>& blk, int2 pages, int slot,
                                              const bf16_t* __restrict__ k_pool, const bf16_t* __restrict__ v_pool,
                                              int kvh, int KVH, int page_shift, LaneOffsets off) {
#pragma unroll
    for (int t = 0; t < 2; ++t) {
        const int pg = __builtin_amdgcn_readlane(pages.x, 2 * slot + t);                    // wave-uniform
        const int in_page = __builtin_amdgcn_readlane(pages.y, 2 * slot + t);
        const __amdgpu_buffer_rsrc_t kbuf =
            uniform_buffer(k_pool + ((((size_t)pg << page_shift) + in_page) * KVH + kvh) * D);
        const __amdgpu_buffer_rsrc_t vbuf =
            uniform_buffer(v_pool + ((((size_t)pg * KVH + kvh) * D) << page_shift) + in_page);
#pragma unroll
        for (int c = 0; c < D / 32; ++c)
            blk.k[t][c].u = __builtin_amdgcn_raw_buffer_load_b128(kbuf, off.k, 64 * c, 0);
#pragma unroll
        for (int dt = 0; dt < D / 16; ++dt)
            blk.v[dt][t] = __builtin_amdgcn_raw_buffer_load_b64(vbuf, off.v, (32 * dt) << page_shift, 0);
    }
}

// One block of 32 keys against the wavefront's heads.
template <int D, int HPW>
__device__ __forceinline__ void attend_block(KVBlock<D>& blk, HeadState<D, HPW>& st, const PFrag (&qf)[HPW][D / 32],
                                             int key0, int nh, const TileView& tv, int g, float scale_log2) {
    constexpr int NDC = D / 32, NDT = D / 16;
    // values of keys nobody may see (beyond the newest key) can hold anything: clear them
    if (key0 + 31 > tv.last_key) {
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            const int k0 = key0 + 16 * t + 4 * g;
            const uint32_t keep0 = ((k0 <= tv.last_key) ? 0x0000ffffu : 0u) | ((k0 + 1 <= tv.last_key) ? 0xffff0000u : 0u);
            const uint32_t keep1 = ((k0 + 2 <= tv.last_key) ? 0x0000ffffu : 0u) | ((k0 + 3 <= tv.last_key) ? 0xffff0000u : 0u);
#pragma unroll
            for (int dt = 0; dt < NDT; ++dt) {
                blk.v[dt][t][0] &= keep0;
                blk.v[dt][t][1] &= keep1;
            }
        }
    }
    // does any (query, key) pair of this block fall outside the causal / window limits?
    const bool edge = (key0 + 31 > tv.pos0) || (key0 < tv.last_lo);
    // all score products first: the matrix unit works on the next head's while the vector unit
    // does the softmax of this one
    f32x4_t sc[HPW][2];
#pragma unroll
    for (int hh = 0; hh < HPW; ++hh) {
        if (hh >= nh) continue;                                  // wave-uniform
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            f32x4_t acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int c = 0; c < NDC; ++c)
                acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(blk.k[t][c].b, qf[hh][c].b, acc, 0, 0, 0);
            sc[hh][t] = acc;
        }
    }
#pragma unroll
    for (int hh = 0; hh < HPW; ++hh) {
        if (hh >= nh) continue;                                  // wave-uniform
        if (edge) {
#pragma unroll
            for (int t = 0; t < 2; ++t)
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const int kj = key0 + 16 * t + 4 * g + i;
                    if (kj > tv.my_pos || kj < tv.my_lo) sc[hh][t][i] = -INFINITY;
                }
        }
        // this lane's largest score of the block (scale > 0: the maximum commutes with it)
        float lm = max3(-INFINITY, sc[hh][0][0], sc[hh][0][1]);
        lm = max3(lm, sc[hh][0][2], sc[hh][0][3]);
        lm = max3(lm, sc[hh][1][0], sc[hh][1][1]);
        lm = max3(lm, sc[hh][1][2], sc[hh][1][3]);
        // The running reference m of a column moves only when the block's maximum exceeds it by more
        // than PF_SLACK (in units of log2): until then the weights are exp2(s - m) <= 2^PF_SLACK instead of
        // <= 1, which changes nothing but their common scale (it cancels against the sum), and the
        // rescaling of the accumulators, the expensive part of a block on the vector unit, becomes rare.
        // Each column decides for itself and one that stays multiplies by exactly 1, so a query's result
        // does not depend on the other queries of its tile. Whether any column moves is asked of the lanes'
        // own maxima first (a column's maximum exceeds the limit exactly when one of its four lanes' does), so
        // the exchange between the lanes of a column is as rare as the rescaling.
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
                pr[t][i] = __builtin_amdgcn_exp2f(fmaf(sc[hh][t][i], scale_log2, neg_m));
                st.l[hh] += pr[t][i];
            }
        PFrag pt;
        pt.u = u32x4_t{pk_bf16(pr[0][0], pr[0][1]), pk_bf16(pr[0][2], pr[0][3]), pk_bf16(pr[1][0], pr[1][1]),
                       pk_bf16(pr[1][2], pr[1][3])};
#pragma unroll
        for (int dt = 0; dt < NDT; ++dt) {
            PFrag vf;
            vf.u = u32x4_t{blk.v[dt][0][0], blk.v[dt][0][1], blk.v[dt][1][0], blk.v[dt][1][1]};
            st.o[hh][dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf.b, pt.b, st.o[hh][dt], 0, 0, 0);
        }
    }
}

// tiles: int32 [n_tiles][4] = (request index in the step, first row of the tile in the flat batch,
//                              tokens in the tile (1..16), position of its first token)
// A block is KS wavefronts on the same tile and heads; wavefront j takes the key blocks kb with
// kb % KS == j and the partial results are merged through LDS in wavefront order. Which blocks a
// wavefront takes depends on absolute positions only, and a block in which a token sees no key
// changes nothing for it, so a token's bits do not depend on the tile it falls into.
// With pair != 0 a block takes tile b and then tile n_tiles - 1 - b: in a table sorted by the
// number of keys a tile sees, the longest goes with the shortest and every block has the same work
// (the lower triangle of a prompt, folded).
template <int D, int HPW, int KS>
__global__ __launch_bounds__(64 * KS) void attn_prefill_mfma_kernel(
    const bf16_t* __restrict__ q, int q_stride, bf16_t* __restrict__ out, int out_stride,
    const bf16_t* __restrict__ k_pool, const bf16_t* __restrict__ v_pool, const int* __restrict__ block_tables,
    int table_width, const int* __restrict__ tiles, int n_tiles, int pair, int H, int KVH, int page_shift,
    float scale_log2, int window) {
    constexpr int NDC = D / 32, NDT = D / 16;
    __shared__ float s_m[KS][16], s_l[KS][16];
    __shared__ float s_o[KS][16][D + 1];
    // the wavefront index in a scalar register: everything derived from it (its key blocks, their
    // pages, the branches on them) stays wave-uniform
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / TM_WAVE);
    const int lane = threadIdx.x % TM_WAVE, r = lane % 16, g = lane / 16;
    const int G = H / KVH;
    const int splits = (G + HPW - 1) / HPW;
    const int kvh = blockIdx.y / splits, split = blockIdx.y % splits;
    const int h0 = kvh * G + split * HPW;
    const int nh = (G - split * HPW) < HPW ? (G - split * HPW) : HPW;
    LaneOffsets off;
    off.k = (uint32_t)(((size_t)r * KVH * D + 8 * g) * sizeof(bf16_t));
    off.v = (uint32_t)((((size_t)r << page_shift) + 4 * g) * sizeof(bf16_t));
    const int other = n_tiles - 1 - (int)blockIdx.x;
    const int n_mine = (pair && other > (int)blockIdx.x) ? 2 : 1;

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
        const int kb0 = first_key / 32, kb1 = tv.last_key / 32;
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

        // Two register sets take turns: one is worked on while the other's loads are in flight. The
        // load after the last block repeats it, unused, so that no load hides behind a branch.
        int kb = kb0 + ((wave - kb0) & (KS - 1));                    // first block >= kb0 of this wavefront
        KVBlock<D> ba, bb;
        int2 pages = lane_pages<KS>(kb, lane, first_tile, last_tile, table, page_shift);
        int slot = 0;                                                // block kb is slot `slot` of `pages`
        if (kb <= kb1) load_kv_block<D>(ba, pages, 0, k_pool, v_pool, kvh, KVH, page_shift, off);
        while (kb <= kb1) {
            if (slot == 31) {                                        // the next block starts a new set of pages
                pages = lane_pages<KS>(kb + KS, lane, first_tile, last_tile, table, page_shift);
                slot = -1;
            }
            load_kv_block<D>(bb, pages, slot + 1, k_pool, v_pool, kvh, KVH, page_shift, off);
            attend_block<D, HPW>(ba, st, qf, kb * 32, nh, tv, g, scale_log2);
            kb += KS;
            ++slot;
            if (kb > kb1) break;
            if (slot == 31) {
                pages = lane_pages<KS>(kb + KS, lane, first_tile, last_tile, table, page_shift);
                slot = -1;
            }
            load_kv_block<D>(ba, pages, slot + 1, k_pool, v_pool, kvh, KVH, page_shift, off);
            attend_block<D, HPW>(bb, st, qf, kb * 32, nh, tv, g, scale_log2);
            kb += KS;
            ++slot;
        }

        // merge the wavefronts' partials head by head, in wavefront order; lane: d = 16 dt + 4 g + i of token r
#pragma unroll
        for (int hh = 0; hh < HPW; ++hh) {
            if (hh >= nh) continue;                                  // block-uniform
            float lsum = st.l[hh];
            lsum += __shfl_xor(lsum, 16, TM_WAVE);
            lsum += __shfl_xor(lsum, 32, TM_WAVE);
            if (g == 0) {
                s_m[wave][r] = st.m[hh];
                s_l[wave][r] = lsum;
            }
#pragma unroll
            for (int dt = 0; dt < NDT; ++dt)
#pragma unroll
                for (int i = 0; i < 4; ++i) s_o[wave][r][16 * dt + 4 * g + i] = st.o[hh][dt][i];
            __syncthreads();
            for (int idx = threadIdx.x; idx < 16 * (D / 2); idx += 64 * KS) {
                const int col = idx / (D / 2), d = 2 * (idx % (D / 2));
                if (col >= valid) continue;
                float mm = s_m[0][col];
#pragma unroll
                for (int w = 1; w < KS; ++w) mm = fmaxf(mm, s_m[w][col]);
                float ll = 0.f, o0 = 0.f, o1 = 0.f;
#pragma unroll
                for (int w = 0; w < KS; ++w) {
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
}

// Heads a wavefront takes and wavefronts a block has, by head size (registers decide). Up to head size 64 a
// wavefront can hold four heads, which quarters the loads of a long prompt's keys; a short step, whose blocks of
// two heads a wavefront still fit the chip in one round, takes those instead: twice the blocks, half as long
// (512 tokens at the 0.5B shape: 13.4 to 9.8 us; a head's arithmetic is the same either way, so its bits are).
template <int D> struct PrefillShape { static constexpr int HPW = D <= 64 ? 4 : 2, KS = D <= 64 ? 8 : 4; };

template <int D, int HPW>
static void launch_split_keys(const void* q, int q_stride, void* out, int out_stride, const void* k_pool, const void* v_pool,
                              const int* block_tables, int table_width, const int* tiles, int n_tiles, int H, int KVH,
                              int page_shift, float scale_log2, int window, hipStream_t stream) {
    constexpr int KS = PrefillShape<D>::KS;
    const int splits = (H / KVH + HPW - 1) / HPW;
    // fold the table in two once the folded launch still gives every CU a block
    const int pair = (long long)(n_tiles / 2) * KVH * splits >= 256 ? 1 : 0;
    dim3 grid(pair ? (n_tiles + 1) / 2 : n_tiles, KVH * splits);
    attn_prefill_mfma_kernel<D, HPW, KS><<<grid, 64 * KS, 0, stream>>>(
        (const bf16_t*)q, q_stride, (bf16_t*)out, out_stride, (const bf16_t*)k_pool, (const bf16_t*)v_pool, block_tables,
        table_width, tiles, n_tiles, pair, H, KVH, page_shift, scale_log2, window);
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
    int page_shift = 0;
    while ((1 << page_shift) < page) ++page_shift;
    const float scale_log2 = scale * 1.4426950408889634f;
    if ((long long)KVH * ((G + 1) / 2) > 65535) return TM_ERR_ARG;
#define TM_SPLIT_ARGS q, q_stride, out, out_stride, k_pool, v_pool, block_tables, table_width, tiles, n_tiles, H, KVH, \
                      page_shift, scale_log2, window, stream
#define TM_PREFILL_CASE(DD)                                                                                       \
    case DD: {                                                                                                    \
        constexpr int HPW = PrefillShape<DD>::HPW;                                                                \
        if (HPW > 2 && G > 2 && (long long)n_tiles * KVH * ((G + 1) / 2) <= TM_PREFILL_ONE_ROUND)                 \
            launch_split_keys<DD, 2>(TM_SPLIT_ARGS);                                                              \
        else                                                                                                      \
            launch_split_keys<DD, HPW>(TM_SPLIT_ARGS);                                                            \
        break;                                                                                                    \
    }
    switch (D) {
        TM_PREFILL_CASE(32)
        TM_PREFILL_CASE(64)
        TM_PREFILL_CASE(96)
        TM_PREFILL_CASE(128)
        default:
            return TM_ERR_ARG;
    }
#undef TM_PREFILL_CASE
#undef TM_SPLIT_ARGS
    TM_CHECK_LAUNCH();
    return TM_OK;
}
