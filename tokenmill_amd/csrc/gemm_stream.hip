// Matrix products of a step with 17 to 64 tokens at any width, each with its layer's own epilogue: q|k|v with
// bias, rotary and cache write; gate|up with SiLU*up; a plain product with bias whose rounded result is stored or
// added into the 32-bit residual stream (the output and down projections).
//
// With at most 64 rows a product is bound by reading its matrix once. The matrix comes in strip order (api.h), the
// copy the decode kernels for up to 16 tokens read, whatever its strips' height (16, 8 or 4 rows): a wavefront
// always multiplies two tiles of 16 matrix rows (a "unit": the two halves of 16 rotary pairs, 16 gate rows and
// the 16 up rows that meet them, or 32 consecutive rows), each tile made of 1, 2 or 4 packed strips, with all
// row tiles of the activations (1 to 4 tiles of 16 tokens), so a 16-byte piece of the matrix is used for up to
// 64 tokens.
//
// A block has KS x US wavefronts: US units side by side, each unit's K split over KS wavefronts. The block walks K
// in rounds of ST_KCH k-steps per wavefront. The activations of a round (for each of the KS ranges of K a window
// of ST_KCH k-steps, all rows) are read from the cache in whole lines by all threads together, go through LDS,
// and serve all US units from there: the cache sees them once a block, not once a wavefront, and a wavefront
// reads them in the matrix unit's layout without asking the cache for half lines. The matrix streams from HBM
// straight into registers: as soon as a k-step's products are issued its registers are asked for the same
// k-step of the next round, so every wavefront keeps ST_KCH k-steps of two strips in flight while it multiplies.
// Every load is without a condition, at an address clamped into valid memory. At the end the KS partial sums of
// a unit are added through LDS in wavefront order, tile by tile, and wavefront t mod KS of the unit does the
// epilogue of row tile t.
//
// Which k goes to which wavefront depends on the matrix's shape alone, never on the number of tokens: a token's
// result does not depend on its batch-mates. Everything is rounded where the unfused path stores a bfloat16
// tensor, so both agree up to the order of 32-bit sums (reference src/infer/model/layers.py:142-150,60-64,
// 163-164; src/infer/kv/paged_cache.py:40-43; src/infer/model/qwen2.py:22-23).
#include "common.h"
#include "api.h"
#include "fused_common.h"

#define ST_EPI_QKV 0
#define ST_EPI_SILU 1
#define ST_EPI_PLAIN 2
#define ST_KCH 4            // k-steps of a round, per wavefront
#define ST_WD 8             // k-steps of the matrix a wavefront has in registers or on their way (a multiple of ST_KCH)
// the matrix is read once and never again: loads that do not displace the activations in the caches
#define ST_WLOAD(p) __builtin_nontemporal_load((const u32x4_t*)(p))
#define ST_XPAD 16          // padding of an LDS row of activations, in elements: rows 288 bytes apart, which the operand loads (lane (r, g): 16 bytes of row r at piece g) read free of bank conflicts; with 8 (272 bytes) they take twice as long

struct StreamArgs {
    FusedArgs f;            // activations X [M, K], the packed matrix, and what the q|k|v and SiLU epilogues need
    int rows;               // height of the packed strips (16, 8 or 4)
    int n_strips;           // strips the packed matrix has in all (SiLU: in each half)
    // the plain epilogue
    int N;
    void* C;                // [M, N] rows ldc apart, or null with accum
    int ldc, c_f32;
    float* accum;           // [M, N] rows ldacc apart: += the result rounded to bfloat16
    int ldacc;
    float* parts;           // K split over gridDim.y groups of blocks: [group][M][N] gets the 32-bit partial sums
};

struct StreamUnit {
    int nA, nB;             // first matrix rows of the two tiles
    int pA, pB;             // the packed strips their first rows lie in
    int head, jt;           // q|k|v: the head and which slice of it
};

template <int EPI>
__device__ __forceinline__ StreamUnit stream_unit_of(const StreamArgs& a, int u) {
    StreamUnit t;
    t.head = t.jt = 0;
    if (EPI == ST_EPI_QKV) {
        const int per_head = a.f.D / 32;
        t.head = u / per_head;
        t.jt = u % per_head;
        if (t.head < a.f.H + a.f.KVH) {                              // the two halves of 16 rotary pairs
            t.nA = t.head * a.f.D + 16 * t.jt;
            t.nB = t.nA + a.f.D / 2;
        } else {
            t.nA = t.head * a.f.D + 32 * t.jt;
            t.nB = t.nA + 16;
        }
        t.pA = t.nA / a.rows;
        t.pB = t.nB / a.rows;
    } else if (EPI == ST_EPI_SILU) {                                 // gate rows and the up rows that meet them
        t.nA = 16 * u;
        t.nB = a.f.I + 16 * u;
        t.pA = u;
        t.pB = a.f.up_strip0 + u;
    } else {
        t.nA = 32 * u;
        t.nB = t.nA + 16;
        t.pA = t.nA / a.rows;
        t.pB = t.nB / a.rows;
    }
    return t;
}

// Bytes of LDS a block needs: the activations of a round, or (whichever is more) the partial sums of two tiles.
__host__ __device__ constexpr int stream_lds_bytes(int NT, int KS, int US) {
    const int window = KS * NT * 16 * (ST_KCH * 32 + ST_XPAD) * 2;
    const int sums = 2 * KS * US * 2 * 64 * 4 * 4;
    return window > sums ? window : sums;
}

// NT: 16-token tiles of the activations (1..4). KS: wavefronts that split a unit's K. US: units of a block.
template <int EPI, int NT, int KS, int US>
__global__ __launch_bounds__(64 * KS * US) void gemm_stream_kernel(const StreamArgs a, const int n_units) {
    extern __shared__ __align__(16) unsigned char smem_raw[];
    constexpr int WAVES = KS * US, THREADS = 64 * WAVES;
    constexpr int XROW = ST_KCH * 32 + ST_XPAD;                      // elements of an LDS row: a window of K, padded
    constexpr int ROWS_X = NT * 16;
    bf16_t* xs = (bf16_t*)smem_raw;                                  // [KS][ROWS_X][XROW]
    const FusedArgs& f = a.f;
    // the tokens of this block: all of them, or (gridDim.z > 1) the NT tiles from tok0 on
    const int tok0 = blockIdx.z * (NT * 16);
    const int K = f.K, M = f.M - tok0 < NT * 16 ? f.M - tok0 : NT * 16;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / TM_WAVE), lane = threadIdx.x % TM_WAVE;
    const int kw = wave % KS, uw = wave / KS;                        // which range of K, which unit of the block
    const int r = lane % 16, g = lane / 16;
    const int ksteps = (K + 31) / 32;
    // the k-steps of this block: all of them, or one of gridDim.y equal parts (a plain product with few rows of output)
    const int per_block = (ksteps + gridDim.y - 1) / gridDim.y;
    const int k_begin = blockIdx.y * per_block;
    const int k_stop = k_begin + per_block < ksteps ? k_begin + per_block : ksteps;
    const int per = (per_block + KS - 1) / KS;
    const int ks0 = k_begin + kw * per < k_stop ? k_begin + kw * per : k_stop;
    const int ks1 = ks0 + per < k_stop ? ks0 + per : k_stop;
    const int last_ks = ksteps - 1;
    const int u_mine = blockIdx.x * US + uw;
    const bool have_unit = u_mine < n_units;                         // (the last block may hold fewer units)
    const StreamUnit cu = stream_unit_of<EPI>(a, have_unit ? u_mine : n_units - 1);

    // this lane's piece of a k-step of tile A / B: row r of the tile lies in packed strip p + r / rows, row r % rows
    const int frag = 32 * a.rows;
    const int sub = r / a.rows, rr = r % a.rows;
    const int last_strip = (EPI == ST_EPI_SILU ? 2 : 1) * a.n_strips - 1;
    const int sA = cu.pA + sub < last_strip ? cu.pA + sub : last_strip;       // (a strip that does not exist: rows beyond
    const int sB = cu.pB + sub < last_strip ? cu.pB + sub : last_strip;       //  the matrix, whose results nobody stores)
    const bf16_t* wA = f.W + (size_t)sA * ksteps * frag + (g * a.rows + rr) * 8;
    const bf16_t* wB = f.W + (size_t)sB * ksteps * frag + (g * a.rows + rr) * 8;
    auto w_at = [&](int ks) { return (size_t)(ks < last_ks ? ks : last_ks) * frag; };

    // The activations of a round: KS windows of ST_KCH k-steps (64 bytes a row each), all rows. Thread i takes the
    // 16-byte pieces i, i + THREADS, ...: consecutive lanes read one row's window as a run, whole lines at a time.
    constexpr int PIECES_ROW = ST_KCH * 4;
    constexpr int PIECES = KS * ROWS_X * PIECES_ROW;
    constexpr int XL = (PIECES + THREADS - 1) / THREADS;
    const int k_end = K;
    u32x4_t xv[XL];
    auto load_x = [&](int round) {
#pragma unroll
        for (int i = 0; i < XL; ++i) {
            const int p = threadIdx.x + i * THREADS;
            const int win = p / (ROWS_X * PIECES_ROW), in = p % (ROWS_X * PIECES_ROW);
            const int row = in / PIECES_ROW, piece = in % PIECES_ROW;
            int k = (k_begin + (win < KS ? win : KS - 1) * per + round * ST_KCH) * 32 + piece * 8;
            k = k + 8 <= k_end ? k : 0;                               // beyond the row: a piece that exists (zeroed when stored)
            xv[i] = *(const u32x4_t*)(f.X + (size_t)(tok0 + (row < M ? row : M - 1)) * f.ldx + k);
        }
    };
    auto store_x = [&](int round) {
#pragma unroll
        for (int i = 0; i < XL; ++i) {
            const int p = threadIdx.x + i * THREADS;
            if (PIECES % THREADS == 0 || p < PIECES) {
                const int win = p / (ROWS_X * PIECES_ROW), in = p % (ROWS_X * PIECES_ROW);
                const int row = in / PIECES_ROW, piece = in % PIECES_ROW;
                const int k = (k_begin + win * per + round * ST_KCH) * 32 + piece * 8;
                // beyond K the packed matrix holds zeros: the activations there must be zeros too (0 * anything stays 0)
                const u32x4_t v = k + 8 <= k_end ? xv[i] : u32x4_t{0, 0, 0, 0};
                *(u32x4_t*)(xs + ((size_t)win * ROWS_X + row) * XROW + piece * 8) = v;
            }
        }
    };

    f32x4_t accA[NT], accB[NT];
#pragma unroll
    for (int t = 0; t < NT; ++t) {
        accA[t] = f32x4_t{0.f, 0.f, 0.f, 0.f};
        accB[t] = f32x4_t{0.f, 0.f, 0.f, 0.f};
    }
    const int rounds = (per + ST_KCH - 1) / ST_KCH;                  // the same for every wavefront of the block
    // What the q|k|v epilogue needs from memory, where a wavefront owns one token tile (tile kw): the token's position,
    // cache slot and the bias are asked for before anything else (loads come back in the order they were issued, so
    // these are not behind the matrix), the rotary row, whose address hangs on the position, after the first round.
    constexpr bool PRE = EPI == ST_EPI_QKV && NT <= KS;
    int pre_pos = 0, pre_slot = -1;
    float pre_bA[4] = {0.f, 0.f, 0.f, 0.f}, pre_bB[4] = {0.f, 0.f, 0.f, 0.f};
    f32x4_t pre_cs = {0.f, 0.f, 0.f, 0.f}, pre_sn = {0.f, 0.f, 0.f, 0.f};
    if constexpr (PRE) {
        const int tok = tok0 + (16 * kw + r < M ? 16 * kw + r : M - 1);    // (tile kw may not exist: a token that does)
        pre_pos = f.positions[tok];
        pre_slot = f.slots ? f.slots[tok] : -1;
        if (f.bias) {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int ia = cu.nA + 4 * g + i, ib = cu.nB + 4 * g + i;
                pre_bA[i] = f.bias_f32 ? ((const float*)f.bias)[ia] : bf16_to_f32(((const bf16_t*)f.bias)[ia]);
                pre_bB[i] = f.bias_f32 ? ((const float*)f.bias)[ib] : bf16_to_f32(((const bf16_t*)f.bias)[ib]);
            }
        }
    }
    // The matrix runs ST_WD k-steps ahead of the products, in registers: the activations of a k-step need to be in
    // LDS only when it is multiplied, so how much of the matrix a wavefront has in flight is not bound by LDS.
    FFrag fa[ST_WD], fb[ST_WD];
    load_x(0);
#pragma unroll
    for (int j = 0; j < ST_WD; ++j) {
        fa[j].u = ST_WLOAD(wA + w_at(ks0 + j));
        fb[j].u = ST_WLOAD(wB + w_at(ks0 + j));
    }
    const bf16_t* x_mine = xs + ((size_t)kw * ROWS_X + r) * XROW + 8 * g;
    for (int round0 = 0; round0 < rounds; round0 += ST_WD / ST_KCH) {
#pragma unroll
        for (int sr = 0; sr < ST_WD / ST_KCH; ++sr) {
            const int round = round0 + sr;
            if (round < rounds) {                                     // the same for the whole block
                store_x(round);
                __syncthreads();
                if (round + 1 < rounds) load_x(round + 1);            // on their way while this round multiplies
                if constexpr (PRE) {
                    if (round == 0 && cu.head < f.H + f.KVH) {        // the position has arrived with the first activations
                        const size_t at = (size_t)pre_pos * (f.D / 2) + 16 * cu.jt + 4 * g;
                        pre_cs = *(const f32x4_t*)(f.cos_t + at);
                        pre_sn = *(const f32x4_t*)(f.sin_t + at);
                    }
                }
                const int base = ks0 + round * ST_KCH;
#pragma unroll
                for (int j = 0; j < ST_KCH; ++j) {
                    const int slot = sr * ST_KCH + j;                 // a compile-time register index
                    if (base + j < ks1) {                             // the same for all lanes of the wavefront
#pragma unroll
                        for (int t = 0; t < NT; ++t) {
                            FFrag x;
                            x.u = *(const u32x4_t*)(x_mine + (size_t)(16 * t) * XROW + 32 * j);
                            accA[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fa[slot].b, x.b, accA[t], 0, 0, 0);
                            accB[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fb[slot].b, x.b, accB[t], 0, 0, 0);
                        }
                    }
                    if (base + j + ST_WD < ks1) {   // these registers are free: they take the k-step ST_WD further on
                        fa[slot].u = ST_WLOAD(wA + w_at(base + j + ST_WD));
                        fb[slot].u = ST_WLOAD(wB + w_at(base + j + ST_WD));
                    }
                }
                __syncthreads();                                      // everybody has read this round's activations
            }
        }
    }

    float (*red)[KS * US][2][64][4] = (float (*)[KS * US][2][64][4])smem_raw;    // [2 tiles in turn][wavefront][A, B][lane][4]
    // tile by tile: the partial sums meet in LDS and are added in wavefront order by the wavefront that owns the tile
#pragma unroll
    for (int t = 0; t < NT; ++t) {
        float (*buf)[2][64][4] = red[t & 1];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            buf[wave][0][lane][i] = accA[t][i];
            buf[wave][1][lane][i] = accB[t][i];
        }
        __syncthreads();
        if (kw != t % KS || !have_unit) continue;
        if (16 * t + r >= M) continue;
        const int tok = tok0 + 16 * t + r;
        float sA[4], sB[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            float va = buf[uw * KS][0][lane][i], vb = buf[uw * KS][1][lane][i];
#pragma unroll
            for (int w = 1; w < KS; ++w) {
                va += buf[uw * KS + w][0][lane][i];
                vb += buf[uw * KS + w][1][lane][i];
            }
            sA[i] = va;
            sB[i] = vb;
        }
        // lane: token tok, matrix rows nA + 4g + i and nB + 4g + i
        if constexpr (EPI == ST_EPI_SILU) {
            const int col = cu.nA + 4 * g;
            if (col < f.I) {
                float v[4];
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const float gt = fd_round(sA[i]), up = fd_round(sB[i]);
                    v[i] = gt / (1.f + expf(-gt)) * up;
                }
                bf16_t* dst = f.act_out + (size_t)tok * f.I + col;
                if (col + 4 <= f.I) {
                    *(uint2*)dst = uint2{fd_pack(v[0], v[1]), fd_pack(v[2], v[3])};
                } else {
                    for (int i = 0; i < 4 && col + i < f.I; ++i) dst[i] = f32_to_bf16(v[i]);
                }
            }
        } else if constexpr (EPI == ST_EPI_QKV) {
            float xA[4], xB[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                float bA = pre_bA[i], bB = pre_bB[i];
                if (!PRE && f.bias) {
                    const int ia = cu.nA + 4 * g + i, ib = cu.nB + 4 * g + i;
                    bA = f.bias_f32 ? ((const float*)f.bias)[ia] : bf16_to_f32(((const bf16_t*)f.bias)[ia]);
                    bB = f.bias_f32 ? ((const float*)f.bias)[ib] : bf16_to_f32(((const bf16_t*)f.bias)[ib]);
                }
                xA[i] = fd_round(sA[i] + bA);
                xB[i] = fd_round(sB[i] + bB);
            }
            const int slot = PRE ? pre_slot : (f.slots ? f.slots[tok] : -1);
            if (cu.head < f.H + f.KVH) {
                const int half = f.D / 2;
                const int j0 = 16 * cu.jt + 4 * g;                                   // pair index of element 0
                f32x4_t cs = pre_cs, sn = pre_sn;
                if (!PRE) {
                    const size_t at = (size_t)f.positions[tok] * half + j0;
                    cs = *(const f32x4_t*)(f.cos_t + at);
                    sn = *(const f32x4_t*)(f.sin_t + at);
                }
                float y1[4], y2[4];
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    rotate_pair(xA[i], xB[i], cs[i], sn[i], y1[i], y2[i]);
                }
                bf16_t* dst = nullptr;
                if (cu.head < f.H)
                    dst = f.q_out + (size_t)tok * f.H * f.D + (size_t)cu.head * f.D + j0;
                else if (slot >= 0)
                    dst = f.k_pool + ((size_t)slot * f.KVH + (cu.head - f.H)) * f.D + j0;
                if (dst) {
                    *(uint2*)dst = uint2{fd_pack(y1[0], y1[1]), fd_pack(y1[2], y1[3])};
                    *(uint2*)(dst + half) = uint2{fd_pack(y2[0], y2[1]), fd_pack(y2[2], y2[3])};
                }
            } else if (slot >= 0) {
                const int vh = cu.head - f.H - f.KVH;
                const int pg = slot >> f.page_shift, in_page = slot & ((1 << f.page_shift) - 1);
                const int d0 = 32 * cu.jt + 4 * g;
                bf16_t* dst = f.v_pool + ((((size_t)pg * f.KVH + vh) * f.D + d0) << f.page_shift) + in_page;
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    dst[(size_t)i << f.page_shift] = f32_to_bf16(xA[i]);
                    dst[(size_t)(i + 16) << f.page_shift] = f32_to_bf16(xB[i]);
                }
            }
        } else {
#pragma unroll
            for (int half = 0; half < 2; ++half) {
                const int nf = (half ? cu.nB : cu.nA) + 4 * g;
                if (nf >= a.N) continue;
                const float* s = half ? sB : sA;
                float v[4];
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    float b = 0.f;
                    if (f.bias && nf + i < a.N && blockIdx.y == 0)
                        b = f.bias_f32 ? ((const float*)f.bias)[nf + i] : bf16_to_f32(((const bf16_t*)f.bias)[nf + i]);
                    v[i] = s[i] + b;
                }
                const bool whole = nf + 4 <= a.N;
                if (a.parts) {          // this block's share of K: 32-bit, unrounded, for whoever adds the parts up
                    float* dst = a.parts + ((size_t)blockIdx.y * f.M + tok) * a.N + nf;
                    if (whole && (a.N % 4) == 0) {
                        *(f32x4_t*)dst = f32x4_t{v[0], v[1], v[2], v[3]};
                    } else {
                        for (int i = 0; i < 4 && nf + i < a.N; ++i) dst[i] = v[i];
                    }
                } else if (a.accum) {          // the rounded result goes into the 32-bit residual stream (each element has one owner)
                    float* dst = a.accum + (size_t)tok * a.ldacc + nf;
                    if (whole && (a.ldacc % 4) == 0 && ((uintptr_t)a.accum % 16) == 0) {
                        f32x4_t cur = *(const f32x4_t*)dst;
#pragma unroll
                        for (int i = 0; i < 4; ++i) cur[i] += fd_round(v[i]);
                        *(f32x4_t*)dst = cur;
                    } else {
                        for (int i = 0; i < 4 && nf + i < a.N; ++i) dst[i] += fd_round(v[i]);
                    }
                } else if (a.c_f32) {
                    float* dst = (float*)a.C + (size_t)tok * a.ldc + nf;
                    for (int i = 0; i < 4 && nf + i < a.N; ++i) dst[i] = v[i];
                } else {
                    bf16_t* dst = (bf16_t*)a.C + (size_t)tok * a.ldc + nf;
                    if (whole && (a.ldc % 4) == 0 && ((uintptr_t)a.C % 8) == 0) {
                        *(uint2*)dst = uint2{fd_pack(v[0], v[1]), fd_pack(v[2], v[3])};
                    } else {
                        for (int i = 0; i < 4 && nf + i < a.N; ++i) dst[i] = f32_to_bf16(v[i]);
                    }
                }
            }
        }
    }
}

// How a block is made for a matrix: KS wavefronts split a unit's K, US units share the activations in LDS. From
// the matrix's shape alone (never from the number of tokens: that keeps a token's sums in one order).
//
// A CU holds one block of these kernels (at 128 registers a lane a CU has room for 16 wavefronts), so a launch
// should be one round of at most 256 blocks, as close to 256 as the units allow: US = the fewest units a block
// that leave at most 256 blocks, and two wavefronts a unit from three units a block on (four with two units,
// eight with one). Measured on an MI355X, 8 / 32 / 64 tokens (us): gate|up 7B (1,184 units) 2 x 5 = 237 blocks:
// 53 / 50 / 55 (2 x 8 = 148 blocks: 58 / 61 / 68; 2 x 6: 54 / 53 / 57; 3 x 5: 48 / 50 / 78; 1 x 4 = 296 blocks: - / 60 / 73;
// 4 x 4: - / 70 / 100); gate|up 32B (1,728 units) 2 x 8 = 216 blocks: 95 / 98 / 101 (2 x 7 = 247: 94 / 97 / 106, a few registers spilled; 2 x 6 = 288
// blocks, a second round: 133 / 134 / 142; 1 x 4: - / 97 / 110); gate|up 0.5B (304 units) 4 x 2: - / 9 / 13 (8 x 1: - / 14 / 21);
// q|k|v 7B (144 units) 8 x 1: - / 17 / 25 (4 x 2: - / 20 / 27).
static void stream_config(int n_units, int* ks, int* us) {
    int u = (n_units + 255) / 256;
    if (u > 6) u = 8;                           // (seven units, 14 wavefronts, need a few registers more than the 128 there are)
    *us = u;
    *ks = u == 1 ? 8 : u == 2 ? 4 : 2;
}

// The same for a plain product whose K is split over `parts` groups of blocks, which leave 32-bit partial sums
// (1: not split). From the matrix's shape alone.
static void stream_plain_shape(int N, int K, int* parts, int* ks, int* us) {
    const int n_units = (N + 31) / 32, ksteps = (K + 31) / 32;
    // Wide outputs over a K that gives every wavefront four k-steps: eight groups of blocks, two wavefronts a unit, and
    // the fewest units a block that leave at most 256 blocks. Measured on an MI355X, 8 / 32 / 64 tokens (us): 7B down
    // (112 units, K 18,944) 8 groups of 2 x 4 = 224 blocks: 27 / 29 / 34 (3 x 4: 26 / 29 / 33; 4 x 4: 26 / 29 / 41; 4 groups
    // of 4 x 2: - / 30 / 39; 8 of 2 x 8 = 112 blocks: - / 36 / 42; unsplit - / 56 / 81; the library's product with its
    // algorithm chosen by timing - / 52 / 69); 7B o: 8 / 10 / 13 (4 groups of 4 x 2: - / 10 / 13); 32B down (160 units,
    // K 27,648) 8 groups of 2 x 5 = 256 blocks: 52 / 51 / 57 (2 x 8 = 160 blocks: 56 / 58 / 65; 3 x 5: 51 / 52 / 143; 4 groups
    // of 4 x 2: - / 65 / 92); 32B o: 12.5 / 14 / 17 (2 x 8: 14 / 16 / 19; 4 groups of 4 x 2: - / 17 / 27).
    if (n_units >= 96 && ksteps >= 64) {
        *parts = 8;
        *ks = 2;
        *us = (n_units + 31) / 32 < 7 ? (n_units + 31) / 32 : 8;
        return;
    }
    // Narrow outputs: the fewest groups (a power of two, at most 8) that give the matrix about 400 blocks' worth of
    // units, as long as a wavefront (of the four that split a block's share of K) keeps four k-steps to itself:
    // 0.5B down 8 groups: 8 / 11 us at 32 / 64 tokens against 10 / 10 us. 1: not worth splitting (the library's
    // product is the faster one then).
    int p = 1;
    while (p < 8 && n_units * p < 384) p *= 2;
    while (p > 1 && ksteps / (p * 4) < 4) p /= 2;
    *parts = p;
    stream_config(n_units * p, ks, us);
}

template <int EPI, int NT, int KS, int US>
static int launch_stream_config(const StreamArgs& a, int n_units, int kparts, int row_parts, hipStream_t stream) {
    constexpr int lds = stream_lds_bytes(NT, KS, US);
    static bool raised = false;
    if (lds > 48 * 1024 && !raised) {
        if (hipFuncSetAttribute((const void*)gemm_stream_kernel<EPI, NT, KS, US>, hipFuncAttributeMaxDynamicSharedMemorySize,
                                lds) != hipSuccess)
            return TM_ERR_LAUNCH;
        raised = true;
    }
    gemm_stream_kernel<EPI, NT, KS, US><<<dim3((n_units + US - 1) / US, kparts, row_parts), 64 * KS * US, lds, stream>>>(a, n_units);
    TM_CHECK_LAUNCH();
    return TM_OK;
}

template <int EPI, int NT>
static int launch_stream_tiles(const StreamArgs& a, int n_units, int kparts, int row_parts, int ks, int us, hipStream_t stream) {
    switch (ks * 16 + us) {                     // the shapes stream_config and stream_plain_shape name
        case 4 * 16 + 2: return launch_stream_config<EPI, NT, 4, 2>(a, n_units, kparts, row_parts, stream);
        case 8 * 16 + 1: return launch_stream_config<EPI, NT, 8, 1>(a, n_units, kparts, row_parts, stream);
        case 2 * 16 + 3: return launch_stream_config<EPI, NT, 2, 3>(a, n_units, kparts, row_parts, stream);
        case 2 * 16 + 4: return launch_stream_config<EPI, NT, 2, 4>(a, n_units, kparts, row_parts, stream);
        case 2 * 16 + 5: return launch_stream_config<EPI, NT, 2, 5>(a, n_units, kparts, row_parts, stream);
        case 2 * 16 + 6: return launch_stream_config<EPI, NT, 2, 6>(a, n_units, kparts, row_parts, stream);
        case 2 * 16 + 8: return launch_stream_config<EPI, NT, 2, 8>(a, n_units, kparts, row_parts, stream);
        default: return TM_ERR_ARG;
    }
}

// kparts == 1: the block's shape from the number of units; else the caller's (stream_plain_shape).
template <int EPI>
static int launch_stream(const StreamArgs& a, int n_units, hipStream_t stream, int kparts = 1, int ks = 0, int us = 0) {
    if (ks == 0) stream_config(n_units, &ks, &us);
    int tiles = (a.f.M + 15) / 16, row_parts = 1;
    // gate|up over a matrix small enough that reading it twice from the cache costs little, in blocks of 8 wavefronts
    // of which a CU holds two when they carry two tiles of tokens (124 registers instead of 164): the further tiles
    // go to blocks of their own (0.5B shape, a decode step of 48 / 64 requests 1.65 / 1.88 to 1.54 / 1.73 ms together
    // with the same for q|k|v in gemm_panel.hip; at the 7B shape's q|k|v, whose matrix is 33 MB, it lost: 25 us
    // against 20 us at 64 rows)
    if (EPI == ST_EPI_SILU && ks * us <= 8 && n_units <= 512 && tiles > 2) {
        row_parts = 2;
        tiles = 2;
    }
    switch (tiles) {
        case 1: return launch_stream_tiles<EPI, 1>(a, n_units, kparts, row_parts, ks, us, stream);
        case 2: return launch_stream_tiles<EPI, 2>(a, n_units, kparts, row_parts, ks, us, stream);
        case 3: return launch_stream_tiles<EPI, 3>(a, n_units, kparts, row_parts, ks, us, stream);
        default: return launch_stream_tiles<EPI, 4>(a, n_units, kparts, row_parts, ks, us, stream);
    }
}

static bool stream_common_ok(int M, int K, const void* X, int ldx, const void* W, int rows) {
    return M > 0 && M <= 64 && K > 0 && (K % 8) == 0 && ldx >= K && (ldx % 8) == 0 && X && W && ((uintptr_t)X % 16) == 0 &&
           ((uintptr_t)W % 16) == 0 && (rows == 16 || rows == 8 || rows == 4);
}

// Does the stream family take M tokens of width K? (Any K that is a multiple of 8, up to 64 tokens.)
extern "C" int tm_gemm_stream_fits(int M, int K) { return M > 0 && M <= 64 && K > 0 && (K % 8) == 0 ? 1 : 0; }

// q_out[M, H*D], K cache, V cache <- rope(X Wqkv^T + b) for up to 64 tokens; X bfloat16 [M, K] (rows ldx apart) is the
// normed input; W the [(H + 2 KVH) D, K] matrix packed in strips of `rows` rows; the rest as for tm_panel_qkv_rope.
extern "C" int tm_stream_qkv_rope(const void* X, int ldx, int M, int K, const void* W, int rows, const void* bias,
                                  int bias_dtype, void* q_out, int H, int KVH, int D, const float* cos_t,
                                  const float* sin_t, const int* positions, const int* slots, void* k_pool,
                                  void* v_pool, int page, hipStream_t stream) {
    if (M == 0) return TM_OK;
    if (!stream_common_ok(M, K, X, ldx, W, rows) || H <= 0 || KVH <= 0 || D <= 0 || D % 32 || !cos_t || !sin_t || !positions ||
        !q_out || ((uintptr_t)q_out % 8) || page <= 0 || (page & (page - 1)))
        return TM_ERR_ARG;
    if (slots && (!k_pool || !v_pool)) return TM_ERR_ARG;
    StreamArgs a{};
    FusedArgs& f = a.f;
    f.X = (const bf16_t*)X; f.ldx = ldx; f.M = M; f.K = K;
    f.W = (const bf16_t*)W; f.bias = bias; f.bias_f32 = bias_dtype == TM_F32;
    f.q_out = (bf16_t*)q_out; f.H = H; f.KVH = KVH; f.D = D; f.cos_t = cos_t; f.sin_t = sin_t;
    f.positions = positions; f.slots = slots; f.k_pool = (bf16_t*)k_pool; f.v_pool = (bf16_t*)v_pool;
    f.page_shift = 0;
    while ((1 << f.page_shift) < page) ++f.page_shift;
    a.rows = rows;
    a.n_strips = ((H + 2 * KVH) * D + rows - 1) / rows;
    return launch_stream<ST_EPI_QKV>(a, (H + 2 * KVH) * (D / 32), stream);
}

// act[M, I] <- silu(X Wg^T) * (X Wu^T) for up to 64 tokens; W = [Wg; Wu], each half packed in strips of 16 rows.
extern "C" int tm_stream_gate_up_silu(const void* X, int ldx, int M, int K, const void* W, void* act_out, int I,
                                      hipStream_t stream) {
    if (M == 0) return TM_OK;
    if (!stream_common_ok(M, K, X, ldx, W, 16) || I <= 0 || !act_out || ((uintptr_t)act_out % 8) || (I % 4)) return TM_ERR_ARG;
    StreamArgs a{};
    FusedArgs& f = a.f;
    f.X = (const bf16_t*)X; f.ldx = ldx; f.M = M; f.K = K;
    f.W = (const bf16_t*)W; f.act_out = (bf16_t*)act_out; f.I = I;
    const int units = (I + 15) / 16;
    f.up_strip0 = units;
    a.rows = 16;
    a.n_strips = units;
    return launch_stream<ST_EPI_SILU>(a, units, stream);
}

// C[M, N] = X W^T + bias (bfloat16, or float32 with out_f32), or with accum (float32 [M, N], rows ldacc apart)
// accum += round_bfloat16(X W^T + bias) and C is not written; up to 64 tokens; W [N, K] packed in strips of `rows` rows.
extern "C" int tm_stream_linear(const void* X, int ldx, int M, int K, const void* W, int rows, int N, const void* bias,
                                int bias_dtype, void* C, int ldc, int out_f32, float* accum, int ldacc,
                                hipStream_t stream) {
    if (M == 0) return TM_OK;
    if (!stream_common_ok(M, K, X, ldx, W, rows) || N <= 0 || (!C && !accum) || (C && ldc < N) || (accum && ldacc < N))
        return TM_ERR_ARG;
    StreamArgs a{};
    FusedArgs& f = a.f;
    f.X = (const bf16_t*)X; f.ldx = ldx; f.M = M; f.K = K;
    f.W = (const bf16_t*)W; f.bias = bias; f.bias_f32 = bias_dtype == TM_F32;
    a.rows = rows;
    a.n_strips = (N + rows - 1) / rows;
    a.N = N; a.C = accum ? nullptr : C; a.ldc = ldc; a.c_f32 = out_f32; a.accum = accum; a.ldacc = ldacc;
    return launch_stream<ST_EPI_PLAIN>(a, (N + 31) / 32, stream);
}

// Groups of blocks a plain product's K is split over: enough that a matrix with few rows still has a few thousand
// wavefronts streaming it, each with a few rounds of k-steps to itself. From the matrix's shape alone.
extern "C" int tm_stream_linear_parts(int N, int K) {
    int parts = 1, ks = 0, us = 0;
    stream_plain_shape(N, K, &parts, &ks, &us);
    return parts;
}

extern "C" int tm_stream_linear_split(const void* X, int ldx, int M, int K, const void* W, int rows, int N, const void* bias,
                                      int bias_dtype, float* parts, hipStream_t stream) {
    if (M == 0) return TM_OK;
    if (!stream_common_ok(M, K, X, ldx, W, rows) || N <= 0 || !parts) return TM_ERR_ARG;
    StreamArgs a{};
    FusedArgs& f = a.f;
    f.X = (const bf16_t*)X; f.ldx = ldx; f.M = M; f.K = K;
    f.W = (const bf16_t*)W; f.bias = bias; f.bias_f32 = bias_dtype == TM_F32;
    a.rows = rows;
    a.n_strips = (N + rows - 1) / rows;
    a.N = N; a.parts = parts;
    int kparts = 1, ks = 0, us = 0;
    stream_plain_shape(N, K, &kparts, &ks, &us);
    return launch_stream<ST_EPI_PLAIN>(a, (N + 31) / 32, stream, kparts, ks, us);
}
