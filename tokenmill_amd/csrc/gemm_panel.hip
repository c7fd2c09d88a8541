// The q|k|v product of a decode step with 9 to 64 tokens of a narrow model (a width of at most 1,024), with
// its layer's own epilogue (bias + rotary + cache write), behind a norm that ran as a kernel of its own.
//
// With this many rows a block cannot afford to compute the norm itself (every block would read all
// rows of the residual stream), and it cannot read its activations from the cache k-step by k-step
// (a wavefront would wait for the cache at every step, and all blocks ask for the same lines at once).
// So the normed input x [M, K] (bfloat16, a few tens of KB) is copied once per block into LDS, each
// block starting at another row so that the blocks do not all want the same line at the same time,
// while the block's matrix strips are already on their way from HBM; then the four wavefronts, which
// split K, multiply their strips with all row tiles of x out of LDS, their partial sums are added
// through LDS in wavefront order, and wavefront t does the epilogue of row tile t.
//
// The matrix is read in strip order (tm_pack_layout in api.h) like the decode kernels for fewer rows,
// the strips pair up the same way (the two halves of a rotary pair), and everything is
// rounded where the unfused path stores a bfloat16 tensor, so both paths agree up to the order of
// 32-bit sums (reference src/infer/model/layers.py:142-147,60-64,163-164; src/infer/kv/paged_cache.py:40-43).
// Which k goes to which wavefront depends on K alone: a token's result does not depend on how many
// other tokens the step holds.
#include "common.h"
#include "api.h"
#include "fused_common.h"

#define PN_WAVES 4
#define PN_KCH 8            // k-steps a wavefront holds: K <= 4 * 8 * 32 = 1024

// NT: 16-row tiles of x a block takes (1..4). ROWS: rows of a matrix strip (16 or 8).
template <int ROWS, int NT>
__global__ __launch_bounds__(64 * PN_WAVES, 1) void gemm_panel_kernel(const FusedArgs a, const int n_units) {
    extern __shared__ __align__(16) unsigned char smem_raw[];
    // the tokens of this block: all of them, or (gridDim.y > 1) the NT tiles from tok0 on
    const int tok0 = blockIdx.y * (NT * 16);
    const int K = a.K, M = a.M - tok0 < NT * 16 ? a.M - tok0 : NT * 16;
    const int xstride = K + FD_XPAD;
    bf16_t* xs = (bf16_t*)smem_raw;                                  // [NT * 16][K + FD_XPAD]
    float* red = (float*)(smem_raw + (size_t)NT * 16 * xstride * sizeof(bf16_t));   // [waves][2][NT][64][5]
    auto red_at = [&](int w, int ab, int t, int l) { return red + ((((size_t)w * 2 + ab) * NT + t) * 64 + l) * 5; };
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / TM_WAVE), lane = threadIdx.x % TM_WAVE;
    const int r = lane % 16, g = lane / 16;

    const int ksteps = (K + 31) / 32;
    const int per = (ksteps + PN_WAVES - 1) / PN_WAVES;
    const int ks0 = wave * per;
    const int ks1 = ks0 + per < ksteps ? ks0 + per : ksteps;
    int u = blockIdx.x;
    FusedUnit cu = fused_unit_of<FD_EPI_QKV, ROWS>(a, u, r);

    // This wavefront's epilogue is that of row tile `wave`: token 16 wave + r. Its position comes by
    // scalar loads (addresses the same in every lane), which are counted apart from the vector loads.
    const int tile = wave;
    const int tok = 16 * tile + r;
    const bool epi_wave = tile < NT;
    const bool epi_lane = epi_wave && tok < M && 4 * g < ROWS;
    int tok_pos = 0;
    if (epi_wave) {
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const int ti = 16 * tile + i;
            const int pos_i = a.positions[tok0 + (ti < M ? ti : 0)];
            tok_pos = r == i ? pos_i : tok_pos;
        }
    }

    // the matrix first: it has the longest way
    constexpr int FRAG = 32 * ROWS;
    const int lane_off = (g * ROWS + (r < ROWS ? r : 0)) * 8;
    auto strip_pointer = [&](int strip) { return a.W + (size_t)strip * ksteps * FRAG + lane_off; };
    const bf16_t* wA = strip_pointer(cu.sA);
    const bf16_t* wB = strip_pointer(cu.sB);
    FFrag fa[PN_KCH], fb[PN_KCH];
    auto load_group = [&]() {
#pragma unroll
        for (int j = 0; j < PN_KCH; ++j) {
            const bool in = cu.rows_ok && ks0 + j < ks1;
            fa[j].u = in ? *(const u32x4_t*)(wA + (size_t)(ks0 + j) * FRAG) : u32x4_t{0, 0, 0, 0};
            fb[j].u = in ? *(const u32x4_t*)(wB + (size_t)(ks0 + j) * FRAG) : u32x4_t{0, 0, 0, 0};
        }
    };
    load_group();

    // what the epilogue needs from memory, asked for now and kept as loaded (every lane loads, from
    // entries that exist; the lanes without an epilogue do not look at what came)
    struct EpilogueInputs {
        f32x4_t bias_f[2];
        uint2 bias_h[2];
        f32x4_t cos, sin;
        int slot;
    };
    const int bias_kind = !a.bias ? 0 : (a.bias_f32 ? 2 : 1);
    auto epilogue_inputs = [&](const FusedUnit& t) {
        EpilogueInputs e;
        const int ge = 4 * g < ROWS ? 4 * g : 0;
        const int ia = t.nA + ge, ib = t.nB + ge;
        if (bias_kind == 2) {
            e.bias_f[0] = *(const f32x4_t*)((const float*)a.bias + ia);
            e.bias_f[1] = *(const f32x4_t*)((const float*)a.bias + ib);
        } else if (bias_kind == 1) {
            e.bias_h[0] = *(const uint2*)((const bf16_t*)a.bias + ia);
            e.bias_h[1] = *(const uint2*)((const bf16_t*)a.bias + ib);
        }
        const int jt = t.head < a.H + a.KVH ? t.jt : 0;          // value heads have no rotary row
        const size_t at = (size_t)tok_pos * (a.D / 2) + ROWS * jt + ge;
        e.cos = *(const f32x4_t*)(a.cos_t + at);
        e.sin = *(const f32x4_t*)(a.sin_t + at);
        e.slot = (a.slots ? a.slots : a.positions)[tok0 + (tok < M ? tok : 0)];
        return e;
    };
    EpilogueInputs e_next = epilogue_inputs(cu);

    // x into LDS, 16 bytes a thread and load, every load of a thread in flight at once (K <= 1024: at most
    // 8 NT of them); block b starts at row b
    {
        const int per_row = K / 8;
        const int pieces = M * per_row;
        const int row_shift = blockIdx.x % M;
        constexpr int XL = 8 * NT;
        u32x4_t v[XL];
#pragma unroll
        for (int i = 0; i < XL; ++i) {
            const int p = threadIdx.x + i * 64 * PN_WAVES;
            const int pc = p < pieces ? p : 0;
            int row = pc / per_row + row_shift;
            row = row < M ? row : row - M;
            v[i] = *(const u32x4_t*)(a.X + (size_t)(tok0 + row) * a.ldx + (pc % per_row) * 8);
        }
#pragma unroll
        for (int i = 0; i < XL; ++i) {
            const int p = threadIdx.x + i * 64 * PN_WAVES;
            if (p < pieces) {
                int row = p / per_row + row_shift;
                row = row < M ? row : row - M;
                *(u32x4_t*)(xs + (size_t)row * xstride + (p % per_row) * 8) = v[i];
            }
        }
        // rows M .. 16 NT - 1 of x stay as they are: they only feed result columns of tokens that do
        // not exist, which no lane stores
    }
    __syncthreads();

    for (;;) {
        const EpilogueInputs e = e_next;
        f32x4_t accA[NT], accB[NT];
#pragma unroll
        for (int t = 0; t < NT; ++t) {
            accA[t] = f32x4_t{0.f, 0.f, 0.f, 0.f};
            accB[t] = f32x4_t{0.f, 0.f, 0.f, 0.f};
        }
#pragma unroll
        for (int j = 0; j < PN_KCH; ++j) {
            const int k = (ks0 + j) * 32 + 8 * g;
            const bool in = ks0 + j < ks1 && k < K;
#pragma unroll
            for (int t = 0; t < NT; ++t) {
                FFrag xf;
                xf.u = in ? *(const u32x4_t*)(xs + (size_t)(16 * t + r) * xstride + k) : u32x4_t{0, 0, 0, 0};
                accA[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fa[j].b, xf.b, accA[t], 0, 0, 0);
                accB[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fb[j].b, xf.b, accB[t], 0, 0, 0);
            }
        }
        // partial sums of the wavefronts, added in wavefront order by the wavefront that owns the tile
#pragma unroll
        for (int t = 0; t < NT; ++t)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                red_at(wave, 0, t, lane)[i] = accA[t][i];
                red_at(wave, 1, t, lane)[i] = accB[t][i];
            }
        __syncthreads();

        // the next unit's matrix goes out before this unit's epilogue
        const int un = u + gridDim.x;
        const bool more = un < n_units;
        const FusedUnit done = cu;
        if (more) {
            cu = fused_unit_of<FD_EPI_QKV, ROWS>(a, un, r);
            wA = strip_pointer(cu.sA);
            wB = strip_pointer(cu.sB);
            load_group();
            e_next = epilogue_inputs(cu);
        }

        if (epi_lane) {
            float sA[4], sB[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                float va = red_at(0, 0, tile, lane)[i], vb = red_at(0, 1, tile, lane)[i];
#pragma unroll
                for (int w = 1; w < PN_WAVES; ++w) {
                    va += red_at(w, 0, tile, lane)[i];
                    vb += red_at(w, 1, tile, lane)[i];
                }
                sA[i] = va;
                sB[i] = vb;
            }
            // lane: token tok, rows nA + 4g + i and nB + 4g + i
            f32x4_t bA = {0.f, 0.f, 0.f, 0.f}, bB = {0.f, 0.f, 0.f, 0.f};
            if (bias_kind == 2) {
                bA = e.bias_f[0];
                bB = e.bias_f[1];
            } else if (bias_kind == 1) {
                bA = f32x4_t{__uint_as_float(e.bias_h[0].x << 16), __uint_as_float(e.bias_h[0].x & 0xffff0000u),
                             __uint_as_float(e.bias_h[0].y << 16), __uint_as_float(e.bias_h[0].y & 0xffff0000u)};
                bB = f32x4_t{__uint_as_float(e.bias_h[1].x << 16), __uint_as_float(e.bias_h[1].x & 0xffff0000u),
                             __uint_as_float(e.bias_h[1].y << 16), __uint_as_float(e.bias_h[1].y & 0xffff0000u)};
            }
            float xA[4], xB[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                xA[i] = fd_round(sA[i] + bA[i]);
                xB[i] = fd_round(sB[i] + bB[i]);
            }
            const int slot = a.slots ? e.slot : -1;
            if (done.head < a.H + a.KVH) {
                const int half = a.D / 2;
                const int j0 = ROWS * done.jt + 4 * g;                       // pair index of element 0
                float y1[4], y2[4];
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    rotate_pair(xA[i], xB[i], e.cos[i], e.sin[i], y1[i], y2[i]);
                }
                bf16_t* dst = nullptr;
                if (done.head < a.H)
                    dst = a.q_out + (size_t)(tok0 + tok) * a.H * a.D + (size_t)done.head * a.D + j0;
                else if (slot >= 0)
                    dst = a.k_pool + ((size_t)slot * a.KVH + (done.head - a.H)) * a.D + j0;
                if (dst) {
                    *(uint2*)dst = uint2{fd_pack(y1[0], y1[1]), fd_pack(y1[2], y1[3])};
                    *(uint2*)(dst + half) = uint2{fd_pack(y2[0], y2[1]), fd_pack(y2[2], y2[3])};
                }
            } else if (slot >= 0) {
                const int vh = done.head - a.H - a.KVH;
                const int pg = slot >> a.page_shift, in_page = slot & ((1 << a.page_shift) - 1);
                const int d0 = 2 * ROWS * done.jt + 4 * g;
                bf16_t* dst = a.v_pool + ((((size_t)pg * a.KVH + vh) * a.D + d0) << a.page_shift) + in_page;
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    dst[(size_t)i << a.page_shift] = f32_to_bf16(xA[i]);
                    dst[(size_t)(i + ROWS) << a.page_shift] = f32_to_bf16(xB[i]);
                }
            }
        }
        if (!more) break;
        __syncthreads();                                                 // the sums have been read: red is free again
        u = un;
    }
}

static int panel_lds_bytes(int tiles, int K) {
    return tiles * 16 * (K + FD_XPAD) * (int)sizeof(bf16_t) + PN_WAVES * 2 * tiles * 64 * 5 * (int)sizeof(float);
}

// Can the panel products take M tokens of width K? (x and the partial sums must fit a block's LDS, and
// a wavefront holds its whole share of K in registers.)
extern "C" int tm_gemm_panel_fits(int M, int K) {
    if (M <= 0 || M > 64 || K <= 0 || (K % 8) || K > PN_WAVES * PN_KCH * 32) return 0;
    return panel_lds_bytes((M + 15) / 16, K) + 1024 <= 160 * 1024 ? 1 : 0;
}

template <int ROWS, int NT>
static int launch_panel_tiles(const FusedArgs& a, int n_units, int blocks, int row_parts, hipStream_t stream) {
    const int lds = panel_lds_bytes(NT, a.K);
    static int raised = 0;          // largest dynamic LDS size this kernel has been allowed so far
    if (lds > 48 * 1024 && lds > raised) {
        if (hipFuncSetAttribute((const void*)gemm_panel_kernel<ROWS, NT>, hipFuncAttributeMaxDynamicSharedMemorySize,
                                lds) != hipSuccess)
            return TM_ERR_LAUNCH;
        raised = lds;
    }
    gemm_panel_kernel<ROWS, NT><<<dim3(blocks, row_parts), 64 * PN_WAVES, lds, stream>>>(a, n_units);
    TM_CHECK_LAUNCH();
    return TM_OK;
}

template <int ROWS>
static int launch_panel(const FusedArgs& a, int n_units, hipStream_t stream) {
    // one block a CU (x fills most of its LDS): beyond that a block takes several units after one copy of x. With
    // fewer units than half the chip's CUs the tiles of tokens are dealt to groups of blocks (the matrix is small:
    // read again from the cache), as many groups as still give at most a block a CU.
    const int blocks = n_units < 256 ? n_units : 256;
    const int all_tiles = (a.M + 15) / 16, room = 256 / blocks;
    int row_parts = room < all_tiles ? room : all_tiles;
    const int tiles = (all_tiles + row_parts - 1) / row_parts;
    row_parts = (all_tiles + tiles - 1) / tiles;
    switch (tiles) {
        case 1: return launch_panel_tiles<ROWS, 1>(a, n_units, blocks, row_parts, stream);
        case 2: return launch_panel_tiles<ROWS, 2>(a, n_units, blocks, row_parts, stream);
        case 3: return launch_panel_tiles<ROWS, 3>(a, n_units, blocks, row_parts, stream);
        default: return launch_panel_tiles<ROWS, 4>(a, n_units, blocks, row_parts, stream);
    }
}

static bool panel_common_ok(int M, int K, const void* X, int ldx, const void* W) {
    return tm_gemm_panel_fits(M, K) && ldx >= K && (ldx % 8) == 0 && X && W && ((uintptr_t)X % 16) == 0 &&
           ((uintptr_t)W % 16) == 0;
}

// q_out[M, H*D], K cache, V cache <- rope(X Wqkv^T + b) for up to 64 tokens; X bfloat16 [M, K] (rows ldx apart)
// is the normed input. W, bias, tables and pools as for tm_fused_norm_qkv_rope.
extern "C" int tm_panel_qkv_rope(const void* X, int ldx, int M, int K, const void* W, const void* bias, int bias_dtype,
                                 void* q_out, int H, int KVH, int D, const float* cos_t, const float* sin_t,
                                 const int* positions, const int* slots, void* k_pool, void* v_pool, int page,
                                 hipStream_t stream) {
    if (M == 0) return TM_OK;
    if (!panel_common_ok(M, K, X, ldx, W) || H <= 0 || KVH <= 0 || D <= 0 || D % 32 || !cos_t || !sin_t || !positions ||
        !q_out || ((uintptr_t)q_out % 8) || page <= 0 || (page & (page - 1)))
        return TM_ERR_ARG;
    if (slots && (!k_pool || !v_pool)) return TM_ERR_ARG;
    if (bias && ((uintptr_t)bias % 16)) return TM_ERR_ARG;
    FusedArgs a{};
    a.X = (const bf16_t*)X; a.ldx = ldx; a.M = M; a.K = K;
    a.W = (const bf16_t*)W; a.bias = bias; a.bias_f32 = bias_dtype == TM_F32;
    a.q_out = (bf16_t*)q_out; a.H = H; a.KVH = KVH; a.D = D; a.cos_t = cos_t; a.sin_t = sin_t;
    a.positions = positions; a.slots = slots; a.k_pool = (bf16_t*)k_pool; a.v_pool = (bf16_t*)v_pool;
    a.page_shift = 0;
    while ((1 << a.page_shift) < page) ++a.page_shift;
    const int units16 = (H + 2 * KVH) * (D / 32);
    if (tm_fused_qkv_strip_rows(H, KVH, D, K) == 16) return launch_panel<16>(a, units16, stream);
    return launch_panel<8>(a, 2 * units16, stream);
}
