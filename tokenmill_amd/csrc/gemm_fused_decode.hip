// Decode-step products with the RMSNorm in front and the layer's own epilogue behind, for at most 16
// tokens (bfloat16 weights and activations, 32-bit residual stream and sums).
//
//   x = weight * round(resid * rsqrt(mean(resid^2) + eps))     (reference src/infer/model/layers.py:41-44)
//   is computed by every block into LDS (a few KB of L2 reads against a matrix streamed from HBM), then
//
//   QKV epilogue  : y = x Wqkv^T + b; q and k rotated by their token's position; q to a dense
//                   [M, H*D] buffer, k and v straight to their cache slots
//                   (reference src/infer/model/layers.py:142-147,60-64; src/infer/kv/paged_cache.py:40-43)
//   SiLU epilogue : act = silu(x Wgate^T) * (x Wup^T)          (reference src/infer/model/layers.py:163-164)
//
// A block owns two strips of 16 matrix rows whose results meet in the epilogue (the two halves of a
// rotary pair; gate and up). Its four wavefronts split K; partial sums are added through LDS in
// wavefront order. Everything is rounded where the unfused path stores a bfloat16 tensor, so both
// paths agree up to the order of 32-bit sums.
#include "common.h"
#include "api.h"
#include "fused_common.h"

// ROWS: rows of a strip (16 or 8). Short strips leave rows of the MFMA tile empty (their lanes load
// nothing) and double the number of units, for matrices that would otherwise give fewer blocks
// than the chip has CUs. A block takes the units u = blockIdx.x, + gridDim.x, ...: the norm is
// computed once and serves all of them.
// PIPE: a wavefront's K range is longer than one group of FD_KCH steps, and two register groups take
// turns so that loads are always in flight (more registers; not worth them when one group holds it all).
// WAVES: wavefronts of a block (4, or 8 for a long K: they split K, and the norm's rows, between them).
template <int EPI, int ROWS, bool PIPE, int WAVES>
__global__ __launch_bounds__(64 * WAVES, WAVES == 4 ? 2 : 1) void fused_norm_gemm_kernel(const FusedArgs a,
                                                                                        const int n_units) {
    constexpr int KCH = PIPE ? FD_KCH_PIPE : FD_KCH;
    constexpr int THREADS = 64 * WAVES;
    extern __shared__ __align__(16) unsigned char smem_raw[];
    bf16_t* xs = (bf16_t*)smem_raw;                                  // [4, 8 or 16 rows][K + FD_XPAD]
    __shared__ float red[WAVES][2][64][4 + 1];
    const int K = a.K, M = a.M;
    const int xstride = K + FD_XPAD;
    const int wave = threadIdx.x / TM_WAVE, lane = threadIdx.x % TM_WAVE;
    const int r = lane % 16, g = lane / 16;

    auto unit_of = [&](int u) { return fused_unit_of<EPI, ROWS>(a, u, r); };

    const int ksteps = (K + 31) / 32;
    const int per = (ksteps + WAVES - 1) / WAVES;
    const int ks0 = wave * per;
    const int ks1 = ks0 + per < ksteps ? ks0 + per : ksteps;
    int u = blockIdx.x;
    FusedUnit cu = unit_of(u);
    // The matrix comes in strip order: the 16-byte piece of lane (r, g) for k-step ks of strip s lies at
    // ((s * ksteps + ks) * 4 + g) * ROWS + r pieces, so a wavefront's load is one run of ROWS * 64 bytes
    // and a strip is one run of memory; rows and k beyond the matrix are zeros there.
    constexpr int FRAG = 32 * ROWS;                                  // bfloat16 values of a (strip, k-step)
    const int lane_off = (g * ROWS + (r < ROWS ? r : 0)) * 8;
    auto strip_pointer = [&](int strip) { return a.W + (size_t)strip * ksteps * FRAG + lane_off; };
    const bf16_t* wA = strip_pointer(cu.sA);
    const bf16_t* wB = strip_pointer(cu.sB);
    auto load_group = [&](auto& ga, auto& gb, int base, bool rows_ok) {
#pragma unroll
        for (int j = 0; j < KCH; ++j) {
            const bool in = rows_ok && base + j < ks1;
            ga[j].u = in ? *(const u32x4_t*)(wA + (size_t)(base + j) * FRAG) : u32x4_t{0, 0, 0, 0};
            gb[j].u = in ? *(const u32x4_t*)(wB + (size_t)(base + j) * FRAG) : u32x4_t{0, 0, 0, 0};
        }
    };
    // What the epilogue will need from memory is asked for long before it is used, and in an order
    // that lets the long loads go first in effect: loads come back in the order they were issued, so
    // the token's position and cache slot (a few bytes from the cache, and the rotary row's address
    // hangs on the position) are asked for BEFORE the matrix, and can be waited for while the matrix
    // is still on its way; the bias and the rotary row follow the matrix and are not looked at (not
    // even widened) until the epilogue.
    const int tok = r;                                               // the epilogue's token of this lane
    const bool epi_lane = wave == 0 && tok < M && 4 * g < ROWS;
    // The positions are read at addresses that are the same in every lane, which makes them scalar
    // loads: those are counted apart from the vector loads, so waiting for them does not wait for the
    // matrix. Each lane then picks its token's.
    int tok_pos = 0;
    if constexpr (EPI == FD_EPI_QKV) {
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const int pos_i = a.positions[i < M ? i : 0];
            tok_pos = tok == i ? pos_i : tok_pos;
        }
    }
    __builtin_amdgcn_sched_barrier(0);
    // matrix loads of the first group go out before the norm is computed
    FFrag fa[KCH], fb[KCH], fa2[PIPE ? KCH : 1], fb2[PIPE ? KCH : 1];
    load_group(fa, fb, ks0, cu.rows_ok);
    if constexpr (PIPE) load_group(fa2, fb2, ks0 + KCH, cu.rows_ok);
    __builtin_amdgcn_sched_barrier(0);

    struct EpilogueInputs {
        union {
            f32x4_t f;              // four rows of a strip as loaded: a 32-bit bias, or
            uint2 h;                // a bfloat16 one (only the kind there is gets loaded and read)
        } bias[2];
        f32x4_t cos, sin;
        int slot;                   // (every lane loads, the lanes without a token from entry 0; what came is
    };                              // looked at only where it is meant: a load under a test is waited for where the test ends)
    const int bias_kind = !a.bias ? 0 : (a.bias_f32 ? 2 : 1);       // the same for every lane
    auto epilogue_inputs = [&](const FusedUnit& t) {
        EpilogueInputs e;
        if constexpr (EPI == FD_EPI_QKV) {
            // lanes beyond the strip's rows (4 g >= ROWS) have no epilogue: they read what group 0 reads
            const int ge = 4 * g < ROWS ? 4 * g : 0;
            const int ia = t.nA + ge, ib = t.nB + ge;               // (the bias is 16-byte aligned)
            if (bias_kind == 2) {
                e.bias[0].f = *(const f32x4_t*)((const float*)a.bias + ia);
                e.bias[1].f = *(const f32x4_t*)((const float*)a.bias + ib);
            } else if (bias_kind == 1) {
                e.bias[0].h = *(const uint2*)((const bf16_t*)a.bias + ia);
                e.bias[1].h = *(const uint2*)((const bf16_t*)a.bias + ib);
            }
            // value heads have no rotary row: they read that of the first pair and do not use it
            const int jt = t.head < a.H + a.KVH ? t.jt : 0;
            const size_t at = (size_t)tok_pos * (a.D / 2) + ROWS * jt + (4 * g < ROWS ? 4 * g : 0);
            e.cos = *(const f32x4_t*)(a.cos_t + at);
            e.sin = *(const f32x4_t*)(a.sin_t + at);
            e.slot = (a.slots ? a.slots : a.positions)[tok < M ? tok : 0];
        }
        return e;
    };
    EpilogueInputs e_next = epilogue_inputs(cu);

    // x = norm(resid) into LDS. A row is shared by TPR threads of one wavefront (256 threads: 16 rows x 16
    // threads, 8 x 32, or 4 x 64); each keeps its first FD_RC vectors in registers between the two passes.
    const int mpad = fused_rows(M);
    {
        const int tpr = THREADS / mpad < TM_WAVE ? THREADS / mpad : TM_WAVE;
        const int row = threadIdx.x / tpr, sub = threadIdx.x % tpr;
        bf16_t* xrow = xs + (size_t)row * xstride;
        const int step = 4 * tpr;
        if (row < M) {
            const float* src = a.resid + (size_t)row * K;
            // The norm's weights of the first group are asked for with the row itself: they depend on
            // nothing, and asked for after the sum of squares they would cost a trip to memory of their
            // own. (Two kinds of loads behind one run-time test would each be waited for singly: the
            // test on the weights' type stands outside the loops.)
            const bool w16 = !a.norm_w_f32;
            auto widen = [](const uint2 wv) {
                return f32x4_t{__uint_as_float(wv.x << 16), __uint_as_float(wv.x & 0xffff0000u),
                               __uint_as_float(wv.y << 16), __uint_as_float(wv.y & 0xffff0000u)};
            };
            uint2 wraw[FD_RC];
            if (w16) {
#pragma unroll
                for (int j = 0; j < FD_RC; ++j) {
                    const int c = sub * 4 + j * step;
                    wraw[j] = c < K ? *(const uint2*)((const bf16_t*)a.norm_w + c) : uint2{0u, 0u};
                }
            }
            f32x4_t cache[FD_RC];
            float ss = 0.f;
#pragma unroll
            for (int j = 0; j < FD_RC; ++j) {
                const int c = sub * 4 + j * step;
                cache[j] = c < K ? *(const f32x4_t*)(src + c) : f32x4_t{0.f, 0.f, 0.f, 0.f};
                ss += cache[j][0] * cache[j][0] + cache[j][1] * cache[j][1] + cache[j][2] * cache[j][2] +
                      cache[j][3] * cache[j][3];
            }
            // the rest of a long row in groups of FD_RC loads that are in flight together
            for (int c0 = sub * 4 + FD_RC * step; c0 < K; c0 += FD_RC * step) {
                f32x4_t v[FD_RC];
#pragma unroll
                for (int j = 0; j < FD_RC; ++j)
                    v[j] = c0 + j * step < K ? *(const f32x4_t*)(src + c0 + j * step) : f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int j = 0; j < FD_RC; ++j)
                    ss += v[j][0] * v[j][0] + v[j][1] * v[j][1] + v[j][2] * v[j][2] + v[j][3] * v[j][3];
            }
            for (int off = 1; off < tpr; off <<= 1) ss += __shfl_xor(ss, off, TM_WAVE);
            const float rs = rsqrtf(ss / (float)K + a.eps);
            auto emit = [&](int c, const f32x4_t v, const f32x4_t w) {
                uint2 pk;
                pk.x = fd_pack(w[0] * fd_round(v[0] * rs), w[1] * fd_round(v[1] * rs));
                pk.y = fd_pack(w[2] * fd_round(v[2] * rs), w[3] * fd_round(v[3] * rs));
                *(uint2*)(xrow + c) = pk;
            };
            {
                f32x4_t w[FD_RC];
                if (w16) {
#pragma unroll
                    for (int j = 0; j < FD_RC; ++j) w[j] = widen(wraw[j]);
                } else {
#pragma unroll
                    for (int j = 0; j < FD_RC; ++j) {
                        const int c = sub * 4 + j * step;
                        w[j] = c < K ? *(const f32x4_t*)((const float*)a.norm_w + c) : f32x4_t{0.f, 0.f, 0.f, 0.f};
                    }
                }
#pragma unroll
                for (int j = 0; j < FD_RC; ++j) {
                    const int c = sub * 4 + j * step;
                    if (c < K) emit(c, cache[j], w[j]);
                }
            }
            // the rest of a long row: the values again and their weights, a group in flight together
            for (int c0 = sub * 4 + FD_RC * step; c0 < K; c0 += FD_RC * step) {
                f32x4_t v[FD_RC], w[FD_RC];
                if (w16) {
                    uint2 raw[FD_RC];
#pragma unroll
                    for (int j = 0; j < FD_RC; ++j) {
                        const bool in = c0 + j * step < K;
                        v[j] = in ? *(const f32x4_t*)(src + c0 + j * step) : f32x4_t{0.f, 0.f, 0.f, 0.f};
                        raw[j] = in ? *(const uint2*)((const bf16_t*)a.norm_w + c0 + j * step) : uint2{0u, 0u};
                    }
#pragma unroll
                    for (int j = 0; j < FD_RC; ++j) w[j] = widen(raw[j]);
                } else {
#pragma unroll
                    for (int j = 0; j < FD_RC; ++j) {
                        const bool in = c0 + j * step < K;
                        v[j] = in ? *(const f32x4_t*)(src + c0 + j * step) : f32x4_t{0.f, 0.f, 0.f, 0.f};
                        w[j] = in ? *(const f32x4_t*)((const float*)a.norm_w + c0 + j * step) : f32x4_t{0.f, 0.f, 0.f, 0.f};
                    }
                }
#pragma unroll
                for (int j = 0; j < FD_RC; ++j)
                    if (c0 + j * step < K) emit(c0 + j * step, v[j], w[j]);
            }
        }
        // rows M..mpad-1 of x stay as they are, and the lanes of tokens beyond mpad read rows below it
        // again: they only feed result columns of tokens that do not exist, which no lane stores
    }
    __syncthreads();

    const bf16_t* xr = xs + (size_t)(r & (mpad - 1)) * xstride + 8 * g;
    f32x4_t accA, accB;
    auto multiply_group = [&](const auto& ga, const auto& gb, int base) {
#pragma unroll
        for (int j = 0; j < KCH; ++j) {
            const int k = (base + j) * 32;
            FFrag xf;
            xf.u = (base + j < ks1 && k + 8 * g < K) ? *(const u32x4_t*)(xr + k) : u32x4_t{0, 0, 0, 0};
            accA = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ga[j].b, xf.b, accA, 0, 0, 0);
            accB = __builtin_amdgcn_mfma_f32_16x16x32_bf16(gb[j].b, xf.b, accB, 0, 0, 0);
        }
    };
    for (;;) {
        const EpilogueInputs e = e_next;                                 // asked for before this unit's products began
        accA = f32x4_t{0.f, 0.f, 0.f, 0.f};
        accB = f32x4_t{0.f, 0.f, 0.f, 0.f};
        if constexpr (PIPE) {
            // fa holds group `base` and fa2 the one after it, loaded or on their way: two groups are
            // always in flight while one is multiplied
            for (int base = ks0; base < ks1; base += 2 * KCH) {
                multiply_group(fa, fb, base);
                if (base + 2 * KCH < ks1) load_group(fa, fb, base + 2 * KCH, cu.rows_ok);
                if (base + KCH >= ks1) break;
                multiply_group(fa2, fb2, base + KCH);
                if (base + 3 * KCH < ks1) load_group(fa2, fb2, base + 3 * KCH, cu.rows_ok);
            }
        } else {
            for (int base = ks0; base < ks1; base += KCH) {
                if (base != ks0) load_group(fa, fb, base, cu.rows_ok);
                multiply_group(fa, fb, base);
            }
        }
        // partial sums of the wavefronts, added in wavefront order
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            red[wave][0][lane][i] = accA[i];
            red[wave][1][lane][i] = accB[i];
        }
        __syncthreads();

        // the next unit's first loads go out before this unit's epilogue
        const int un = u + gridDim.x;
        const bool more = un < n_units;
        const FusedUnit done = cu;
        if (more) {
            cu = unit_of(un);
            wA = strip_pointer(cu.sA);
            wB = strip_pointer(cu.sB);
            load_group(fa, fb, ks0, cu.rows_ok);
            if constexpr (PIPE) load_group(fa2, fb2, ks0 + KCH, cu.rows_ok);
            e_next = epilogue_inputs(cu);
        }

        if (epi_lane) {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                float sa = red[0][0][lane][i], sb = red[0][1][lane][i];
#pragma unroll
                for (int w = 1; w < WAVES; ++w) {
                    sa += red[w][0][lane][i];
                    sb += red[w][1][lane][i];
                }
                accA[i] = sa;
                accB[i] = sb;
            }
            // lane: token r, rows nA + 4g + i and nB + 4g + i
            if (EPI == FD_EPI_SILU) {
                const int col = done.nA + 4 * g;
                if (col < a.I) {
                    float v[4];
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        const float gt = fd_round(accA[i]), up = fd_round(accB[i]);
                        v[i] = gt / (1.f + expf(-gt)) * up;
                    }
                    bf16_t* dst = a.act_out + (size_t)tok * a.I + col;
                    if (col + 4 <= a.I) {
                        *(uint2*)dst = uint2{fd_pack(v[0], v[1]), fd_pack(v[2], v[3])};
                    } else {
                        for (int i = 0; i < 4 && col + i < a.I; ++i) dst[i] = f32_to_bf16(v[i]);
                    }
                }
            } else {
                f32x4_t bA = {0.f, 0.f, 0.f, 0.f}, bB = {0.f, 0.f, 0.f, 0.f};
                if (bias_kind == 2) {
                    bA = e.bias[0].f;
                    bB = e.bias[1].f;
                } else if (bias_kind == 1) {
                    bA = f32x4_t{__uint_as_float(e.bias[0].h.x << 16), __uint_as_float(e.bias[0].h.x & 0xffff0000u),
                                 __uint_as_float(e.bias[0].h.y << 16), __uint_as_float(e.bias[0].h.y & 0xffff0000u)};
                    bB = f32x4_t{__uint_as_float(e.bias[1].h.x << 16), __uint_as_float(e.bias[1].h.x & 0xffff0000u),
                                 __uint_as_float(e.bias[1].h.y << 16), __uint_as_float(e.bias[1].h.y & 0xffff0000u)};
                }
                float xA[4], xB[4];
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    xA[i] = fd_round(accA[i] + bA[i]);
                    xB[i] = fd_round(accB[i] + bB[i]);
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
                        dst = a.q_out + (size_t)tok * a.H * a.D + (size_t)done.head * a.D + j0;
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
        }
        if (!more) break;
        __syncthreads();                                                 // the sums have been read: red is free again
        u = un;
    }
}

static int fused_lds_bytes(int M, int K) { return fused_rows(M) * (K + FD_XPAD) * (int)sizeof(bf16_t); }

template <int EPI, int ROWS, bool PIPE, int WAVES>
static int launch_fused_shape(const FusedArgs& a, int n_units, int blocks, hipStream_t stream) {
    const int lds = fused_lds_bytes(a.M, a.K);
    if (lds + (int)sizeof(float) * WAVES * 2 * 64 * 5 + 1024 > 160 * 1024) return TM_ERR_ARG;
    static int raised = 0;          // largest dynamic LDS size this kernel has been allowed so far
    if (lds > 48 * 1024 && lds > raised) {
        if (hipFuncSetAttribute((const void*)fused_norm_gemm_kernel<EPI, ROWS, PIPE, WAVES>,
                                hipFuncAttributeMaxDynamicSharedMemorySize, lds) != hipSuccess)
            return TM_ERR_LAUNCH;
        raised = lds;
    }
    fused_norm_gemm_kernel<EPI, ROWS, PIPE, WAVES><<<blocks, 64 * WAVES, lds, stream>>>(a, n_units);
    TM_CHECK_LAUNCH();
    return TM_OK;
}

// A long K gets 8 wavefronts a block (shorter K ranges, a faster norm); whether a wavefront's range
// needs more than one register group of loads decides the pipelined variant.
template <int EPI, int ROWS>
static int launch_fused(const FusedArgs& a, int n_units, int blocks, hipStream_t stream) {
    const int ksteps = (a.K + 31) / 32;
    if (a.K >= 2048) {
        return (ksteps + 7) / 8 > FD_KCH ? launch_fused_shape<EPI, ROWS, true, 8>(a, n_units, blocks, stream)
                                         : launch_fused_shape<EPI, ROWS, false, 8>(a, n_units, blocks, stream);
    }
    return (ksteps + 3) / 4 > FD_KCH ? launch_fused_shape<EPI, ROWS, true, 4>(a, n_units, blocks, stream)
                                     : launch_fused_shape<EPI, ROWS, false, 4>(a, n_units, blocks, stream);
}

static bool fused_common_ok(int M, int K, const void* resid, const void* W) {
    return M > 0 && M <= 16 && K > 0 && K % 8 == 0 && ((uintptr_t)resid % 16) == 0 && ((uintptr_t)W % 16) == 0;
}

// Rows of a strip of the packed q|k|v matrix that tm_fused_norm_qkv_rope reads: strips of 16 rows where
// they give the chip enough blocks, else of 8; a long K runs one block of 8 wavefronts a CU, and more
// blocks than CUs would mean a second round for a few of them.
extern "C" int tm_fused_qkv_strip_rows(int H, int KVH, int D, int K) {
    const int units16 = (H + 2 * KVH) * (D / 32);
    const bool one_block_a_cu = K >= 2048;
    return (units16 >= 256 || (one_block_a_cu && units16 >= 128)) ? 16 : 8;
}

// q_out[M, H*D], K cache, V cache <- rope(norm(resid) Wqkv^T + b).  Needs M <= 16, D % 32 == 0, a
// rotary table over the whole head, page a power of two. W: the [(H + 2 KVH) D, K] matrix packed in
// strips of tm_fused_qkv_strip_rows(H, KVH, D, K) rows.
extern "C" int tm_fused_norm_qkv_rope(const float* resid, const void* norm_w, int norm_w_dtype, float eps, int M,
                                      int K, const void* W, const void* bias, int bias_dtype, void* q_out, int H,
                                      int KVH, int D, const float* cos_t, const float* sin_t, const int* positions,
                                      const int* slots, void* k_pool, void* v_pool, int page, hipStream_t stream) {
    if (M == 0) return TM_OK;
    if (!fused_common_ok(M, K, resid, W) || H <= 0 || KVH <= 0 || D <= 0 || D % 32 || !cos_t || !sin_t || !positions ||
        !q_out || ((uintptr_t)q_out % 8) || page <= 0 || (page & (page - 1)) || !(eps > 0.f))
        return TM_ERR_ARG;
    if (slots && (!k_pool || !v_pool)) return TM_ERR_ARG;
    if (bias && ((uintptr_t)bias % 16)) return TM_ERR_ARG;          // read four rows at a time
    FusedArgs a{};
    a.resid = resid; a.norm_w = norm_w; a.norm_w_f32 = norm_w_dtype == TM_F32; a.eps = eps; a.M = M; a.K = K;
    a.W = (const bf16_t*)W; a.bias = bias; a.bias_f32 = bias_dtype == TM_F32;
    a.q_out = (bf16_t*)q_out; a.H = H; a.KVH = KVH; a.D = D; a.cos_t = cos_t; a.sin_t = sin_t;
    a.positions = positions; a.slots = slots; a.k_pool = (bf16_t*)k_pool; a.v_pool = (bf16_t*)v_pool;
    a.page_shift = 0;
    while ((1 << a.page_shift) < page) ++a.page_shift;
    const int units16 = (H + 2 * KVH) * (D / 32);
    if (tm_fused_qkv_strip_rows(H, KVH, D, K) == 16) return launch_fused<FD_EPI_QKV, 16>(a, units16, units16, stream);
    return launch_fused<FD_EPI_QKV, 8>(a, 2 * units16, 2 * units16, stream);
}

// act[M, I] <- silu(norm(resid) Wg^T) * (norm(resid) Wu^T).  Needs M <= 16. W: Wg [I, K] and Wu [I, K]
// each packed in strips of 16 rows, Wu behind Wg.
extern "C" int tm_fused_norm_gate_up_silu(const float* resid, const void* norm_w, int norm_w_dtype, float eps, int M,
                                          int K, const void* W, void* act_out, int I, hipStream_t stream) {
    if (M == 0) return TM_OK;
    if (!fused_common_ok(M, K, resid, W) || I <= 0 || !act_out || ((uintptr_t)act_out % 8) || (I % 4) || !(eps > 0.f))
        return TM_ERR_ARG;
    FusedArgs a{};
    a.resid = resid; a.norm_w = norm_w; a.norm_w_f32 = norm_w_dtype == TM_F32; a.eps = eps; a.M = M; a.K = K;
    a.W = (const bf16_t*)W; a.act_out = (bf16_t*)act_out; a.I = I;
    // One round of blocks, every block with the same number of units (as few as leave at most a block a CU), after one
    // norm for all of them: the 0.5B shape's 304 units as 152 blocks of two (a decode step of 8 requests 0.980 to
    // 0.960 ms against 304 blocks of one, of which some CUs held two; 256 blocks of one or two: 0.980), the 7B
    // shape's 1,184 as 237 blocks of five (the same as 256 blocks of four or five).
    const int units = (I + 15) / 16;
    a.up_strip0 = units;
    const int per_block = (units + 255) / 256;
    return launch_fused<FD_EPI_SILU, 16>(a, units, (units + per_block - 1) / per_block, stream);
}
