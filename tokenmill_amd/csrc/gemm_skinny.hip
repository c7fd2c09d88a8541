// C[M, N] = A[M, K] * W[N, K]^T (+ bias) for few rows (M <= 64) on MFMA, bfloat16 in, 32-bit sums.
//
// With so few rows the product is bound by reading W once. Each wavefront streams a strip of 16
// rows of W (16-byte loads straight into the MFMA A operand: 16 rows x 32 k per instruction) and
// multiplies it with all M activations rows (B operand, 16 tokens per tile). The result tile holds,
// per lane, four consecutive output features of one token.
//
//   split mode : the WAVES wavefronts of a block share one strip and split K between them; their
//                partial sums are added through LDS in wavefront order (for matrices with few rows,
//                so that enough wavefronts are in flight).
//   row mode   : each of the 4 wavefronts of a block has a strip of its own (matrices with many
//                rows, such as the output head).
//
// The K range of each wavefront and the order of all additions depend only on K and the mode,
// never on M: a token's result does not depend on how many other tokens the call holds.
// Fused epilogues: bias; silu(gate) * up for a stacked [gate; up] matrix (reference
// src/infer/model/layers.py:163-164), with gate and up rounded to bfloat16 first as if stored.
//
// The matrix is read row-major [N, K], or (decode steps, at most 16 tokens) in strip order: the
// 16-byte piece of lane (r, g) for k-step ks of strip s lies at ((s * ksteps + ks) * 4 + g) * ROWS + r
// pieces, so that a wavefront's load is one run of ROWS * 64 bytes instead of ROWS pieces a row
// apart (measured on an MI355X: 15% more bytes a second from HBM). Both give the same bits.
#include "common.h"
#include "api.h"

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));

union Frag {
    u32x4_t u;
    bf16x8_t b;
};

__device__ __forceinline__ Frag load_frag(const bf16_t* row, int k, int K, bool row_ok) {
    Frag f;
    if (row_ok && k < K)
        f.u = *(const u32x4_t*)(row + k);
    else
        f.u = u32x4_t{0, 0, 0, 0};
    return f;
}

template <typename TC>
__device__ __forceinline__ void store4(TC* dst, const float v[4], int n_left);

template <>
__device__ __forceinline__ void store4<float>(float* dst, const float v[4], int n_left) {
    if (n_left >= 4 && ((uintptr_t)dst % 16) == 0) {
        *(f32x4_t*)dst = f32x4_t{v[0], v[1], v[2], v[3]};
    } else {
        for (int i = 0; i < 4 && i < n_left; ++i) dst[i] = v[i];
    }
}

template <>
__device__ __forceinline__ void store4<bf16_t>(bf16_t* dst, const float v[4], int n_left) {
    if (n_left >= 4 && ((uintptr_t)dst % 8) == 0) {
        uint2 pk;
        pk.x = (uint32_t)f32_to_bf16(v[0]) | ((uint32_t)f32_to_bf16(v[1]) << 16);
        pk.y = (uint32_t)f32_to_bf16(v[2]) | ((uint32_t)f32_to_bf16(v[3]) << 16);
        *(uint2*)dst = pk;
    } else {
        for (int i = 0; i < 4 && i < n_left; ++i) dst[i] = f32_to_bf16(v[i]);
    }
}

__device__ __forceinline__ float bias_at(const void* bias, int bias_f32, int n) {
    return bias_f32 ? ((const float*)bias)[n] : bf16_to_f32(((const bf16_t*)bias)[n]);
}

// NT: tiles of 16 tokens. WAVES: wavefronts per block. SPLIT: they share a strip and split K.
// SILU: W is [2 * N, K] = [gate; up] and the output is silu(gate) * up, N wide.
// ROWS: rows of W in a strip (16, 8 or 4). A short strip leaves rows of the MFMA tile empty (their
// lanes load nothing), which costs nothing here, and gives a matrix with few rows enough strips,
// and so enough blocks, to have loads in flight on every CU of the chip.
// PACKED: W is in strip order, strips of ROWS rows, rows and k beyond the matrix zero-filled; with SILU
// the up rows' strips start at strip `up_strip0` (each half packed by itself).
template <int NT, int WAVES, bool SPLIT, bool SILU, typename TC, int ROWS = 16, bool PACKED = false>
__global__ __launch_bounds__(WAVES * 64) void gemm_skinny_kernel(const bf16_t* __restrict__ A, int lda,
                                                                 const bf16_t* __restrict__ W,
                                                                 const void* __restrict__ bias, int bias_f32,
                                                                 TC* __restrict__ C, int ldc, int M, int N, int K,
                                                                 float* __restrict__ accum, int ldacc,
                                                                 int up_strip0 = 0) {
    constexpr int NACC = SILU ? 2 : 1;
    // k-steps in flight per wavefront (fewer where 16 wavefronts share the register file)
    constexpr int KCH = (WAVES > 4 && SILU && NT > 2) ? 4 : ((WAVES > 4 && NT == 1 && !SILU) ? 12 : ((WAVES > 4 || NT > 2 || SILU) ? 8 : 16));
    __shared__ float red[SPLIT ? WAVES : 1][64][4 + 1];        // one accumulator tile at a time
    const int wave = threadIdx.x / TM_WAVE, lane = threadIdx.x % TM_WAVE;
    const int r = lane % 16, g = lane / 16;
    const int strip = SPLIT ? blockIdx.x : blockIdx.x * WAVES + wave;
    const int n0 = strip * ROWS;
    // K range of this wavefront, in steps of 32
    const int ksteps = (K + 31) / 32;
    int ks0 = 0, ks1 = ksteps;
    if (SPLIT) {
        const int per = (ksteps + WAVES - 1) / WAVES;
        ks0 = wave * per;
        ks1 = ks0 + per < ksteps ? ks0 + per : ksteps;
    }
    constexpr int FRAG = 32 * ROWS;             // packed: bfloat16 values of a (strip, k-step)
    const bool w_ok = r < ROWS && (PACKED || n0 + r < N);
    const bf16_t* wrow;
    const bf16_t* urow = nullptr;
    if constexpr (PACKED) {
        const int lane_off = (g * ROWS + (r < ROWS ? r : 0)) * 8;
        wrow = W + (size_t)strip * ksteps * FRAG + lane_off;
        if (SILU) urow = W + (size_t)(up_strip0 + strip) * ksteps * FRAG + lane_off;
    } else {
        wrow = W + (size_t)(n0 + r) * K + 8 * g;
        if (SILU) urow = W + (size_t)(N + n0 + r) * K + 8 * g;
    }
    // offset of k-step ks from wrow / urow, and how far a lane's eight values may reach
    auto w_at = [&](int ks) { return PACKED ? ks * FRAG : ks * 32; };
    const int w_end = PACKED ? ksteps * FRAG : K - 8 * g;
    const bf16_t* arow[NT];
    bool a_ok[NT];
#pragma unroll
    for (int t = 0; t < NT; ++t) {
        a_ok[t] = 16 * t + r < M;
        arow[t] = A + (size_t)(16 * t + r) * lda + 8 * g;
    }
    f32x4_t acc[NACC][NT];
#pragma unroll
    for (int a = 0; a < NACC; ++a)
#pragma unroll
        for (int t = 0; t < NT; ++t) acc[a][t] = f32x4_t{0.f, 0.f, 0.f, 0.f};
    // What the accumulate epilogue will read is asked for now: it arrives while the matrix streams.
    const int nf = n0 + 4 * g;                  // this lane's output features nf + i (i = 0..3) of token 16t + r
    const bool acc_fast = accum && nf + 4 <= N && (ldacc % 4) == 0 && ((uintptr_t)accum % 16) == 0;
    f32x4_t resid_cur[NT];
    if (acc_fast && (!SPLIT || wave == 0) && 4 * g < ROWS) {
#pragma unroll
        for (int t = 0; t < NT; ++t)
            resid_cur[t] = 16 * t + r < M ? *(const f32x4_t*)(accum + (size_t)(16 * t + r) * ldacc + nf) : f32x4_t{0.f, 0.f, 0.f, 0.f};
    }

    if (n0 < N) {
        // KCH k-steps at a time with every load issued before the first product: a wavefront's whole
        // K range is at most one or two such groups, so it waits for memory once or twice, not per step.
        for (int base = ks0; base < ks1; base += KCH) {
            // With one tile of tokens (decode steps) the activations are asked for first: loads come back
            // in the order they were issued, and these few rows come from the cache long before the
            // matrix arrives from HBM. With more tiles there are no registers for that.
            Frag af[NT == 1 ? KCH : 1], wf[KCH], uf[SILU ? KCH : 1];
            if constexpr (NT == 1) {
#pragma unroll
                for (int j = 0; j < KCH; ++j)
                    af[j] = load_frag(arow[0], (base + j) * 32, K - 8 * g, a_ok[0] && base + j < ks1);
            }
#pragma unroll
            for (int j = 0; j < KCH; ++j) {
                const bool in = base + j < ks1;
                wf[j] = load_frag(wrow, w_at(base + j), w_end, w_ok && in);
                if (SILU) uf[j] = load_frag(urow, w_at(base + j), w_end, w_ok && in);
            }
#pragma unroll
            for (int j = 0; j < KCH; ++j) {
                const bool in = base + j < ks1;
#pragma unroll
                for (int t = 0; t < NT; ++t) {
                    Frag a1;
                    if constexpr (NT == 1) a1 = af[j];
                    else a1 = load_frag(arow[t], (base + j) * 32, K - 8 * g, a_ok[t] && in);
                    acc[0][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[j].b, a1.b, acc[0][t], 0, 0, 0);
                    if (SILU) acc[1][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(uf[j].b, a1.b, acc[1][t], 0, 0, 0);
                }
            }
        }
    }
    if (SPLIT) {
#pragma unroll
        for (int a = 0; a < NACC; ++a)
#pragma unroll
            for (int t = 0; t < NT; ++t) {
#pragma unroll
                for (int i = 0; i < 4; ++i) red[wave][lane][i] = acc[a][t][i];
                __syncthreads();
                if (wave == 0) {
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        float v = red[0][lane][i];
                        for (int w = 1; w < WAVES; ++w) v += red[w][lane][i];
                        acc[a][t][i] = v;
                    }
                }
                __syncthreads();
            }
        if (wave != 0) return;
    }
    if (n0 >= N) return;
    if (4 * g >= ROWS) return;
#pragma unroll
    for (int t = 0; t < NT; ++t) {
        const int tok = 16 * t + r;
        if (tok >= M || nf >= N) continue;
        float v[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            float x = acc[0][t][i];
            if (bias && nf + i < N) x += bias_at(bias, bias_f32, nf + i);
            if (SILU) {
                const float gt = bf16_to_f32(f32_to_bf16(x));
                const float up = bf16_to_f32(f32_to_bf16(acc[1][t][i]));
                x = gt / (1.f + expf(-gt)) * up;
            }
            v[i] = x;
        }
        if (accum) {            // the rounded result goes into the 32-bit residual stream (each element has one owner)
            float* dst = accum + (size_t)tok * ldacc + nf;
            if (acc_fast) {
                f32x4_t cur = resid_cur[t];
#pragma unroll
                for (int i = 0; i < 4; ++i) cur[i] += bf16_to_f32(f32_to_bf16(v[i]));
                *(f32x4_t*)dst = cur;
            } else {
                for (int i = 0; i < 4 && nf + i < N; ++i) dst[i] += bf16_to_f32(f32_to_bf16(v[i]));
            }
        } else {
            store4<TC>(C + (size_t)tok * ldc + nf, v, N - nf);
        }
    }
}

template <int NT, bool SILU, typename TC>
static int launch_skinny(const void* A, int lda, const void* W, const void* bias, int bias_f32, void* C, int ldc,
                         int M, int N, int K, float* accum, int ldacc, hipStream_t stream) {
    const int strips = (N + 15) / 16;
    if (NT == 1 && !SILU && strips < 192) {    // few rows and few tokens: short strips, so that every CU gets a block
        const bool r8 = (N + 7) / 8 >= 192;
        const int n_strips = r8 ? (N + 7) / 8 : (N + 3) / 4;
#define TM_SHORT(WV, RW)                                                                                         \
    gemm_skinny_kernel<1, WV, true, false, TC, RW><<<n_strips, 64 * WV, 0, stream>>>(                            \
        (const bf16_t*)A, lda, (const bf16_t*)W, bias, bias_f32, (TC*)C, ldc, M, N, K, accum, ldacc)
        if (K < 2048) {
            if (r8) TM_SHORT(4, 8); else TM_SHORT(4, 4);
        } else {
            if (r8) TM_SHORT(16, 8); else TM_SHORT(16, 4);
        }
#undef TM_SHORT
        TM_CHECK_LAUNCH();
        return TM_OK;
    }
    if (strips >= 2048) {                      // many rows: a strip per wavefront
        gemm_skinny_kernel<NT, 4, false, SILU, TC><<<(strips + 3) / 4, 256, 0, stream>>>(
            (const bf16_t*)A, lda, (const bf16_t*)W, bias, bias_f32, (TC*)C, ldc, M, N, K, accum, ldacc);
    } else if (strips >= 256 || K < 2048) {    // a block of 4 wavefronts per strip
        gemm_skinny_kernel<NT, 4, true, SILU, TC><<<strips, 256, 0, stream>>>(
            (const bf16_t*)A, lda, (const bf16_t*)W, bias, bias_f32, (TC*)C, ldc, M, N, K, accum, ldacc);
    } else {                                   // few rows, long K: 16 wavefronts per strip
        gemm_skinny_kernel<NT, 16, true, SILU, TC><<<strips, 1024, 0, stream>>>(
            (const bf16_t*)A, lda, (const bf16_t*)W, bias, bias_f32, (TC*)C, ldc, M, N, K, accum, ldacc);
    }
    TM_CHECK_LAUNCH();
    return TM_OK;
}

template <bool SILU, typename TC>
static int launch_skinny_nt(const void* A, int lda, const void* W, const void* bias, int bias_f32, void* C, int ldc,
                            int M, int N, int K, float* accum, int ldacc, hipStream_t stream) {
    switch ((M + 15) / 16) {
        case 1: return launch_skinny<1, SILU, TC>(A, lda, W, bias, bias_f32, C, ldc, M, N, K, accum, ldacc, stream);
        case 2: return launch_skinny<2, SILU, TC>(A, lda, W, bias, bias_f32, C, ldc, M, N, K, accum, ldacc, stream);
        case 3: return launch_skinny<3, SILU, TC>(A, lda, W, bias, bias_f32, C, ldc, M, N, K, accum, ldacc, stream);
        case 4: return launch_skinny<4, SILU, TC>(A, lda, W, bias, bias_f32, C, ldc, M, N, K, accum, ldacc, stream);
        default: return TM_ERR_ARG;
    }
}

// silu == 0: C[M, N] = A W^T + bias, W [N, K].   silu == 1: C[M, N] = silu(A Wg^T) * (A Wu^T), W = [Wg; Wu] [2N, K].
// A, W bfloat16; C bfloat16 (out_dtype 1) or float32 (0); bias bfloat16 or float32 or null.
// accum != null: nothing is stored to C; the bfloat16-rounded result is added to accum[M, N] (float32, row
// stride ldacc) instead: the residual add of the layer, done by the product that feeds it.
// Needs M <= 64, K % 8 == 0, lda % 8 == 0 and 16-byte aligned A and W.
extern "C" int tm_gemm_skinny(const void* A, int lda, const void* W, const void* bias, int bias_dtype, void* C,
                              int ldc, int M, int N, int K, int out_dtype, int silu, float* accum, int ldacc,
                              hipStream_t stream) {
    if (M <= 0 || N <= 0) return TM_OK;
    if (accum && (silu || ldacc < N)) return TM_ERR_ARG;
    if (!accum && !C) return TM_ERR_ARG;
    if (M > 64 || K <= 0 || (K % 8) || (lda % 8) || lda < K || ldc < N || ((uintptr_t)A % 16) || ((uintptr_t)W % 16))
        return TM_ERR_ARG;
    if (silu && bias) return TM_ERR_ARG;
    const int bias_f32 = bias_dtype == TM_F32;
    if (out_dtype == TM_BF16)
        return silu ? launch_skinny_nt<true, bf16_t>(A, lda, W, bias, bias_f32, C, ldc, M, N, K, accum, ldacc, stream)
                    : launch_skinny_nt<false, bf16_t>(A, lda, W, bias, bias_f32, C, ldc, M, N, K, accum, ldacc, stream);
    if (out_dtype == TM_F32 && !silu)
        return launch_skinny_nt<false, float>(A, lda, W, bias, bias_f32, C, ldc, M, N, K, accum, ldacc, stream);
    return TM_ERR_ARG;
}

// Rows of a strip that tm_gemm_skinny_packed wants a plain [N, K] matrix (no SiLU) packed in: 16, or
// 8 or 4 for a matrix with so few rows that 16-row strips would leave CUs without a block.
extern "C" int tm_skinny_strip_rows(int N, int K) {
    (void)K;
    if ((N + 15) / 16 >= 192) return 16;
    return (N + 7) / 8 >= 192 ? 8 : 4;
}

template <bool SILU, typename TC, int ROWS>
static int launch_skinny_packed(const void* A, int lda, const void* W, const void* bias, int bias_f32, void* C, int ldc,
                                int M, int N, int K, float* accum, int ldacc, int up_strip0, hipStream_t stream) {
    const int strips = (N + ROWS - 1) / ROWS;
#define TM_PACKED(WV, SPL, BLOCKS)                                                                               \
    gemm_skinny_kernel<1, WV, SPL, SILU, TC, ROWS, true><<<BLOCKS, 64 * WV, 0, stream>>>(                        \
        (const bf16_t*)A, lda, (const bf16_t*)W, bias, bias_f32, (TC*)C, ldc, M, N, K, accum, ldacc, up_strip0)
    if (ROWS == 16 && strips >= 2048) TM_PACKED(4, false, (strips + 3) / 4);      // many rows: a strip per wavefront
    else if (K < 2048 || (ROWS == 16 && strips >= 256)) TM_PACKED(4, true, strips);
    else TM_PACKED(16, true, strips);
#undef TM_PACKED
    TM_CHECK_LAUNCH();
    return TM_OK;
}

// tm_gemm_skinny for at most 16 rows with the matrix in strip order (tm_pack_layout in api.h): strips of
// `rows` rows (16, 8 or 4; 16 with silu, where Wg and Wu are each packed by themselves, Wu behind Wg).
extern "C" int tm_gemm_skinny_packed(const void* A, int lda, const void* W, int rows, const void* bias, int bias_dtype,
                                     void* C, int ldc, int M, int N, int K, int out_dtype, int silu, float* accum,
                                     int ldacc, hipStream_t stream) {
    if (M <= 0 || N <= 0) return TM_OK;
    if (accum && (silu || ldacc < N)) return TM_ERR_ARG;
    if (!accum && !C) return TM_ERR_ARG;
    if (M > 16 || K <= 0 || (K % 8) || (lda % 8) || lda < K || ldc < N || ((uintptr_t)A % 16) || ((uintptr_t)W % 16) ||
        (rows != 16 && rows != 8 && rows != 4) || (silu && (rows != 16 || bias)))
        return TM_ERR_ARG;
    const int bias_f32 = bias_dtype == TM_F32;
    const int up_strip0 = (N + 15) / 16;
#define TM_PACKED_ROWS(SILU_, TC_)                                                                               \
    switch (rows) {                                                                                              \
        case 16: return launch_skinny_packed<SILU_, TC_, 16>(A, lda, W, bias, bias_f32, C, ldc, M, N, K, accum, ldacc, up_strip0, stream); \
        case 8: if (!SILU_) return launch_skinny_packed<false, TC_, 8>(A, lda, W, bias, bias_f32, C, ldc, M, N, K, accum, ldacc, 0, stream); break; \
        default: if (!SILU_) return launch_skinny_packed<false, TC_, 4>(A, lda, W, bias, bias_f32, C, ldc, M, N, K, accum, ldacc, 0, stream); break; \
    }
    if (out_dtype == TM_BF16) {
        if (silu) { TM_PACKED_ROWS(true, bf16_t) } else { TM_PACKED_ROWS(false, bf16_t) }
    } else if (out_dtype == TM_F32 && !silu) {
        TM_PACKED_ROWS(false, float)
    }
#undef TM_PACKED_ROWS
    return TM_ERR_ARG;
}
