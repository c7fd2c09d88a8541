// C[M, N] = A[M, K] * W[N, K]^T (+ bias[N]), everything float32, on the 32-bit matrix unit
// (v_mfma_f32_16x16x4_f32: 32-bit products and sums, no reduced-precision inputs): the matrix product
// of prompt-sized steps of the true 32-bit path                (reference src/infer/model/layers.py:144,
// 150,163-164 run with float32 parameters, src/infer/model/loader.py:32-35).
//
// A block of four wavefronts computes a BM x BN tile of C; A and W tiles of 16 k go through LDS, the
// next tile's global loads are in flight while the current one is multiplied. A lane of the matrix
// instruction carries k = 4 g + s (g = lane / 16) in its s-th instruction of a tile, so one 16-byte LDS
// read feeds four instructions. Which k meet in which instruction, and the order of the instructions,
// depend on K alone: a row's result does not depend on the other rows of the call or on the tile
// it falls into. The sum over K is taken in blocks of 128: the matrix unit's accumulators hold one block's
// sum and are added to the running total at the block's end. One chain of additions over all of K loses
// sqrt(K / 4) roundings' worth of accuracy (3e-6 of the result at K = 7,680, ten times what a blocked
// library product loses); in blocks it is the chain of a block and then the chain of the blocks.
#include "common.h"
#include "api.h"

typedef float mf_f32x4 __attribute__((ext_vector_type(4)));

#define MF_BK 16
#define MF_STRIDE 20        // floats per LDS row: 16 + 4, so that the 16-byte reads of 16 rows hit 64 different banks
#define MF_BLOCK_STEPS 8    // tiles of 16 k whose sum is taken by itself before it joins the total

template <int BM, int BN>
__global__ __launch_bounds__(256) void gemm_nt_mfma_f32_kernel(const float* __restrict__ A, int lda,
                                                               const float* __restrict__ W,
                                                               const float* __restrict__ bias, float* __restrict__ C,
                                                               int ldc, int M, int N, int K) {
    constexpr int TI = BM / 32, TJ = BN / 32;                 // 16 x 16 tiles of a wavefront's (BM/2) x (BN/2) share
    constexpr int A_LOADS = BM / 64, W_LOADS = BN / 64;       // 16-byte global loads per thread and tile
    __shared__ __align__(16) float As[2][BM][MF_STRIDE];
    __shared__ __align__(16) float Ws[2][BN][MF_STRIDE];
    const int tid = threadIdx.x;
    const int wave = tid / TM_WAVE, lane = tid % TM_WAVE;
    const int wm = wave / 2, wn = wave % 2;
    const int r = lane % 16, g = lane / 16;
    const int m0 = blockIdx.y * BM, n0 = blockIdx.x * BN;
    const int lrow = tid / 4, lq = tid % 4;                   // this thread's row and 4-k piece of a tile

    // No load stands under a test (a tested load is waited for where the test ends, one at a time): rows
    // beyond the matrices read their first rows instead, and what those give is never stored; K is a
    // multiple of the tile's 16, so no piece lies beyond it.
    mf_f32x4 ra[A_LOADS], rw[W_LOADS];
    const float* a_src[A_LOADS];
    const float* w_src[W_LOADS];
#pragma unroll
    for (int e = 0; e < A_LOADS; ++e) {
        const int m = m0 + lrow + 64 * e;
        a_src[e] = A + (size_t)(m < M ? m : 0) * lda + 4 * lq;
    }
#pragma unroll
    for (int e = 0; e < W_LOADS; ++e) {
        const int n = n0 + lrow + 64 * e;
        w_src[e] = W + (size_t)(n < N ? n : 0) * K + 4 * lq;
    }
    auto gload = [&](int k0) {
#pragma unroll
        for (int e = 0; e < A_LOADS; ++e) ra[e] = *(const mf_f32x4*)(a_src[e] + k0);
#pragma unroll
        for (int e = 0; e < W_LOADS; ++e) rw[e] = *(const mf_f32x4*)(w_src[e] + k0);
    };
    auto sstore = [&](int buf) {
#pragma unroll
        for (int e = 0; e < A_LOADS; ++e) *(mf_f32x4*)&As[buf][lrow + 64 * e][4 * lq] = ra[e];
#pragma unroll
        for (int e = 0; e < W_LOADS; ++e) *(mf_f32x4*)&Ws[buf][lrow + 64 * e][4 * lq] = rw[e];
    };

    mf_f32x4 acc[TI][TJ], total[TI][TJ];
#pragma unroll
    for (int i = 0; i < TI; ++i)
#pragma unroll
        for (int j = 0; j < TJ; ++j) acc[i][j] = total[i][j] = mf_f32x4{0.f, 0.f, 0.f, 0.f};

    const int steps = (K + MF_BK - 1) / MF_BK;
    gload(0);
    sstore(0);
    __syncthreads();
    int buf = 0;
    for (int it = 0; it < steps; ++it) {
        const bool more = it + 1 < steps;
        if (more) gload((it + 1) * MF_BK);
        mf_f32x4 a4[TI], w4[TJ];
#pragma unroll
        for (int i = 0; i < TI; ++i) a4[i] = *(const mf_f32x4*)&As[buf][wm * (BM / 2) + 16 * i + r][4 * g];
#pragma unroll
        for (int j = 0; j < TJ; ++j) w4[j] = *(const mf_f32x4*)&Ws[buf][wn * (BN / 2) + 16 * j + r][4 * g];
#pragma unroll
        for (int s = 0; s < 4; ++s)
#pragma unroll
            for (int i = 0; i < TI; ++i)
#pragma unroll
                for (int j = 0; j < TJ; ++j)
                    // rows of the instruction's result: n (from W), columns: m (from A)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x4f32(w4[j][s], a4[i][s], acc[i][j], 0, 0, 0);
        if ((it + 1) % MF_BLOCK_STEPS == 0 || !more) {           // a block of K ends: its sum joins the total
#pragma unroll
            for (int i = 0; i < TI; ++i)
#pragma unroll
                for (int j = 0; j < TJ; ++j) {
                    total[i][j] += acc[i][j];
                    acc[i][j] = mf_f32x4{0.f, 0.f, 0.f, 0.f};
                }
        }
        if (more) sstore(buf ^ 1);
        __syncthreads();
        buf ^= 1;
    }
    // lane (r, g) holds C[m = tile row r][n = 4 g .. 4 g + 3] of every tile
#pragma unroll
    for (int i = 0; i < TI; ++i) {
        const int m = m0 + wm * (BM / 2) + 16 * i + r;
        if (m >= M) continue;
#pragma unroll
        for (int j = 0; j < TJ; ++j) {
            const int n = n0 + wn * (BN / 2) + 16 * j + 4 * g;
            if (n >= N) continue;                              // N is a multiple of 4: a piece is whole or absent
            mf_f32x4 v = total[i][j];
            if (bias) {
                const mf_f32x4 b = *(const mf_f32x4*)(bias + n);
                v += b;
            }
            *(mf_f32x4*)(C + (size_t)m * ldc + n) = v;
        }
    }
}

// Can the matrix-unit kernel take this product? (float32 everywhere, K a multiple of 16, N of 4, rows 16-byte aligned)
extern "C" int tm_gemm_f32_mfma_fits(const void* A, int lda, const void* W, const void* bias, const void* C, int ldc,
                                     int M, int N, int K) {
    return M > 0 && N > 0 && K > 0 && K % MF_BK == 0 && N % 4 == 0 && lda % 4 == 0 && ldc % 4 == 0 && lda >= K && ldc >= N &&
           ((uintptr_t)A % 16) == 0 && ((uintptr_t)W % 16) == 0 && ((uintptr_t)C % 16) == 0 && ((uintptr_t)bias % 16) == 0;
}

extern "C" int tm_gemm_f32_mfma(const float* A, int lda, const float* W, const float* bias, float* C, int ldc, int M,
                                int N, int K, hipStream_t stream) {
    if (M <= 0 || N <= 0) return TM_OK;
    if (!tm_gemm_f32_mfma_fits(A, lda, W, bias, C, ldc, M, N, K)) return TM_ERR_ARG;
    // 64 x 128 tiles where they still give every CU a block, else 64 x 64. (128 x 128 tiles were the faster ones while
    // one set of accumulators sufficed; with the running total beside the block's sum they leave two wavefronts a
    // SIMD instead of three and are the slower ones: 21.2 ms against 20.8 ms for the 2,048-token prefill.)
    const long long mid = (long long)((M + 63) / 64) * ((N + 127) / 128);
    if (mid >= 256) {
        dim3 grid((N + 127) / 128, (M + 63) / 64);
        if (grid.y > 65535u) return TM_ERR_ARG;
        gemm_nt_mfma_f32_kernel<64, 128><<<grid, 256, 0, stream>>>(A, lda, W, bias, C, ldc, M, N, K);
    } else {
        dim3 grid((N + 63) / 64, (M + 63) / 64);
        if (grid.y > 65535u) return TM_ERR_ARG;
        gemm_nt_mfma_f32_kernel<64, 64><<<grid, 256, 0, stream>>>(A, lda, W, bias, C, ldc, M, N, K);
    }
    TM_CHECK_LAUNCH();
    return TM_OK;
}
