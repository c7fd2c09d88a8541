// C[M, N] = A[M, K] * W[N, K]^T (+ bias[N])   -- torch's F.linear with W stored [out, in]
//                                    (reference src/infer/model/layers.py:144,150,163-164;
//                                     src/infer/model/qwen2.py:51-52)
//
// gemm_nt_tiled: an LDS-tiled kernel on the vector ALU with 32-bit multiply-adds only. It is the
// matrix product of the true 32-bit path for shapes the 32-bit matrix-unit kernel (gemm_f32_mfma.hip)
// does not take, and the fallback of the bfloat16 path for shapes its MFMA kernels refuse. Each output element is accumulated over k = 0..K-1 in ascending order by one
// thread, so a row's result does not depend on how many other rows the call holds.
#include "common.h"
#include "api.h"

#define GT_BM 64
#define GT_BN 64
#define GT_BK 16

template <typename TA, typename TB, typename TC>
__global__ __launch_bounds__(256) void gemm_nt_tiled_kernel(const TA* __restrict__ A, int lda,
                                                            const TA* __restrict__ W,
                                                            const TB* __restrict__ bias,
                                                            TC* __restrict__ C, int ldc, int M, int N, int K) {
    __shared__ float As[GT_BK][GT_BM + 4];
    __shared__ float Ws[GT_BK][GT_BN + 4];
    const int tid = threadIdx.x;
    const int tx = tid % 16, ty = tid / 16;
    const int m0 = blockIdx.y * GT_BM, n0 = blockIdx.x * GT_BN;
    // the sum over K in blocks of 128: a block's sum is taken by itself and then joins the total (one chain of
    // additions over all of K loses sqrt(K) roundings' worth of accuracy, blocks lose the chain of a block and then
    // the chain of the blocks); where the blocks end depends on K alone
    float acc[4][4], total[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = total[i][j] = 0.f;

    for (int k0 = 0; k0 < K; k0 += GT_BK) {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const int idx = tid + e * 256;          // 0 .. 1023
            const int r = idx / GT_BK, c = idx % GT_BK;
            const int k = k0 + c;
            float a = 0.f, w = 0.f;
            if (k < K) {
                if (m0 + r < M) a = Elem<TA>::load(A + (size_t)(m0 + r) * lda + k);
                if (n0 + r < N) w = Elem<TA>::load(W + (size_t)(n0 + r) * K + k);
            }
            As[c][r] = a;
            Ws[c][r] = w;
        }
        __syncthreads();
#pragma unroll
        for (int kk = 0; kk < GT_BK; ++kk) {
            float a[4], w[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) a[i] = As[kk][ty * 4 + i];
#pragma unroll
            for (int j = 0; j < 4; ++j) w[j] = Ws[kk][tx * 4 + j];
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], w[j], acc[i][j]);
        }
        if ((k0 / GT_BK + 1) % 8 == 0 || k0 + GT_BK >= K) {
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    total[i][j] += acc[i][j];
                    acc[i][j] = 0.f;
                }
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int m = m0 + ty * 4 + i;
        if (m >= M) continue;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int n = n0 + tx * 4 + j;
            if (n >= N) continue;
            float v = total[i][j];
            if (bias) v += Elem<TB>::load(bias + n);
            Elem<TC>::store(C + (size_t)m * ldc + n, v);
        }
    }
}

template <typename TA, typename TB, typename TC>
static int launch_tiled(const void* A, int lda, const void* W, const void* bias, void* C, int ldc, int M, int N,
                        int K, hipStream_t stream) {
    dim3 grid((N + GT_BN - 1) / GT_BN, (M + GT_BM - 1) / GT_BM);
    gemm_nt_tiled_kernel<TA, TB, TC><<<grid, 256, 0, stream>>>((const TA*)A, lda, (const TA*)W, (const TB*)bias,
                                                               (TC*)C, ldc, M, N, K);
    TM_CHECK_LAUNCH();
    return TM_OK;
}

// gemv_f32: the same product for at most 16 rows of A in 32-bit (a decode step of the true 32-bit
// path), bound by reading W once. A block of four wavefronts takes GV_ROWS rows of W; the
// wavefronts split K into four contiguous ranges, a lane takes the slices k = 256 i + 4 lane .. + 3
// of its wavefront's range in ascending i, the lanes' sums are added by a fixed tree and the
// wavefronts' in wavefront order: the order of additions depends on K only, so a row's result
// does not depend on the other rows of the call. 32-bit multiply-adds only.
#define GV_ROWS 4

typedef float gv_f32x4 __attribute__((ext_vector_type(4)));

template <int MT>
__global__ __launch_bounds__(256) void gemv_f32_kernel(const float* __restrict__ A, int lda,
                                                       const float* __restrict__ W,
                                                       const float* __restrict__ bias, float* __restrict__ C,
                                                       int ldc, int M, int N, int K) {
    __shared__ float red[4][GV_ROWS][MT];
    const int wave = threadIdx.x / TM_WAVE, lane = threadIdx.x % TM_WAVE;
    const int n0 = blockIdx.x * GV_ROWS;
    const int slices = (K + 255) / 256;                     // 256 = 64 lanes x 4 elements
    const int per = (slices + 3) / 4;
    const int s0 = wave * per, s1 = s0 + per < slices ? s0 + per : slices;
    float acc[GV_ROWS][MT];
#pragma unroll
    for (int r = 0; r < GV_ROWS; ++r)
#pragma unroll
        for (int m = 0; m < MT; ++m) acc[r][m] = 0.f;
    for (int sl = s0; sl < s1; ++sl) {
        const int k = sl * 256 + 4 * lane;
        if (k >= K) continue;                               // K is a multiple of 4: a slice is whole or absent
        gv_f32x4 w[GV_ROWS];
#pragma unroll
        for (int r = 0; r < GV_ROWS; ++r)
            w[r] = n0 + r < N ? *(const gv_f32x4*)(W + (size_t)(n0 + r) * K + k) : gv_f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int m = 0; m < MT; ++m) {
            const gv_f32x4 a = m < M ? *(const gv_f32x4*)(A + (size_t)m * lda + k) : gv_f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int r = 0; r < GV_ROWS; ++r) {
                float v = acc[r][m];
                v = fmaf(a[0], w[r][0], v);
                v = fmaf(a[1], w[r][1], v);
                v = fmaf(a[2], w[r][2], v);
                v = fmaf(a[3], w[r][3], v);
                acc[r][m] = v;
            }
        }
    }
#pragma unroll
    for (int r = 0; r < GV_ROWS; ++r)
#pragma unroll
        for (int m = 0; m < MT; ++m) {
            const float v = wave_sum(acc[r][m]);
            if (lane == 0) red[wave][r][m] = v;
        }
    __syncthreads();
    const int r = threadIdx.x / MT, m = threadIdx.x % MT;
    if (r < GV_ROWS && m < M && n0 + r < N) {
        float v = red[0][r][m] + red[1][r][m];
        v += red[2][r][m];
        v += red[3][r][m];
        if (bias) v += bias[n0 + r];
        C[(size_t)m * ldc + n0 + r] = v;
    }
}

// C[M, N] (float32) = A[M, K] W[N, K]^T + bias, all float32, M <= 16, K % 4 == 0, 16-byte aligned rows.
extern "C" int tm_gemv_f32(const float* A, int lda, const float* W, const float* bias, float* C, int ldc, int M,
                           int N, int K, hipStream_t stream) {
    if (M <= 0 || N <= 0) return TM_OK;
    if (M > 16 || K <= 0 || (K % 4) || (lda % 4) || lda < K || ldc < N || ((uintptr_t)A % 16) || ((uintptr_t)W % 16))
        return TM_ERR_ARG;
    const unsigned blocks = (unsigned)((N + GV_ROWS - 1) / GV_ROWS);
    if (M <= 4)
        gemv_f32_kernel<4><<<blocks, 256, 0, stream>>>(A, lda, W, bias, C, ldc, M, N, K);
    else if (M <= 8)
        gemv_f32_kernel<8><<<blocks, 256, 0, stream>>>(A, lda, W, bias, C, ldc, M, N, K);
    else
        gemv_f32_kernel<16><<<blocks, 256, 0, stream>>>(A, lda, W, bias, C, ldc, M, N, K);
    TM_CHECK_LAUNCH();
    return TM_OK;
}

extern "C" int tm_gemm_nt_tiled(const void* A, int lda, const void* W, const void* bias, int bias_dtype,
                                void* C, int ldc, int M, int N, int K, int in_dtype, int out_dtype,
                                hipStream_t stream) {
    if (M <= 0 || N <= 0) return TM_OK;
    if (K <= 0 || lda < K || ldc < N) return TM_ERR_ARG;
    if ((size_t)((M + GT_BM - 1) / GT_BM) > 65535u) return TM_ERR_ARG;
    if (!bias) bias_dtype = in_dtype;
    if (in_dtype == TM_F32 && out_dtype == TM_F32 && bias_dtype == TM_F32)
        return launch_tiled<float, float, float>(A, lda, W, bias, C, ldc, M, N, K, stream);
    if (in_dtype == TM_BF16 && out_dtype == TM_BF16 && bias_dtype == TM_BF16)
        return launch_tiled<bf16_t, bf16_t, bf16_t>(A, lda, W, bias, C, ldc, M, N, K, stream);
    if (in_dtype == TM_BF16 && out_dtype == TM_BF16 && bias_dtype == TM_F32)
        return launch_tiled<bf16_t, float, bf16_t>(A, lda, W, bias, C, ldc, M, N, K, stream);
    if (in_dtype == TM_BF16 && out_dtype == TM_F32 && bias_dtype == TM_BF16)
        return launch_tiled<bf16_t, bf16_t, float>(A, lda, W, bias, C, ldc, M, N, K, stream);
    if (in_dtype == TM_BF16 && out_dtype == TM_F32 && bias_dtype == TM_F32)
        return launch_tiled<bf16_t, float, float>(A, lda, W, bias, C, ldc, M, N, K, stream);
    return TM_ERR_ARG;
}
