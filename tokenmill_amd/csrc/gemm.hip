// C[M, N] = A[M, K] * W[N, K]^T (+ bias[N])   -- torch's F.linear with W stored [out, in]
//                                    (reference src/infer/model/layers.py:144,150,163-164;
//                                     src/infer/model/qwen2.py:51-52)
//
// gemm_nt_tiled: an LDS-tiled kernel on the vector ALU with 32-bit multiply-adds only. It is the
// matrix product of the true 32-bit path, and the fallback of the bfloat16 path for shapes its
// MFMA kernels refuse. Each output element is accumulated over k = 0..K-1 in ascending order by one
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
    float acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = 0.f;

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
            float v = acc[i][j];
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
