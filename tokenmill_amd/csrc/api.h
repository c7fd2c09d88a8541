// C interface of the kernel library (libtokenmill_hip.so). Every function returns 0 on success,
// TM_ERR_ARG (1) for sizes or types the kernel does not run, TM_ERR_LAUNCH (2) if the launch failed.
// Pointers are device pointers; `stream` is a hipStream_t. dtype codes: 0 = float32, 1 = bfloat16.
#pragma once
#include <hip/hip_runtime.h>

extern "C" {

int tm_embed_gather(const void* table, int dtype, const int* ids, float* out, int T, int hidden, int vocab,
                    hipStream_t stream);

int tm_add_rmsnorm(float* resid, const void* delta, const int* rows, const void* weight, int w_dtype, void* out,
                   int dtype, int R, int hidden, float eps, hipStream_t stream);

// The same with what is to be added given as 32-bit partial sums parts[p * stride + i] (p < n_parts) of a product whose
// K was split over blocks: added in the order of p, rounded to `dtype`, then as above. tm_sum_parts: that rounded sum alone.
int tm_add_rmsnorm_parts(float* resid, const float* parts, int n_parts, size_t stride, const int* rows, const void* weight,
                         int w_dtype, void* out, int dtype, int R, int hidden, float eps, hipStream_t stream);
int tm_sum_parts(const float* parts, int n_parts, size_t stride, void* out, int dtype, size_t n, hipStream_t stream);

int tm_rope_kv_write(void* qkv, int dtype, int T, int H, int KVH, int D, int rot, const float* cos_t,
                     const float* sin_t, const int* positions, const int* slots, void* k_pool, void* v_pool,
                     int page, int write_kv, hipStream_t stream);

int tm_silu_mul(const void* gu, void* out, int dtype, int T, int I, hipStream_t stream);

int tm_convert(const void* in, int in_dtype, void* out, int out_dtype, long long n, hipStream_t stream);

int tm_gemm_nt_tiled(const void* A, int lda, const void* W, const void* bias, int bias_dtype, void* C, int ldc,
                     int M, int N, int K, int in_dtype, int out_dtype, hipStream_t stream);

// The float32 product on the 32-bit matrix unit: all operands float32, K a multiple of 16, N and the row strides of 4,
// 16-byte aligned (tm_gemm_f32_mfma_fits says whether a product is taken).
int tm_gemm_f32_mfma_fits(const void* A, int lda, const void* W, const void* bias, const void* C, int ldc, int M, int N,
                          int K);
int tm_gemm_f32_mfma(const float* A, int lda, const float* W, const float* bias, float* C, int ldc, int M, int N, int K,
                     hipStream_t stream);

int tm_attn_paged_generic(const void* q, int q_stride, void* out, int out_stride, const void* k_pool,
                          const void* v_pool, const int* block_tables, int table_width, const int* seq_of_token,
                          const int* positions, int T, int H, int KVH, int D, int page, float scale, int window,
                          int dtype, hipStream_t stream);

int tm_gemm_skinny(const void* A, int lda, const void* W, const void* bias, int bias_dtype, void* C, int ldc, int M,
                   int N, int K, int out_dtype, int silu, float* accum, int ldacc, hipStream_t stream);

// Strip order of a bfloat16 matrix W [N, K] for the decode-step products ("packed", strips of R = 16, 8 or 4
// rows): with KS = ceil(K / 32) k-steps, packed[((s * KS + ks) * 4 + g) * R + r][i] = W[s * R + r][32 ks + 8 g + i]
// for i < 8, zero where the row or the k does not exist; ceil(N / R) strips in all. A wavefront's
// 16-byte loads of one k-step of one strip are then one run of R * 64 bytes. A stacked matrix whose
// parts meet in an epilogue (gate and up) is packed part by part, each part's strips behind the other's.
int tm_skinny_strip_rows(int N, int K);
int tm_fused_qkv_strip_rows(int H, int KVH, int D, int K);
int tm_gemm_skinny_packed(const void* A, int lda, const void* W, int rows, const void* bias, int bias_dtype, void* C,
                          int ldc, int M, int N, int K, int out_dtype, int silu, float* accum, int ldacc,
                          hipStream_t stream);

int tm_attn_decode_mfma(const void* q, int q_stride, void* out, int out_stride, const void* k_pool,
                        const void* v_pool, const int* block_tables, int table_width, const int* context_lens,
                        float* part_o, float* part_ml, int max_chunks, int S, int H, int KVH, int D, int page,
                        float scale, int window, hipStream_t stream);

int tm_fused_norm_qkv_rope(const float* resid, const void* norm_w, int norm_w_dtype, float eps, int M, int K,
                           const void* W, const void* bias, int bias_dtype, void* q_out, int H, int KVH, int D,
                           const float* cos_t, const float* sin_t, const int* positions, const int* slots,
                           void* k_pool, void* v_pool, int page, hipStream_t stream);

int tm_fused_norm_gate_up_silu(const float* resid, const void* norm_w, int norm_w_dtype, float eps, int M, int K,
                               const void* W, void* act_out, int I, hipStream_t stream);

int tm_gemm_panel_fits(int M, int K);
int tm_panel_qkv_rope(const void* X, int ldx, int M, int K, const void* W, const void* bias, int bias_dtype, void* q_out,
                      int H, int KVH, int D, const float* cos_t, const float* sin_t, const int* positions,
                      const int* slots, void* k_pool, void* v_pool, int page, hipStream_t stream);

// The same products for up to 64 tokens at any width (K a multiple of 8), the matrix streamed once from its packed
// copy in strips of `rows` rows (16, 8 or 4), and the plain product with bias whose result is stored or, rounded to
// bfloat16, added into a 32-bit tensor (gemm_stream.hip).
int tm_gemm_stream_fits(int M, int K);
int tm_stream_qkv_rope(const void* X, int ldx, int M, int K, const void* W, int rows, const void* bias, int bias_dtype,
                       void* q_out, int H, int KVH, int D, const float* cos_t, const float* sin_t, const int* positions,
                       const int* slots, void* k_pool, void* v_pool, int page, hipStream_t stream);
int tm_stream_gate_up_silu(const void* X, int ldx, int M, int K, const void* W, void* act_out, int I, hipStream_t stream);
int tm_stream_linear(const void* X, int ldx, int M, int K, const void* W, int rows, int N, const void* bias, int bias_dtype,
                     void* C, int ldc, int out_f32, float* accum, int ldacc, hipStream_t stream);
// The plain product with K split over tm_stream_linear_parts(N, K) groups of blocks (a number from the matrix's shape
// alone; 1: not worth splitting): parts[p][M][N] (float32, M * N elements apart) receives the 32-bit partial sums,
// the bias in part 0, for tm_add_rmsnorm_parts or tm_sum_parts to add up.
int tm_stream_linear_parts(int N, int K);
int tm_stream_linear_split(const void* X, int ldx, int M, int K, const void* W, int rows, int N, const void* bias,
                           int bias_dtype, float* parts, hipStream_t stream);

int tm_attn_prefill_mfma(const void* q, int q_stride, void* out, int out_stride, const void* k_pool,
                         const void* v_pool, const int* block_tables, int table_width, const int* tiles, int n_tiles,
                         int H, int KVH, int D, int page, float scale, int window, hipStream_t stream);

// The same attention with the keys and values of a tile staged through LDS once for all query heads of a kv
// head (attention_prefill_shared.hip); same operands, out rows 8-byte aligned.
int tm_attn_prefill_shared(const void* q, int q_stride, void* out, int out_stride, const void* k_pool,
                           const void* v_pool, const int* block_tables, int table_width, const int* tiles, int n_tiles,
                           int H, int KVH, int D, int page, float scale, int window, hipStream_t stream);
int tm_attn_prefill_shared_takes(int H, int KVH, int D);

int tm_gemv_f32(const float* A, int lda, const float* W, const float* bias, float* C, int ldc, int M, int N, int K,
                hipStream_t stream);

// How a caller wants the library's algorithm for a product chosen (tm_gemm_library): see gemm_library.hip.
struct TmTune {
    int candidates;     // 0 or 1: the library's first choice, untimed; n: up to n candidates are timed, the fastest kept
    int after;          // the call of a shape (with the matrix of its first call) at which that happens; 1: at once
    int every;          // a shape timed at its first call also tries every algorithm the library holds for the types
};
int tm_gemm_library(const void* A, int lda, const void* W, int ldw, const void* bias, int bias_dtype, void* C, int ldc,
                    int out_f32, int M, int N, int K, void* workspace, size_t workspace_bytes, const TmTune* tune,
                    hipStream_t stream);

int tm_attn_prefill_f32(const void* q, int q_stride, void* out, int out_stride, const void* k_pool,
                        const void* v_pool, const int* block_tables, int table_width, const int* tiles, int n_tiles,
                        int H, int KVH, int D, int page, float scale, int window, hipStream_t stream);

int tm_argmax_work_chunks(int V);
int tm_argmax_rows(const float* logits, int R, int V, int* out, float* work_v, int* work_i, hipStream_t stream);

// The argmax again, for callers that cannot allocate device memory: code under HIP graph capture, tight
// serving loops, harnesses that forbid hipMalloc. (The reference has no counterpart: its argmax is a
// torch call that allocates as it likes.) Same result as tm_argmax_rows. The chunk candidates of the
// two-stage path go to a fixed array of 512 KiB that each GPU holds from the library's load to the
// process's end; the call allocates nothing and frees nothing. R * tm_argmax_work_chunks(V) may be at
// most tm_argmax_rows_static_max_pairs() (65,536: 256 rows of a 1M-entry vocabulary, 1,724 rows of
// 151,936 entries); more is refused with TM_ERR_ARG before anything is launched. All calls on one GPU
// share that GPU's array: two calls whose kernels can overlap there (different streams, or threads
// without an order between them) race; calls on one stream are ordered and safe. The device of
// `stream` must be the current device.
int tm_argmax_rows_static_max_pairs(void);
int tm_argmax_rows_static(const float* logits, int R, int V, int* out, hipStream_t stream);

size_t tm_sample_work_bytes(int R, int V);
int tm_sample_rows(const float* logits, int R, int V, const float* temperature, const int* top_k,
                   const float* top_p, const float* u, int* out, void* work, size_t work_bytes, int stages,
                   hipStream_t stream);

}  // extern "C"
