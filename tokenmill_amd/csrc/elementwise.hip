// Row-wise kernels: embedding rows, residual add + RMSNorm, rotary position encoding fused with
// the cache write, SiLU(gate)*up, type conversion.
//
// Exactness: the residual stream is 32-bit; sums of squares, the reciprocal root and the rotation
// are 32-bit; a bfloat16 result is rounded once, where the tensor is stored.
#include "common.h"
#include "api.h"

// ------------------------------------------------------------------------------------------
// embedding rows -> 32-bit residual stream           (reference src/infer/model/qwen2.py:46)
// ------------------------------------------------------------------------------------------
template <typename T>
__global__ void embed_gather_kernel(const T* __restrict__ table, const int* __restrict__ ids,
                                    float* __restrict__ out, int hidden, int vocab) {
    const int t = blockIdx.x;
    int id = ids[t];
    id = id < 0 ? 0 : (id >= vocab ? vocab - 1 : id);       // the host rejects such ids; never read outside
    const T* row = table + (size_t)id * hidden;
    float* o = out + (size_t)t * hidden;
    for (int c = threadIdx.x; c < hidden; c += blockDim.x) o[c] = Elem<T>::load(row + c);
}

extern "C" int tm_embed_gather(const void* table, int dtype, const int* ids, float* out, int T,
                               int hidden, int vocab, hipStream_t stream) {
    if (T <= 0) return TM_OK;
    if (hidden <= 0 || vocab <= 0) return TM_ERR_ARG;
    if (dtype == TM_F32)
        embed_gather_kernel<float><<<T, 256, 0, stream>>>((const float*)table, ids, out, hidden, vocab);
    else if (dtype == TM_BF16)
        embed_gather_kernel<bf16_t><<<T, 256, 0, stream>>>((const bf16_t*)table, ids, out, hidden, vocab);
    else
        return TM_ERR_ARG;
    TM_CHECK_LAUNCH();
    return TM_OK;
}

// ------------------------------------------------------------------------------------------
// residual += delta ; out = weight * round(residual * rsqrt(mean(residual^2) + eps))
//                                                    (reference src/infer/model/layers.py:41-44,
//                                                     src/infer/model/qwen2.py:22-23)
// rows == nullptr: row r of the residual is updated in place.
// rows != nullptr: row rows[r] is read (residual + delta), nothing is written back, out row r.
// ------------------------------------------------------------------------------------------
// What is still to be added to the residual stream: a tensor of the model's type, or the partial sums of a product
// whose K was split over blocks (32-bit, `parts` of them, `stride` elements apart), which are added in their
// order and rounded to the model's type first, as the product's own epilogue would have stored them.
template <typename T>
struct Pending {
    const T* delta;
    const float* parts;
    int n_parts;
    size_t stride;
    __device__ __forceinline__ bool any() const { return delta || parts; }
    __device__ __forceinline__ float at(size_t i) const {
        if (delta) return Elem<T>::load(delta + i);
        float s = parts[i];
        for (int p = 1; p < n_parts; ++p) s += parts[p * stride + i];
        return Elem<T>::round(s);
    }
};

template <typename T, typename WT>
__global__ void add_rmsnorm_kernel(float* __restrict__ resid, const Pending<T> pending,
                                   const int* __restrict__ rows, const WT* __restrict__ weight,
                                   T* __restrict__ out, int hidden, float eps) {
    __shared__ float red[4];
    const int r = blockIdx.x;
    const size_t src = rows ? (size_t)rows[r] : (size_t)r;
    float* x = resid + src * hidden;
    const bool d = pending.any();
    T* o = out + (size_t)r * hidden;
    float ss = 0.f;
    for (int c = threadIdx.x; c < hidden; c += 256) {
        float v = x[c];
        if (d) v += pending.at(src * hidden + c);
        if (d && !rows) x[c] = v;
        ss += v * v;
    }
    ss = block_sum<256>(ss, red);
    const float rs = rsqrtf(ss / (float)hidden + eps);
    for (int c = threadIdx.x; c < hidden; c += 256) {
        float v = x[c];
        if (d && rows) v += pending.at(src * hidden + c);   // in-place rows already hold the sum
        const float n = Elem<T>::round(v * rs);            // rounded BEFORE the weight multiplies
        Elem<T>::store(o + c, Elem<WT>::load(weight + c) * n);
    }
}

// The same for widths that are a multiple of 4 and at most 16,384: every thread (256, 512 or 1,024 of them) keeps
// its (up to four) 4-element groups of the row in registers, so the row is read once.
typedef float ew_f32x4 __attribute__((ext_vector_type(4)));

template <typename T> struct Vec4;
template <> struct Vec4<float> {
    static __device__ __forceinline__ ew_f32x4 load(const float* p) { return *(const ew_f32x4*)p; }
    static __device__ __forceinline__ void store(float* p, ew_f32x4 v) { *(ew_f32x4*)p = v; }
};
template <> struct Vec4<bf16_t> {
    static __device__ __forceinline__ ew_f32x4 load(const bf16_t* p) {
        const uint2 u = *(const uint2*)p;
        return ew_f32x4{__uint_as_float(u.x << 16), __uint_as_float(u.x & 0xffff0000u), __uint_as_float(u.y << 16),
                        __uint_as_float(u.y & 0xffff0000u)};
    }
    static __device__ __forceinline__ void store(bf16_t* p, ew_f32x4 v) {
        uint2 u;
        u.x = (uint32_t)f32_to_bf16(v[0]) | ((uint32_t)f32_to_bf16(v[1]) << 16);
        u.y = (uint32_t)f32_to_bf16(v[2]) | ((uint32_t)f32_to_bf16(v[3]) << 16);
        *(uint2*)p = u;
    }
};

#define ADD_NORM_MAX_PARTS 8       // most partial sums the vector kernel adds (more: the plain kernel)

template <typename T, typename WT, int THREADS>
__global__ __launch_bounds__(THREADS) void add_rmsnorm_vec_kernel(float* __restrict__ resid, const Pending<T> pending,
                                                              const int* __restrict__ rows,
                                                              const WT* __restrict__ weight, T* __restrict__ out,
                                                              int hidden, float eps) {
    __shared__ float red[THREADS / 64];
    const int r = blockIdx.x;
    const size_t src = rows ? (size_t)rows[r] : (size_t)r;
    float* x = resid + src * hidden;
    const T* d = pending.delta ? pending.delta + src * hidden : nullptr;
    const float* ps = pending.parts ? pending.parts + src * hidden : nullptr;
    T* o = out + (size_t)r * hidden;
    const int groups = hidden / 4;
    ew_f32x4 v[4];
    float ss = 0.f;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int gidx = threadIdx.x + i * THREADS;
        v[i] = ew_f32x4{0.f, 0.f, 0.f, 0.f};
        if (gidx < groups) {
            v[i] = Vec4<float>::load(x + 4 * gidx);
            if (d) {
                v[i] += Vec4<T>::load(d + 4 * gidx);
                if (!rows) Vec4<float>::store(x + 4 * gidx, v[i]);
            } else if (ps) {
                // all parts asked for at once (a part that does not exist: part 0 again, not counted), then added in order
                ew_f32x4 part[ADD_NORM_MAX_PARTS];
#pragma unroll
                for (int p = 0; p < ADD_NORM_MAX_PARTS; ++p)
                    part[p] = Vec4<float>::load(ps + (size_t)(p < pending.n_parts ? p : 0) * pending.stride + 4 * gidx);
                ew_f32x4 sum = part[0];
#pragma unroll
                for (int p = 1; p < ADD_NORM_MAX_PARTS; ++p)
                    if (p < pending.n_parts) sum += part[p];
#pragma unroll
                for (int k = 0; k < 4; ++k) v[i][k] += Elem<T>::round(sum[k]);
                if (!rows) Vec4<float>::store(x + 4 * gidx, v[i]);
            }
            ss += v[i][0] * v[i][0] + v[i][1] * v[i][1] + v[i][2] * v[i][2] + v[i][3] * v[i][3];
        }
    }
    ss = block_sum<THREADS>(ss, red);
    const float rs = rsqrtf(ss / (float)hidden + eps);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int gidx = threadIdx.x + i * THREADS;
        if (gidx < groups) {
            const ew_f32x4 w = Vec4<WT>::load(weight + 4 * gidx);
            ew_f32x4 y;
#pragma unroll
            for (int k = 0; k < 4; ++k) y[k] = w[k] * Elem<T>::round(v[i][k] * rs);   // rounded BEFORE the weight multiplies
            Vec4<T>::store(o + 4 * gidx, y);
        }
    }
}

template <typename T, typename WT>
static void launch_add_rmsnorm(float* resid, const void* delta, const float* parts, int n_parts, size_t stride,
                               const int* rows, const void* weight, void* out, int R, int hidden, float eps,
                               hipStream_t stream) {
    const bool vec = hidden % 4 == 0 && hidden <= 16384 && ((uintptr_t)resid % 16) == 0 && ((uintptr_t)weight % 16) == 0 &&
                     ((uintptr_t)out % 16) == 0 && (!delta || ((uintptr_t)delta % 16) == 0) &&
                     (!parts || (((uintptr_t)parts % 16) == 0 && stride % 4 == 0 && n_parts <= ADD_NORM_MAX_PARTS));
    const Pending<T> pending{(const T*)delta, parts, n_parts, stride};
    // a thread for every 4-element group where 1,024 reach (measured on an MI355X, 64 rows with 4 partial sums: width
    // 3,584 6.5 us with 256 threads, 4.9 with 512, 4.5 with 1,024; width 5,120 5.7 with 512, 5.1 with 1,024; width 896
    // 3.4 us with any); from the width alone: the sum of squares has one order per model
    const int threads = hidden <= 1024 ? 256 : hidden <= 2048 ? 512 : 1024;
    if (vec && threads == 256)
        add_rmsnorm_vec_kernel<T, WT, 256><<<R, 256, 0, stream>>>(resid, pending, rows, (const WT*)weight, (T*)out, hidden, eps);
    else if (vec && threads == 512)
        add_rmsnorm_vec_kernel<T, WT, 512><<<R, 512, 0, stream>>>(resid, pending, rows, (const WT*)weight, (T*)out, hidden, eps);
    else if (vec)
        add_rmsnorm_vec_kernel<T, WT, 1024><<<R, 1024, 0, stream>>>(resid, pending, rows, (const WT*)weight, (T*)out, hidden, eps);
    else
        add_rmsnorm_kernel<T, WT><<<R, 256, 0, stream>>>(resid, pending, rows, (const WT*)weight, (T*)out, hidden, eps);
}

static int add_rmsnorm_any(float* resid, const void* delta, const float* parts, int n_parts, size_t stride, const int* rows,
                           const void* weight, int w_dtype, void* out, int dtype, int R, int hidden, float eps,
                           hipStream_t stream) {
    if (R <= 0) return TM_OK;
    if (hidden <= 0 || !(eps > 0.f)) return TM_ERR_ARG;
    if (dtype == TM_F32 && w_dtype == TM_F32)
        launch_add_rmsnorm<float, float>(resid, delta, parts, n_parts, stride, rows, weight, out, R, hidden, eps, stream);
    else if (dtype == TM_BF16 && w_dtype == TM_BF16)
        launch_add_rmsnorm<bf16_t, bf16_t>(resid, delta, parts, n_parts, stride, rows, weight, out, R, hidden, eps, stream);
    else if (dtype == TM_BF16 && w_dtype == TM_F32)
        launch_add_rmsnorm<bf16_t, float>(resid, delta, parts, n_parts, stride, rows, weight, out, R, hidden, eps, stream);
    else
        return TM_ERR_ARG;
    TM_CHECK_LAUNCH();
    return TM_OK;
}

extern "C" int tm_add_rmsnorm(float* resid, const void* delta, const int* rows, const void* weight,
                              int w_dtype, void* out, int dtype, int R, int hidden, float eps,
                              hipStream_t stream) {
    return add_rmsnorm_any(resid, delta, nullptr, 0, 0, rows, weight, w_dtype, out, dtype, R, hidden, eps, stream);
}

// The same, with what is to be added given as the 32-bit partial sums of a product whose K was split over blocks:
// parts[p * stride + i], p < n_parts, added in the order of p and rounded to `dtype` before they meet the residual.
extern "C" int tm_add_rmsnorm_parts(float* resid, const float* parts, int n_parts, size_t stride, const int* rows,
                                    const void* weight, int w_dtype, void* out, int dtype, int R, int hidden, float eps,
                                    hipStream_t stream) {
    if (!parts || n_parts < 1 || n_parts > 16) return TM_ERR_ARG;
    return add_rmsnorm_any(resid, nullptr, parts, n_parts, stride, rows, weight, w_dtype, out, dtype, R, hidden, eps, stream);
}

// out[i] = round(sum over p of parts[p * stride + i]) in `dtype`: the partial sums as the tensor the product would
// have stored.
template <typename T>
__global__ void sum_parts_kernel(const float* __restrict__ parts, int n_parts, size_t stride, T* __restrict__ out, size_t n) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    float s = parts[i];
    for (int p = 1; p < n_parts; ++p) s += parts[p * stride + i];
    Elem<T>::store(out + i, s);
}

extern "C" int tm_sum_parts(const float* parts, int n_parts, size_t stride, void* out, int dtype, size_t n,
                            hipStream_t stream) {
    if (n == 0) return TM_OK;
    if (!parts || n_parts < 1 || !out) return TM_ERR_ARG;
    const unsigned blocks = (unsigned)((n + 255) / 256);
    if (dtype == TM_BF16) sum_parts_kernel<bf16_t><<<blocks, 256, 0, stream>>>(parts, n_parts, stride, (bf16_t*)out, n);
    else if (dtype == TM_F32) sum_parts_kernel<float><<<blocks, 256, 0, stream>>>(parts, n_parts, stride, (float*)out, n);
    else return TM_ERR_ARG;
    TM_CHECK_LAUNCH();
    return TM_OK;
}

// ------------------------------------------------------------------------------------------
// Rotary position encoding of q and k in place, then k and v of every token to its cache slot.
//   qkv row = [H heads of q | KVH heads of k | KVH heads of v], each D wide.
//   pairs (j, j + rot/2) for j < rot/2; elements >= rot pass through
//                                                    (reference src/infer/model/layers.py:55-64;
//                                                     cache write: src/infer/kv/paged_cache.py:40-43)
//   cos/sin: [max_pos, rot/2] 32-bit; cos == nullptr means no rotation (cache write only).
//   slot = page * page_size + place in the page; slot < 0: k and v are not stored (padding rows).
//   K pool [pages, page_size, KVH, D]; V pool [pages, KVH, D, page_size]: the values of one page
//   lie key-contiguous for each (head, d), which is how the MFMA attention kernels read them.
// ------------------------------------------------------------------------------------------
template <typename T>
__global__ void rope_kv_write_kernel(T* __restrict__ qkv, int H, int KVH, int D, int rot,
                                     const float* __restrict__ cos_t, const float* __restrict__ sin_t,
                                     const int* __restrict__ positions, const int* __restrict__ slots,
                                     T* __restrict__ k_pool, T* __restrict__ v_pool, int page, int write_kv) {
    // one block per token; its threads walk (head, pair) for q and k and (head, d) for v
    const int t = blockIdx.x;
    const int width = (H + 2 * KVH) * D;
    T* row = qkv + (size_t)t * width;
    const int slot = slots ? slots[t] : -1;
    const bool store = write_kv && slot >= 0;
    const int half = rot / 2;
    const float* c = cos_t ? cos_t + (size_t)positions[t] * half : nullptr;
    const float* s = cos_t ? sin_t + (size_t)positions[t] * half : nullptr;
    if (cos_t) {
        for (int idx = threadIdx.x; idx < (H + KVH) * half; idx += blockDim.x) {
            const int hh = idx / half, j = idx - hh * half;
            T* x = row + (size_t)hh * D;
            const float x1 = Elem<T>::load(x + j), x2 = Elem<T>::load(x + j + half);
            float y1, y2;
            rotate_pair(x1, x2, c[j], s[j], y1, y2);
            Elem<T>::store(x + j, y1);
            Elem<T>::store(x + j + half, y2);
            if (store && hh >= H) {
                T* dst = k_pool + ((size_t)slot * KVH + (hh - H)) * D;
                Elem<T>::store(dst + j, y1);
                Elem<T>::store(dst + j + half, y2);
            }
        }
    }
    if (!store) return;
    // the part of k that is not rotated (all of it without a table) and v
    const int tail = D - rot * (cos_t ? 1 : 0);
    const int k_from = cos_t ? rot : 0;
    for (int idx = threadIdx.x; idx < KVH * tail; idx += blockDim.x) {
        const int kvh = idx / tail, j = k_from + idx - kvh * tail;
        k_pool[((size_t)slot * KVH + kvh) * D + j] = row[(size_t)(H + kvh) * D + j];
    }
    const int pg = slot / page, in_page = slot % page;
    for (int idx = threadIdx.x; idx < KVH * D; idx += blockDim.x) {
        const int kvh = idx / D, j = idx - kvh * D;
        v_pool[(((size_t)pg * KVH + kvh) * D + j) * page + in_page] = row[(size_t)(H + KVH + kvh) * D + j];
    }
}

extern "C" int tm_rope_kv_write(void* qkv, int dtype, int T, int H, int KVH, int D, int rot,
                                const float* cos_t, const float* sin_t, const int* positions,
                                const int* slots, void* k_pool, void* v_pool, int page, int write_kv,
                                hipStream_t stream) {
    if (T <= 0) return TM_OK;
    if (H <= 0 || KVH <= 0 || D <= 0 || rot < 0 || rot > D || (rot & 1)) return TM_ERR_ARG;
    if (cos_t && (!sin_t || !positions)) return TM_ERR_ARG;
    if (write_kv && (!slots || !k_pool || !v_pool || page <= 0)) return TM_ERR_ARG;
    const int grid = T;
    if (dtype == TM_F32)
        rope_kv_write_kernel<float><<<grid, 256, 0, stream>>>((float*)qkv, H, KVH, D, rot, cos_t, sin_t, positions,
                                                            slots, (float*)k_pool, (float*)v_pool, page, write_kv);
    else if (dtype == TM_BF16)
        rope_kv_write_kernel<bf16_t><<<grid, 256, 0, stream>>>((bf16_t*)qkv, H, KVH, D, rot, cos_t, sin_t,
                                                             positions, slots, (bf16_t*)k_pool, (bf16_t*)v_pool,
                                                             page, write_kv);
    else
        return TM_ERR_ARG;
    TM_CHECK_LAUNCH();
    return TM_OK;
}

// ------------------------------------------------------------------------------------------
// out[t, i] = silu(gu[t, i]) * gu[t, I + i]           (reference src/infer/model/layers.py:164)
// ------------------------------------------------------------------------------------------
template <typename T>
__global__ void silu_mul_kernel(const T* __restrict__ gu, T* __restrict__ out, int I, size_t total) {
    for (size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
         idx += (size_t)gridDim.x * blockDim.x) {
        const size_t t = idx / I;
        const int i = (int)(idx - t * I);
        const float g = Elem<T>::load(gu + t * 2 * I + i);
        const float u = Elem<T>::load(gu + t * 2 * I + I + i);
        Elem<T>::store(out + idx, g / (1.f + expf(-g)) * u);
    }
}

// bfloat16 rows whose width is a multiple of 8: eight elements (16 bytes) per thread and step
__global__ void silu_mul_bf16x8_kernel(const bf16_t* __restrict__ gu, bf16_t* __restrict__ out, int I, size_t groups) {
    const int per_row = I / 8;
    for (size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x; idx < groups;
         idx += (size_t)gridDim.x * blockDim.x) {
        const size_t t = idx / per_row;
        const int i = (int)(idx - t * per_row) * 8;
        const uint4 gv = *(const uint4*)(gu + t * 2 * I + i);
        const uint4 uv = *(const uint4*)(gu + t * 2 * I + I + i);
        const uint32_t gw[4] = {gv.x, gv.y, gv.z, gv.w}, uw[4] = {uv.x, uv.y, uv.z, uv.w};
        uint32_t ow[4];
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const float g0 = __uint_as_float(gw[k] << 16), g1 = __uint_as_float(gw[k] & 0xffff0000u);
            const float u0 = __uint_as_float(uw[k] << 16), u1 = __uint_as_float(uw[k] & 0xffff0000u);
            const float r0 = g0 / (1.f + expf(-g0)) * u0, r1 = g1 / (1.f + expf(-g1)) * u1;
            ow[k] = (uint32_t)f32_to_bf16(r0) | ((uint32_t)f32_to_bf16(r1) << 16);
        }
        *(uint4*)(out + t * I + i) = uint4{ow[0], ow[1], ow[2], ow[3]};
    }
}

extern "C" int tm_silu_mul(const void* gu, void* out, int dtype, int T, int I, hipStream_t stream) {
    if (T <= 0) return TM_OK;
    if (I <= 0) return TM_ERR_ARG;
    const size_t total = (size_t)T * I;
    if (dtype == TM_BF16 && I % 8 == 0 && ((uintptr_t)gu % 16) == 0 && ((uintptr_t)out % 16) == 0) {
        const size_t groups = total / 8;
        size_t want = (groups + 255) / 256;
        silu_mul_bf16x8_kernel<<<(int)(want < 65536 ? want : 65536), 256, 0, stream>>>((const bf16_t*)gu, (bf16_t*)out,
                                                                                  I, groups);
        TM_CHECK_LAUNCH();
        return TM_OK;
    }
    size_t want = (total + 255) / 256;
    const int blocks = (int)(want < 16384 ? want : 16384);
    if (dtype == TM_F32)
        silu_mul_kernel<float><<<blocks, 256, 0, stream>>>((const float*)gu, (float*)out, I, total);
    else if (dtype == TM_BF16)
        silu_mul_kernel<bf16_t><<<blocks, 256, 0, stream>>>((const bf16_t*)gu, (bf16_t*)out, I, total);
    else
        return TM_ERR_ARG;
    TM_CHECK_LAUNCH();
    return TM_OK;
}

// ------------------------------------------------------------------------------------------
// type conversion of a flat array
// ------------------------------------------------------------------------------------------
template <typename TI, typename TO>
__global__ void convert_kernel(const TI* __restrict__ in, TO* __restrict__ out, size_t n) {
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x)
        Elem<TO>::store(out + i, Elem<TI>::load(in + i));
}

extern "C" int tm_convert(const void* in, int in_dtype, void* out, int out_dtype, long long n,
                          hipStream_t stream) {
    if (n <= 0) return TM_OK;
    size_t want = ((size_t)n + 255) / 256;
    const int blocks = (int)(want < 16384 ? want : 16384);
    if (in_dtype == TM_BF16 && out_dtype == TM_F32)
        convert_kernel<bf16_t, float><<<blocks, 256, 0, stream>>>((const bf16_t*)in, (float*)out, (size_t)n);
    else if (in_dtype == TM_F32 && out_dtype == TM_BF16)
        convert_kernel<float, bf16_t><<<blocks, 256, 0, stream>>>((const float*)in, (bf16_t*)out, (size_t)n);
    else
        return TM_ERR_ARG;
    TM_CHECK_LAUNCH();
    return TM_OK;
}
