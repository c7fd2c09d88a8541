// What the two bfloat16 prefill attention kernels share: operand fragments, the softmax state of a
// wavefront's heads, and what a wavefront knows about the tile of query tokens it works on.
#pragma once
#include "common.h"

#define PF_SLACK 8.f        // how far (log2 units) a score may exceed the running reference before it moves

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));

union PFrag {
    u32x4_t u;
    bf16x8_t b;
};

typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef float f32x2_t __attribute__((ext_vector_type(2)));

// two floats -> packed bfloat16 (round to nearest even, one instruction on gfx950)
__device__ __forceinline__ uint32_t pk_bf16(float a, float b) {
    const bf16x2_t v = __builtin_convertvector(f32x2_t{a, b}, bf16x2_t);
    return *(const uint32_t*)&v;
}

// max(a, b, c) in the nesting the compiler turns into one three-operand maximum. A two-operand
// maximum of values whose origin it cannot see (matrix-unit results, lane swaps) costs it an extra
// instruction per operand (it first makes signalling NaNs quiet); the three-operand form does not,
// so the reductions below are chains of these, started from a constant.
__device__ __forceinline__ float max3(float a, float b, float c) { return fmaxf(fmaxf(a, b), c); }

// maximum over the four lanes (r, 0..3) that hold one query column
__device__ __forceinline__ float column_max(float v) {
    const uint32_t u = __float_as_uint(v);
    const auto a = __builtin_amdgcn_permlane32_swap(u, u, false, false);     // lanes l and l ^ 32
    const float m32 = max3(-INFINITY, __uint_as_float(a[0]), __uint_as_float(a[1]));
    const uint32_t w = __float_as_uint(m32);
    const auto b = __builtin_amdgcn_permlane16_swap(w, w, false, false);     // lanes l and l ^ 16
    return max3(-INFINITY, __uint_as_float(b[0]), __uint_as_float(b[1]));
}

// Running softmax state of the query heads a wavefront works on.
//   m: running maximum of (score * scale * log2 e) of this lane's column; l: this lane's share of
//   the running sum (its 8 keys of every block), reduced over the lanes of a column at the end
template <int D, int HPW>
struct HeadState {
    float m[HPW], l[HPW];
    f32x4_t o[HPW][D / 16];
};

// What a wavefront knows about the tile it works on (all wave-uniform but my_pos and my_lo).
struct TileView {
    int pos0;               // position of the tile's first query
    int last_key;           // newest key any query of the tile sees
    int last_lo;            // oldest key the tile's last query sees (0 without a window)
    int my_pos, my_lo;      // this lane's query column: its position and the oldest key it sees
};
