// What the decode-step products that end in a layer's own epilogue share: their arguments, the pair
// of matrix strips a block multiplies, small helpers.
#pragma once
#include "common.h"

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));
typedef float f32x2_t __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));

union FFrag {
    u32x4_t u;
    bf16x8_t b;
};

__device__ __forceinline__ uint32_t fd_pack(float a, float b) {
    const bf16x2_t v = __builtin_convertvector(f32x2_t{a, b}, bf16x2_t);
    return *(const uint32_t*)&v;
}

__device__ __forceinline__ float fd_round(float a) { return bf16_to_f32(f32_to_bf16(a)); }

#define FD_EPI_QKV 0
#define FD_EPI_SILU 1
#define FD_KCH 8            // k-steps of one register group of matrix loads, per wavefront (one group in all)
#define FD_KCH_PIPE 6       // the same where two groups take turns
#define FD_XPAD 16          // padding of an LDS row of x, in elements: with K a multiple of 32 the rows are 32 bytes more than a multiple of 64 apart, which the operand loads read free of bank conflicts (with 8 they take twice as long)
#define FD_RC 8             // 4-element vectors of a residual row a thread keeps in registers

// rows of x a block keeps in LDS for M tokens
__host__ __device__ __forceinline__ int fused_rows(int M) { return M <= 4 ? 4 : (M <= 8 ? 8 : 16); }

struct FusedArgs {
    // norm + product
    const float* resid;     // [M, K] (the kernel that starts at the norm)
    const bf16_t* X;        // [M, K], rows ldx apart: the normed input (the kernel that starts behind the norm)
    int ldx;
    const void* norm_w;     // [K]
    int norm_w_f32;
    float eps;
    int M, K;
    const bf16_t* W;        // the matrix in strip order (see tm_pack_layout in api.h), strips of the kernel's ROWS
    int up_strip0;          // SiLU epilogue: index of the first strip of the up rows
    const void* bias;       // [rows] or null
    int bias_f32;
    // QKV epilogue
    bf16_t* q_out;          // [M, H*D]
    int H, KVH, D;
    const float* cos_t;     // [max_pos, D/2]
    const float* sin_t;
    const int* positions;   // [M]
    const int* slots;       // [M]; < 0: not stored
    bf16_t* k_pool;         // [pages, page, KVH, D]
    bf16_t* v_pool;         // [pages, KVH, D, page]
    int page_shift;
    // SiLU epilogue
    bf16_t* act_out;        // [M, I]
    int I;
};

// The two strips of ROWS matrix rows a block multiplies together ("unit" u).
struct FusedUnit {
    int nA, nB;             // first rows of the strips
    int sA, sB;             // their indices in the packed matrix
    int head, jt;           // QKV: the head and which slice of it
    bool rows_ok;           // this lane's rows exist
};


// Unit u of a product whose strips have ROWS rows.
template <int EPI, int ROWS>
__device__ __forceinline__ FusedUnit fused_unit_of(const FusedArgs& a, int u, int r) {
    FusedUnit t;
    t.head = 0;
    t.jt = 0;
    t.rows_ok = r < ROWS;
    if (EPI == FD_EPI_QKV) {
        const int per_head = a.D / (2 * ROWS);
        t.head = u / per_head;
        t.jt = u % per_head;
        if (t.head < a.H + a.KVH) {                                  // the two halves of ROWS rotary pairs
            t.nA = t.head * a.D + ROWS * t.jt;
            t.nB = t.nA + a.D / 2;
        } else {
            t.nA = t.head * a.D + 2 * ROWS * t.jt;
            t.nB = t.nA + ROWS;
        }
        t.sA = t.nA / ROWS;                                          // D % 32 == 0: every strip starts on a multiple of ROWS
        t.sB = t.nB / ROWS;
    } else {                                                         // gate rows and the up rows that meet them
        t.nA = ROWS * u;
        t.nB = a.I + ROWS * u;
        t.sA = u;
        t.sB = a.up_strip0 + u;                                      // (rows beyond I are zeros in the packed matrix)
    }
    return t;
}
