// The rules by which a step's kernels are chosen, in one place: the row counts up to which each family of
// matrix-product kernels is preferred, and when the decode attention splits a context over blocks. The step
// program (step_program.hip) is the only code that applies them; the Python side reads the numbers through
// tm_rule() where it sizes a buffer or checks an argument, and never decides by them.
#pragma once

// --- matrix products (bfloat16) ----------------------------------------------------------------------
// up to this many rows the kernels that stream the matrix once win: the products over packed matrices with
// the layer's epilogue (bias, rotary + cache write, SiLU*up, residual add), and the ones that start at the norm
constexpr int TM_SKINNY_ROWS = 16;
// ... while the model is narrow. They keep all of K of every row in LDS (or re-read the rows per block); beyond a
// width of 1,024 the products that stream the matrix through windows of K (gemm_stream.hip, with the partial sums
// of the output and down projections added by the next norm) take over at fewer rows, the wider the earlier.
// Measured on an MI355X, a decode step (ms) with this family against the stream family: width 896 (0.5B shape)
// 16 rows 1.16 against 1.23; width 1,536 (12 layers of 8,960) 8 rows 0.82 against 0.86, 16 rows 0.95 against 0.92;
// width 2,048 (12 layers of 11,008) 4 rows 0.85 against 0.99, 8 rows 0.90 against 1.00, 16 rows 1.10 against 1.06;
// width 3,584 (7B) 1 row 3.38 against 3.53, 4 rows 3.45 against 3.53, 8 rows 3.72 against 3.63, 16 rows 4.42 against
// 3.84; width 5,120 (32B, 16 layers) 1 row 3.64 against 3.49, 4 rows 3.80 against 3.44, 8 rows 4.10 against 3.56,
// 16 rows 4.92 against 3.81. The two families do not mix within a layer: the kernels that start at the norm need the
// residual stream complete, the stream family leaves partial sums for the norm.
inline int tm_skinny_rows(int hidden) { return hidden <= 1024 ? TM_SKINNY_ROWS : hidden < 3072 ? 8 : hidden < 4096 ? 4 : 0; }
// ... and the two of them that start at the norm (q|k|v, gate|up) at most to 8 rows: with 9 to 16 rows in LDS a CU
// holds one block (0.5B shape, 16 rows: 1.195 ms a step against 1.156 with the panel kernels behind a norm of its own)
inline int tm_from_norm_rows(int hidden) { const int s = tm_skinny_rows(hidden); return s < 8 ? s : 8; }
// q|k|v keeps the normed input in LDS behind a norm of its own up to this many rows where it fits (a width of at
// most 1,024): its matrix is small enough that the copy of the input is most of any kernel's work (measured at the
// 0.5B shape, 64 rows: 10.9 us against 14.9 us streamed). gate|up had such a kernel too; the stream product, with
// the tiles of tokens dealt to two groups of blocks beyond 32 rows, is as fast or faster at every row count (0.5B
// shape, a decode step of 12 / 24 / 32 / 48 requests: 1.07 / 1.29 / 1.34 / 1.54 ms against 1.08 / 1.32 / 1.38 / 1.54 ms).
constexpr int TM_PANEL_QKV_ROWS = 64;
// up to this many rows the products stream the packed matrix once for several row tiles, with their epilogues
constexpr int TM_STREAM_ROWS = 64;
// (a plain product of 17 to 64 rows, such as the output and down projections, is streamed where splitting its K over
// groups of blocks pays: tm_stream_linear_parts in gemm_stream.hip; else it is the library's)
// most rows one launch of the skinny product takes at all
constexpr int TM_SKINNY_MAX_ROWS = 64;
// most rows the 32-bit matrix-vector product takes
constexpr int TM_GEMV_F32_ROWS = 16;

// --- decode attention ---------------------------------------------------------------------------------
constexpr int TM_DECODE_CHUNK = 256;        // keys per block of the split decode attention
constexpr int TM_DECODE_SPLIT_PAIRS = 192;  // below this many (request, kv head) pairs the split kernels run

inline int tm_decode_chunks(int max_context) { return (max_context + TM_DECODE_CHUNK - 1) / TM_DECODE_CHUNK; }

// Does a decode step of `requests` single tokens split its contexts over blocks (and need the scratch
// memory for their partial results)?
inline bool tm_decode_splits(int requests, int kv_heads, int max_context) {
    return requests * kv_heads < TM_DECODE_SPLIT_PAIRS && tm_decode_chunks(max_context) > 1;
}

// --- prefill attention (bfloat16) ---------------------------------------------------------------------
// Two kernels: one whose wavefronts each load their own key blocks and split a tile's keys among them (many
// short chains: best for short prompts and for small head sizes), and one that stages a tile's keys and values
// through LDS once for all query heads of a kv head (twice the rate at head sizes above 64 from about a thousand
// tokens on, where the first is held back by one wavefront a SIMD). The second needs at least three wavefronts'
// worth of heads (two heads a wavefront) to fill a CU, and a launch of at least a block a CU.
inline bool tm_prefill_shares_keys(int D, int H, int KVH, int n_tiles) {
    const int G = H / KVH;
    return D > 64 && G >= 5 && G <= 16 && (long long)n_tiles * KVH >= 256;
}

// The split-keys kernel at head sizes up to 64 takes two heads a wavefront instead of four while the blocks that
// gives are no more than the chip runs at once (one a CU).
constexpr int TM_PREFILL_ONE_ROUND = 256;
