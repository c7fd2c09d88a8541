// C interface of the step program: a decoder's launch sequence as a list of operations that the parts
// describe once, run by one call per run of consecutive operations (step_program.hip). All pointers are
// device pointers unless said otherwise; dtype codes as in api.h (0 = float32, 1 = bfloat16, -1 = none).
#pragma once
#include <hip/hip_runtime.h>
#include <stddef.h>

#include "api.h"

#define TM_MAX_GROUPS 8

extern "C" {

struct TmLinear {               // y = x W^T + b, W [N, K]
    const void* w;              // row-major [N, K]
    const void* packed;         // the same matrix in strip order (api.h), or null
    const void* bias;           // [N] or null
    int packed_rows;            // rows of a strip of `packed`
    int packed_parts;           // 1, or 2 when a stacked matrix was packed part by part (gate, up)
    int bias_dtype;             // -1 without bias
    int N, K;
    int dtype;                  // type of w
    int library_first;          // the owner asks for the library's product at any row count (an output head)
};

struct TmNorm {                 // weight * round(x * rsqrt(mean(x^2) + eps)); w null: the operation has no norm of
    const void* w;              // its own and is always handed its input already normed (TmStream::x)
    int w_dtype;
    float eps;
};

struct TmEmbedOp {              // resid = table[token_ids]
    const void* table;          // [V, hidden]
    int dtype;
    int V, hidden;
};

struct TmAttentionOp {          // resid += o(attention(rope(qkv(norm(resid)))))
    TmNorm norm;
    TmLinear qkv, o;
    const float* cos_t;         // [max_positions, rot / 2], or null when rot == 0
    const float* sin_t;
    void* k_pool;               // [pages, page, KVH, D]
    void* v_pool;               // [pages, KVH, D, page]
    int H, KVH, D;
    float scale;
    int window;                 // 0: every key
    int rot;                    // rotary width (0: no rotation)
    int max_positions;          // rows of the rotary tables
    int page;
    int group;                  // which of the step's block tables and slot mappings
    int write;                  // 0: this call reads a cache that another call writes
};

struct TmFfnOp {                // resid += down(silu(gate(n)) * up(n)), n = norm(resid)
    TmNorm norm;
    TmLinear gate_up, down;
    int I;
};

struct TmFinalOp {              // logits = head(norm(resid[rows]))
    TmNorm norm;
    TmLinear head;
};

struct TmStep {                 // one step's metadata: host scalars and device arrays (int32)
    int T, S, R;                // tokens, requests, logit rows
    int num_decode;             // the last num_decode requests bring one token each
    int max_context_len;        // >= every request's length after this step
    int max_decode_context;     // >= the length of every single-token request
    int n_tiles;
    int num_groups;
    const int* token_ids;       // [T]
    const int* positions;       // [T]
    const int* seq_of_token;    // [T]
    const int* context_lens;    // [S]
    const int* logit_rows;      // [R]
    const int* prefill_tiles;   // [n_tiles, 4]
    const int* block_tables[TM_MAX_GROUPS];     // [S, table_width[g]]
    const int* slot_mapping[TM_MAX_GROUPS];     // [T]
    int table_width[TM_MAX_GROUPS];
};

// What crosses from one operation to the next, and into and out of a run of operations.
struct TmStream {
    float* resid;               // the 32-bit residual stream [T, hidden]; null only with accumulate == 0 and x or qkv given
    const void* delta;          // in: a result [T, hidden] (model type) still to be added to resid, or null;
                                // out: what the run's last operation left to be added (it lies in the workspace), or null
    const void* x;              // in: the first operation's input [T, hidden], already normed (its norm is skipped), or null
    const void* qkv;            // in: q|k|v [T, (H + 2 KVH) D] of the first operation (an attention), already projected,
                                // position-encoded and stored in the cache (only attention and output projection run), or null
    int accumulate;             // 0: nothing is added into resid by an operation's last product: its result is left in `delta`
};

struct TmProgram;

// how an operation was computed, counted per program (tm_program_counters fills TM_PROGRAM_COUNTERS numbers)
enum {
    TM_QKV_FROM_NORM = 0,       // q|k|v by the kernel that starts at the norm (at most 16 tokens)
    TM_QKV_PANEL,               // ... by the kernel that keeps the normed input in LDS (17 to 64 tokens)
    TM_QKV_STREAM,              // ... by the kernel that streams the packed matrix for up to 64 tokens
    TM_QKV_PLAIN,               // ... by a product, then rotation and cache write
    TM_GATE_UP_FROM_NORM,
    TM_GATE_UP_STREAM,
    TM_GATE_UP_PLAIN,           // a product with the SiLU*up epilogue, or a product and then SiLU*up
    TM_PREFILL_SPLIT_KEYS,      // bfloat16 attention of prompt portions: wavefronts split a tile's key blocks
    TM_PREFILL_SHARED_KEYS,     // ... a tile's keys and values staged through LDS for all heads of a kv head
    TM_PROGRAM_COUNTERS
};
void tm_program_counters(const TmProgram* p, long long* out);

// The spans of a run that a profile tells apart. While labels are asked for (TM_RUN_LABELS), `hook(user, op,
// label, 1)` is called on the host before the span's launches and `hook(user, op, label, 0)` after them; op is
// the operation's index in the program.
enum { TM_LABEL_EMBED = 0, TM_LABEL_QKV, TM_LABEL_ATTENTION, TM_LABEL_O_PROJ, TM_LABEL_GATE_UP, TM_LABEL_DOWN,
       TM_LABEL_NORM, TM_LABEL_HEAD, TM_LABELS };
typedef void (*TmHook)(void* user, int op, int label, int begin);

enum { TM_RUN_LABELS = 1,           // call the hook around every labelled span
       TM_RUN_TUNE_AT_ONCE = 2 };   // a library product's algorithms are timed at this call (the step is about to be captured)

TmProgram* tm_program_create(int dtype, int hidden);
void tm_program_destroy(TmProgram* p);
// Each returns the new operation's index, or -1 for a description the library does not run.
int tm_program_add_embedding(TmProgram* p, const TmEmbedOp* e);
int tm_program_add_attention(TmProgram* p, const TmAttentionOp* a);
int tm_program_add_feed_forward(TmProgram* p, const TmFfnOp* f);
int tm_program_add_head(TmProgram* p, const TmFinalOp* f);
void tm_program_set_hook(TmProgram* p, TmHook hook, void* user);
// The library products of this program time up to `candidates` algorithms per shape (0: the library's first choice).
int tm_program_set_tune(TmProgram* p, int candidates, int every);
size_t tm_program_workspace_bytes(const TmProgram* p, int T, int R, int num_decode, int max_decode_context);
// Runs operations [first, first + count) on `stream`. workspace: at least tm_program_workspace_bytes(...) bytes,
// 256-byte aligned, the same for every run of one step; library_workspace: what the library products may use;
// logits: float [R, vocab], written by a head operation. flags: TM_RUN_*.
int tm_program_run(const TmProgram* p, int first, int count, const TmStep* s, TmStream* io, void* workspace,
                   size_t workspace_bytes, void* library_workspace, size_t library_workspace_bytes, float* logits,
                   int flags, hipStream_t stream);

// One product by the rules the program's operations use: out[M, N] = x[M, K] W^T + b in `out_dtype`, or with
// `accum` (float32 [M, N], row stride ldacc) the result, rounded to the matrix's type, added there where a kernel
// does that in its epilogue (tm_linear_accumulates says whether; then `out` is not written).
int tm_linear_accumulates(const TmLinear* L, int x_dtype, const void* x, int ldx, int M);
int tm_linear_run(const TmLinear* L, int x_dtype, const void* x, int ldx, int M, void* out, int ldc, int out_dtype,
                  float* accum, int ldacc, void* library_workspace, size_t library_workspace_bytes, const TmTune* tune,
                  hipStream_t stream);

// A number of choose.h by name ("skinny_rows", "panel_qkv_rows", "stream_rows", "skinny_max_rows", "gemv_f32_rows",
// "decode_chunk", "decode_split_pairs"); -1 for a name it does not know.
int tm_rule(const char* name);
// Chunks a decode step's contexts are split into, or 0 if this step does not split them.
int tm_decode_split_chunks(int requests, int kv_heads, int max_context);

}  // extern "C"
