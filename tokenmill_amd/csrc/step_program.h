// C interface of the step program: a decoder's launch sequence as a list of operations that the parts
// fill once, run by one call per step (step_program.hip). All pointers are device pointers unless said
// otherwise; dtype codes as in api.h (0 = float32, 1 = bfloat16, -1 = none).
#pragma once
#include <hip/hip_runtime.h>
#include <stddef.h>

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

struct TmNorm {                 // weight * round(x * rsqrt(mean(x^2) + eps))
    const void* w;
    int w_dtype;
    float eps;
};

struct TmEmbedOp {
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

struct TmProgram;

// how an operation was computed, counted per program (tm_program_counters fills TM_PROGRAM_COUNTERS numbers)
enum {
    TM_QKV_FROM_NORM = 0,       // q|k|v by the kernel that starts at the norm (at most 16 tokens)
    TM_QKV_PANEL,               // ... by the kernel that keeps the normed input in LDS (17 to 48 tokens)
    TM_QKV_PLAIN,               // ... by a product, then rotation and cache write
    TM_GATE_UP_FROM_NORM,
    TM_GATE_UP_PANEL,
    TM_GATE_UP_PLAIN,           // a product with the SiLU*up epilogue, or a product and then SiLU*up
    TM_PROGRAM_COUNTERS
};
void tm_program_counters(const TmProgram* p, long long* out);

TmProgram* tm_program_create(int dtype, int hidden);
void tm_program_destroy(TmProgram* p);
int tm_program_set_embedding(TmProgram* p, const TmEmbedOp* e);
int tm_program_add_attention(TmProgram* p, const TmAttentionOp* a);
int tm_program_add_feed_forward(TmProgram* p, const TmFfnOp* f);
int tm_program_set_final(TmProgram* p, const TmFinalOp* f);
size_t tm_program_workspace_bytes(const TmProgram* p, int T, int R, int num_decode, int max_decode_context);
// workspace: at least tm_program_workspace_bytes(...) bytes, 256-byte aligned; library_workspace: what the
// library products may use; logits: float [R, vocab]. Runs the whole step on `stream`.
int tm_program_run(const TmProgram* p, const TmStep* s, void* workspace, size_t workspace_bytes, void* library_workspace,
                   size_t library_workspace_bytes, float* logits, hipStream_t stream);

}  // extern "C"
