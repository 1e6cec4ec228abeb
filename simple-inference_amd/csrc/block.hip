// One pre-norm block (attention with rotation over the paged cache, SwiGLU feed-forward, RMS norms) of a step of
// many rows, as one call: the launches that the parts' own calls would make one by one, in the same order, on the
// same buffers.  Nothing is computed here; it spares the host the way through the interpreter between the launches,
// which in a step of a few hundred tokens of a small model takes longer than the GPU needs for them.  The matrix
// products and the matrix-core attention live in other libraries: the caller hands their entry points in.
#include "common.h"

extern "C" {
int sia_add_rmsnorm(float* residual, const void* delta, const float* weight, void* out, const int* rows, int n_out,
                    int hidden, float eps, int dtype, hipStream_t stream);
int sia_swiglu(const void* gu, void* out, int n_tokens, int inter, int dtype, hipStream_t stream);
int sia_rope_kv_write(void* qkv, int row_stride, const float* cos_table, const float* sin_table, const int* positions,
                      const int* seq_of_token, const int* block_table, int table_width, void* k_pages, void* v_pages,
                      int n_tokens, int n_heads, int n_kv, int head_dim, int rotary_dim, int page_size, int dtype,
                      hipStream_t stream);
}

typedef int (*ProductFn)(const void* X, const void* W, void* Y, int M, int N, int K, int out_float, hipStream_t stream);
typedef int (*DecodeFn)(const void* q, int q_row_stride, const void* k_pages, const void* v_pages,
                        const int* block_table, int table_width, const int* cu_q, const int* kv_len, void* out,
                        float* ws_acc, float* ws_ml, int n_seqs, int n_heads, int n_kv, int page_size, float scale,
                        int window, int max_splits, hipStream_t stream);
typedef int (*PrefillFn)(const void* q, int q_row_stride, const void* k_pages, const void* v_pages,
                         const int* block_table, int table_width, const int* cu_q, const int* kv_len, void* out,
                         int seq_begin, int seq_end, int n_tiles, int n_tiles_split, int n_tiles_long, int q_bound,
                         int kv_bound, int n_heads, int n_kv, int page_size, float scale, int window,
                         hipStream_t stream);

// What a block owns: its weights (bfloat16 matrices [out, in], float gains) and its constants.
struct SiaBlockOwn {
    const float* mixer_norm_gain;
    const void* w_qkv;
    const void* w_o;
    const float* feed_forward_norm_gain;
    const void* w_gate_up;
    const void* w_down;
    const float* cos_table;  // null without rotation
    const float* sin_table;
    float mixer_norm_eps, feed_forward_norm_eps, scale;
    int hidden, n_heads, n_kv, head_dim, rotary_dim, inter, window;
};

// What a step owns, the same for every block of the same geometry: its metadata, the buffers between the launches
// (bfloat16, each used by one block after the other) and how its attention is launched.
struct SiaBlockStep {
    ProductFn product;
    DecodeFn attend_single;   // sequences that bring one token
    PrefillFn attend_runs;    // the others
    float* residual;          // [tokens, hidden]
    void* normed;             // [tokens, hidden]
    void* qkv;                // [tokens, (n_heads + 2 n_kv) head_dim]
    void* attended;           // [tokens, n_heads head_dim]
    void* mixed;              // [tokens, hidden]: the mixer's output
    void* gate_up;            // [tokens, 2 inter]
    void* activated;          // [tokens, inter]
    void* fed;                // [tokens, hidden]: the feed-forward's output, the delta of the next block
    const int* positions;
    const int* seq_of_token;
    const int* cu_q;
    const int* kv_len;
    float* ws_acc;
    float* ws_ml;
    int n_tokens, n_seqs, n_single, max_splits, n_tiles, n_tiles_split, n_tiles_long, q_bound, kv_bound;
};

#define SIA_STEP(call)             \
    do {                           \
        const int rc_ = (call);    \
        if (rc_ != 0) return rc_;  \
    } while (0)

// residual += delta (where there is one); then the block.  Leaves the block's last product in S->fed, not yet added.
// block_table [n_seqs, table_width], k_pages, v_pages: the block's cache in this step.  0, or the first launch's error.
SIA_EXPORT int sia_prenorm_block(const SiaBlockOwn* B, const SiaBlockStep* S, const void* delta, const int* block_table,
                                 int table_width, void* k_pages, void* v_pages, int page_size, hipStream_t stream) {
    if (!B || !S || !S->product || !S->attend_runs || S->n_tokens <= 0 || S->n_tokens > 65535) return SIA_BAD_ARGUMENT;
    const int M = S->n_tokens, H = B->hidden, Q = B->n_heads * B->head_dim;
    const int qkv_width = (B->n_heads + 2 * B->n_kv) * B->head_dim;
    SIA_STEP(sia_add_rmsnorm(S->residual, delta, B->mixer_norm_gain, S->normed, nullptr, M, H, B->mixer_norm_eps,
                             SIA_BF16, stream));
    SIA_STEP(S->product(S->normed, B->w_qkv, S->qkv, M, qkv_width, H, 0, stream));
    SIA_STEP(sia_rope_kv_write(S->qkv, qkv_width, B->cos_table, B->sin_table, S->positions, S->seq_of_token,
                               block_table, table_width, k_pages, v_pages, M, B->n_heads, B->n_kv, B->head_dim,
                               B->rotary_dim, page_size, SIA_BF16, stream));
    if (S->n_single > 0) {
        if (!S->attend_single) return SIA_BAD_ARGUMENT;
        SIA_STEP(S->attend_single(S->qkv, qkv_width, k_pages, v_pages, block_table, table_width, S->cu_q, S->kv_len,
                                  S->attended, S->ws_acc, S->ws_ml, S->n_single, B->n_heads, B->n_kv, page_size,
                                  B->scale, B->window, S->max_splits, stream));
    }
    if (S->n_single < S->n_seqs)
        SIA_STEP(S->attend_runs(S->qkv, qkv_width, k_pages, v_pages, block_table, table_width, S->cu_q, S->kv_len,
                                S->attended, S->n_single, S->n_seqs, S->n_tiles, S->n_tiles_split, S->n_tiles_long,
                                S->q_bound, S->kv_bound, B->n_heads, B->n_kv, page_size, B->scale, B->window, stream));
    SIA_STEP(S->product(S->attended, B->w_o, S->mixed, M, H, Q, 0, stream));
    SIA_STEP(sia_add_rmsnorm(S->residual, S->mixed, B->feed_forward_norm_gain, S->normed, nullptr, M, H,
                             B->feed_forward_norm_eps, SIA_BF16, stream));
    SIA_STEP(S->product(S->normed, B->w_gate_up, S->gate_up, M, 2 * B->inter, H, 0, stream));
    SIA_STEP(sia_swiglu(S->gate_up, S->activated, M, B->inter, SIA_BF16, stream));
    SIA_STEP(S->product(S->activated, B->w_down, S->fed, M, H, B->inter, 0, stream));
    return 0;
}
