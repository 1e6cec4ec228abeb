// Rotary position encoding of q and k, fused with the write of k and v into the cache pages.
//
// One workgroup per token.  The projected row is [q heads | k heads | v heads], each head
// head_dim wide.  q is rotated in place; k is rotated and stored at the token's position in
// its page; v is stored as it is.  Rotation pairs element i with i + rotary_dim/2 (reference:
// ops/rope.py:167-182):  a' = a cos - b sin,  b' = b cos + a sin,  with float cos/sin taken from
// a table row of the token's absolute position (reference: ops/rope.py:108-118) and float
// arithmetic, rounded once (reference: kernels/rope_kernel.py:131-154).  Elements beyond
// rotary_dim pass through.
//
// Page layout:  keys   [page][kv_head][offset][dim]
//               values [page][kv_head][dim][offset]      (positions innermost)
// The page of position p of sequence s is block_table[s][p / page_size].
#include "common.h"

template <typename T>
__global__ void rope_kv_write_kernel(T* __restrict__ qkv, int row_stride,
                                     const float* __restrict__ cos_table, const float* __restrict__ sin_table,
                                     const int* __restrict__ positions, const int* __restrict__ seq_of_token,
                                     const int* __restrict__ block_table, int table_width,
                                     T* __restrict__ k_pages, T* __restrict__ v_pages,
                                     int n_heads, int n_kv, int head_dim, int rotary_dim, int page_size) {
    const int n = blockIdx.x;
    const int pos = positions[n];
    const int half = rotary_dim / 2;
    T* row = qkv + (size_t)n * row_stride;
    const float* cs = cos_table + (size_t)pos * half;
    const float* sn = sin_table + (size_t)pos * half;

    // q: in place, one thread per rotary pair.
    for (int i = threadIdx.x; i < n_heads * half; i += blockDim.x) {
        const int h = i / half, j = i % half;
        T* x = row + h * head_dim;
        const float a = to_float(x[j]), b = to_float(x[j + half]);
        const float c = cs[j], s = sn[j];
        x[j] = from_float<T>(a * c - b * s);
        x[j + half] = from_float<T>(b * c + a * s);
    }
    if (n_kv == 0) return;

    const int seq = seq_of_token[n];
    const int page = block_table[(size_t)seq * table_width + pos / page_size];
    if (page < 0) return;  // never for a token the step owns; keeps a bad table from writing out of bounds
    const int off = pos % page_size;
    const T* k_row = row + n_heads * head_dim;
    const T* v_row = k_row + n_kv * head_dim;

    for (int i = threadIdx.x; i < n_kv * head_dim; i += blockDim.x) {
        const int h = i / head_dim, d = i % head_dim;
        const T* x = k_row + h * head_dim;
        float val;
        if (d < half) {
            val = to_float(x[d]) * cs[d] - to_float(x[d + half]) * sn[d];
        } else if (d < rotary_dim) {
            val = to_float(x[d]) * cs[d - half] + to_float(x[d - half]) * sn[d - half];
        } else {
            val = to_float(x[d]);
        }
        k_pages[(((size_t)page * n_kv + h) * page_size + off) * head_dim + d] = from_float<T>(val);
        v_pages[(((size_t)page * n_kv + h) * head_dim + d) * page_size + off] = v_row[i];
    }
}

SIA_EXPORT int sia_rope_kv_write(void* qkv, int row_stride, const float* cos_table, const float* sin_table,
                                 const int* positions, const int* seq_of_token, const int* block_table,
                                 int table_width, void* k_pages, void* v_pages, int n_tokens, int n_heads,
                                 int n_kv, int head_dim, int rotary_dim, int page_size, int dtype,
                                 hipStream_t stream) {
    if (n_tokens <= 0) return 0;
    if (rotary_dim < 0 || rotary_dim > head_dim || (rotary_dim & 1)) return SIA_BAD_ARGUMENT;
    if (n_kv > 0 && (!k_pages || !v_pages || !block_table || page_size <= 0)) return SIA_BAD_ARGUMENT;
    if (rotary_dim > 0 && (!cos_table || !sin_table)) return SIA_BAD_ARGUMENT;
    dim3 grid(n_tokens), block(256);
#define LAUNCH(T)                                                                                         \
    hipLaunchKernelGGL(rope_kv_write_kernel<T>, grid, block, 0, stream, (T*)qkv, row_stride, cos_table,   \
                       sin_table, positions, seq_of_token, block_table, table_width, (T*)k_pages,         \
                       (T*)v_pages, n_heads, n_kv, head_dim, rotary_dim, page_size)
    if (dtype == SIA_F32) LAUNCH(float);
    else if (dtype == SIA_BF16) LAUNCH(bf16_t);
    else return SIA_BAD_ARGUMENT;
#undef LAUNCH
    return SIA_LAUNCH_CHECK();
}
