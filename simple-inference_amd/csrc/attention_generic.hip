// Attention over the paged cache for any mix of prompt portions and decoded tokens:
// the plain kernel.  It takes every head size up to 256, any number of heads and groups,
// any page size and both element types, and is the kernel of the 32-bit path.
//
// One wavefront per (token, query head).  Keys are visited in chunks of 64 absolute
// positions (chunk c covers positions 64c .. 64c+63), so a token's result depends on its
// own position and keys only: not on how the prompt was cut into steps, on the other
// rows of the batch, or on which pages hold the keys.
//
//   s_j = (q . k_j) * scale                                   scale after the dot
//   visible: j <= pos, and j > pos - window if window > 0
//   online softmax over chunks: m' = max(m, max_j s_j); p_j = exp(s_j - m');
//   l = l * exp(m - m') + sum_j p_j;  acc = acc * exp(m - m') + sum_j p_j v_j;  o = acc / l
// (reference: kernels/attention_kernel.py:184-251, :516-586).  Everything is float.
#include "common.h"

#define ATTN_MAX_HEAD_DIM 256

template <typename T>
__global__ __launch_bounds__(SIA_WAVE) void attention_generic_kernel(
    const T* __restrict__ q, int q_row_stride, const T* __restrict__ k_pages, const T* __restrict__ v_pages,
    const int* __restrict__ block_table, int table_width, const int* __restrict__ seq_of_token,
    const int* __restrict__ positions, T* __restrict__ out, int n_heads, int n_kv, int head_dim,
    int page_size, float scale, int window) {
    __shared__ float q_s[ATTN_MAX_HEAD_DIM];
    __shared__ float p_s[SIA_WAVE];
    __shared__ int page_s[SIA_WAVE];

    const int n = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
    const int seq = seq_of_token[n];
    const int pos = positions[n];
    const int hk = h / (n_heads / n_kv);
    const int lo = window > 0 ? max(0, pos - window + 1) : 0;
    const int* table = block_table + (size_t)seq * table_width;

    const T* q_row = q + (size_t)n * q_row_stride + h * head_dim;
    for (int d = lane; d < head_dim; d += SIA_WAVE) q_s[d] = to_float(q_row[d]);
    __syncthreads();

    float m = -INFINITY, l = 0.f;
    float acc[ATTN_MAX_HEAD_DIM / SIA_WAVE] = {0.f, 0.f, 0.f, 0.f};

    for (int c0 = (lo / SIA_WAVE) * SIA_WAVE; c0 <= pos; c0 += SIA_WAVE) {
        const int j = c0 + lane;
        const bool visible = j >= lo && j <= pos;
        float s = -INFINITY;
        int page = -1;
        if (visible) page = table[j / page_size];
        if (page >= 0) {  // a missing page (never for a visible key of a sound table) gives NaN, not a fault
            const T* kp = k_pages + (((size_t)page * n_kv + hk) * page_size + (j % page_size)) * head_dim;
            float dot = 0.f;
            for (int d = 0; d < head_dim; ++d) dot += q_s[d] * to_float(kp[d]);
            s = dot * scale;
        }
        const float m_new = fmaxf(m, wave_max(s));  // finite: every chunk holds a visible key
        const float p = (visible && page >= 0) ? expf(s - m_new) : 0.f;
        const float alpha = expf(m - m_new);        // exp(-inf) = 0 on the first chunk
        l = l * alpha + wave_sum(p);
        m = m_new;
        p_s[lane] = p;
        page_s[lane] = page;
        __syncthreads();
        const int j_first = max(lo, c0) - c0, j_last = min(pos, c0 + SIA_WAVE - 1) - c0;
#pragma unroll
        for (int dd = 0; dd < ATTN_MAX_HEAD_DIM / SIA_WAVE; ++dd) {
            const int d = lane + dd * SIA_WAVE;
            if (d < head_dim) {
                float a = acc[dd] * alpha;
                for (int jj = j_first; jj <= j_last; ++jj) {
                    if (page_s[jj] < 0) continue;
                    const T* vp = v_pages + (((size_t)page_s[jj] * n_kv + hk) * head_dim + d) * page_size +
                                  ((c0 + jj) % page_size);
                    a += p_s[jj] * to_float(*vp);
                }
                acc[dd] = a;
            }
        }
        __syncthreads();
    }

    T* o = out + ((size_t)n * n_heads + h) * head_dim;
    const float inv = 1.f / l;
#pragma unroll
    for (int dd = 0; dd < ATTN_MAX_HEAD_DIM / SIA_WAVE; ++dd) {
        const int d = lane + dd * SIA_WAVE;
        if (d < head_dim) o[d] = from_float<T>(acc[dd] * inv);
    }
}

// The largest head size any attention kernel of this package takes (a model is checked against it when it is built).
SIA_EXPORT int sia_attention_max_head_dim() { return ATTN_MAX_HEAD_DIM; }

SIA_EXPORT int sia_attention_generic(const void* q, int q_row_stride, const void* k_pages, const void* v_pages,
                                     const int* block_table, int table_width, const int* seq_of_token,
                                     const int* positions, void* out, int n_tokens, int n_heads, int n_kv,
                                     int head_dim, int page_size, float scale, int window, int dtype,
                                     hipStream_t stream) {
    if (n_tokens <= 0) return 0;
    if (head_dim <= 0 || head_dim > ATTN_MAX_HEAD_DIM || n_kv <= 0 || n_heads % n_kv || page_size <= 0 ||
        n_heads > 65535)
        return SIA_BAD_ARGUMENT;
    dim3 grid(n_tokens, n_heads), block(SIA_WAVE);
#define LAUNCH(T)                                                                                              \
    hipLaunchKernelGGL(attention_generic_kernel<T>, grid, block, 0, stream, (const T*)q, q_row_stride,         \
                       (const T*)k_pages, (const T*)v_pages, block_table, table_width, seq_of_token, positions, \
                       (T*)out, n_heads, n_kv, head_dim, page_size, scale, window)
    if (dtype == SIA_F32) LAUNCH(float);
    else if (dtype == SIA_BF16) LAUNCH(bf16_t);
    else return SIA_BAD_ARGUMENT;
#undef LAUNCH
    return SIA_LAUNCH_CHECK();
}
