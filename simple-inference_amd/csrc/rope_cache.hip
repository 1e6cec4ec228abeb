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

// The same with 8 elements a thread (head_dim, rotary_dim / 2 and the row stride multiples of 8): a work
// item is a pair of 8-element pieces (i, i + rotary_dim / 2) of a q or k head, an unrotated piece of a k
// head, or a piece of a v head.  All of a token's loads are independent of one another.
template <typename T>
__global__ void rope_kv_write_vec_kernel(T* __restrict__ qkv, int row_stride, const float* __restrict__ cos_table,
                                         const float* __restrict__ sin_table, const int* __restrict__ positions,
                                         const int* __restrict__ seq_of_token, const int* __restrict__ block_table,
                                         int table_width, T* __restrict__ k_pages, T* __restrict__ v_pages,
                                         int n_heads, int n_kv, int head_dim, int rotary_dim, int page_size,
                                         int v_group) {
    const int n = blockIdx.x;
    const int pos = positions[n];
    const int half = rotary_dim / 2, pairs = half / 8, plain = (head_dim - rotary_dim) / 8, pieces = head_dim / 8;
    T* row = qkv + (size_t)n * row_stride;
    const float* cs = cos_table + (size_t)pos * half;
    const float* sn = sin_table + (size_t)pos * half;
    int page = -1, off = 0;
    if (n_kv > 0) {
        page = block_table[(size_t)seq_of_token[n] * table_width + pos / page_size];
        off = pos % page_size;
    }
    const int items_q = n_heads * pairs, items_kr = n_kv * pairs, items_kp = n_kv * plain;
    const int items_v = v_group ? 0 : n_kv * pieces;
    // with v_group the workgroup's last wave does nothing but the values (below), beside the others and not behind
    // them: what a token's workgroup takes is a chain of a few dependent loads, and two chains in turn last twice as long
    const int rotating = v_group ? (int)blockDim.x - SIA_WAVE : (int)blockDim.x;
    for (int item = threadIdx.x; item < items_q + items_kr + items_kp + items_v && (int)threadIdx.x < rotating;
         item += rotating) {
        if (item < items_q + items_kr) {  // a rotated pair of q (in place) or of k (into the page)
            const bool is_q = item < items_q;
            const int it = is_q ? item : item - items_q;
            const int h = it / pairs, j = (it % pairs) * 8;
            T* x = row + (is_q ? h : n_heads + h) * head_dim;
            Vec8<T> va, vb;
            Vec8<float> vc, vs;
            va.load(x + j);
            vb.load(x + j + half);
            vc.load(cs + j);
            vs.load(sn + j);
            float a[8], b[8], c[8], s[8], ra[8], rb[8];
            va.get(a); vb.get(b); vc.get(c); vs.get(s);
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                ra[i] = a[i] * c[i] - b[i] * s[i];
                rb[i] = b[i] * c[i] + a[i] * s[i];
            }
            va.set(ra);
            vb.set(rb);
            if (is_q) {
                va.store(x + j);
                vb.store(x + j + half);
            } else if (page >= 0) {
                T* dst = k_pages + (((size_t)page * n_kv + h) * page_size + off) * head_dim;
                va.store(dst + j);
                vb.store(dst + j + half);
            }
        } else if (item < items_q + items_kr + items_kp) {  // dims of k beyond the rotation
            const int it = item - items_q - items_kr;
            const int h = it / plain, j = rotary_dim + (it % plain) * 8;
            Vec8<T> v;
            v.load(row + (n_heads + h) * head_dim + j);
            if (page >= 0) v.store(k_pages + (((size_t)page * n_kv + h) * page_size + off) * head_dim + j);
        } else if (page >= 0 && v_group == 0) {  // v: 8 dims, each to its own row of the page (positions are innermost there)
            const int it = item - items_q - items_kr - items_kp;
            const int h = it / pieces, j = (it % pieces) * 8;
            const T* x = row + (n_heads + n_kv + h) * head_dim + j;
            T* dst = v_pages + (((size_t)page * n_kv + h) * head_dim + j) * page_size + off;
#pragma unroll
            for (int i = 0; i < 8; ++i) dst[(size_t)i * page_size] = x[i];
        }
    }
    if (v_group == 0 || page < 0 || (int)threadIdx.x < rotating) return;
    const int lane = threadIdx.x - rotating;
    // v, for pages of 8 or 16 positions and more.  Positions are innermost in a page, so where v_group consecutive
    // tokens of one sequence fill an aligned run of a page, their workgroups share the work by dims, not by tokens:
    // each takes a slice of the (head, dim) rows and writes all the group's positions of a row at once (16 or 32
    // contiguous bytes in bfloat16, neighbouring lanes neighbouring rows), instead of one element per token and row.
    const int seq = seq_of_token[n];
    const int place = off % v_group, first = n - place, rows = n_kv * head_dim;
    const bool whole = first >= 0 && first + v_group <= (int)gridDim.x && seq_of_token[first] == seq &&
                       seq_of_token[first + v_group - 1] == seq && positions[first] == pos - place &&
                       positions[first + v_group - 1] == pos - place + v_group - 1;
    if (!whole) {  // an incomplete group: every token writes its own values
        const T* x = row + (n_heads + n_kv) * head_dim;
        for (int i = lane; i < rows; i += SIA_WAVE)
            v_pages[((size_t)page * rows + i) * page_size + off] = x[i];
        return;
    }
    constexpr int V_MAX = 16;
    const int slice = (rows + v_group - 1) / v_group;
    const T* x0 = qkv + (size_t)first * row_stride + (n_heads + n_kv) * head_dim;
    for (int i = place * slice + lane; i < min(rows, (place + 1) * slice); i += SIA_WAVE) {
        __attribute__((aligned(16))) T vals[V_MAX];
#pragma unroll
        for (int j = 0; j < V_MAX; ++j) vals[j] = j < v_group ? x0[(size_t)j * row_stride + i] : T(0);
        T* dst = v_pages + ((size_t)page * rows + i) * page_size + (off - place);
        constexpr int PER = 16 / sizeof(T);  // elements of a 16-byte store
#pragma unroll
        for (int j = 0; j < V_MAX; j += PER)
            if (j < v_group) *reinterpret_cast<uint4*>(dst + j) = *reinterpret_cast<const uint4*>(vals + j);
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
    dim3 grid(n_tokens);
    const bool vec = head_dim % 8 == 0 && rotary_dim % 16 == 0 && row_stride % 8 == 0;
    // tokens whose values one workgroup writes together (0: every token its own); needs runs aligned to 16 bytes
    const int v_group = (n_kv > 0 && n_tokens > 1 && page_size % 16 == 0) ? 16 : (n_kv > 0 && n_tokens > 1 && page_size % 8 == 0) ? 8 : 0;
    const int items = vec ? (n_heads + n_kv) * (rotary_dim / 16) + n_kv * ((head_dim - rotary_dim) / 8 + head_dim / 8) : 0;
    // with v_group one wave more, which writes the values
    // With many tokens a thread takes four items in turn: workgroups of fewer waves, so that all of a long step's are
    // on the chip at once (2,048 tokens: 14.0 -> 11.4 us; 512 tokens are faster with a thread for every item).
    const int per = n_tokens >= 1024 ? 4 : 1;
    const int want = (items + per - 1) / per;
    dim3 block(vec ? min(1024 - SIA_WAVE, max(SIA_WAVE, (want + SIA_WAVE - 1) / SIA_WAVE * SIA_WAVE)) + (v_group ? SIA_WAVE : 0)
                   : 256);
#define LAUNCH(T)                                                                                             \
    do {                                                                                                      \
        if (vec)                                                                                              \
            hipLaunchKernelGGL(rope_kv_write_vec_kernel<T>, grid, block, 0, stream, (T*)qkv, row_stride,      \
                               cos_table, sin_table, positions, seq_of_token, block_table, table_width,       \
                               (T*)k_pages, (T*)v_pages, n_heads, n_kv, head_dim, rotary_dim, page_size,      \
                               v_group);                                                                      \
        else                                                                                                  \
            hipLaunchKernelGGL(rope_kv_write_kernel<T>, grid, block, 0, stream, (T*)qkv, row_stride,          \
                               cos_table, sin_table, positions, seq_of_token, block_table, table_width,       \
                               (T*)k_pages, (T*)v_pages, n_heads, n_kv, head_dim, rotary_dim, page_size);     \
    } while (0)
    if (dtype == SIA_F32) LAUNCH(float);
    else if (dtype == SIA_BF16) LAUNCH(bf16_t);
    else return SIA_BAD_ARGUMENT;
#undef LAUNCH
    return SIA_LAUNCH_CHECK();
}
