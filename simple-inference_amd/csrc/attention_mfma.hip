// bfloat16 attention over the paged cache on the matrix cores (v_mfma_f32_16x16x32_bf16).
//
// Compiled once per head size: -DSIA_HEAD_DIM=<multiple of 16, up to 256>.
//
// Both kernels work on tiles of 64 keys at absolute positions 64t .. 64t+63 and keep the
// transposed problem, so that neither the scores nor the probabilities ever leave registers:
//
//   S^T[key, q] = K[key, :] . Q[q, :]          A = 16 key rows x 32 dims, B = Q^T, 4 x D/32 MFMAs
//   online softmax down each q column           a column lives in the 4 lanes {r, r+16, r+32, r+48}
//   O^T[d, q] += V^T[d, keys] . P^T[keys, q]    A = 16 dims x 32 keys, B = P^T, D/16 x 2 MFMAs
//
// An MFMA 16x16x32 gives lane (r = lane % 16, g = lane / 16) rows g*4 .. g*4+3 of column r of its
// result, and wants from it 8 consecutive k of row/column r, k = g*8 .. g*8+7, as operands.  The key
// rows of the score MFMAs are loaded in the order  key(row m of block 2c+h) = 32c + 8(m/4) + 4h + m%4,
// so that what a lane holds of S^T after the four score blocks is exactly the 2 x 8 keys
// 32c + 8g + (0..7) that it must supply as P^T to the two value MFMAs: no shuffle, no LDS.
// Keys are read straight from the pages ([page][kv_head][offset][dim], 16 bytes a lane), values too
// ([page][kv_head][dim][offset]: 8 consecutive positions of one dim are 16 bytes).
//
// Scores are float, scaled after the dot; softmax statistics and the output accumulator are float;
// probabilities are rounded to bfloat16 for the value product (reference: kernels/attention_kernel.py:
// 184-251 does the same in its prefill kernel).
//
// decode:  one wave per (split of the keys, kv head, sequence); the query heads that share the kv
//          head are the q columns (at most 16).  Partial (m, l, acc) per split go to a workspace and
//          a second kernel combines them in split order.
// prefill: one wave per 16*NQ consecutive tokens of one query head; 4 waves a workgroup.
#include "common.h"

#ifndef SIA_HEAD_DIM
#error "compile with -DSIA_HEAD_DIM=<head size>"
#endif

constexpr int HD = SIA_HEAD_DIM;
static_assert(HD % 16 == 0 && HD >= 16 && HD <= 256, "head size must be a multiple of 16 up to 256");
constexpr int KSTEPS = (HD + 31) / 32;
constexpr int DBLOCKS = HD / 16;
constexpr int TILE = 64;

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float floatx4;

__device__ __forceinline__ bf16x8 load8(const bf16_t* p) {
    return __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(p));
}
__device__ __forceinline__ bf16x8 zero8() {
    return __builtin_bit_cast(bf16x8, make_uint4(0u, 0u, 0u, 0u));
}
__device__ __forceinline__ uint32_t pack2(float lo, float hi) {
    return (uint32_t)float_to_bf16(lo) | ((uint32_t)float_to_bf16(hi) << 16);
}

// One tile of 64 keys starting at absolute position kb, for NQ groups of 16 q columns.
//   lo[n], hi[n]: visible keys of this lane's column in group n (hi < lo: none).
//   load_lo, load_hi: wave-uniform range outside which keys are not read (their pages may not exist).
template <int NQ>
__device__ __forceinline__ void attn_tile(const bf16x8 (&q)[NQ][KSTEPS], const bf16_t* __restrict__ kp,
                                          const bf16_t* __restrict__ vp, const int* __restrict__ table,
                                          int ps_log2, int n_kv, int hk, int kb, const int (&lo)[NQ],
                                          const int (&hi)[NQ], int load_lo, int load_hi, float scale,
                                          float (&m)[NQ], float (&l)[NQ], floatx4 (&acc)[NQ][DBLOCKS]) {
    const int lane = threadIdx.x & 63, r = lane & 15, g = lane >> 4;
    const int ps = 1 << ps_log2;
    floatx4 s[NQ][4];

#pragma unroll
    for (int b = 0; b < 4; ++b) {
        const int c = b >> 1, h = b & 1;
        const int key = kb + c * 32 + (r >> 2) * 8 + h * 4 + (r & 3);
        const bf16_t* krow = nullptr;
        if (key >= load_lo && key <= load_hi) {
            const int page = table[key >> ps_log2];
            if (page >= 0) krow = kp + (((size_t)page * n_kv + hk) * ps + (key & (ps - 1))) * HD;
        }
#pragma unroll
        for (int n = 0; n < NQ; ++n) s[n][b] = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int ks = 0; ks < KSTEPS; ++ks) {
            const int d0 = ks * 32 + g * 8;
            const bf16x8 a = (krow != nullptr && d0 < HD) ? load8(krow + d0) : zero8();
#pragma unroll
            for (int n = 0; n < NQ; ++n)
                s[n][b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, q[n][ks], s[n][b], 0, 0, 0);
        }
    }

    bf16x8 p[NQ][2];
#pragma unroll
    for (int n = 0; n < NQ; ++n) {
        float mx = -INFINITY;
#pragma unroll
        for (int b = 0; b < 4; ++b)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int key = kb + (b >> 1) * 32 + g * 8 + (b & 1) * 4 + i;
                const float v = (key >= lo[n] && key <= hi[n]) ? s[n][b][i] * scale : -INFINITY;
                s[n][b][i] = v;
                mx = fmaxf(mx, v);
            }
        mx = fmaxf(mx, __shfl_xor(mx, 16, SIA_WAVE));
        mx = fmaxf(mx, __shfl_xor(mx, 32, SIA_WAVE));
        const float m_new = fmaxf(m[n], mx);
        const float m_use = (m_new == -INFINITY) ? 0.f : m_new;  // a column that has seen no key yet
        const float alpha = __expf(m[n] - m_use);
        float sum = 0.f;
#pragma unroll
        for (int b = 0; b < 4; ++b)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const float e = __expf(s[n][b][i] - m_use);
                s[n][b][i] = e;
                sum += e;
            }
        sum += __shfl_xor(sum, 16, SIA_WAVE);
        sum += __shfl_xor(sum, 32, SIA_WAVE);
        l[n] = l[n] * alpha + sum;
        m[n] = m_new;
#pragma unroll
        for (int db = 0; db < DBLOCKS; ++db) acc[n][db] *= alpha;
#pragma unroll
        for (int c = 0; c < 2; ++c) {
            uint4 u;
            u.x = pack2(s[n][2 * c][0], s[n][2 * c][1]);
            u.y = pack2(s[n][2 * c][2], s[n][2 * c][3]);
            u.z = pack2(s[n][2 * c + 1][0], s[n][2 * c + 1][1]);
            u.w = pack2(s[n][2 * c + 1][2], s[n][2 * c + 1][3]);
            p[n][c] = __builtin_bit_cast(bf16x8, u);
        }
    }

#pragma unroll
    for (int c = 0; c < 2; ++c) {
        const int key0 = kb + c * 32 + g * 8;
        const bf16_t* vbase = nullptr;
        if (key0 <= load_hi && key0 + 7 >= load_lo) {
            const int page = table[key0 >> ps_log2];
            if (page >= 0) vbase = vp + ((size_t)page * n_kv + hk) * HD * ps + (key0 & (ps - 1));
        }
#pragma unroll
        for (int db = 0; db < DBLOCKS; ++db) {
            const bf16x8 a = vbase != nullptr ? load8(vbase + (size_t)(db * 16 + r) * ps) : zero8();
#pragma unroll
            for (int n = 0; n < NQ; ++n)
                acc[n][db] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, p[n][c], acc[n][db], 0, 0, 0);
        }
    }
}

// q operand of column r: 8 dims d0 .. d0+7 of that column's query row (zeros if the column is unused).
__device__ __forceinline__ void load_q(bf16x8 (&q)[KSTEPS], const bf16_t* row, int g) {
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ++ks) {
        const int d0 = ks * 32 + g * 8;
        q[ks] = (row != nullptr && d0 < HD) ? load8(row + d0) : zero8();
    }
}

// ---------------------------------------------------------------------------------------------------
// decode: sequences with one new token each
// ---------------------------------------------------------------------------------------------------
__global__ __launch_bounds__(SIA_WAVE) void attn_decode_kernel(
    const bf16_t* __restrict__ q, int q_row_stride, const bf16_t* __restrict__ kp, const bf16_t* __restrict__ vp,
    const int* __restrict__ block_table, int table_width, const int* __restrict__ cu_q,
    const int* __restrict__ kv_len, float* __restrict__ ws_acc, float* __restrict__ ws_ml, int n_heads, int n_kv,
    int ps_log2, float scale, int window, int split_keys, int max_splits) {
    const int split = blockIdx.x, hk = blockIdx.y, seq = blockIdx.z;
    const int lane = threadIdx.x, r = lane & 15, g = lane >> 4;
    const int pos = kv_len[seq] - 1;
    const int lo_all = window > 0 ? max(0, pos - window + 1) : 0;
    const int s_lo = max(lo_all, split * split_keys);
    const int s_hi = min(pos, split * split_keys + split_keys - 1);
    if (s_hi < s_lo) return;

    const int group = n_heads / n_kv;
    const int token = cu_q[seq];
    const int head = hk * group + r;
    bf16x8 qf[1][KSTEPS];
    load_q(qf[0], r < group ? q + (size_t)token * q_row_stride + head * HD : nullptr, g);

    const int lo[1] = {r < group ? s_lo : 1}, hi[1] = {r < group ? s_hi : 0};
    float m[1] = {-INFINITY}, l[1] = {0.f};
    floatx4 acc[1][DBLOCKS];
#pragma unroll
    for (int db = 0; db < DBLOCKS; ++db) acc[0][db] = floatx4{0.f, 0.f, 0.f, 0.f};

    const int* table = block_table + (size_t)seq * table_width;
    for (int kb = (s_lo / TILE) * TILE; kb <= s_hi; kb += TILE)
        attn_tile<1>(qf, kp, vp, table, ps_log2, n_kv, hk, kb, lo, hi, s_lo, s_hi, scale, m, l, acc);

    if (r < group) {
        const size_t slot = ((size_t)seq * n_heads + head) * max_splits + split;
        if (g == 0) {
            ws_ml[slot * 2] = m[0];
            ws_ml[slot * 2 + 1] = l[0];
        }
        float* dst = ws_acc + slot * HD;
#pragma unroll
        for (int db = 0; db < DBLOCKS; ++db)
            *reinterpret_cast<floatx4*>(dst + db * 16 + g * 4) = acc[0][db];
    }
}

// Combines the splits of each (sequence, head) in split order.
__global__ __launch_bounds__(SIA_WAVE) void attn_decode_combine_kernel(
    const float* __restrict__ ws_acc, const float* __restrict__ ws_ml, const int* __restrict__ cu_q,
    const int* __restrict__ kv_len, bf16_t* __restrict__ out, int n_heads, int window, int split_keys,
    int max_splits) {
    const int head = blockIdx.x, seq = blockIdx.y, lane = threadIdx.x;
    const int pos = kv_len[seq] - 1;
    const int lo_all = window > 0 ? max(0, pos - window + 1) : 0;
    const int first = lo_all / split_keys, last = pos / split_keys;
    const size_t base = ((size_t)seq * n_heads + head) * max_splits;
    float mx = -INFINITY;
    for (int s = first; s <= last; ++s) mx = fmaxf(mx, ws_ml[(base + s) * 2]);
    float denom = 0.f;
    float o[(HD + SIA_WAVE - 1) / SIA_WAVE] = {0.f};
    for (int s = first; s <= last; ++s) {
        const float w = __expf(ws_ml[(base + s) * 2] - mx);
        denom += w * ws_ml[(base + s) * 2 + 1];
#pragma unroll
        for (int dd = 0; dd < (HD + SIA_WAVE - 1) / SIA_WAVE; ++dd) {
            const int d = lane + dd * SIA_WAVE;
            if (d < HD) o[dd] += w * ws_acc[(base + s) * HD + d];
        }
    }
    const int token = cu_q[seq];
    bf16_t* dst = out + ((size_t)token * n_heads + head) * HD;
    const float inv = 1.f / denom;
#pragma unroll
    for (int dd = 0; dd < (HD + SIA_WAVE - 1) / SIA_WAVE; ++dd) {
        const int d = lane + dd * SIA_WAVE;
        if (d < HD) dst[d] = float_to_bf16(o[dd] * inv);
    }
}

// ---------------------------------------------------------------------------------------------------
// prefill: runs of several tokens (works for single tokens too, without splitting the keys)
// ---------------------------------------------------------------------------------------------------
constexpr int PF_NQ = 2;                   // groups of 16 tokens per wave
constexpr int PF_WAVES = 4;
constexpr int PF_ROWS = PF_WAVES * PF_NQ * 16;  // tokens per workgroup

__global__ __launch_bounds__(PF_WAVES* SIA_WAVE) void attn_prefill_kernel(
    const bf16_t* __restrict__ q, int q_row_stride, const bf16_t* __restrict__ kp, const bf16_t* __restrict__ vp,
    const int* __restrict__ block_table, int table_width, const int* __restrict__ cu_q,
    const int* __restrict__ kv_len, bf16_t* __restrict__ out, int n_heads, int n_kv, int ps_log2, float scale,
    int window, int seq_begin, int seq_end) {
    // which sequence and which of its row tiles this workgroup has
    int tile = blockIdx.x, seq = seq_begin;
    for (; seq < seq_end; ++seq) {
        const int tiles = (cu_q[seq + 1] - cu_q[seq] + PF_ROWS - 1) / PF_ROWS;
        if (tile < tiles) break;
        tile -= tiles;
    }
    if (seq >= seq_end) return;
    const int head = blockIdx.y, hk = head / (n_heads / n_kv);
    const int wave = threadIdx.x / SIA_WAVE, lane = threadIdx.x & 63, r = lane & 15, g = lane >> 4;
    const int q_begin = cu_q[seq], q_len = cu_q[seq + 1] - q_begin;
    const int first_pos = kv_len[seq] - q_len;
    const int row0 = tile * PF_ROWS + wave * PF_NQ * 16;  // this wave's first row within the sequence's run
    if (row0 >= q_len) return;
    const int row_last = min(q_len - 1, row0 + PF_NQ * 16 - 1);

    bf16x8 qf[PF_NQ][KSTEPS];
    int lo[PF_NQ], hi[PF_NQ];
    float m[PF_NQ], l[PF_NQ];
    floatx4 acc[PF_NQ][DBLOCKS];
#pragma unroll
    for (int n = 0; n < PF_NQ; ++n) {
        const int row = row0 + n * 16 + r;
        const bool live = row < q_len;
        const int qpos = first_pos + row;
        load_q(qf[n], live ? q + (size_t)(q_begin + row) * q_row_stride + head * HD : nullptr, g);
        hi[n] = live ? qpos : 0;
        lo[n] = live ? (window > 0 ? max(0, qpos - window + 1) : 0) : 1;
        m[n] = -INFINITY;
        l[n] = 0.f;
#pragma unroll
        for (int db = 0; db < DBLOCKS; ++db) acc[n][db] = floatx4{0.f, 0.f, 0.f, 0.f};
    }
    const int load_hi = first_pos + row_last;
    const int load_lo = window > 0 ? max(0, first_pos + row0 - window + 1) : 0;
    const int* table = block_table + (size_t)seq * table_width;
    for (int kb = (load_lo / TILE) * TILE; kb <= load_hi; kb += TILE)
        attn_tile<PF_NQ>(qf, kp, vp, table, ps_log2, n_kv, hk, kb, lo, hi, load_lo, load_hi, scale, m, l, acc);

#pragma unroll
    for (int n = 0; n < PF_NQ; ++n) {
        const int row = row0 + n * 16 + r;
        if (row >= q_len) continue;
        const float inv = 1.f / l[n];
        bf16_t* dst = out + ((size_t)(q_begin + row) * n_heads + head) * HD;
#pragma unroll
        for (int db = 0; db < DBLOCKS; ++db) {
            uint2 u;
            u.x = pack2(acc[n][db][0] * inv, acc[n][db][1] * inv);
            u.y = pack2(acc[n][db][2] * inv, acc[n][db][3] * inv);
            *reinterpret_cast<uint2*>(dst + db * 16 + g * 4) = u;
        }
    }
}

// ---------------------------------------------------------------------------------------------------
// entry points
// ---------------------------------------------------------------------------------------------------
static int log2_exact(int v) {
    int l = 0;
    while ((1 << l) < v) ++l;
    return (1 << l) == v ? l : -1;
}

SIA_EXPORT int sia_attn_mfma_head_dim() { return HD; }

// Sequences 0 .. n_seqs-1 of the step, each with exactly one new token.  ws_acc holds
// n_seqs * n_heads * max_splits * head_dim floats and ws_ml twice n_seqs * n_heads * max_splits;
// max_splits * split_keys must cover the longest sequence.
SIA_EXPORT int sia_attn_decode(const void* q, int q_row_stride, const void* k_pages, const void* v_pages,
                               const int* block_table, int table_width, const int* cu_q, const int* kv_len,
                               void* out, float* ws_acc, float* ws_ml, int n_seqs, int n_heads, int n_kv,
                               int page_size, float scale, int window, int split_keys, int max_splits,
                               hipStream_t stream) {
    if (n_seqs <= 0) return 0;
    const int ps_log2 = log2_exact(page_size);
    if (ps_log2 < 3 || n_kv <= 0 || n_heads % n_kv || n_heads / n_kv > 16 || split_keys % TILE || split_keys <= 0 ||
        max_splits <= 0 || n_kv > 65535 || n_seqs > 65535 || q_row_stride % 8)
        return SIA_BAD_ARGUMENT;
    hipLaunchKernelGGL(attn_decode_kernel, dim3(max_splits, n_kv, n_seqs), dim3(SIA_WAVE), 0, stream,
                       (const bf16_t*)q, q_row_stride, (const bf16_t*)k_pages, (const bf16_t*)v_pages, block_table,
                       table_width, cu_q, kv_len, ws_acc, ws_ml, n_heads, n_kv, ps_log2, scale, window, split_keys,
                       max_splits);
    hipLaunchKernelGGL(attn_decode_combine_kernel, dim3(n_heads, n_seqs), dim3(SIA_WAVE), 0, stream, ws_acc, ws_ml,
                       cu_q, kv_len, (bf16_t*)out, n_heads, window, split_keys, max_splits);
    return SIA_LAUNCH_CHECK();
}

// Sequences seq_begin .. seq_end-1 of the step; n_tiles = sum over them of ceil(q_len / rows per workgroup).
SIA_EXPORT int sia_attn_prefill_rows() { return PF_ROWS; }

SIA_EXPORT int sia_attn_prefill(const void* q, int q_row_stride, const void* k_pages, const void* v_pages,
                                const int* block_table, int table_width, const int* cu_q, const int* kv_len,
                                void* out, int seq_begin, int seq_end, int n_tiles, int n_heads, int n_kv,
                                int page_size, float scale, int window, hipStream_t stream) {
    if (seq_end <= seq_begin || n_tiles <= 0) return 0;
    const int ps_log2 = log2_exact(page_size);
    if (ps_log2 < 3 || n_kv <= 0 || n_heads % n_kv || n_heads > 65535 || q_row_stride % 8) return SIA_BAD_ARGUMENT;
    hipLaunchKernelGGL(attn_prefill_kernel, dim3(n_tiles, n_heads), dim3(PF_WAVES * SIA_WAVE), 0, stream,
                       (const bf16_t*)q, q_row_stride, (const bf16_t*)k_pages, (const bf16_t*)v_pages, block_table,
                       table_width, cu_q, kv_len, (bf16_t*)out, n_heads, n_kv, ps_log2, scale, window, seq_begin,
                       seq_end);
    return SIA_LAUNCH_CHECK();
}
