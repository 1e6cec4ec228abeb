// bfloat16 attention over the paged cache on the matrix cores (v_mfma_f32_16x16x32_bf16).
//
// Compiled once per head size: -DSIA_HEAD_DIM=<multiple of 16, up to 256>.
//
// Both kernels walk the keys in tiles of 32 absolute positions (32t .. 32t+31) and keep the
// transposed problem, so that neither scores nor probabilities ever leave registers:
//
//   S^T[key, q] = K[key, :] . Q[q, :]          A = 16 key rows x 32 dims, B = Q^T, 2 x D/32 MFMAs
//   online softmax down each q column           a column lives in the 4 lanes {r, r+16, r+32, r+48}
//   O^T[d, q] += V^T[d, keys] . P^T[keys, q]    A = 16 dims x 32 keys, B = P^T, D/16 MFMAs
//
// An MFMA 16x16x32 gives lane (r = lane % 16, g = lane / 16) rows g*4 .. g*4+3 of column r of its
// result, and wants from it 8 consecutive k of row/column r, k = g*8 .. g*8+7, as operands.  The key
// rows of the two score MFMAs (h = 0, 1) are loaded in the order  key(row m) = 8(m/4) + 4h + m%4,
// so that what a lane holds of S^T afterwards is exactly the 8 keys 8g + (0..7) that it must supply
// as P^T to the value MFMAs: no shuffle, no LDS.  Keys are read straight from the pages
// ([page][kv_head][offset][dim], 16 bytes a lane), values too ([page][kv_head][dim][offset]: 8
// consecutive positions of one dim are 16 bytes).
//
// The loads of tile t+1 (16 KiB of keys and values a wave) are issued before the arithmetic of tile
// t: two register stages, used alternately.  The block-table entries a wave needs are held one per
// lane (64 consecutive entries) and fetched by lane shuffle, so that no load's address waits for
// another load.
//
// Scores are float, scaled after the dot; softmax statistics and the output accumulator are float;
// probabilities are rounded to bfloat16 for the value product (reference:
// kernels/attention_kernel.py:184-251 does the same in its prefill kernel).
//
// decode:  four waves per (split of the keys, kv head, sequence), each a contiguous quarter of the
//          split; the query heads that share the kv head are the q columns (at most 16).  The four
//          partial results are merged through LDS; (m, l, acc) per split go to a workspace and a
//          second kernel combines the splits in order.
// prefill: one wave per 16*NQ consecutive tokens of one query head; 4 waves a workgroup.
#include "common.h"

#ifndef SIA_HEAD_DIM
#error "compile with -DSIA_HEAD_DIM=<head size>"
#endif

constexpr int HD = SIA_HEAD_DIM;
static_assert(HD % 16 == 0 && HD >= 16 && HD <= 256, "head size must be a multiple of 16 up to 256");
constexpr int KSTEPS = (HD + 31) / 32;
constexpr int DBLOCKS = HD / 16;
constexpr int TILE = 32;

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

// 64 consecutive entries of a sequence's block table, one per lane.
struct PageWindow {
    int base;  // index of the entry that lane 0 holds
    int mine;
};

__device__ __forceinline__ void pages_load(PageWindow& w, const int* __restrict__ table, int table_width,
                                           int first, int lane) {
    w.base = first;
    w.mine = table[min(first + lane, table_width - 1)];
}

__device__ __forceinline__ int pages_get(const PageWindow& w, int index) {
    return max(__shfl(w.mine, index - w.base, SIA_WAVE), 0);
}

// Keys and values of one tile of 32 positions, as MFMA operands.
struct Stage {
    bf16x8 k[2][KSTEPS];
    bf16x8 v[DBLOCKS];
};

// Loads the tile at absolute position kb.  [load_lo, load_hi] is the wave-uniform range of keys whose
// pages exist; it must meet the tile.  Addresses of keys outside it are clamped into it, so every
// load is unconditional; what a clamped load brings is masked (scores) or multiplied by a zero
// probability (values).  The pages only ever hold finite numbers.
__device__ __forceinline__ void load_stage(Stage& st, const bf16_t* __restrict__ kp, const bf16_t* __restrict__ vp,
                                           const PageWindow& pages, int ps_log2, int n_kv, int hk, int kb,
                                           int load_lo, int load_hi) {
    const int lane = threadIdx.x & 63, r = lane & 15, g = lane >> 4;
    const int ps = 1 << ps_log2;
    const int t_lo = max(kb, load_lo), t_hi = min(kb + TILE - 1, load_hi);
#pragma unroll
    for (int h = 0; h < 2; ++h) {
        const int key = min(max(kb + (r >> 2) * 8 + h * 4 + (r & 3), t_lo), t_hi);
        const int page = pages_get(pages, key >> ps_log2);
        const bf16_t* row = kp + (((size_t)page * n_kv + hk) * ps + (key & (ps - 1))) * HD;
#pragma unroll
        for (int ks = 0; ks < KSTEPS; ++ks) {
            const int d0 = ks * 32 + g * 8;
            if (HD % 32 == 0 || ks < KSTEPS - 1)
                st.k[h][ks] = load8(row + d0);
            else
                st.k[h][ks] = d0 < HD ? load8(row + d0) : zero8();
        }
    }
    const int key0 = min(max(kb + g * 8, t_lo & ~7), t_hi & ~7);
    const int page = pages_get(pages, key0 >> ps_log2);
    const bf16_t* vbase = vp + ((size_t)page * n_kv + hk) * HD * ps + (key0 & (ps - 1));
#pragma unroll
    for (int db = 0; db < DBLOCKS; ++db) st.v[db] = load8(vbase + (size_t)(db * 16 + r) * ps);
}

// Scores, online softmax and value product of one loaded tile, for NQ groups of 16 q columns.
//   lo[n], hi[n]: visible keys of this lane's column in group n (hi < lo: none).
template <int NQ>
__device__ __forceinline__ void compute_stage(const Stage& st, const bf16x8 (&q)[NQ][KSTEPS], int kb,
                                              const int (&lo)[NQ], const int (&hi)[NQ], float scale,
                                              float (&m)[NQ], float (&l)[NQ], floatx4 (&acc)[NQ][DBLOCKS]) {
    const int g = (threadIdx.x & 63) >> 4;
    floatx4 s[NQ][2];
#pragma unroll
    for (int h = 0; h < 2; ++h) {
#pragma unroll
        for (int n = 0; n < NQ; ++n) s[n][h] = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int ks = 0; ks < KSTEPS; ++ks)
#pragma unroll
            for (int n = 0; n < NQ; ++n)
                s[n][h] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(st.k[h][ks], q[n][ks], s[n][h], 0, 0, 0);
    }
    bf16x8 p[NQ];
#pragma unroll
    for (int n = 0; n < NQ; ++n) {
        float mx = -INFINITY;
#pragma unroll
        for (int h = 0; h < 2; ++h)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int key = kb + g * 8 + h * 4 + i;
                const float v = (key >= lo[n] && key <= hi[n]) ? s[n][h][i] * scale : -INFINITY;
                s[n][h][i] = v;
                mx = fmaxf(mx, v);
            }
        mx = fmaxf(mx, __shfl_xor(mx, 16, SIA_WAVE));
        mx = fmaxf(mx, __shfl_xor(mx, 32, SIA_WAVE));
        const float m_new = fmaxf(m[n], mx);
        const float m_use = (m_new == -INFINITY) ? 0.f : m_new;  // a column that has seen no key yet
        const float alpha = __expf(m[n] - m_use);
        float sum = 0.f;
#pragma unroll
        for (int h = 0; h < 2; ++h)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const float e = __expf(s[n][h][i] - m_use);
                s[n][h][i] = e;
                sum += e;
            }
        sum += __shfl_xor(sum, 16, SIA_WAVE);
        sum += __shfl_xor(sum, 32, SIA_WAVE);
        l[n] = l[n] * alpha + sum;
        m[n] = m_new;
#pragma unroll
        for (int db = 0; db < DBLOCKS; ++db) acc[n][db] *= alpha;
        uint4 u;
        u.x = pack2(s[n][0][0], s[n][0][1]);
        u.y = pack2(s[n][0][2], s[n][0][3]);
        u.z = pack2(s[n][1][0], s[n][1][1]);
        u.w = pack2(s[n][1][2], s[n][1][3]);
        p[n] = __builtin_bit_cast(bf16x8, u);
    }
#pragma unroll
    for (int db = 0; db < DBLOCKS; ++db)
#pragma unroll
        for (int n = 0; n < NQ; ++n)
            acc[n][db] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(st.v[db], p[n], acc[n][db], 0, 0, 0);
}

// All tiles that meet [range_lo, range_hi] (range_lo <= range_hi), two register stages in turn.
template <int NQ>
__device__ __forceinline__ void attend_range(const bf16x8 (&q)[NQ][KSTEPS], const bf16_t* __restrict__ kp,
                                             const bf16_t* __restrict__ vp, const int* __restrict__ table,
                                             int table_width, int ps_log2, int n_kv, int hk, int range_lo,
                                             int range_hi, const int (&lo)[NQ], const int (&hi)[NQ], float scale,
                                             float (&m)[NQ], float (&l)[NQ], floatx4 (&acc)[NQ][DBLOCKS]) {
    const int lane = threadIdx.x & 63;
    const int kb_first = (range_lo / TILE) * TILE, kb_last = (range_hi / TILE) * TILE;
    PageWindow pages;
    pages_load(pages, table, table_width, range_lo >> ps_log2, lane);
    // Before a tile is loaded the window must hold its entries; it is moved when a tile's last entry
    // lies beyond it (every 64 pages).
    auto ensure = [&](int kb) {
        const int last_entry = min(kb + TILE - 1, range_hi) >> ps_log2;
        if (last_entry >= pages.base + SIA_WAVE)
            pages_load(pages, table, table_width, max(kb, range_lo) >> ps_log2, lane);
    };
    Stage a, b;
    load_stage(a, kp, vp, pages, ps_log2, n_kv, hk, kb_first, range_lo, range_hi);
    for (int kb = kb_first; kb <= kb_last; kb += 2 * TILE) {
        const int kb1 = min(kb + TILE, kb_last);  // past the end: the last tile again, never computed
        ensure(kb1);
        load_stage(b, kp, vp, pages, ps_log2, n_kv, hk, kb1, range_lo, range_hi);
        compute_stage<NQ>(a, q, kb, lo, hi, scale, m, l, acc);
        const int kb2 = min(kb + 2 * TILE, kb_last);
        ensure(kb2);
        load_stage(a, kp, vp, pages, ps_log2, n_kv, hk, kb2, range_lo, range_hi);
        if (kb + TILE <= kb_last) compute_stage<NQ>(b, q, kb + TILE, lo, hi, scale, m, l, acc);
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
constexpr int DEC_WAVES = 4;

__global__ __launch_bounds__(DEC_WAVES* SIA_WAVE) void attn_decode_kernel(
    const bf16_t* __restrict__ q, int q_row_stride, const bf16_t* __restrict__ kp, const bf16_t* __restrict__ vp,
    const int* __restrict__ block_table, int table_width, const int* __restrict__ cu_q,
    const int* __restrict__ kv_len, float* __restrict__ ws_acc, float* __restrict__ ws_ml, int n_heads, int n_kv,
    int ps_log2, float scale, int window, int split_keys, int max_splits) {
    extern __shared__ float lds[];  // [DEC_WAVES][group][HD + 2]
    const int split = blockIdx.x, hk = blockIdx.y, seq = blockIdx.z;
    const int wave = threadIdx.x / SIA_WAVE, lane = threadIdx.x & 63, r = lane & 15, g = lane >> 4;
    const int pos = kv_len[seq] - 1;
    const int lo_all = window > 0 ? max(0, pos - window + 1) : 0;
    const int s_lo = max(lo_all, split * split_keys);
    const int s_hi = min(pos, split * split_keys + split_keys - 1);
    if (s_hi < s_lo) return;  // the whole workgroup: this split holds no visible key

    const int group = n_heads / n_kv;
    const int part = split_keys / DEC_WAVES;
    const int w_lo = max(s_lo, split * split_keys + wave * part);
    const int w_hi = min(s_hi, split * split_keys + wave * part + part - 1);

    float m[1] = {-INFINITY}, l[1] = {0.f};
    floatx4 acc[1][DBLOCKS];
#pragma unroll
    for (int db = 0; db < DBLOCKS; ++db) acc[0][db] = floatx4{0.f, 0.f, 0.f, 0.f};

    if (w_lo <= w_hi) {  // wave-uniform
        const int token = cu_q[seq];
        bf16x8 qf[1][KSTEPS];
        load_q(qf[0], r < group ? q + (size_t)token * q_row_stride + (hk * group + r) * HD : nullptr, g);
        const int lo[1] = {r < group ? w_lo : 1}, hi[1] = {r < group ? w_hi : 0};
        attend_range<1>(qf, kp, vp, block_table + (size_t)seq * table_width, table_width, ps_log2, n_kv, hk, w_lo,
                        w_hi, lo, hi, scale, m, l, acc);
    }

    constexpr int ROW = HD + 2;
    if (r < group) {
        float* mine = lds + (size_t)(wave * group + r) * ROW;
        if (g == 0) {
            mine[HD] = m[0];
            mine[HD + 1] = l[0];
        }
#pragma unroll
        for (int db = 0; db < DBLOCKS; ++db)
#pragma unroll
            for (int i = 0; i < 4; ++i) mine[db * 16 + g * 4 + i] = acc[0][db][i];
    }
    __syncthreads();
    for (int idx = threadIdx.x; idx < group * HD; idx += DEC_WAVES * SIA_WAVE) {
        const int c = idx / HD, d = idx % HD;
        float mx = -INFINITY;
#pragma unroll
        for (int w = 0; w < DEC_WAVES; ++w) mx = fmaxf(mx, lds[(size_t)(w * group + c) * ROW + HD]);
        float o = 0.f, lsum = 0.f;
#pragma unroll
        for (int w = 0; w < DEC_WAVES; ++w) {
            const float* row = lds + (size_t)(w * group + c) * ROW;
            const float wgt = __expf(row[HD] - mx);  // a wave without keys has m = -inf: weight 0
            o += wgt * row[d];
            lsum += wgt * row[HD + 1];
        }
        const size_t slot = ((size_t)seq * n_heads + hk * group + c) * max_splits + split;
        ws_acc[slot * HD + d] = o;
        if (d == 0) {
            ws_ml[slot * 2] = mx;
            ws_ml[slot * 2 + 1] = lsum;
        }
    }
}

// Combines the splits of each (sequence, head): out = sum_s w_s acc_s / sum_s w_s l_s with
// w_s = exp(m_s - max m), summed in split order, eight splits' loads in flight at a time.
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
    for (int s0 = first; s0 <= last; s0 += SIA_WAVE) {
        const int s = s0 + lane;
        mx = fmaxf(mx, s <= last ? ws_ml[(base + s) * 2] : -INFINITY);
    }
    mx = wave_max(mx);
    float denom = 0.f;
    constexpr int DD = (HD + SIA_WAVE - 1) / SIA_WAVE;
    float o[DD];
#pragma unroll
    for (int dd = 0; dd < DD; ++dd) o[dd] = 0.f;
    for (int s0 = first; s0 <= last; s0 += 8) {
        float w[8], part[8][DD];
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const int s = min(s0 + j, last);  // a clamped slot is read again with weight 0
            const bool live = s0 + j <= last;
            w[j] = live ? __expf(ws_ml[(base + s) * 2] - mx) : 0.f;
            denom += live ? w[j] * ws_ml[(base + s) * 2 + 1] : 0.f;
#pragma unroll
            for (int dd = 0; dd < DD; ++dd) {
                const int d = lane + dd * SIA_WAVE;
                part[j][dd] = d < HD ? ws_acc[(base + s) * HD + d] : 0.f;
            }
        }
#pragma unroll
        for (int j = 0; j < 8; ++j)
#pragma unroll
            for (int dd = 0; dd < DD; ++dd) o[dd] += w[j] * part[j][dd];
    }
    const int token = cu_q[seq];
    bf16_t* dst = out + ((size_t)token * n_heads + head) * HD;
    const float inv = 1.f / denom;
#pragma unroll
    for (int dd = 0; dd < DD; ++dd) {
        const int d = lane + dd * SIA_WAVE;
        if (d < HD) dst[d] = float_to_bf16(o[dd] * inv);
    }
}

// ---------------------------------------------------------------------------------------------------
// prefill: runs of several tokens (works for single tokens too, without splitting the keys)
// ---------------------------------------------------------------------------------------------------
constexpr int PF_NQ = 2;                        // groups of 16 tokens per wave
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
    const int range_hi = first_pos + row_last;
    const int range_lo = window > 0 ? max(0, first_pos + row0 - window + 1) : 0;
    attend_range<PF_NQ>(qf, kp, vp, block_table + (size_t)seq * table_width, table_width, ps_log2, n_kv, hk,
                        range_lo, range_hi, lo, hi, scale, m, l, acc);

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
// max_splits * split_keys must cover the longest sequence; split_keys is a multiple of 128.
SIA_EXPORT int sia_attn_decode(const void* q, int q_row_stride, const void* k_pages, const void* v_pages,
                               const int* block_table, int table_width, const int* cu_q, const int* kv_len,
                               void* out, float* ws_acc, float* ws_ml, int n_seqs, int n_heads, int n_kv,
                               int page_size, float scale, int window, int split_keys, int max_splits,
                               hipStream_t stream) {
    if (n_seqs <= 0) return 0;
    const int ps_log2 = log2_exact(page_size);
    if (ps_log2 < 3 || n_kv <= 0 || n_heads % n_kv || n_heads / n_kv > 16 || split_keys % (DEC_WAVES * TILE) ||
        split_keys <= 0 || max_splits <= 0 || n_kv > 65535 || n_seqs > 65535 || q_row_stride % 8 || table_width <= 0)
        return SIA_BAD_ARGUMENT;
    const size_t lds_bytes = (size_t)DEC_WAVES * (n_heads / n_kv) * (HD + 2) * sizeof(float);
    if (lds_bytes > 64 * 1024) return SIA_BAD_ARGUMENT;
    hipLaunchKernelGGL(attn_decode_kernel, dim3(max_splits, n_kv, n_seqs), dim3(DEC_WAVES * SIA_WAVE), lds_bytes,
                       stream, (const bf16_t*)q, q_row_stride, (const bf16_t*)k_pages, (const bf16_t*)v_pages,
                       block_table, table_width, cu_q, kv_len, ws_acc, ws_ml, n_heads, n_kv, ps_log2, scale, window,
                       split_keys, max_splits);
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
    if (ps_log2 < 3 || n_kv <= 0 || n_heads % n_kv || n_heads > 65535 || q_row_stride % 8 || table_width <= 0)
        return SIA_BAD_ARGUMENT;
    hipLaunchKernelGGL(attn_prefill_kernel, dim3(n_tiles, n_heads), dim3(PF_WAVES * SIA_WAVE), 0, stream,
                       (const bf16_t*)q, q_row_stride, (const bf16_t*)k_pages, (const bf16_t*)v_pages, block_table,
                       table_width, cu_q, kv_len, (bf16_t*)out, n_heads, n_kv, ps_log2, scale, window, seq_begin,
                       seq_end);
    return SIA_LAUNCH_CHECK();
}
