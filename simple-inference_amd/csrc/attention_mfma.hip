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
// decode:  workgroups of four waves; a (kv head, sequence) is shared by as many of them ("splits") as its own
//          number of visible key tiles says (decode_splits below: a power of two that leaves a wave some four
//          tiles), never by how many sequences the step holds or how long the others are: the grid is sized for
//          the longest sequence the step may hold, and workgroups beyond a sequence's own count leave at once.
//          The sequence's tiles are dealt evenly, in order, to these waves (runs differ by a tile at most); the
//          query heads that share the kv head are the q columns (at most 16).  A workgroup's four partial results
//          are merged through LDS; (m, l, acc) per split go to a workspace and a second kernel combines the
//          splits in order (a sequence with a single split writes its result itself).  So a sequence's result
//          depends on its own keys and length only, bit for bit, whatever else is in the batch.
// prefill: 128 consecutive tokens of one query head a workgroup (64 for head sizes over 128), as 4 waves of 32
//          tokens or 8 waves of 16; the waves share each tile of keys and values through LDS (two stages;
//          head sizes whose stages fit 64 KiB, the others load operands straight from the pages).
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
// Two floats to two bfloat16 (round to nearest even) with the hardware's packed conversion.
typedef __attribute__((__vector_size__(2 * sizeof(__bf16)))) __bf16 bf16x2;
typedef __attribute__((__vector_size__(2 * sizeof(float)))) float floatx2;
__device__ __forceinline__ uint32_t pack2(float lo, float hi) {
    const floatx2 f = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(f, bf16x2));
}
// 2^x by the hardware instruction; arguments here are <= 0 or -inf, results in [0, 1].
__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }
constexpr float LOG2E = 1.4426950408889634f;

// Maximum and sum over the four lanes r, r+16, r+32, r+48 that share a q column, for every lane, by the
// register swaps between the wave's rows of 16 lanes (no trip through LDS as a general lane shuffle makes):
// v_permlane16_swap exchanges rows 1, 3 of its first operand with rows 0, 2 of its second, v_permlane32_swap
// the upper half of the first with the lower half of the second; either way the two results hold, lane by
// lane, the two values to combine.  The sum is (row 0 + row 1) + (row 2 + row 3) in every lane.
__device__ __forceinline__ float column_max(float v) {
    uint32_t u = __float_as_uint(v);
    const auto a = __builtin_amdgcn_permlane16_swap(u, u, false, false);
    u = __float_as_uint(fmaxf(__uint_as_float(a[0]), __uint_as_float(a[1])));
    const auto b = __builtin_amdgcn_permlane32_swap(u, u, false, false);
    return fmaxf(__uint_as_float(b[0]), __uint_as_float(b[1]));
}
__device__ __forceinline__ float column_sum(float v) {
    uint32_t u = __float_as_uint(v);
    const auto a = __builtin_amdgcn_permlane16_swap(u, u, false, false);
    u = __float_as_uint(__uint_as_float(a[0]) + __uint_as_float(a[1]));
    const auto b = __builtin_amdgcn_permlane32_swap(u, u, false, false);
    return __uint_as_float(b[0]) + __uint_as_float(b[1]);
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

// What a wave keeps of the softmax of its q columns, per group n of 16 columns.  A column (one query) lives in the
// four lanes r, r + 16, r + 32, r + 48, each of which sees 8 of a tile's 32 keys.
//   m:   the column's *reference*, in units of log2: exponentials are taken as 2^(s * scale_log2 - m).  It follows
//        the running maximum lazily: it moves up to the maximum only when the maximum has grown more than
//        SOFTMAX_SLACK beyond it.  Exponentials are then at most 2^SOFTMAX_SLACK instead of 1, which float sums and
//        bfloat16 probabilities hold just as well, and (m, l, acc) stay a consistent triple, so acc / l is the
//        same value.  The same in all four lanes of a column.
//   mu:  m, or 0 while the column has seen no key (m = -inf).
//   l:   this lane's part of the sum of exponentials (its 8 keys of every tile); the four lanes' parts are added
//        once, at the end (finish_sums).
// The point of the lazy reference: a tile on which no column's reference moves (nearly all of them) costs no
// exchange between lanes and no rescaling of the accumulators (4 * DBLOCKS registers a column group), only a
// maximum, a multiply-add and an exponential per score.  Whether a column's reference moves depends on that
// column's scores alone, never on its neighbours in the wave.
constexpr float SOFTMAX_SLACK = 8.f;

template <int NQ>
struct Softmax {
    float m[NQ], mu[NQ], l[NQ];
    __device__ __forceinline__ void start() {
#pragma unroll
        for (int n = 0; n < NQ; ++n) {
            m[n] = -INFINITY;
            mu[n] = 0.f;
            l[n] = 0.f;
        }
    }
    // after the last tile: l becomes the column's whole sum, in every lane
    __device__ __forceinline__ void finish_sums() {
#pragma unroll
        for (int n = 0; n < NQ; ++n) l[n] = column_sum(l[n]);
    }
};

// max without the quieting of signalling NaNs that fmaxf owes the standard (scores are never NaN)
__device__ __forceinline__ float max2(float a, float b) { return __builtin_fmaxf(a, b); }

// Masks the scores of a tile, updates the softmax state of each q column, rescales the accumulators where a
// reference moved, and returns the tile's probabilities as the P^T operand.
//   lo[n], hi[n]: visible keys of this lane's column in group n (hi < lo: none).
//   scale_log2 = scale * log2(e) > 0.
// A tile that every column of the wave sees whole skips the masking (the test is wave-uniform).
template <int NQ>
__device__ __forceinline__ void softmax_update(floatx4 (&s)[NQ][2], int kb, const int (&lo)[NQ], const int (&hi)[NQ],
                                               float scale_log2, Softmax<NQ>& sm, floatx4 (&acc)[NQ][DBLOCKS],
                                               bf16x8 (&p)[NQ]) {
    const int g = (threadIdx.x & 63) >> 4;
    float top[NQ];
    bool grew = false;
#pragma unroll
    for (int n = 0; n < NQ; ++n) {
        if (!__all(kb >= lo[n] && kb + TILE - 1 <= hi[n])) {
#pragma unroll
            for (int h = 0; h < 2; ++h)
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const int key = kb + g * 8 + h * 4 + i;
                    if (key < lo[n] || key > hi[n]) s[n][h][i] = -INFINITY;
                }
        }
        top[n] = max2(max2(max2(s[n][0][0], s[n][0][1]), max2(s[n][0][2], s[n][0][3])),
                      max2(max2(s[n][1][0], s[n][1][1]), max2(s[n][1][2], s[n][1][3]))) * scale_log2;
        grew |= top[n] > sm.m[n] + SOFTMAX_SLACK;   // also a column's first visible key (m = -inf)
    }
    if (__builtin_expect(__any(grew), 0)) {
#pragma unroll
        for (int n = 0; n < NQ; ++n) {
            const float mx = column_max(top[n]);
            const bool moved = mx > sm.m[n] + SOFTMAX_SLACK;
            const float alpha = moved ? fast_exp2(sm.m[n] - mx) : 1.f;   // from -inf: 0 (there is nothing yet)
            sm.m[n] = moved ? mx : sm.m[n];
            sm.mu[n] = sm.m[n] == -INFINITY ? 0.f : sm.m[n];
            sm.l[n] *= alpha;
#pragma unroll
            for (int db = 0; db < DBLOCKS; ++db) acc[n][db] *= alpha;
        }
    }
#pragma unroll
    for (int n = 0; n < NQ; ++n) {
        float sum = 0.f;
#pragma unroll
        for (int h = 0; h < 2; ++h)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const float e = fast_exp2(fmaf(s[n][h][i], scale_log2, -sm.mu[n]));
                s[n][h][i] = e;
                sum += e;
            }
        sm.l[n] += sum;
        uint4 u;
        u.x = pack2(s[n][0][0], s[n][0][1]);
        u.y = pack2(s[n][0][2], s[n][0][3]);
        u.z = pack2(s[n][1][0], s[n][1][1]);
        u.w = pack2(s[n][1][2], s[n][1][3]);
        p[n] = __builtin_bit_cast(bf16x8, u);
    }
}

// Scores, online softmax and value product of one tile held in registers.
template <int NQ>
__device__ __forceinline__ void compute_stage(const Stage& st, const bf16x8 (&q)[NQ][KSTEPS], int kb,
                                              const int (&lo)[NQ], const int (&hi)[NQ], float scale,
                                              Softmax<NQ>& sm, floatx4 (&acc)[NQ][DBLOCKS]) {
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
    softmax_update<NQ>(s, kb, lo, hi, scale, sm, acc, p);
#pragma unroll
    for (int db = 0; db < DBLOCKS; ++db)
#pragma unroll
        for (int n = 0; n < NQ; ++n)
            acc[n][db] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(st.v[db], p[n], acc[n][db], 0, 0, 0);
}

// Called before a tile is computed; the default does nothing.
struct NoHook {
    __device__ __forceinline__ void operator()(int) const {}
};

// The tiles w_first, w_first + TILE, ..., w_last, whose block-table entries the window holds; two register
// stages in turn: the loads of tile t+1 are issued before the arithmetic of tile t.  `before(kb)` runs before the
// arithmetic of the tile at kb (it may hand the state on and start it afresh).
template <int NQ, typename Hook>
__device__ __forceinline__ void attend_tiles(const PageWindow& pages, int w_first, int w_last,
                                             const bf16x8 (&q)[NQ][KSTEPS], const bf16_t* __restrict__ kp,
                                             const bf16_t* __restrict__ vp, int ps_log2, int n_kv, int hk,
                                             int range_lo, int range_hi, const int (&lo)[NQ], const int (&hi)[NQ],
                                             float scale, Softmax<NQ>& sm, floatx4 (&acc)[NQ][DBLOCKS], Hook& before) {
    Stage a, b;
    load_stage(a, kp, vp, pages, ps_log2, n_kv, hk, w_first, range_lo, range_hi);
    for (int kb = w_first; kb <= w_last; kb += 2 * TILE) {
        const int kb1 = min(kb + TILE, w_last);  // past the end: the last tile again, never computed
        load_stage(b, kp, vp, pages, ps_log2, n_kv, hk, kb1, range_lo, range_hi);
        before(kb);
        compute_stage<NQ>(a, q, kb, lo, hi, scale, sm, acc);
        const int kb2 = min(kb + 2 * TILE, w_last);
        load_stage(a, kp, vp, pages, ps_log2, n_kv, hk, kb2, range_lo, range_hi);
        if (kb + TILE <= w_last) {
            before(kb + TILE);
            compute_stage<NQ>(b, q, kb + TILE, lo, hi, scale, sm, acc);
        }
    }
}

// All tiles that meet [range_lo, range_hi] (range_lo <= range_hi).  The block-table window (64 entries,
// starting at the page of the first tile it serves) is loaded outside the pipelined loop, once per 64
// pages: a load inside it would make every iteration wait for all outstanding loads.
template <int NQ, typename Hook>
__device__ __forceinline__ void attend_range(const bf16x8 (&q)[NQ][KSTEPS], const bf16_t* __restrict__ kp,
                                             const bf16_t* __restrict__ vp, const int* __restrict__ table,
                                             int table_width, int ps_log2, int n_kv, int hk, int range_lo,
                                             int range_hi, const int (&lo)[NQ], const int (&hi)[NQ], float scale,
                                             Softmax<NQ>& sm, floatx4 (&acc)[NQ][DBLOCKS], Hook& before) {
    const int lane = threadIdx.x & 63;
    const int kb_first = (range_lo / TILE) * TILE, kb_last = (range_hi / TILE) * TILE;
    for (int w_first = kb_first; w_first <= kb_last;) {
        const int first_page = w_first >> ps_log2;
        const int w_end = (first_page + SIA_WAVE) << ps_log2;  // first key beyond the window, a multiple of TILE
        PageWindow pages;
        pages_load(pages, table, table_width, first_page, lane);
        attend_tiles<NQ>(pages, w_first, min(kb_last, w_end - TILE), q, kp, vp, ps_log2, n_kv, hk, range_lo, range_hi,
                         lo, hi, scale, sm, acc, before);
        w_first = w_end;
    }
}

template <int NQ>
__device__ __forceinline__ void attend_range(const bf16x8 (&q)[NQ][KSTEPS], const bf16_t* __restrict__ kp,
                                             const bf16_t* __restrict__ vp, const int* __restrict__ table,
                                             int table_width, int ps_log2, int n_kv, int hk, int range_lo,
                                             int range_hi, const int (&lo)[NQ], const int (&hi)[NQ], float scale,
                                             Softmax<NQ>& sm, floatx4 (&acc)[NQ][DBLOCKS]) {
    NoHook none;
    attend_range<NQ>(q, kp, vp, table, table_width, ps_log2, n_kv, hk, range_lo, range_hi, lo, hi, scale, sm, acc,
                     none);
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
constexpr int DEC_TILES_PER_SPLIT = 16;  // a split is worth taking from this many tiles (512 keys) on
constexpr int DEC_MAX_SPLITS = 32;
constexpr int DEC_FOLD_LDS = 128 * 1024;  // most LDS a workgroup that does all splits may take for their states

// Workgroups that share one (sequence, kv head) with n_tiles visible key tiles: the largest power of two that
// leaves every workgroup DEC_TILES_PER_SPLIT tiles, at most DEC_MAX_SPLITS.  A function of the sequence's own
// length only; host and device use the same one.
__host__ __device__ inline int decode_splits(int n_tiles) {
    int s = 1;
    while (s < DEC_MAX_SPLITS && 2 * s * DEC_TILES_PER_SPLIT <= n_tiles) s *= 2;
    return s;
}

// out = sum_s w_s acc_s / sum_s w_s l_s over the splits of one (sequence, head), with w_s = 2^(m_s - max m) (the
// maxima are kept in units of log2; a split without keys has m = -inf and weight 0).  One element: `at(s)` gives
// split s's (acc, m, l).  Summed in split order with fused multiply-adds, the same wherever it is called from.
template <typename At>
__device__ __forceinline__ float merge_splits(int n_splits, float mx, At at) {
    float o = 0.f, denom = 0.f;
    for (int s0 = 0; s0 < n_splits; s0 += 4) {  // four splits' loads in flight at a time
        float acc[4], m[4], l[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) at(min(s0 + j, n_splits - 1), acc[j], m[j], l[j]);  // past the end: the last again, weight 0
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const float w = s0 + j < n_splits ? fast_exp2(m[j] - mx) : 0.f;
            denom = __builtin_fmaf(w, l[j], denom);
            o = __builtin_fmaf(w, acc[j], o);
        }
    }
    return o * (1.f / denom);
}

// The states of the four runs of one split, merged for one element of one query head: the split's (acc, m, l).
// `row(w)` is run w's state of that head: acc[HD], m, l.  The same arithmetic wherever it is called from.
template <typename Row>
__device__ __forceinline__ void merge_waves(Row row, int d, float& o, float& mx, float& lsum) {
    const float* rows[4];
#pragma unroll
    for (int w = 0; w < 4; ++w) rows[w] = row(w);
    mx = -INFINITY;
#pragma unroll
    for (int w = 0; w < 4; ++w) mx = fmaxf(mx, rows[w][HD]);
    const float mx_use = (mx == -INFINITY) ? 0.f : mx;  // no run had a key: all weights 0, the split counts for nothing
    o = 0.f;
    lsum = 0.f;
#pragma unroll
    for (int w = 0; w < 4; ++w) {
        const float wgt = fast_exp2(rows[w][HD] - mx_use);  // a run without keys has m = -inf: weight 0
        o += wgt * rows[w][d];
        lsum += wgt * rows[w][HD + 1];
    }
}

// One wave's state, finished, into its row of LDS (lanes whose column is no query head of the group write nothing).
__device__ __forceinline__ void leave_state(float* mine, Softmax<1>& sm, const floatx4 (&acc)[1][DBLOCKS], int g,
                                            bool writes) {
    sm.finish_sums();
    if (!writes) return;
    if (g == 0) {
        mine[HD] = sm.m[0];
        mine[HD + 1] = sm.l[0];
    }
#pragma unroll
    for (int db = 0; db < DBLOCKS; ++db)
#pragma unroll
        for (int i = 0; i < 4; ++i) mine[db * 16 + g * 4 + i] = acc[0][db][i];
}

// A sequence's visible key tiles are dealt evenly, in order, to n_splits * DEC_WAVES runs (every run contiguous,
// runs differ by one tile at most); the four runs of a split are merged, then the splits, always with the same
// arithmetic, so that how the runs are spread over workgroups changes no bit:
//   DEC_PLAIN   grid (kv heads, sequences, splits), 4 waves: a workgroup is one split, a wave one run; the combine
//               kernel merges the splits.
//   DEC_FOLD    grid (kv heads, sequences, 1), 4 waves: one workgroup does it all.  Each of its waves walks n_splits
//               runs that follow one another as one stream of tiles (its loads never stop at a run's end), leaves
//               each run's state in LDS as it passes the run's end, and the workgroup merges runs and splits
//               itself.  For steps of so many sequences that the splits are not needed to fill the device: no
//               partial results in memory and no second kernel.
//   DEC_SPREAD  grid (kv heads, sequences, runs), 1 wave: a workgroup is one run and leaves its state in the
//               workspace; the combine kernel merges runs and splits.  For steps of so few sequences that their
//               splits alone leave most compute units idle.
enum DecodeMode { DEC_PLAIN = 0, DEC_FOLD = 1, DEC_SPREAD = 2 };

__global__ __launch_bounds__(DEC_WAVES* SIA_WAVE) void attn_decode_kernel(
    const bf16_t* __restrict__ q, int q_row_stride, const bf16_t* __restrict__ kp, const bf16_t* __restrict__ vp,
    const int* __restrict__ block_table, int table_width, const int* __restrict__ cu_q,
    const int* __restrict__ kv_len, float* __restrict__ ws_acc, float* __restrict__ ws_ml,
    bf16_t* __restrict__ out, int n_heads, int n_kv, int ps_log2, float scale, int window, int max_splits, int mode) {
    const bool fold = mode == DEC_FOLD, spread = mode == DEC_SPREAD;
    static_assert(DEC_WAVES == 4, "merge_waves merges four runs");
    extern __shared__ float lds[];  // [runs of the workgroup][group][HD + 2]
    // splits are the slowest index of the grid: the workgroups that leave at once (splits a sequence does not
    // have) then come last, not interleaved with the others, which the chip deals out to its dies in turn
    const int hk = blockIdx.x, seq = blockIdx.y;
    const int wave = threadIdx.x / SIA_WAVE, lane = threadIdx.x & 63, r = lane & 15, g = lane >> 4;
    const int pos = kv_len[seq] - 1;
    const int lo_all = window > 0 ? max(0, pos - window + 1) : 0;
    const int t_first = lo_all / TILE, n_tiles = pos / TILE - t_first + 1;
    const int n_splits = min(decode_splits(n_tiles), max_splits);
    // the whole workgroup leaves: the grid is sized for the longest sequence there may be
    if (!fold && (int)blockIdx.z >= (spread ? n_splits * DEC_WAVES : n_splits)) return;
    scale *= LOG2E;  // exponentials are taken as powers of two
    const int group = n_heads / n_kv;
    const int* table = block_table + (size_t)seq * table_width;
    bf16x8 qf[1][KSTEPS];
    load_q(qf[0], r < group ? q + (size_t)seq * q_row_stride + (hk * group + r) * HD : nullptr, g);
    const int n_runs = n_splits * DEC_WAVES;
    constexpr int ROW = HD + 2;
    auto run_begin = [&](int run) { return t_first + (int)(((long long)run * n_tiles) / n_runs); };  // its first tile

    // this wave's runs: one (of this workgroup's split), or with fold n_splits in a row
    const int mine_n = fold ? n_splits : 1;
    const int run0 = fold ? wave * n_splits : spread ? blockIdx.z : blockIdx.z * DEC_WAVES + wave;
    const int first = run_begin(run0), end = run_begin(run0 + mine_n);
    Softmax<1> sm;
    sm.start();
    floatx4 acc[1][DBLOCKS];
#pragma unroll
    for (int db = 0; db < DBLOCKS; ++db) acc[0][db] = floatx4{0.f, 0.f, 0.f, 0.f};
    // the row of LDS of run `run0 + j`: with fold rows are in order of runs, else the wave's own
    auto row_of = [&](int j) { return lds + (size_t)((fold ? run0 + j : wave) * group + min(r, group - 1)) * ROW; };
    struct AtRunEnds {  // before the tile at kb: every run that ends at or before it hands its state on
        int done, run_end;
        const int mine_n, run0, r, g, group;
        Softmax<1>& sm;
        floatx4 (&acc)[1][DBLOCKS];
        decltype(run_begin)& begin;
        decltype(row_of)& row;
        __device__ __forceinline__ void pass() {
            float* mine = row(done);
            Softmax<1> left = sm;
            leave_state(mine, left, acc, g, r < group);
            sm.start();
#pragma unroll
            for (int db = 0; db < DBLOCKS; ++db) acc[0][db] = floatx4{0.f, 0.f, 0.f, 0.f};
            ++done;
            run_end = begin(run0 + done + 1);
        }
        __device__ __forceinline__ void operator()(int kb) {
            while (done < mine_n - 1 && kb / TILE >= run_end) pass();  // wave-uniform
        }
    } at_run_ends{0, run_begin(run0 + 1), mine_n, run0, r, g, group, sm, acc, run_begin, row_of};

    if (first < end) {  // wave-uniform
        const int w_lo = max(lo_all, first * TILE), w_hi = min(pos, end * TILE - 1);
        const int lo[1] = {r < group ? w_lo : 1}, hi[1] = {r < group ? w_hi : 0};
        attend_range<1>(qf, kp, vp, table, table_width, ps_log2, n_kv, hk, w_lo, w_hi, lo, hi, scale, sm, acc,
                        at_run_ends);
    }
    while (at_run_ends.done < mine_n - 1) at_run_ends.pass();  // runs without tiles of their own
    if (spread) {  // the run's state of every query head of the group: [sequence][head][run][HD + 2] in ws_acc
        const size_t slot = ((size_t)seq * n_heads + hk * group + min(r, group - 1)) * (max_splits * DEC_WAVES) + run0;
        leave_state(ws_acc + slot * ROW, sm, acc, g, r < group);
        return;
    }
    leave_state(row_of(mine_n - 1), sm, acc, g, r < group);
    __syncthreads();

    for (int idx = threadIdx.x; idx < group * HD; idx += DEC_WAVES * SIA_WAVE) {
        const int c = idx / HD, d = idx % HD;
        bf16_t* dst = out + ((size_t)cu_q[seq] * n_heads + hk * group + c) * HD + d;
        if (!fold || n_splits == 1) {
            float o, mx, lsum;
            merge_waves([&](int w) { return lds + (size_t)(w * group + c) * ROW; }, d, o, mx, lsum);
            if (n_splits == 1) {  // nothing to combine with: this is the result
                *dst = float_to_bf16(o * (1.f / lsum));
                continue;
            }
            const size_t slot = ((size_t)seq * n_heads + hk * group + c) * max_splits + blockIdx.z;
            ws_acc[slot * HD + d] = o;
            if (d == 0) {
                ws_ml[slot * 2] = mx;
                ws_ml[slot * 2 + 1] = lsum;
            }
            continue;
        }
        float mx_all = -INFINITY;
        for (int run = 0; run < n_runs; ++run) mx_all = fmaxf(mx_all, lds[(size_t)(run * group + c) * ROW + HD]);
        *dst = float_to_bf16(merge_splits(n_splits, mx_all, [&](int sp, float& a, float& m, float& l) {
            merge_waves([&](int w) { return lds + (size_t)((sp * DEC_WAVES + w) * group + c) * ROW; }, d, a, m, l);
        }));
    }
}

// Combines what workgroups of their own left in the workspaces for each (sequence, head): the splits' merged states
// (ws_acc [..][split][HD], ws_ml [..][split][2]), or with `runs` the states of all runs (ws_acc [..][run][HD + 2]).
__global__ __launch_bounds__(SIA_WAVE) void attn_decode_combine_kernel(
    const float* __restrict__ ws_acc, const float* __restrict__ ws_ml, const int* __restrict__ cu_q,
    const int* __restrict__ kv_len, bf16_t* __restrict__ out, int n_heads, int max_splits, int window, int runs) {
    const int head = blockIdx.x, seq = blockIdx.y, lane = threadIdx.x;
    const int pos = kv_len[seq] - 1;
    const int lo_all = window > 0 ? max(0, pos - window + 1) : 0;
    const int n_splits = min(decode_splits(pos / TILE - lo_all / TILE + 1), max_splits);
    bf16_t* dst = out + ((size_t)cu_q[seq] * n_heads + head) * HD;
    if (runs) {
        constexpr int ROW = HD + 2;
        const float* mine = ws_acc + ((size_t)seq * n_heads + head) * (max_splits * DEC_WAVES) * ROW;
        float mx = -INFINITY;  // a lane a run: the loads go out together
        for (int run = lane; run < n_splits * DEC_WAVES; run += SIA_WAVE) mx = fmaxf(mx, mine[(size_t)run * ROW + HD]);
        mx = wave_max(mx);
        for (int d = lane; d < HD; d += SIA_WAVE)
            dst[d] = float_to_bf16(merge_splits(n_splits, mx, [&](int sp, float& acc, float& m, float& l) {
                merge_waves([&](int w) { return mine + (size_t)(sp * DEC_WAVES + w) * ROW; }, d, acc, m, l);
            }));
        return;
    }
    if (n_splits == 1) return;  // its one workgroup wrote the result itself
    const size_t base = ((size_t)seq * n_heads + head) * max_splits;
    float mx = -INFINITY;
    for (int s = lane; s < n_splits; s += SIA_WAVE) mx = fmaxf(mx, ws_ml[(base + s) * 2]);
    mx = wave_max(mx);
    for (int d = lane; d < HD; d += SIA_WAVE)
        dst[d] = float_to_bf16(merge_splits(n_splits, mx, [&](int s, float& acc, float& m, float& l) {
            acc = ws_acc[(base + s) * HD + d];
            m = ws_ml[(base + s) * 2];
            l = ws_ml[(base + s) * 2 + 1];
        }));
}

// ---------------------------------------------------------------------------------------------------
// prefill: runs of several tokens (works for single tokens too, without splitting the keys)
// ---------------------------------------------------------------------------------------------------
// Four shapes of workgroup.  Wide: 128 tokens, 4 waves of 32 tokens each, one tile of keys a step (fewest
// instructions and reads from LDS per MFMA: the fastest when there are workgroups enough to keep two on every
// compute unit).  Split: 64 tokens, 8 waves: waves 0-3 take 16 tokens each and the even tiles of keys, waves 4-7
// the same tokens and the odd tiles, two tiles a step, and the two halves are merged through LDS at the end: half
// as many steps for the last tokens of a prompt, whose many keys set the time of a short prompt or portion.
// Paired: the same with 32 tokens a wave (128 tokens a workgroup), between the two: half the steps of the wide
// shape, half the reads from LDS per MFMA of the split one (6 to 8 % faster than 8 waves of 16 tokens that each
// take every tile, from 1,280 to 2,560 tokens at 24 heads; 10 to 17 % faster than the split shape from 1,024).  Long: 256 tokens, 8 waves of 32.  Head sizes above
// 128 take 4 waves of 16 tokens.
constexpr int PF_ROWS = HD <= 128 ? 128 : 64;  // tokens per wide workgroup
constexpr int PF_ROWS_SPLIT = 64;              // tokens per split workgroup
constexpr int PF_ROWS_LONG = 256;              // tokens per workgroup of 8 waves of 32 tokens
// Key and value tiles are shared by the workgroup's waves through LDS (two stages).  A 128-bit read takes the
// 64 banks in four passes of 16 lanes, and the lanes of a pass are not neighbours: the first takes lanes 0-3,
// 12-15, 20-23 and 24-27 (measured: rows of 16 lanes, one 16-byte piece each, are read without a conflict when the
// rows lie an odd multiple of 32 bytes apart, and in twice the time when the row is padded by 16 bytes only).
constexpr int K_STRIDE = HD + ((HD / 16) % 2 == 0 ? 16 : 0);  // elements per key row: an odd multiple of 32 bytes
constexpr int V_STRIDE = TILE + 16;                           // elements per dim row (32 positions + pad): 96 bytes
constexpr int K_CHUNKS = TILE * HD / 8;         // 16-byte pieces of a key tile (a value tile has as many)
constexpr bool PF_USE_LDS = (2 * (TILE * K_STRIDE + HD * V_STRIDE) * 2) <= 64 * 1024;

// What one thread of a workgroup of TEAM threads carries from global memory to LDS for one tile.
typedef __attribute__((__vector_size__(4 * sizeof(uint32_t)))) uint32_t u32x4;  // a plain 16-byte register value
template <int TEAM>
struct TileRegs {
    static constexpr int PER_THREAD = (K_CHUNKS + TEAM - 1) / TEAM;
    u32x4 k[PER_THREAD];
    u32x4 v[PER_THREAD];
};

// Where a thread's pieces of a tile lie, as far as that does not depend on the tile: worked out once per workgroup.
// Key piece c is (key c / (HD/8) of the tile, dims 8 (c % (HD/8)) ..); value pieces are ordered (page segment, dim,
// group of 8 positions), so that consecutive threads read consecutive 16 bytes of a page.  With that order a
// thread's key piece and its value piece lie in the same page segment of the tile, whatever the page size, so one
// look-up of the page serves both.
template <int TEAM>
struct FetchPlan {
    static constexpr int PER_THREAD = (K_CHUNKS + TEAM - 1) / TEAM;
    int k_key[PER_THREAD], k_off[PER_THREAD];  // key within the tile; element offset of the piece within its page
    int v_key[PER_THREAD], v_off[PER_THREAD];  // first of its 8 positions within the tile; offset within the page
    __device__ __forceinline__ void make(int ps_log2, int hk) {
        const int ps = 1 << ps_log2;
        const int seg_keys = min(ps, TILE);            // positions of one page inside a tile
        const int seg_chunks = HD * (seg_keys / 8);    // 16-byte pieces of one page's values inside a tile
#pragma unroll
        for (int i = 0; i < PER_THREAD; ++i) {
            const int c = min((int)threadIdx.x + i * TEAM, K_CHUNKS - 1);
            k_key[i] = c / (HD / 8);
            k_off[i] = hk * ps * HD + (c % (HD / 8)) * 8;
            const int seg = c / seg_chunks, rest = c % seg_chunks;
            const int d = rest / (seg_keys / 8), j = rest % (seg_keys / 8);
            v_key[i] = seg * seg_keys + j * 8;
            v_off[i] = (hk * HD + d) * ps;
        }
    }
};

// The pages of a thread's pieces of the tile at kb, looked up a step before the tile's loads are issued, so that no
// load's address waits for the exchange between lanes.  Keys outside [lo, hi] are clamped into it (see load_stage);
// a key piece and its value piece then still lie in one page: both are clamped into the same range, whose ends lie
// in pages of their own only as a whole.
template <int TEAM>
__device__ __forceinline__ void tile_lookup(int (&page)[TileRegs<TEAM>::PER_THREAD], const FetchPlan<TEAM>& plan,
                                            const PageWindow& pages, int ps_log2, int kb, int lo, int hi) {
    const int t_lo = max(kb, lo), t_hi = min(kb + TILE - 1, hi);
#pragma unroll
    for (int i = 0; i < TileRegs<TEAM>::PER_THREAD; ++i) {
        const int key = min(max(kb + plan.k_key[i], t_lo), t_hi);
        page[i] = pages_get(pages, key >> ps_log2);
    }
}

// Issues the global loads of the tile at kb, whose pages tile_lookup found.  page_stride: elements of one page
// (keys and values alike).
template <int TEAM>
__device__ __forceinline__ void tile_fetch(TileRegs<TEAM>& t, const FetchPlan<TEAM>& plan, const bf16_t* __restrict__ kp,
                                           const bf16_t* __restrict__ vp, const int (&page)[TileRegs<TEAM>::PER_THREAD],
                                           int ps_log2, unsigned page_stride, int kb, int lo, int hi) {
    const int ps_mask = (1 << ps_log2) - 1;
    const int t_lo = max(kb, lo), t_hi = min(kb + TILE - 1, hi);
    const int v_lo = t_lo & ~7, v_hi = t_hi & ~7;
#pragma unroll
    for (int i = 0; i < TileRegs<TEAM>::PER_THREAD; ++i) {
        if (K_CHUNKS % TEAM != 0 && (int)threadIdx.x + i * TEAM >= K_CHUNKS) break;
        const int key = min(max(kb + plan.k_key[i], t_lo), t_hi);
        const int key0 = min(max(kb + plan.v_key[i], v_lo), v_hi);
        const size_t page_at = (size_t)(unsigned)page[i] * page_stride;
        t.k[i] = *reinterpret_cast<const u32x4*>(kp + page_at + (unsigned)(plan.k_off[i] + (key & ps_mask) * HD));
        t.v[i] = *reinterpret_cast<const u32x4*>(vp + page_at + (unsigned)(plan.v_off[i] + (key0 & ps_mask)));
    }
}

// Writes a fetched tile into an LDS stage.  Key rows are stored in the order the score MFMAs read them
// (row 16h + m holds key 8(m/4) + 4h + m%4), so that the 16 lanes of a read take 16 consecutive rows.
template <int TEAM>
__device__ __forceinline__ void tile_store(const TileRegs<TEAM>& t, bf16_t* __restrict__ k_lds, bf16_t* __restrict__ v_lds,
                                           int ps_log2) {
    const int ps = 1 << ps_log2;
    const int seg_keys = min(ps, TILE);
    const int seg_chunks = HD * (seg_keys / 8);
#pragma unroll
    for (int i = 0; i < TileRegs<TEAM>::PER_THREAD; ++i) {
        const int c = threadIdx.x + i * TEAM;
        if (K_CHUNKS % TEAM != 0 && c >= K_CHUNKS) break;
        const int key = c / (HD / 8);
        const int row = ((key >> 2) & 1) * 16 + (key >> 3) * 4 + (key & 3);
        *reinterpret_cast<u32x4*>(k_lds + row * K_STRIDE + (c % (HD / 8)) * 8) = t.k[i];
        const int seg = c / seg_chunks, rest = c % seg_chunks;
        const int d = rest / (seg_keys / 8), j = rest % (seg_keys / 8);
        *reinterpret_cast<u32x4*>(v_lds + d * V_STRIDE + seg * seg_keys + j * 8) = t.v[i];
    }
}

// Scores, online softmax and value product of one tile held in an LDS stage.  With EARLY all key operands of the
// tile are read before the first score MFMA and all value operands before the softmax, so that a read's latency
// passes behind the arithmetic in front of it instead of in front of the two MFMAs that use it (4 % at 2,048 tokens;
// these shapes hold one workgroup a compute unit whatever they do, so the registers are there); without it every
// operand is read right before its MFMAs, which the 256-token shape, that has most arithmetic per read, likes
// better by 3 %.
template <int NQ, bool EARLY>
__device__ __forceinline__ void compute_from_lds(const bf16_t* __restrict__ k_lds, const bf16_t* __restrict__ v_lds,
                                                 const bf16x8 (&q)[NQ][KSTEPS], int kb, const int (&lo)[NQ],
                                                 const int (&hi)[NQ], float scale, Softmax<NQ>& sm,
                                                 floatx4 (&acc)[NQ][DBLOCKS]) {
    const int lane = threadIdx.x & 63, r = lane & 15, g = lane >> 4;
    auto key_operand = [&](int h, int ks) {
        const int d0 = ks * 32 + g * 8;
        if (HD % 32 == 0 || ks < KSTEPS - 1) return load8(k_lds + (h * 16 + r) * K_STRIDE + d0);
        return d0 < HD ? load8(k_lds + (h * 16 + r) * K_STRIDE + d0) : zero8();
    };
    auto value_operand = [&](int db) { return load8(v_lds + (db * 16 + r) * V_STRIDE + g * 8); };
    bf16x8 ka[2][KSTEPS], va[DBLOCKS];
    if (EARLY) {
#pragma unroll
        for (int h = 0; h < 2; ++h)
#pragma unroll
            for (int ks = 0; ks < KSTEPS; ++ks) ka[h][ks] = key_operand(h, ks);
    }
    floatx4 s[NQ][2];
#pragma unroll
    for (int h = 0; h < 2; ++h) {
#pragma unroll
        for (int n = 0; n < NQ; ++n) s[n][h] = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int ks = 0; ks < KSTEPS; ++ks) {
            const bf16x8 a = EARLY ? ka[h][ks] : key_operand(h, ks);
#pragma unroll
            for (int n = 0; n < NQ; ++n) s[n][h] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, q[n][ks], s[n][h], 0, 0, 0);
        }
    }
    if (EARLY) {
#pragma unroll
        for (int db = 0; db < DBLOCKS; ++db) va[db] = value_operand(db);
    }
    bf16x8 p[NQ];
    softmax_update<NQ>(s, kb, lo, hi, scale, sm, acc, p);
#pragma unroll
    for (int db = 0; db < DBLOCKS; ++db) {
        const bf16x8 a = EARLY ? va[db] : value_operand(db);
#pragma unroll
        for (int n = 0; n < NQ; ++n) acc[n][db] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, p[n], acc[n][db], 0, 0, 0);
    }
}

// PF_NQ groups of 16 tokens per wave; PF_WAVES waves, of which each KSPLIT-th part takes the same tokens and
// every KSPLIT-th tile of keys: ROWS = PF_NQ * 16 * PF_WAVES / KSPLIT tokens per workgroup.  KTILES tiles of keys
// are staged per step (and barrier); with KSPLIT = 1 every wave takes them one after the other, which at 8 waves
// of 16 tokens is 7 % faster with two tiles than with one (fewer barriers a key) and changes no bit.
template <int PF_NQ, int PF_WAVES, int KSPLIT, int KTILES>
__global__ __launch_bounds__(PF_WAVES* SIA_WAVE) void attn_prefill_kernel(
    const bf16_t* __restrict__ q, int q_row_stride, const bf16_t* __restrict__ kp, const bf16_t* __restrict__ vp,
    const int* __restrict__ block_table, int table_width, const int* __restrict__ cu_q,
    const int* __restrict__ kv_len, bf16_t* __restrict__ out, int n_heads, int n_kv, int ps_log2, float scale,
    int window, int seq_begin, int seq_end) {
    constexpr int ROW_WAVES = PF_WAVES / KSPLIT;
    constexpr int ROWS = ROW_WAVES * PF_NQ * 16;
    constexpr int TEAM = PF_WAVES * SIA_WAVE;
    extern __shared__ __align__(16) unsigned char pf_lds[];
    // The chip has 8 dies (XCDs), each with an L2 of its own, and hands workgroups to them in turn.  The
    // workgroup ids are renumbered so that each die gets a contiguous range: the query heads that share a
    // kv head, and the row tiles of one head, then read their keys and values through one L2.
    scale *= LOG2E;  // exponentials are taken as powers of two
    const int n_blocks = gridDim.x * gridDim.y;
    int vid = blockIdx.y * gridDim.x + blockIdx.x;
    int head, tile;
    if (n_heads % 8 == 0) {
        // a die's heads take turns tile by tile, so that on every die the workgroups with most keys (see below)
        // start first and the short ones fill the compute units up at the end
        const int heads_here = n_heads / 8, die = vid % 8, turn = vid / 8;
        head = die * heads_here + turn % heads_here;
        tile = turn / heads_here;
    } else {
        if (n_blocks % 8 == 0) vid = (vid % 8) * (n_blocks / 8) + vid / 8;
        head = vid / gridDim.x;
        tile = vid % gridDim.x;
    }
    // which sequence and which of its row tiles this workgroup has; late tiles (most keys) come first
    int seq = seq_begin;
    for (; seq < seq_end; ++seq) {
        const int tiles = (cu_q[seq + 1] - cu_q[seq] + ROWS - 1) / ROWS;
        if (tile < tiles) {
            tile = tiles - 1 - tile;
            break;
        }
        tile -= tiles;
    }
    if (seq >= seq_end) return;
    const int hk = head / (n_heads / n_kv);
    const int wave = threadIdx.x / SIA_WAVE, lane = threadIdx.x & 63, r = lane & 15, g = lane >> 4;
    const int row_wave = wave % ROW_WAVES, part = wave / ROW_WAVES;  // which tokens, which tiles of a step
    const int q_begin = cu_q[seq], q_len = cu_q[seq + 1] - q_begin;
    const int first_pos = kv_len[seq] - q_len;
    const int row0 = tile * ROWS + row_wave * PF_NQ * 16;  // this wave's first row within the sequence's run
    const bool wave_live = row0 < q_len;
    const int row_last = min(q_len - 1, row0 + PF_NQ * 16 - 1);
    const int* table = block_table + (size_t)seq * table_width;

    bf16x8 qf[PF_NQ][KSTEPS];
    int lo[PF_NQ], hi[PF_NQ];
    Softmax<PF_NQ> sm;
    sm.start();
    floatx4 acc[PF_NQ][DBLOCKS];
#pragma unroll
    for (int n = 0; n < PF_NQ; ++n) {
        const int row = row0 + n * 16 + r;
        const bool live = row < q_len;
        const int qpos = first_pos + row;
        load_q(qf[n], live ? q + (size_t)(q_begin + row) * q_row_stride + head * HD : nullptr, g);
        hi[n] = live ? qpos : 0;
        lo[n] = live ? (window > 0 ? max(0, qpos - window + 1) : 0) : 1;
#pragma unroll
        for (int db = 0; db < DBLOCKS; ++db) acc[n][db] = floatx4{0.f, 0.f, 0.f, 0.f};
    }

    if constexpr (PF_USE_LDS) {
        // LDS: [2 stages][KTILES tiles] of (keys, values)
        constexpr int TILE_ELEMS = TILE * K_STRIDE + HD * V_STRIDE;
        bf16_t* const lds_tiles = reinterpret_cast<bf16_t*>(pf_lds);
#define PF_K_LDS(STAGE, PART) (lds_tiles + ((STAGE) * KTILES + (PART)) * TILE_ELEMS)
#define PF_V_LDS(STAGE, PART) (PF_K_LDS(STAGE, PART) + TILE * K_STRIDE)
        // the workgroup's key range: from the first row's oldest visible key to the last live row's position
        const int blk_rows = min(q_len - tile * ROWS, ROWS);
        const int blk_hi = first_pos + tile * ROWS + blk_rows - 1;
        const int blk_lo = window > 0 ? max(0, first_pos + tile * ROWS - window + 1) : 0;
        const int wave_hi = first_pos + row_last;
        const int wave_lo = window > 0 ? max(0, first_pos + row0 - window + 1) : 0;
        const int kb_first = (blk_lo / TILE) * TILE, kb_last = (blk_hi / TILE) * TILE;
        constexpr int STEP_KEYS = KTILES * TILE;
        constexpr int AHEAD = PF_NQ == 1 ? 4 : 2;
        constexpr bool EARLY = KSPLIT == 2 || KTILES == 1;  // all shapes but the one of 256 tokens
        constexpr bool ONE_TILE = KSPLIT == KTILES;         // a wave takes one tile of a step (tile `part`)
        static_assert(ONE_TILE || KSPLIT == 1, "either each set of waves takes one tile of a step, or every wave all");
        static_assert(AHEAD % 2 == 0, "the LDS stage of a step is its parity within a group of AHEAD");
        FetchPlan<TEAM> plan;
        plan.make(ps_log2, hk);
        const unsigned page_stride = (unsigned)n_kv * HD << ps_log2;
        // AHEAD (two or four) register sets: while the tiles of step t are computed from LDS, those of the steps
        // after it wait in the others (or are still on their way) and the loads of step t+AHEAD are issued.  The
        // block-table window (64 entries from the page of the first tile it serves) is loaded outside the
        // pipelined loop.
        for (int w_first = kb_first, w_end; w_first <= kb_last; w_first = w_end) {
            const int first_page = w_first >> ps_log2;
            w_end = (first_page + SIA_WAVE) << ps_log2;  // first key beyond the window, a multiple of TILE
            const int w_last = min(kb_last, w_end - TILE);
            PageWindow pages;
            pages_load(pages, table, table_width, first_page, lane);
            TileRegs<TEAM> regs[AHEAD][KTILES];
            int found[KTILES][TileRegs<TEAM>::PER_THREAD];  // pages of the tiles whose loads are issued next
// One step: issue the loads of the tiles AHEAD steps ahead into FREE (whose tiles are in LDS by now; their pages
// were looked up a step ago) and look up the pages for the loads of the step after, compute this wave's tile of the
// step at KB from LDS stage STAGE, write the tiles that wait in NEXT (loaded AHEAD - 1 steps ago) into the other
// stage.  With AHEAD = 4 a load has three steps' time to arrive before anybody waits for it:
// with the one or two workgroups a compute unit holds when a prompt is short, nothing else would hide its latency
// (the shapes of 32 tokens a wave have no registers to spare for it and hide it by their number).  (Macros, not
// lambdas: register sets that a closure captures by reference end up in scratch memory.)
#define PF_LOOKUP(KB)                                                                                           \
    _Pragma("unroll") for (int p = 0; p < KTILES; ++p)                                                          \
        tile_lookup<TEAM>(found[p], plan, pages, ps_log2, min((KB) + p * TILE, w_last), blk_lo, blk_hi)
#define PF_FETCH(SET, KB)                                                                                       \
    _Pragma("unroll") for (int p = 0; p < KTILES; ++p)                                                          \
        tile_fetch(SET[p], plan, kp, vp, found[p], ps_log2, page_stride, min((KB) + p * TILE, w_last), blk_lo, blk_hi)
#define PF_STORE(SET, KB, STAGE)                                                                                \
    _Pragma("unroll") for (int p = 0; p < KTILES; ++p)                                                          \
        if ((KB) + p * TILE <= w_last) tile_store(SET[p], PF_K_LDS(STAGE, p), PF_V_LDS(STAGE, p), ps_log2)
#define PF_LIVE(MY_KB) (wave_live && (MY_KB) <= w_last && (MY_KB) <= wave_hi && (MY_KB) + TILE - 1 >= wave_lo)
#define PF_STEP(FREE, NEXT, KB, STAGE)                                                                          \
    do {                                                                                                        \
        PF_FETCH(FREE, (KB) + AHEAD * STEP_KEYS);                                                               \
        PF_LOOKUP((KB) + (AHEAD + 1) * STEP_KEYS);                                                              \
        if (ONE_TILE) { /* the wave's tile is chosen by an address, so that both sets of waves run the same code */ \
            const int mine = KSPLIT == 2 ? part : 0, my_kb = (KB) + mine * TILE;                                \
            if (PF_LIVE(my_kb))                                                                                 \
                compute_from_lds<PF_NQ, EARLY>(PF_K_LDS(STAGE, mine), PF_V_LDS(STAGE, mine), qf, my_kb, lo, hi, \
                                               scale, sm, acc);                                                 \
        } else {                                                                                                \
            _Pragma("unroll") for (int p = 0; p < KTILES; ++p) {                                                \
                const int my_kb = (KB) + p * TILE;                                                              \
                if (PF_LIVE(my_kb))                                                                             \
                    compute_from_lds<PF_NQ, EARLY>(PF_K_LDS(STAGE, p), PF_V_LDS(STAGE, p), qf, my_kb, lo, hi,   \
                                                   scale, sm, acc);                                             \
            }                                                                                                   \
        }                                                                                                       \
        PF_STORE(NEXT, (KB) + STEP_KEYS, (STAGE) ^ 1);                                                          \
        __syncthreads();                                                                                        \
    } while (0)
            // steps past the last tile (to fill a group of AHEAD) load the last tile again, compute and store
            // nothing and keep the barriers in step
#pragma unroll
            for (int j = 0; j < AHEAD; ++j) {
                PF_LOOKUP(w_first + j * STEP_KEYS);
                PF_FETCH(regs[j], w_first + j * STEP_KEYS);
            }
            PF_LOOKUP(w_first + AHEAD * STEP_KEYS);
            PF_STORE(regs[0], w_first, 0);
            __syncthreads();
            for (int kb = w_first; kb <= w_last; kb += AHEAD * STEP_KEYS) {
#pragma unroll
                for (int j = 0; j < AHEAD; ++j)
                    PF_STEP(regs[j], regs[(j + 1) % AHEAD], kb + j * STEP_KEYS, j & 1);
            }
#undef PF_STEP
#undef PF_LIVE
#undef PF_STORE
#undef PF_FETCH
#undef PF_LOOKUP
        }
#undef PF_K_LDS
#undef PF_V_LDS
    } else {
        static_assert(PF_USE_LDS || KSPLIT == 1, "the split shape stages its tiles through LDS");
        if (wave_live) {
            const int range_hi = first_pos + row_last;
            const int range_lo = window > 0 ? max(0, first_pos + row0 - window + 1) : 0;
            attend_range<PF_NQ>(qf, kp, vp, table, table_width, ps_log2, n_kv, hk, range_lo, range_hi, lo, hi, scale,
                                sm, acc);
        }
    }
    sm.finish_sums();

    if constexpr (KSPLIT == 2) {
        // The waves of the second part hand (m, l, acc) to the waves of the first through LDS (the tiles are
        // done with: the loop ended with a barrier), lane to lane, and those merge and write.
        constexpr int PER_LANE = PF_NQ * (DBLOCKS * 4 + 2);
        float* const box = reinterpret_cast<float*>(pf_lds) + (size_t)(row_wave * SIA_WAVE + lane) * PER_LANE;
        if (part == 1) {
#pragma unroll
            for (int n = 0; n < PF_NQ; ++n) {
                float* b = box + n * (DBLOCKS * 4 + 2);
                b[0] = sm.m[n];
                b[1] = sm.l[n];
#pragma unroll
                for (int db = 0; db < DBLOCKS; ++db)
#pragma unroll
                    for (int i = 0; i < 4; ++i) b[2 + db * 4 + i] = acc[n][db][i];
            }
        }
        __syncthreads();
        if (part == 1) return;
#pragma unroll
        for (int n = 0; n < PF_NQ; ++n) {
            const float* b = box + n * (DBLOCKS * 4 + 2);
            const float m_other = b[0], m_new = fmaxf(sm.m[n], m_other);
            const float m_use = (m_new == -INFINITY) ? 0.f : m_new;
            const float w_mine = fast_exp2(sm.m[n] - m_use), w_other = fast_exp2(m_other - m_use);
            sm.l[n] = sm.l[n] * w_mine + b[1] * w_other;
#pragma unroll
            for (int db = 0; db < DBLOCKS; ++db)
#pragma unroll
                for (int i = 0; i < 4; ++i) acc[n][db][i] = acc[n][db][i] * w_mine + b[2 + db * 4 + i] * w_other;
        }
    }
    if (!wave_live) return;

#pragma unroll
    for (int n = 0; n < PF_NQ; ++n) {
        const int row = row0 + n * 16 + r;
        if (row >= q_len) continue;
        const float inv = 1.f / sm.l[n];
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
// Compute units of the current device (asked once per device).
static int compute_units() {
    static int known[64];
    int device = 0;
    if (hipGetDevice(&device) != hipSuccess || device < 0 || device >= 64) return 256;
    if (!known[device]) {
        int n = 0;
        known[device] = (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, device) == hipSuccess && n > 0) ? n : 256;
    }
    return known[device];
}

static int log2_exact(int v) {
    int l = 0;
    while ((1 << l) < v) ++l;
    return (1 << l) == v ? l : -1;
}

SIA_EXPORT int sia_attn_mfma_head_dim() { return HD; }

// Most workgroups that share one (sequence, kv head) when no sequence of the step holds more than kv_bound keys
// (with a window: sees more than the window): what the caller sizes the workspaces and this library its grid by.
SIA_EXPORT int sia_attn_decode_max_splits(int kv_bound, int window) {
    if (kv_bound <= 0) return 1;
    // the visible keys of a sequence of length n span at most this many tiles (a window need not start on a tile)
    const int tiles_all = (kv_bound + TILE - 1) / TILE;
    const int tiles = window > 0 ? min(tiles_all, (window + TILE - 2) / TILE + 1) : tiles_all;
    return decode_splits(tiles);
}

// How a decode step of n_seqs sequences, none with more splits than max_splits, spreads its runs over workgroups.
static DecodeMode decode_mode(int n_seqs, int n_heads, int n_kv, int max_splits) {
    const long long pairs = (long long)n_kv * n_seqs, cus = compute_units();
    const size_t row_bytes = (size_t)(n_heads / n_kv) * (HD + 2) * sizeof(float);
    if (max_splits > 1 && pairs >= cus && DEC_WAVES * row_bytes * max_splits <= (size_t)DEC_FOLD_LDS) return DEC_FOLD;
    // no more splits than compute units: a workgroup for every run.  Not for sequences too short to split: their one
    // workgroup writes the result itself, which costs less than a second kernel that merges runs.
    if (max_splits > 1 && pairs * max_splits <= cus) return DEC_SPREAD;
    return DEC_PLAIN;
}

// Which of the three ways such a step takes (0 plain, 1 fold, 2 spread): for tests and profiles that want to know
// which code ran.
SIA_EXPORT int sia_attn_decode_mode(int n_seqs, int n_heads, int n_kv, int max_splits) {
    if (n_seqs <= 0 || n_kv <= 0 || n_heads % n_kv || max_splits <= 0) return SIA_BAD_ARGUMENT;
    return (int)decode_mode(n_seqs, n_heads, n_kv, max_splits);
}

// Floats of ws_acc and of ws_ml that sia_attn_decode needs for such a step (0: none, the pointer may be null).
SIA_EXPORT long long sia_attn_decode_workspace(int n_seqs, int n_heads, int n_kv, int max_splits, int which) {
    if (n_seqs <= 0 || n_kv <= 0 || n_heads % n_kv || max_splits <= 0) return 0;
    const long long states = (long long)n_seqs * n_heads;
    switch (decode_mode(n_seqs, n_heads, n_kv, max_splits)) {
    case DEC_FOLD: return 0;
    case DEC_SPREAD: return which == 0 ? states * max_splits * DEC_WAVES * (HD + 2) : 0;
    default: return max_splits > 1 ? states * max_splits * (which == 0 ? HD : 2) : 0;
    }
}

// Sequences 0 .. n_seqs-1 of the step, each with exactly one new token, which is row s of q (cu_q[s] = s), and
// none longer than kv_bound.  max_splits = sia_attn_decode_max_splits(kv_bound, window); ws_acc and ws_ml hold
// sia_attn_decode_workspace(.., 0) and (.., 1) floats (neither is read before it is written).
SIA_EXPORT int sia_attn_decode(const void* q, int q_row_stride, const void* k_pages, const void* v_pages,
                               const int* block_table, int table_width, const int* cu_q, const int* kv_len,
                               void* out, float* ws_acc, float* ws_ml, int n_seqs, int n_heads, int n_kv,
                               int page_size, float scale, int window, int max_splits, hipStream_t stream) {
    if (n_seqs <= 0) return 0;
    const int ps_log2 = log2_exact(page_size);
    const int n_splits = max_splits;
    if (ps_log2 < 3 || n_kv <= 0 || n_heads % n_kv || n_heads / n_kv > 16 || n_splits <= 0 ||
        n_splits > DEC_MAX_SPLITS || n_kv > 65535 || n_seqs > 65535 || q_row_stride % 8 || table_width <= 0)
        return SIA_BAD_ARGUMENT;
    const DecodeMode mode = decode_mode(n_seqs, n_heads, n_kv, n_splits);
    if ((sia_attn_decode_workspace(n_seqs, n_heads, n_kv, n_splits, 0) && !ws_acc) ||
        (sia_attn_decode_workspace(n_seqs, n_heads, n_kv, n_splits, 1) && !ws_ml))
        return SIA_BAD_ARGUMENT;
    const size_t row_bytes = (size_t)(n_heads / n_kv) * (HD + 2) * sizeof(float);
    size_t lds_bytes = DEC_WAVES * row_bytes;
    if (lds_bytes > 64 * 1024) return SIA_BAD_ARGUMENT;
    if (mode == DEC_FOLD) {
        lds_bytes *= n_splits;  // a row for every run
        if (lds_bytes > 48 * 1024) {  // beyond the default limit of dynamic LDS
            static bool allowed[64];
            int device = 0;
            if (hipGetDevice(&device) != hipSuccess || device < 0 || device >= 64) return SIA_BAD_ARGUMENT;
            if (!allowed[device]) {
                const hipError_t e = hipFuncSetAttribute((const void*)attn_decode_kernel,
                                                         hipFuncAttributeMaxDynamicSharedMemorySize, DEC_FOLD_LDS);
                if (e != hipSuccess) return (int)e;
                allowed[device] = true;
            }
        }
    }
    const dim3 grid(n_kv, n_seqs, mode == DEC_FOLD ? 1 : mode == DEC_SPREAD ? n_splits * DEC_WAVES : n_splits);
    hipLaunchKernelGGL(attn_decode_kernel, grid, dim3((mode == DEC_SPREAD ? 1 : DEC_WAVES) * SIA_WAVE),
                       mode == DEC_SPREAD ? 0 : lds_bytes, stream, (const bf16_t*)q, q_row_stride,
                       (const bf16_t*)k_pages, (const bf16_t*)v_pages, block_table, table_width, cu_q, kv_len, ws_acc,
                       ws_ml, (bf16_t*)out, n_heads, n_kv, ps_log2, scale, window, n_splits, (int)mode);
    if (mode == DEC_SPREAD || (mode == DEC_PLAIN && n_splits > 1))
        hipLaunchKernelGGL(attn_decode_combine_kernel, dim3(n_heads, n_seqs), dim3(SIA_WAVE), 0, stream, ws_acc,
                           ws_ml, cu_q, kv_len, (bf16_t*)out, n_heads, n_splits, window, mode == DEC_SPREAD ? 1 : 0);
    return SIA_LAUNCH_CHECK();
}

// Sequences seq_begin .. seq_end-1 of the step.  n_tiles = sum over them of ceil(q_len / sia_attn_prefill_rows()),
// n_tiles_split the same with sia_attn_prefill_rows_split() and n_tiles_long with sia_attn_prefill_rows_long()
// (0 if this head size has no such shape).
SIA_EXPORT int sia_attn_prefill_rows() { return PF_ROWS; }
SIA_EXPORT int sia_attn_prefill_rows_split() { return (HD <= 128 && PF_USE_LDS) ? PF_ROWS_SPLIT : 0; }
SIA_EXPORT int sia_attn_prefill_rows_long() { return (HD <= 128 && PF_USE_LDS) ? PF_ROWS_LONG : 0; }

template <int NQ, int WAVES, int KSPLIT, int KTILES = KSPLIT>
static int launch_prefill(int tiles, const void* q, int q_row_stride, const void* k_pages, const void* v_pages,
                          const int* block_table, int table_width, const int* cu_q, const int* kv_len, void* out,
                          int seq_begin, int seq_end, int n_heads, int n_kv, int ps_log2, float scale, int window,
                          hipStream_t stream) {
    constexpr int TILE_ELEMS = TILE * K_STRIDE + HD * V_STRIDE;
    size_t lds_bytes = PF_USE_LDS ? (size_t)2 * KTILES * TILE_ELEMS * sizeof(bf16_t) : 0;
    if (KSPLIT == 2) {
        const size_t merge = (size_t)(WAVES / 2) * SIA_WAVE * NQ * (DBLOCKS * 4 + 2) * sizeof(float);
        if (merge > lds_bytes) lds_bytes = merge;
    }
    const void* fn = reinterpret_cast<const void*>(&attn_prefill_kernel<NQ, WAVES, KSPLIT, KTILES>);
    if (lds_bytes > 48 * 1024) {  // beyond the default limit of dynamic LDS
        const hipError_t e = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes);
        if (e != hipSuccess) return (int)e;
    }
    hipLaunchKernelGGL((attn_prefill_kernel<NQ, WAVES, KSPLIT, KTILES>), dim3(tiles, n_heads), dim3(WAVES * SIA_WAVE),
                       lds_bytes, stream, (const bf16_t*)q, q_row_stride, (const bf16_t*)k_pages,
                       (const bf16_t*)v_pages, block_table, table_width, cu_q, kv_len, (bf16_t*)out, n_heads, n_kv,
                       ps_log2, scale, window, seq_begin, seq_end);
    return SIA_LAUNCH_CHECK();
}

// Which of the four workgroup shapes a launch takes.  n_tiles, n_tiles_split, n_tiles_long: its row tiles at 128, 64
// and 256 tokens a workgroup; q_bound, kv_bound: the most tokens and the most keys of one of its sequences (0: not
// known, taken as a prompt from its start).
enum PrefillShape { PF_SPLIT, PF_PAIRED, PF_WIDE, PF_LONG };
static PrefillShape prefill_shape(int n_tiles, int n_tiles_split, int n_tiles_long, int n_heads, int q_bound,
                                  int kv_bound) {
    // Measured at 24 heads of 128 on 256 compute units.  For a prompt from its start, whose row tiles see from few
    // keys to all, the fastest shape follows the number of workgroups per compute unit: the split shape while all
    // its workgroups are on the chip at once (up to 6/8 of a wide workgroup per compute unit: prompts up to about
    // 1,000 tokens), the paired shape of 128 tokens (two tiles of keys a step, one for each set of waves) up to 15/8
    // (about 2,500 tokens), the wide shape (one tile a step) beyond, and from 36/8 on (about 6,000 tokens) 8 waves
    // of 32 tokens (256 tokens a workgroup, two tiles a step: a tile staged in LDS then serves twice as many tokens).
    const long long wide_groups = (long long)n_tiles * n_heads, cus = compute_units();
    const bool split_fits = n_tiles_split > 0 && wide_groups * 8 <= cus * 6;
    // A portion over a past is another matter: every row tile sees about as many keys, so the launch lasts as many
    // rounds as its workgroups need on the compute units, each as long as the shape's time for that many keys.
    if (split_fits && q_bound > 0 && 2LL * kv_bound >= 3LL * q_bound && (long long)n_tiles_split * n_heads > cus)
        return PF_PAIRED;  // one round of 128 tokens instead of two of 64 (768 to 1,024 tokens: 10 to 30 % less)
    if (!split_fits && q_bound > 0 && kv_bound >= 4LL * q_bound) {
        // time of a round for a given number of keys, relative: a compute unit holds one paired workgroup (128
        // tokens), two wide ones (256) or one long one (256)
        const long long paired = (wide_groups + cus - 1) / cus * 124;
        const long long wide = (wide_groups + 2 * cus - 1) / (2 * cus) * 236;
        const long long lng = n_tiles_long > 0 ? ((long long)n_tiles_long * n_heads + cus - 1) / cus * 222 : paired + wide;
        return lng <= wide && lng <= paired ? PF_LONG : wide <= paired ? PF_WIDE : PF_PAIRED;
    }
    if (split_fits) return PF_SPLIT;
    if (wide_groups * 8 <= cus * 15) return PF_PAIRED;
    if (n_tiles_long > 0 && wide_groups * 8 >= cus * 36) return PF_LONG;
    return PF_WIDE;
}

SIA_EXPORT int sia_attn_prefill(const void* q, int q_row_stride, const void* k_pages, const void* v_pages,
                                const int* block_table, int table_width, const int* cu_q, const int* kv_len,
                                void* out, int seq_begin, int seq_end, int n_tiles, int n_tiles_split, int n_tiles_long,
                                int q_bound, int kv_bound, int n_heads, int n_kv, int page_size, float scale, int window,
                                hipStream_t stream) {
    if (seq_end <= seq_begin || n_tiles <= 0) return 0;
    const int ps_log2 = log2_exact(page_size);
    if (ps_log2 < 3 || n_kv <= 0 || n_heads % n_kv || n_heads > 65535 || q_row_stride % 8 || table_width <= 0)
        return SIA_BAD_ARGUMENT;
#define ARGS q, q_row_stride, k_pages, v_pages, block_table, table_width, cu_q, kv_len, out, seq_begin, seq_end, \
             n_heads, n_kv, ps_log2, scale, window, stream
    if constexpr (HD > 128 || !PF_USE_LDS) {
        return HD > 128 ? launch_prefill<1, PF_ROWS / 16, 1>(n_tiles, ARGS) : launch_prefill<2, PF_ROWS / 32, 1>(n_tiles, ARGS);
    } else {
        switch (prefill_shape(n_tiles, n_tiles_split, n_tiles_long, n_heads, q_bound, kv_bound)) {
            case PF_SPLIT: return launch_prefill<1, 2 * PF_ROWS_SPLIT / 16, 2>(n_tiles_split, ARGS);
            case PF_PAIRED: return launch_prefill<2, 2 * PF_ROWS / 32, 2, 2>(n_tiles, ARGS);
            case PF_LONG: return launch_prefill<2, PF_ROWS_LONG / 32, 1, 2>(n_tiles_long, ARGS);
            default: return launch_prefill<2, PF_ROWS / 32, 1>(n_tiles, ARGS);
        }
    }
#undef ARGS
}
