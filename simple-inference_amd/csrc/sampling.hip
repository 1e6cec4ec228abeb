// Sampling of one token per row of float logits [rows, vocab]: argmax, or temperature with
// optional top-k and top-p and a draw by inverting the cumulative distribution at a uniform
// number that the caller supplies (so that a request's draws do not depend on its batch).
//
// Order of operations (reference: sampling.py:141-173): temperature 0 -> argmax, all else
// ignored.  Otherwise x = logits / T; top-k keeps the values not below the k-th largest
// (ties with it stay; reference: sampling.py:69-84); top-p, over what top-k kept, drops a
// token iff the probability mass of the tokens above it already exceeds p (reference:
// sampling.py:96-129; tokens of equal value are kept or dropped together here, where the
// reference's sort splits them arbitrarily); p <= 0 keeps the top value only.  Then softmax
// over what is left, and the token is the first, in index order, whose cumulative
// probability exceeds u * total.
//
// Every row is spread over SP_CHUNKS workgroups, and the work is a short series of launches:
//   1. the maximum (and its index) of each chunk; the row's histograms are set to zero beside it;
//   2. top-k: the k-th largest value by radix selection over the order-preserving integer image
//      of the floats, 11 + 11 + 10 bits, one counting pass per digit;
//   3. top-p: the lowest kept value the same way, with the probability mass per digit in place of
//      the count;
//   4. the mass of what is kept, for SP_PIECES pieces of consecutive tokens of the row (a piece a wave), and then
//      one wave per row that finds the piece in which the cumulative mass passes u * total and the token in it.
// Probabilities enter every sum as fixed-point integers (exp(x - max) * 2^s with the largest s that keeps
// a row's sum below 2^63: 46 bits for 128,256 entries): integer sums do not depend on their order, so
// histograms can be built with atomics and every workgroup that recomputes a sum gets the same bits.  A
// token whose probability is below 2^-s of the most likely one's counts as zero.  A launch starts by reading
// the digit that the histogram of the launch before it decides, and leaves what has been decided so far in the
// row's workspace for the next (every workgroup of a row computes the same bits and writes them to the same
// place).  Launches whose filter no row asks for are skipped by the caller's hint.
#include "common.h"
#include "no_alloc.h"

#include <cstddef>
#include <mutex>

#define SP_CHUNKS 16
#define SP_THREADS 1024
#define SP_WAVES (SP_THREADS / SIA_WAVE)
#define SP_PASSES 3
#define SP_MAX_BINS 2048
#define SP_COUNT_COPIES 4  // histograms of a workgroup in LDS: lanes that meet in a bin add to different copies
#define SP_MASS_COPIES 3
#define SP_PIECES (SP_CHUNKS * SP_WAVES)  // of a row when the kept mass is summed: one for each wave of each chunk

typedef unsigned long long u64;

__host__ __device__ constexpr int sp_shift(int pass) { return pass == 0 ? 21 : pass == 1 ? 10 : 0; }
__host__ __device__ constexpr int sp_bins(int pass) { return pass == 2 ? 1024 : 2048; }

// What one more digit decided: of the k-th largest key (prefix, k_rem) or of the lowest kept key (the rest).
struct Decided {
    uint32_t prefix;  // the digits found so far
    int k_rem;        // rank of the k-th largest among the keys that share them
    u64 carried;      // mass above the keys that share them
    u64 limit;        // p * total mass
};

// What the launches of one row share.  `mass` and `count` are zero before the first counting launch.
struct SampleRow {
    u64 mass[SP_PASSES][SP_MAX_BINS];
    int count[SP_PASSES][SP_MAX_BINS];
    Decided after_k[SP_PASSES], after_p[SP_PASSES];
    u64 piece_mass[SP_PIECES];  // of the kept tokens
    float chunk_max[SP_CHUNKS];
    int chunk_arg[SP_CHUNKS];
};

__device__ __forceinline__ uint32_t ordered_key(float f) {
    const uint32_t u = __float_as_uint(f);
    return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}

__device__ __forceinline__ u64 fixed_mass(float x, float mx, float one) { return (u64)(expf(x - mx) * one); }

__device__ __forceinline__ void take_better(float& bv, int& bi, float v, int i) {
    if (v > bv || (v == bv && i < bi)) { bv = v; bi = i; }
}

// Sum over the lanes above this one.
template <typename T>
__device__ __forceinline__ T lanes_above_sum(T v) {
    const int lane = threadIdx.x & 63;
    T inc = v;
#pragma unroll
    for (int off = 1; off < SIA_WAVE; off <<= 1) {
        const T other = __shfl_down(inc, off, SIA_WAVE);
        if (lane + off < SIA_WAVE) inc += other;
    }
    return inc - v;
}

// Sum over this lane and the lanes below it.
__device__ __forceinline__ u64 lanes_up_to_sum(u64 v) {
    const int lane = threadIdx.x & 63;
#pragma unroll
    for (int off = 1; off < SIA_WAVE; off <<= 1) {
        const u64 other = __shfl_up(v, off, SIA_WAVE);
        if (lane >= off) v += other;
    }
    return v;
}

// What the passes so far have decided for a row; computed by wave 0 of a workgroup.
struct RowState {
    float T, mx;          // temperature, maximum of x = logit / T
    uint32_t cut_k;       // keep keys >= cut_k (0: all); final after SP_PASSES top-k passes
    uint32_t prefix_k;    // digits of the k-th largest key found so far
    uint32_t cut_p;       // keep keys >= cut_p; final after SP_PASSES top-p passes
    uint32_t prefix_p;    // digits of the lowest kept key found so far
    int wants_k, wants_p; // the row has a top-k / a top-p filter to search for
};

// k-th largest: one more digit.  Lane l owns PER bins from l * PER on; lane 63 the highest.
template <int PER>
__device__ __forceinline__ void refine_top_k(const int* __restrict__ count, int shift, Decided& d) {
    const int lane = threadIdx.x & 63, base = lane * PER;
    int c[PER];
    const int4* src = (const int4*)(count + base);
#pragma unroll
    for (int i = 0; i < PER / 4; ++i) {
        const int4 v = src[i];
        c[4 * i] = v.x; c[4 * i + 1] = v.y; c[4 * i + 2] = v.z; c[4 * i + 3] = v.w;
    }
    int local = 0;
#pragma unroll
    for (int b = 0; b < PER; ++b) local += c[b];
    const int above = lanes_above_sum(local);
    int digit = -1, rank = 0;
    if (above < d.k_rem && d.k_rem <= above + local) {  // the lane that holds the k-th
        int seen = above;
#pragma unroll
        for (int b = PER - 1; b >= 0; --b) {
            if (digit < 0 && seen + c[b] >= d.k_rem) { digit = base + b; rank = d.k_rem - seen; }
            seen += c[b];
        }
    }
    const u64 owner = __ballot(digit >= 0);
    if (!owner) return;  // fewer keys than k under these digits (cannot be: k < vocab)
    const int src_lane = __ffsll((long long)owner) - 1;
    digit = __shfl(digit, src_lane, SIA_WAVE);
    rank = __shfl(rank, src_lane, SIA_WAVE);
    d.prefix |= (uint32_t)digit << shift;
    d.k_rem = rank;
}

// Lowest kept key: one more digit.  A bin holds a kept key iff it is not empty and the mass above it
// (carried + the bins above it) does not exceed the limit; the lowest such bin is taken.  With `first` the
// histogram is the whole row's, and the limit is taken from its total.
template <int PER>
__device__ __forceinline__ void refine_top_p(const u64* __restrict__ mass, int shift, Decided& d, float p, bool first) {
    const int lane = threadIdx.x & 63, base = lane * PER;
    u64 m[PER];
    const ulonglong2* src = (const ulonglong2*)(mass + base);
#pragma unroll
    for (int i = 0; i < PER / 2; ++i) {
        const ulonglong2 v = src[i];
        m[2 * i] = v.x; m[2 * i + 1] = v.y;
    }
    u64 local = 0;
#pragma unroll
    for (int b = 0; b < PER; ++b) local += m[b];
    const u64 higher = lanes_above_sum(local);
    if (first) {
        const u64 total = __shfl(higher + local, 0, SIA_WAVE);  // lane 0 has every other lane above it
        d.limit = (u64)((double)p * (double)total);
    }
    u64 above = d.carried + higher;
    int digit = -1;
    u64 above_digit = 0;
#pragma unroll
    for (int b = PER - 1; b >= 0; --b) {
        if (m[b] > 0 && above <= d.limit) { digit = base + b; above_digit = above; }
        above += m[b];
    }
    const u64 owners = __ballot(digit >= 0);
    if (!owners) return;  // no mass at all under these digits (cannot be: the row's maximum has the mass of one)
    const int src_lane = __ffsll((long long)owners) - 1;  // the lowest lane with a kept bin holds the lowest kept bin
    digit = __shfl(digit, src_lane, SIA_WAVE);
    above_digit = __shfl(above_digit, src_lane, SIA_WAVE);
    d.prefix |= (uint32_t)digit << shift;
    d.carried = above_digit;
}

// The row's state when `k_done` top-k and `p_done` top-p histograms are complete.  The digit of the latest
// histogram is decided here and left in the workspace; the digits before it were left there by the launches
// before.  With negative numbers nothing is decided: every digit is in the workspace.  One whole wave calls it.
__device__ __forceinline__ RowState row_state(SampleRow* __restrict__ ws, float T, int k, float p, int vocab,
                                              int filters, int k_done, int p_done) {
    const int lane = threadIdx.x & 63;
    RowState s;
    s.T = T;
    const float mx = wave_max(lane < SP_CHUNKS ? ws->chunk_max[lane] : -INFINITY);
    s.mx = T > 0.f ? mx / T : mx;
    s.wants_k = (filters & 1) && T > 0.f && k > 0 && k < vocab;
    s.wants_p = (filters & 2) && T > 0.f && p > 0.f && p < 1.f;
    s.cut_k = s.prefix_k = 0;
    if (s.wants_k && k_done != 0) {
        Decided d;
        if (k_done < 0 || (s.wants_p && p_done > 0)) {
            d = ws->after_k[SP_PASSES - 1];  // final since the first launch after the last top-k histogram
        } else {
            if (k_done >= 2) d = ws->after_k[k_done - 2];
            else { d.prefix = 0; d.k_rem = k; }
            d.carried = d.limit = 0;
            const int pass = k_done - 1;
            if (pass == 2) refine_top_k<sp_bins(2) / SIA_WAVE>(ws->count[2], sp_shift(2), d);
            else refine_top_k<sp_bins(0) / SIA_WAVE>(ws->count[pass], sp_shift(pass), d);
            if (lane == 0) ws->after_k[pass] = d;
        }
        s.prefix_k = d.prefix;
        if (k_done < 0 || k_done == SP_PASSES) s.cut_k = d.prefix;
    }
    s.cut_p = s.prefix_p = 0;
    if (T > 0.f && p <= 0.f) s.cut_p = ordered_key(s.mx);  // the top value only
    if (s.wants_p && p_done != 0) {
        Decided d;
        if (p_done < 0) {
            d = ws->after_p[SP_PASSES - 1];
        } else {
            if (p_done >= 2) d = ws->after_p[p_done - 2];
            else { d.prefix = 0; d.k_rem = 0; d.carried = d.limit = 0; }
            const int pass = p_done - 1;
            if (pass == 2) refine_top_p<sp_bins(2) / SIA_WAVE>(ws->mass[2], sp_shift(2), d, p, false);
            else refine_top_p<sp_bins(0) / SIA_WAVE>(ws->mass[pass], sp_shift(pass), d, p, pass == 0);
            if (lane == 0) ws->after_p[pass] = d;
        }
        s.prefix_p = d.prefix;
        if (p_done < 0 || p_done == SP_PASSES) s.cut_p = d.prefix;
    }
    return s;
}

// Every thread of the workgroup gets the state that wave 0 computed.
__device__ __forceinline__ RowState shared_row_state(SampleRow* __restrict__ ws, float T, int k, float p, int vocab,
                                                     int filters, int k_done, int p_done) {
    __shared__ RowState shared;
    if (threadIdx.x < SIA_WAVE) {
        const RowState s = row_state(ws, T, k, p, vocab, filters, k_done, p_done);
        if (threadIdx.x == 0) shared = s;
    }
    __syncthreads();
    return shared;
}

__device__ __forceinline__ void chunk_range(int chunk, int vocab, int& begin, int& end) {
    const int per = (vocab + SP_CHUNKS - 1) / SP_CHUNKS;
    begin = min(vocab, chunk * per);
    end = min(vocab, begin + per);
}

// The logits at i0, i0 + stride, ... below `end`, asked for together so that their latencies overlap; -inf, which
// has no probability mass and is nobody's maximum, where there is none.
#define SP_AT_ONCE 8
__device__ __forceinline__ void load_together(const float* __restrict__ row, int i0, int stride, int end,
                                              float (&v)[SP_AT_ONCE]) {
#pragma unroll
    for (int u = 0; u < SP_AT_ONCE; ++u) v[u] = i0 + u * stride < end ? row[i0 + u * stride] : -INFINITY;
}

#define SP_CLEAR_BYTES (sizeof(u64) * SP_PASSES * SP_MAX_BINS + sizeof(int) * SP_PASSES * SP_MAX_BINS)
static_assert(offsetof(SampleRow, after_k) == SP_CLEAR_BYTES, "the histograms lead the row and are contiguous");
static_assert(SP_CLEAR_BYTES % (sizeof(uint4) * SP_CHUNKS) == 0 && sizeof(SampleRow) % sizeof(uint4) == 0,
              "cleared in 16-byte pieces, a share by each chunk's workgroup");

// 1. maximum and its (lowest) index of each chunk, on the raw logits.  With `clear` each chunk's workgroup also
// sets its share of the row's histograms to zero: the counting launches come after this one.
__global__ __launch_bounds__(SP_THREADS) void sample_max_kernel(const float* __restrict__ logits, int vocab,
                                                                SampleRow* __restrict__ ws, int clear) {
    __shared__ float vals[SP_WAVES];
    __shared__ int idxs[SP_WAVES];
    const int chunk = blockIdx.x, r = blockIdx.y;
    const float* row = logits + (size_t)r * vocab;
    int begin, end;
    chunk_range(chunk, vocab, begin, end);
    float bv = -INFINITY;
    int bi = vocab;
    for (int i0 = begin + threadIdx.x; i0 < end; i0 += SP_AT_ONCE * SP_THREADS) {
        float v[SP_AT_ONCE];
        load_together(row, i0, SP_THREADS, end, v);
#pragma unroll
        for (int u = 0; u < SP_AT_ONCE; ++u)
            if (i0 + u * SP_THREADS < end) take_better(bv, bi, v[u], i0 + u * SP_THREADS);
    }
    if (clear) {
        constexpr int share = (int)(SP_CLEAR_BYTES / sizeof(uint4) / SP_CHUNKS);
        uint4* mine = (uint4*)(ws + r) + chunk * share;
        for (int i = threadIdx.x; i < share; i += SP_THREADS) mine[i] = make_uint4(0, 0, 0, 0);
    }
#pragma unroll
    for (int off = SIA_WAVE / 2; off > 0; off >>= 1) {
        const float ov = __shfl_xor(bv, off, SIA_WAVE);
        const int oi = __shfl_xor(bi, off, SIA_WAVE);
        take_better(bv, bi, ov, oi);
    }
    if (threadIdx.x % SIA_WAVE == 0) { vals[threadIdx.x / SIA_WAVE] = bv; idxs[threadIdx.x / SIA_WAVE] = bi; }
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int w = 1; w < SP_WAVES; ++w) take_better(bv, bi, vals[w], idxs[w]);
        ws[r].chunk_max[chunk] = bv;
        ws[r].chunk_arg[chunk] = bi;
    }
}

// A workgroup's histogram in LDS: COPIES of it, each one element longer than its bins so that the same bin of two
// copies lies in different banks.  A thread adds to the copy of its number.
template <typename T, int COPIES>
struct LocalHistogram {
    T bins[COPIES][SP_MAX_BINS + 1];
    __device__ __forceinline__ void clear(int n_bins) {
        for (int c = 0; c < COPIES; ++c)
            for (int b = threadIdx.x; b < n_bins; b += SP_THREADS) bins[c][b] = 0;
    }
    __device__ __forceinline__ void add(int bin, T v) { atomicAdd(&bins[threadIdx.x % COPIES][bin], v); }
    // adds what the workgroup has counted to the row's histogram
    __device__ __forceinline__ void add_to(T* __restrict__ row_bins, int n_bins) {
        for (int b = threadIdx.x; b < n_bins; b += SP_THREADS) {
            T sum = 0;
#pragma unroll
            for (int c = 0; c < COPIES; ++c) sum += bins[c][b];
            if (sum) atomicAdd(&row_bins[b], sum);
        }
    }
};

// 2. one digit of the k-th largest key: counts of the keys that share the digits found so far
__global__ __launch_bounds__(SP_THREADS) void sample_top_k_kernel(const float* __restrict__ logits,
                                                                  const float* __restrict__ temperature,
                                                                  const int* __restrict__ top_k, int vocab,
                                                                  SampleRow* __restrict__ ws, int filters, int pass) {
    __shared__ LocalHistogram<int, SP_COUNT_COPIES> hist;
    const int chunk = blockIdx.x, r = blockIdx.y;
    const float T = temperature[r];
    const int k = top_k[r];
    if (!(T > 0.f && k > 0 && k < vocab)) return;  // the whole workgroup
    const int bins = sp_bins(pass), shift = sp_shift(pass);
    const float* row = logits + (size_t)r * vocab;
    int begin, end;
    chunk_range(chunk, vocab, begin, end);
    int i0 = begin + threadIdx.x;
    float v[SP_AT_ONCE];
    load_together(row, i0, SP_THREADS, end, v);  // on their way while the row's state is made up
    hist.clear(bins);
    const RowState s = shared_row_state(ws + r, T, k, 1.f, vocab, filters, pass, 0);  // with a barrier
    const uint32_t high_mask = pass == 0 ? 0u : ~((1u << (shift + (pass == 1 ? 11 : 10))) - 1u);
    while (i0 < end) {
#pragma unroll
        for (int u = 0; u < SP_AT_ONCE; ++u) {
            const uint32_t key = ordered_key(v[u] / T);
            if (i0 + u * SP_THREADS < end && (key & high_mask) == s.prefix_k) hist.add((key >> shift) & (bins - 1), 1);
        }
        i0 += SP_AT_ONCE * SP_THREADS;
        if (i0 < end) load_together(row, i0, SP_THREADS, end, v);
    }
    __syncthreads();
    hist.add_to(ws[r].count[pass], bins);
}

// 3. one digit of the lowest kept key: mass of the keys (that top-k kept) that share the digits found so far
__global__ __launch_bounds__(SP_THREADS) void sample_top_p_kernel(const float* __restrict__ logits,
                                                                  const float* __restrict__ temperature,
                                                                  const int* __restrict__ top_k,
                                                                  const float* __restrict__ top_p, int vocab,
                                                                  SampleRow* __restrict__ ws, int filters, int pass,
                                                                  float one) {
    __shared__ LocalHistogram<u64, SP_MASS_COPIES> hist;
    const int chunk = blockIdx.x, r = blockIdx.y;
    const float T = temperature[r], p = top_p[r];
    if (!(T > 0.f && p > 0.f && p < 1.f)) return;  // the whole workgroup
    const int bins = sp_bins(pass), shift = sp_shift(pass);
    const float* row = logits + (size_t)r * vocab;
    int begin, end;
    chunk_range(chunk, vocab, begin, end);
    int i0 = begin + threadIdx.x;
    float v[SP_AT_ONCE];
    load_together(row, i0, SP_THREADS, end, v);  // on their way while the row's state is made up
    hist.clear(bins);
    const RowState s = shared_row_state(ws + r, T, top_k[r], p, vocab, filters, (filters & 1) ? SP_PASSES : 0, pass);
    const uint32_t high_mask = pass == 0 ? 0u : ~((1u << (shift + (pass == 1 ? 11 : 10))) - 1u);
    while (i0 < end) {
#pragma unroll
        for (int u = 0; u < SP_AT_ONCE; ++u) {
            const float x = v[u] / T;
            const uint32_t key = ordered_key(x);
            if (key >= s.cut_k && (key & high_mask) == s.prefix_p) {
                const u64 q = fixed_mass(x, s.mx, one);  // none where there is no token
                if (q) hist.add((key >> shift) & (bins - 1), q);
            }
        }
        i0 += SP_AT_ONCE * SP_THREADS;
        if (i0 < end) load_together(row, i0, SP_THREADS, end, v);
    }
    __syncthreads();
    hist.add_to(ws[r].mass[pass], bins);
}

// The tokens of piece `piece` of a row: a chunk is cut into one piece for each wave of its workgroup.
__device__ __forceinline__ void piece_range(int piece, int vocab, int& begin, int& end) {
    int chunk_begin, chunk_end;
    chunk_range(piece / SP_WAVES, vocab, chunk_begin, chunk_end);
    const int per = (chunk_end - chunk_begin + SP_WAVES - 1) / SP_WAVES;
    begin = min(chunk_end, chunk_begin + (piece % SP_WAVES) * per);
    end = min(chunk_end, begin + per);
}

// Mass of the token with logit `v` if it is kept, else 0 (-inf, which stands for "no token", has none).
__device__ __forceinline__ u64 kept_mass(float v, const RowState& s, uint32_t cut, float one) {
    const float x = v / s.T;
    return ordered_key(x) >= cut ? fixed_mass(x, s.mx, one) : 0;
}

// 4a. mass of each piece's kept tokens
__global__ __launch_bounds__(SP_THREADS) void sample_kept_kernel(const float* __restrict__ logits,
                                                                 const float* __restrict__ temperature,
                                                                 const int* __restrict__ top_k,
                                                                 const float* __restrict__ top_p, int vocab,
                                                                 SampleRow* __restrict__ ws, int filters, float one) {
    const int chunk = blockIdx.x, r = blockIdx.y, lane = threadIdx.x & 63, wave = threadIdx.x / SIA_WAVE;
    const float T = temperature[r];
    if (!(T > 0.f)) return;  // the whole workgroup: a greedy row
    const float* row = logits + (size_t)r * vocab;
    const int piece = chunk * SP_WAVES + wave;
    int begin, end;
    piece_range(piece, vocab, begin, end);
    int i0 = begin + lane;
    float v[SP_AT_ONCE];
    load_together(row, i0, SIA_WAVE, end, v);  // on their way while the row's state is made up
    const RowState s = shared_row_state(ws + r, T, top_k[r], top_p[r], vocab, filters, (filters & 1) ? SP_PASSES : 0,
                                        (filters & 2) ? SP_PASSES : 0);
    const uint32_t cut = max(s.cut_k, s.cut_p);
    u64 sum = 0;
    while (i0 < end) {
#pragma unroll
        for (int u = 0; u < SP_AT_ONCE; ++u) sum += kept_mass(v[u], s, cut, one);
        i0 += SP_AT_ONCE * SIA_WAVE;
        if (i0 < end) load_together(row, i0, SIA_WAVE, end, v);
    }
    sum += lanes_above_sum(sum);  // lane 0 holds the piece's
    if (lane == 0) ws[r].piece_mass[piece] = sum;
}

// 4b. the token: argmax for a greedy row; else the first token, in index order, at which the cumulative mass of
// what is kept exceeds u * total: first the piece, then the token in it.  One wave per row.
__global__ __launch_bounds__(SIA_WAVE) void sample_pick_kernel(const float* __restrict__ logits,
                                                               const float* __restrict__ temperature,
                                                               const int* __restrict__ top_k,
                                                               const float* __restrict__ top_p,
                                                               const float* __restrict__ uniform,
                                                               int* __restrict__ out, int vocab,
                                                               SampleRow* __restrict__ ws, int filters, float one) {
    const int r = blockIdx.x, lane = threadIdx.x;
    const float T = temperature ? temperature[r] : 0.f;
    int pick = -1;
    if (T > 0.f) {
        const RowState s = row_state(ws + r, T, top_k[r], top_p[r], vocab, filters, -1, -1);
        const uint32_t cut = max(s.cut_k, s.cut_p);
        constexpr int each = SP_PIECES / SIA_WAVE;  // lane l looks at pieces each * l onwards
        u64 mine = 0;
#pragma unroll
        for (int j = 0; j < each; ++j) mine += ws[r].piece_mass[lane * each + j];
        u64 up_to = lanes_up_to_sum(mine);
        const u64 total = __shfl(up_to, SIA_WAVE - 1, SIA_WAVE);
        u64 target = (u64)((double)uniform[r] * (double)total);
        if (total > 0 && target >= total) target = total - 1;
        u64 passes = __ballot(up_to > target);
        if (passes) {  // else nothing kept has mass in fixed point
            const int owner = __ffsll((long long)passes) - 1;
            int piece = lane * each;
            u64 before = up_to - mine;
            for (int j = 0; j < each - 1 && before + ws[r].piece_mass[piece] <= target; ++j)
                before += ws[r].piece_mass[piece++];
            piece = __shfl(piece, owner, SIA_WAVE);
            before = __shfl(before, owner, SIA_WAVE);
            const float* row = logits + (size_t)r * vocab;
            int begin, end;
            piece_range(piece, vocab, begin, end);
            for (int i0 = begin; i0 < end && pick < 0; i0 += SP_AT_ONCE * SIA_WAVE) {
                float v[SP_AT_ONCE];
                load_together(row, i0 + lane, SIA_WAVE, end, v);
#pragma unroll
                for (int u = 0; u < SP_AT_ONCE; ++u) {
                    if (pick < 0) {  // the same in every lane
                        up_to = before + lanes_up_to_sum(kept_mass(v[u], s, cut, one));
                        passes = __ballot(up_to > target);
                        if (passes) pick = i0 + u * SIA_WAVE + __ffsll((long long)passes) - 1;
                        before = __shfl(up_to, SIA_WAVE - 1, SIA_WAVE);
                    }
                }
            }
        }
    }
    if (lane == 0) {
        if (pick < 0) {  // a greedy row, or nothing but the row's maximum itself has mass in fixed point: that one
            float bv = -INFINITY;
            int bi = vocab;
            for (int c = 0; c < SP_CHUNKS; ++c) take_better(bv, bi, ws[r].chunk_max[c], ws[r].chunk_arg[c]);
            pick = bi < vocab ? bi : 0;
        }
        out[r] = pick;
    }
}

SIA_EXPORT long long sia_sample_workspace_bytes(int rows) { return (long long)rows * (long long)sizeof(SampleRow); }

// The launches of one call.
static int launch_sampling(const float* logits, const float* temperature, const int* top_k, const float* top_p,
                           const float* uniform, int* out, SampleRow* ws, int rows, int vocab, int filters,
                           hipStream_t stream) {
    const dim3 grid(SP_CHUNKS, rows), block(SP_THREADS);
    int bits = 62;  // fixed point: vocab * 2^bits < 2^63
    while (bits > 0 && ((long long)vocab << bits) >> bits != (long long)vocab) --bits;
    while (bits > 0 && (double)vocab * (double)(1ull << bits) >= 9.2e18) --bits;
    const float one = (float)(1ull << bits);
    hipLaunchKernelGGL(sample_max_kernel, grid, block, 0, stream, logits, vocab, ws, (filters & 3) != 0);
    if (filters & 1)
        for (int pass = 0; pass < SP_PASSES; ++pass)
            hipLaunchKernelGGL(sample_top_k_kernel, grid, block, 0, stream, logits, temperature, top_k, vocab, ws,
                               filters, pass);
    if (filters & 2)
        for (int pass = 0; pass < SP_PASSES; ++pass)
            hipLaunchKernelGGL(sample_top_p_kernel, grid, block, 0, stream, logits, temperature, top_k, top_p, vocab,
                               ws, filters, pass, one);
    if (filters)
        hipLaunchKernelGGL(sample_kept_kernel, grid, block, 0, stream, logits, temperature, top_k, top_p, vocab, ws,
                           filters, one);
    hipLaunchKernelGGL(sample_pick_kernel, dim3(rows), dim3(SIA_WAVE), 0, stream, logits,
                       filters ? temperature : nullptr, top_k, top_p, uniform, out, vocab, ws, filters, one);
    return SIA_LAUNCH_CHECK();
}

// One token per row.  workspace: sia_sample_workspace_bytes(rows) bytes, aligned to 16, which may hold anything
// (what has to start at zero is set to zero by the first launch); calls that share a workspace must not overlap.
// filters: bit 0 set if some row may have a top-k filter, bit 1 if some row may have a top-p filter in (0, 1),
// bit 2 if some row has a temperature above 0; launches for filters that no row has are skipped, and a filter
// whose bit is not set is not applied (rows decide for themselves inside the launches that run).  With
// filters == 0 the parameter pointers may be null: every row takes its argmax.
SIA_EXPORT int sia_sample(const float* logits, const float* temperature, const int* top_k, const float* top_p,
                          const float* uniform, int* out, void* workspace, int rows, int vocab, int filters,
                          hipStream_t stream) {
    if (rows <= 0) return 0;
    if (vocab <= 0 || rows > 65535 || !workspace || ((uintptr_t)workspace & 15)) return SIA_BAD_ARGUMENT;
    if (filters && (!temperature || !top_k || !top_p || !uniform)) return SIA_BAD_ARGUMENT;
    return launch_sampling(logits, temperature, top_k, top_p, uniform, out, (SampleRow*)workspace, rows, vocab, filters,
                           stream);
}

// ---- the same, for callers that cannot allocate -------------------------------------------------------------
// The workspace is a fixed array in device memory that belongs to this library: SIA_SAMPLE_STATIC_MAX_ROWS rows
// (about 4.5 MiB on every GPU the library is used on, until the process ends).  Host code never passes the
// array's name to a kernel: the name is a host-side stand-in, and each GPU holds a copy of its own, so the device
// address is asked for once per device, with that device current, and kept.
static __device__ __align__(256) unsigned char scratch[SIA_SAMPLE_STATIC_MAX_ROWS * sizeof(SampleRow)];

#define SIA_MAX_DEVICES 64
static void* scratch_on_device[SIA_MAX_DEVICES];
static std::mutex scratch_guard;

// Device address of `scratch` on the current device.
static int scratch_address(SampleRow** out) {
    int device = -1;
    hipError_t err = hipGetDevice(&device);
    if (err != hipSuccess) return (int)err;
    if (device < 0 || device >= SIA_MAX_DEVICES) return SIA_BAD_ARGUMENT;
    std::lock_guard<std::mutex> hold(scratch_guard);
    if (!scratch_on_device[device]) {
        void* ptr = nullptr;
        err = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
        if (err != hipSuccess) return (int)err;
        if (!ptr) return SIA_BAD_ARGUMENT;
        scratch_on_device[device] = ptr;
    }
    *out = (SampleRow*)scratch_on_device[device];
    return 0;
}

SIA_EXPORT int sia_sample_static_max_rows(void) { return SIA_SAMPLE_STATIC_MAX_ROWS; }

SIA_EXPORT int sia_sample_static_init(void) {
    SampleRow* ws = nullptr;
    return scratch_address(&ws);
}

SIA_EXPORT int sia_sample_static(const float* logits, const float* temperature, const int* top_k, const float* top_p,
                                 const float* uniform, int* out, int rows, int vocab, int filters,
                                 hipStream_t stream) {
    if (rows <= 0) return 0;
    if (vocab <= 0 || rows > SIA_SAMPLE_STATIC_MAX_ROWS) return SIA_BAD_ARGUMENT;
    if (filters && (!temperature || !top_k || !top_p || !uniform)) return SIA_BAD_ARGUMENT;
    SampleRow* ws = nullptr;
    const int err = scratch_address(&ws);
    if (err) return err;
    // the last call's histograms are still there: the first launch sets them to zero (with a kernel's stores, not
    // a memset, which a caller that records a graph could not rely on)
    return launch_sampling(logits, temperature, top_k, top_p, uniform, out, ws, rows, vocab, filters, stream);
}
