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
//   1. the maximum (and its index) of each chunk;
//   2. top-k: the k-th largest value by radix selection over the order-preserving integer image
//      of the floats, 11 + 11 + 10 bits, one counting pass per digit;
//   3. top-p: the lowest kept value the same way, with the probability mass per digit in place of
//      the count;
//   4. the kept mass of each chunk, then one workgroup per row finds the chunk and the token.
// Probabilities enter every sum as fixed-point integers (exp(x - max) * 2^s with the largest s that keeps
// a row's sum below 2^63: 46 bits for 128,256 entries): integer sums do not depend on their order, so
// histograms can be built with atomics and every workgroup that recomputes a sum gets the same bits.  A
// token whose probability is below 2^-s of the most likely one's counts as zero.  A pass starts by
// recomputing, from the histograms of the passes before it, what those passes decided; nothing but the
// histograms travels between launches.  Launches whose filter no row asks for are skipped by the caller's hint.
#include "common.h"
#include "no_alloc.h"

#include <cstddef>
#include <mutex>

#define SP_CHUNKS 16
#define SP_THREADS 1024
#define SP_PASSES 3
#define SP_MAX_BINS 2048

typedef unsigned long long u64;

__host__ __device__ constexpr int sp_shift(int pass) { return pass == 0 ? 21 : pass == 1 ? 10 : 0; }
__host__ __device__ constexpr int sp_bins(int pass) { return pass == 2 ? 1024 : 2048; }

// What the launches of one row share.  `mass` and `count` start at zero.
struct SampleRow {
    u64 mass[SP_PASSES][SP_MAX_BINS];
    int count[SP_PASSES][SP_MAX_BINS];
    u64 kept[SP_CHUNKS];
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

// What the passes so far have decided for a row; computed by wave 0 of a workgroup.
struct RowState {
    float T, mx;          // temperature, maximum of x = logit / T
    uint32_t cut_k;       // keep keys >= cut_k (0: all); final after SP_PASSES top-k passes
    uint32_t prefix_k;    // digits of the k-th largest key found so far
    int k_rem;            // its rank among the keys that share those digits
    uint32_t cut_p;       // keep keys >= cut_p; final after SP_PASSES top-p passes
    uint32_t prefix_p;    // digits of the lowest kept key found so far
    u64 carried, limit;   // mass above the keys that share those digits; p * total mass
    int wants_k, wants_p; // the row has a top-k / a top-p filter to search for
};

// k-th largest: one more digit.  Lane l owns bins [l * per, (l + 1) * per); lane 63 the highest.
__device__ __forceinline__ void refine_top_k(const int* __restrict__ count, int pass, uint32_t& prefix, int& k_rem) {
    const int lane = threadIdx.x & 63, per = sp_bins(pass) / SIA_WAVE, base = lane * per;
    int local = 0;
    for (int b = 0; b < per; ++b) local += count[base + b];
    const int above = lanes_above_sum(local);
    int digit = -1, rank = 0;
    if (above < k_rem && k_rem <= above + local) {  // the lane that holds the k-th
        int c = above;
        for (int b = base + per - 1; b >= base; --b) {
            if (c + count[b] >= k_rem) { digit = b; rank = k_rem - c; break; }
            c += count[b];
        }
    }
    const u64 owner = __ballot(digit >= 0);
    const int src = owner ? __ffsll((long long)owner) - 1 : 0;
    digit = __shfl(digit, src, SIA_WAVE);
    rank = __shfl(rank, src, SIA_WAVE);
    if (owner) {
        prefix |= (uint32_t)digit << sp_shift(pass);
        k_rem = rank;
    }
}

// Lowest kept key: one more digit.  A bin holds a kept key iff it is not empty and the mass above it
// (carried + the bins above it) does not exceed the limit; the lowest such bin is taken.
__device__ __forceinline__ void refine_top_p(const u64* __restrict__ mass, int pass, uint32_t& prefix, u64& carried,
                                             u64 limit) {
    const int lane = threadIdx.x & 63, per = sp_bins(pass) / SIA_WAVE, base = lane * per;
    u64 local = 0;
    for (int b = 0; b < per; ++b) local += mass[base + b];
    u64 above = carried + lanes_above_sum(local);
    int digit = -1;
    u64 above_digit = 0;
    for (int b = base + per - 1; b >= base; --b) {
        if (mass[b] > 0 && above <= limit) { digit = b; above_digit = above; }
        above += mass[b];
    }
    const u64 owners = __ballot(digit >= 0);
    if (!owners) return;  // no mass at all under these digits (cannot be: the row's maximum has the mass of one)
    const int src = __ffsll((long long)owners) - 1;  // the lowest lane with a kept bin holds the lowest kept bin
    digit = __shfl(digit, src, SIA_WAVE);
    above_digit = __shfl(above_digit, src, SIA_WAVE);
    prefix |= (uint32_t)digit << sp_shift(pass);
    carried = above_digit;
}

// Recomputes the row's state after `k_passes` top-k and `p_passes` top-p passes.  Wave 0 calls it.
__device__ __forceinline__ RowState row_state(const SampleRow* __restrict__ ws, float T, int k, float p, int vocab,
                                              int k_passes, int p_passes) {
    RowState s;
    s.T = T;
    float mx = -INFINITY;
    for (int c = 0; c < SP_CHUNKS; ++c) mx = fmaxf(mx, ws->chunk_max[c]);
    s.mx = T > 0.f ? mx / T : mx;
    s.wants_k = T > 0.f && k > 0 && k < vocab;
    s.wants_p = T > 0.f && p > 0.f && p < 1.f;
    s.cut_k = s.prefix_k = 0;
    s.k_rem = k;
    if (s.wants_k) {
        for (int pass = 0; pass < k_passes; ++pass) refine_top_k(ws->count[pass], pass, s.prefix_k, s.k_rem);
        if (k_passes == SP_PASSES) s.cut_k = s.prefix_k;
    }
    s.cut_p = s.prefix_p = 0;
    s.carried = s.limit = 0;
    if (T > 0.f && p <= 0.f) s.cut_p = ordered_key(s.mx);  // the top value only
    if (s.wants_p && p_passes > 0) {
        const int lane = threadIdx.x & 63, per = sp_bins(0) / SIA_WAVE;
        u64 total = 0;
        for (int b = 0; b < per; ++b) total += ws->mass[0][lane * per + b];
        total += lanes_above_sum(total);            // lane 0 now holds the row's total
        total = __shfl(total, 0, SIA_WAVE);
        s.limit = (u64)((double)p * (double)total);
        for (int pass = 0; pass < p_passes; ++pass) refine_top_p(ws->mass[pass], pass, s.prefix_p, s.carried, s.limit);
        if (p_passes == SP_PASSES) s.cut_p = s.prefix_p;
    }
    return s;
}

// Every thread of the workgroup gets the state that wave 0 computed.
__device__ __forceinline__ RowState shared_row_state(const SampleRow* __restrict__ ws, float T, int k, float p,
                                                     int vocab, int k_passes, int p_passes) {
    __shared__ RowState shared;
    if (threadIdx.x < SIA_WAVE) {
        const RowState s = row_state(ws, T, k, p, vocab, k_passes, p_passes);
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

// 1. maximum and its (lowest) index of each chunk, on the raw logits
__global__ __launch_bounds__(SP_THREADS) void sample_max_kernel(const float* __restrict__ logits, int vocab,
                                                                SampleRow* __restrict__ ws) {
    __shared__ float vals[SP_THREADS / SIA_WAVE];
    __shared__ int idxs[SP_THREADS / SIA_WAVE];
    const int chunk = blockIdx.x, r = blockIdx.y;
    const float* row = logits + (size_t)r * vocab;
    int begin, end;
    chunk_range(chunk, vocab, begin, end);
    float bv = -INFINITY;
    int bi = vocab;
    for (int i = begin + threadIdx.x; i < end; i += SP_THREADS) take_better(bv, bi, row[i], i);
#pragma unroll
    for (int off = SIA_WAVE / 2; off > 0; off >>= 1) {
        const float ov = __shfl_xor(bv, off, SIA_WAVE);
        const int oi = __shfl_xor(bi, off, SIA_WAVE);
        take_better(bv, bi, ov, oi);
    }
    if (threadIdx.x % SIA_WAVE == 0) { vals[threadIdx.x / SIA_WAVE] = bv; idxs[threadIdx.x / SIA_WAVE] = bi; }
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int w = 1; w < SP_THREADS / SIA_WAVE; ++w) take_better(bv, bi, vals[w], idxs[w]);
        ws[r].chunk_max[chunk] = bv;
        ws[r].chunk_arg[chunk] = bi;
    }
}

// 2. one digit of the k-th largest key: counts of the keys that share the digits found so far
__global__ __launch_bounds__(SP_THREADS) void sample_top_k_kernel(const float* __restrict__ logits,
                                                                  const float* __restrict__ temperature,
                                                                  const int* __restrict__ top_k, int vocab,
                                                                  SampleRow* __restrict__ ws, int pass) {
    __shared__ int hist[SP_MAX_BINS];
    const int chunk = blockIdx.x, r = blockIdx.y;
    const float T = temperature[r];
    const int k = top_k[r];
    if (!(T > 0.f && k > 0 && k < vocab)) return;  // the whole workgroup
    const RowState s = shared_row_state(ws + r, T, k, 1.f, vocab, pass, 0);
    const int bins = sp_bins(pass), shift = sp_shift(pass);
    for (int b = threadIdx.x; b < bins; b += SP_THREADS) hist[b] = 0;
    __syncthreads();
    const uint32_t high_mask = pass == 0 ? 0u : ~((1u << (shift + (pass == 1 ? 11 : 10))) - 1u);
    const float* row = logits + (size_t)r * vocab;
    int begin, end;
    chunk_range(chunk, vocab, begin, end);
    for (int i = begin + threadIdx.x; i < end; i += SP_THREADS) {
        const uint32_t key = ordered_key(row[i] / T);
        if ((key & high_mask) == s.prefix_k) atomicAdd(&hist[(key >> shift) & (bins - 1)], 1);
    }
    __syncthreads();
    for (int b = threadIdx.x; b < bins; b += SP_THREADS)
        if (hist[b]) atomicAdd(&ws[r].count[pass][b], hist[b]);
}

// 3. one digit of the lowest kept key: mass of the keys (that top-k kept) that share the digits found so far
__global__ __launch_bounds__(SP_THREADS) void sample_top_p_kernel(const float* __restrict__ logits,
                                                                  const float* __restrict__ temperature,
                                                                  const int* __restrict__ top_k,
                                                                  const float* __restrict__ top_p, int vocab,
                                                                  SampleRow* __restrict__ ws, int pass, float one) {
    __shared__ u64 hist[SP_MAX_BINS];
    const int chunk = blockIdx.x, r = blockIdx.y;
    const float T = temperature[r], p = top_p[r];
    if (!(T > 0.f && p > 0.f && p < 1.f)) return;  // the whole workgroup
    const RowState s = shared_row_state(ws + r, T, top_k[r], p, vocab, SP_PASSES, pass);
    const int bins = sp_bins(pass), shift = sp_shift(pass);
    for (int b = threadIdx.x; b < bins; b += SP_THREADS) hist[b] = 0;
    __syncthreads();
    const uint32_t high_mask = pass == 0 ? 0u : ~((1u << (shift + (pass == 1 ? 11 : 10))) - 1u);
    const float* row = logits + (size_t)r * vocab;
    int begin, end;
    chunk_range(chunk, vocab, begin, end);
    for (int i = begin + threadIdx.x; i < end; i += SP_THREADS) {
        const float x = row[i] / T;
        const uint32_t key = ordered_key(x);
        if (key >= s.cut_k && (key & high_mask) == s.prefix_p) {
            const u64 q = fixed_mass(x, s.mx, one);
            if (q) atomicAdd(&hist[(key >> shift) & (bins - 1)], q);
        }
    }
    __syncthreads();
    for (int b = threadIdx.x; b < bins; b += SP_THREADS)
        if (hist[b]) atomicAdd(&ws[r].mass[pass][b], hist[b]);
}

// 4a. mass of each chunk's kept tokens
__global__ __launch_bounds__(SP_THREADS) void sample_kept_kernel(const float* __restrict__ logits,
                                                                 const float* __restrict__ temperature,
                                                                 const int* __restrict__ top_k,
                                                                 const float* __restrict__ top_p, int vocab,
                                                                 SampleRow* __restrict__ ws, float one) {
    __shared__ u64 sums[SP_THREADS / SIA_WAVE];
    const int chunk = blockIdx.x, r = blockIdx.y;
    const float T = temperature[r];
    if (!(T > 0.f)) return;  // the whole workgroup: a greedy row
    const RowState s = shared_row_state(ws + r, T, top_k[r], top_p[r], vocab, SP_PASSES, SP_PASSES);
    const uint32_t cut = max(s.cut_k, s.cut_p);
    const float* row = logits + (size_t)r * vocab;
    int begin, end;
    chunk_range(chunk, vocab, begin, end);
    u64 sum = 0;
    for (int i = begin + threadIdx.x; i < end; i += SP_THREADS) {
        const float x = row[i] / T;
        if (ordered_key(x) >= cut) sum += fixed_mass(x, s.mx, one);
    }
    sum += lanes_above_sum(sum);  // lane 0 of each wave holds the wave's sum
    if (threadIdx.x % SIA_WAVE == 0) sums[threadIdx.x / SIA_WAVE] = sum;
    __syncthreads();
    if (threadIdx.x == 0) {
        u64 total = 0;
        for (int w = 0; w < SP_THREADS / SIA_WAVE; ++w) total += sums[w];
        ws[r].kept[chunk] = total;
    }
}

// 4b. the token: argmax for a greedy row; else the chunk, then the token, at which the cumulative kept mass
// in index order first exceeds u * total
__global__ __launch_bounds__(SP_THREADS) void sample_pick_kernel(const float* __restrict__ logits,
                                                                 const float* __restrict__ temperature,
                                                                 const int* __restrict__ top_k,
                                                                 const float* __restrict__ top_p,
                                                                 const float* __restrict__ uniform,
                                                                 int* __restrict__ out, int vocab,
                                                                 const SampleRow* __restrict__ ws, float one) {
    __shared__ u64 wave_sum[SP_THREADS / SIA_WAVE];
    __shared__ int picked;
    const int r = blockIdx.x, tid = threadIdx.x, lane = tid & 63, wave = tid / SIA_WAVE;
    const float T = temperature ? temperature[r] : 0.f;
    if (!(T > 0.f)) {
        if (tid == 0) {
            float bv = -INFINITY;
            int bi = vocab;
            for (int c = 0; c < SP_CHUNKS; ++c) take_better(bv, bi, ws[r].chunk_max[c], ws[r].chunk_arg[c]);
            out[r] = bi < vocab ? bi : 0;
        }
        return;
    }
    const RowState s = shared_row_state(ws + r, T, top_k[r], top_p[r], vocab, SP_PASSES, SP_PASSES);
    const uint32_t cut = max(s.cut_k, s.cut_p);
    u64 total = 0;
    for (int c = 0; c < SP_CHUNKS; ++c) total += ws[r].kept[c];
    u64 target = (u64)((double)uniform[r] * (double)total);
    if (total > 0 && target >= total) target = total - 1;
    int chunk = 0;
    u64 before = 0;
    for (; chunk < SP_CHUNKS - 1; ++chunk) {
        if (before + ws[r].kept[chunk] > target) break;
        before += ws[r].kept[chunk];
    }
    // within the chunk: every thread takes a run of consecutive tokens
    const float* row = logits + (size_t)r * vocab;
    int begin, end;
    chunk_range(chunk, vocab, begin, end);
    const int per_thread = (end - begin + SP_THREADS - 1) / SP_THREADS;
    const int i0 = min(end, begin + tid * per_thread), i1 = min(end, i0 + per_thread);
    u64 mine = 0;
    for (int i = i0; i < i1; ++i) {
        const float x = row[i] / T;
        if (ordered_key(x) >= cut) mine += fixed_mass(x, s.mx, one);
    }
    // mass of the threads before this one
    u64 inc = mine;
#pragma unroll
    for (int off = 1; off < SIA_WAVE; off <<= 1) {
        const u64 other = __shfl_up(inc, off, SIA_WAVE);
        if (lane >= off) inc += other;
    }
    if (lane == SIA_WAVE - 1) wave_sum[wave] = inc;
    if (tid == 0) picked = -1;
    __syncthreads();
    u64 cum = before + inc - mine;
    for (int w = 0; w < wave; ++w) cum += wave_sum[w];
    if (cum <= target && target < cum + mine) {  // at most one thread
        for (int i = i0; i < i1; ++i) {
            const float x = row[i] / T;
            if (ordered_key(x) >= cut) {
                cum += fixed_mass(x, s.mx, one);
                if (cum > target) { picked = i; break; }
            }
        }
    }
    __syncthreads();
    if (tid == 0) {
        int pick = picked;
        if (pick < 0) {  // nothing kept has mass in fixed point beyond the row's maximum itself: take that
            float bv = -INFINITY;
            int bi = vocab;
            for (int c = 0; c < SP_CHUNKS; ++c) take_better(bv, bi, ws[r].chunk_max[c], ws[r].chunk_arg[c]);
            pick = bi < vocab ? bi : 0;
        }
        out[r] = pick;
    }
}

SIA_EXPORT long long sia_sample_workspace_bytes(int rows) { return (long long)rows * (long long)sizeof(SampleRow); }

// The launches of one call, on a workspace whose histograms are zero.
static int launch_sampling(const float* logits, const float* temperature, const int* top_k, const float* top_p,
                           const float* uniform, int* out, SampleRow* ws, int rows, int vocab, int filters,
                           hipStream_t stream) {
    const dim3 grid(SP_CHUNKS, rows), block(SP_THREADS);
    int bits = 62;  // fixed point: vocab * 2^bits < 2^63
    while (bits > 0 && ((long long)vocab << bits) >> bits != (long long)vocab) --bits;
    while (bits > 0 && (double)vocab * (double)(1ull << bits) >= 9.2e18) --bits;
    const float one = (float)(1ull << bits);
    hipLaunchKernelGGL(sample_max_kernel, grid, block, 0, stream, logits, vocab, ws);
    if (filters & 1)
        for (int pass = 0; pass < SP_PASSES; ++pass)
            hipLaunchKernelGGL(sample_top_k_kernel, grid, block, 0, stream, logits, temperature, top_k, vocab, ws, pass);
    if (filters & 2)
        for (int pass = 0; pass < SP_PASSES; ++pass)
            hipLaunchKernelGGL(sample_top_p_kernel, grid, block, 0, stream, logits, temperature, top_k, top_p, vocab,
                               ws, pass, one);
    if (filters)
        hipLaunchKernelGGL(sample_kept_kernel, grid, block, 0, stream, logits, temperature, top_k, top_p, vocab, ws,
                           one);
    hipLaunchKernelGGL(sample_pick_kernel, dim3(rows), block, 0, stream, logits, filters ? temperature : nullptr, top_k,
                       top_p, uniform, out, vocab, ws, one);
    return SIA_LAUNCH_CHECK();
}

// One token per row.  workspace: sia_sample_workspace_bytes(rows) bytes, all zero (with filters == 0 they may
// hold anything).  filters: bit 0 set if
// some row may have a top-k filter, bit 1 if some row may have a top-p filter in (0, 1), bit 2 if some row has
// a temperature above 0; launches for filters that no row has are skipped (rows decide for themselves inside
// the launches that run).  With filters == 0 the parameter pointers may be null: every row takes its argmax.
SIA_EXPORT int sia_sample(const float* logits, const float* temperature, const int* top_k, const float* top_p,
                          const float* uniform, int* out, void* workspace, int rows, int vocab, int filters,
                          hipStream_t stream) {
    if (rows <= 0) return 0;
    if (vocab <= 0 || rows > 65535 || !workspace) return SIA_BAD_ARGUMENT;
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

// Zeroes the histograms (the leading members of SampleRow) of the first rows of a workspace.  A kernel, not a
// memset: a caller may be recording a graph, and fill nodes are not reliable in replayed graphs.
#define SP_CLEAR_BYTES (sizeof(u64) * SP_PASSES * SP_MAX_BINS + sizeof(int) * SP_PASSES * SP_MAX_BINS)
static_assert(offsetof(SampleRow, kept) == SP_CLEAR_BYTES, "the histograms lead the row and are contiguous");
static_assert(SP_CLEAR_BYTES % sizeof(uint4) == 0 && sizeof(SampleRow) % sizeof(uint4) == 0, "cleared in 16-byte pieces");
__global__ __launch_bounds__(SP_THREADS) void sample_clear_kernel(SampleRow* __restrict__ ws) {
    const int piece = blockIdx.x * SP_THREADS + threadIdx.x;
    if (piece < (int)(SP_CLEAR_BYTES / sizeof(uint4))) ((uint4*)(ws + blockIdx.y))[piece] = make_uint4(0, 0, 0, 0);
}

SIA_EXPORT int sia_sample_static_max_rows(void) { return SIA_SAMPLE_STATIC_MAX_ROWS; }

SIA_EXPORT int sia_sample_static(const float* logits, const float* temperature, const int* top_k, const float* top_p,
                                 const float* uniform, int* out, int rows, int vocab, int filters,
                                 hipStream_t stream) {
    if (rows <= 0) return 0;
    if (vocab <= 0 || rows > SIA_SAMPLE_STATIC_MAX_ROWS) return SIA_BAD_ARGUMENT;
    if (filters && (!temperature || !top_k || !top_p || !uniform)) return SIA_BAD_ARGUMENT;
    SampleRow* ws = nullptr;
    const int err = scratch_address(&ws);
    if (err) return err;
    if (filters) {  // the last call's histograms are still there
        const int pieces = (int)(SP_CLEAR_BYTES / sizeof(uint4));
        hipLaunchKernelGGL(sample_clear_kernel, dim3((pieces + SP_THREADS - 1) / SP_THREADS, rows), dim3(SP_THREADS), 0,
                           stream, ws);
    }
    return launch_sampling(logits, temperature, top_k, top_p, uniform, out, ws, rows, vocab, filters, stream);
}
