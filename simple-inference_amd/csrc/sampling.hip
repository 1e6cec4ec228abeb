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
// in float over what is left, and the token is the first, in index order, whose cumulative
// probability exceeds u * total.
//
// One workgroup of 1024 threads per row.  The k-th largest value and the top-p cut are
// found by bitwise search over the order-preserving integer image of the floats, one
// counting pass per bit.  The greedy and plain-temperature rows make no such passes.
#include "common.h"

#define SAMPLE_THREADS 1024

__device__ __forceinline__ uint32_t ordered_key(float f) {
    const uint32_t u = __float_as_uint(f);
    return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}

__device__ __forceinline__ int block_sum_int(int v, int* scratch) {
#pragma unroll
    for (int off = SIA_WAVE / 2; off > 0; off >>= 1) v += __shfl_xor(v, off, SIA_WAVE);
    const int wave = threadIdx.x / SIA_WAVE, lane = threadIdx.x % SIA_WAVE;
    if (lane == 0) scratch[wave] = v;
    __syncthreads();
    int total = 0;
    for (int w = 0; w < SAMPLE_THREADS / SIA_WAVE; ++w) total += scratch[w];
    __syncthreads();
    return total;
}

__global__ __launch_bounds__(SAMPLE_THREADS) void sample_kernel(
    const float* __restrict__ logits, const float* __restrict__ temperature, const int* __restrict__ top_k,
    const float* __restrict__ top_p, const float* __restrict__ uniform, int* __restrict__ out, int vocab) {
    __shared__ float fscratch[16];
    __shared__ int iscratch[16];
    __shared__ float chunk_sum[SAMPLE_THREADS];
    __shared__ float best_val[16];
    __shared__ int best_idx[16];
    __shared__ int chosen_chunk;
    __shared__ float chosen_before;

    const int r = blockIdx.x, tid = threadIdx.x;
    const float* row = logits + (size_t)r * vocab;
    const float T = temperature[r];

    if (T == 0.f) {  // argmax, lowest index among equals
        float bv = -INFINITY;
        int bi = vocab;
        for (int i = tid; i < vocab; i += SAMPLE_THREADS) {
            const float v = row[i];
            if (v > bv || (v == bv && i < bi)) { bv = v; bi = i; }
        }
#pragma unroll
        for (int off = SIA_WAVE / 2; off > 0; off >>= 1) {
            const float ov = __shfl_xor(bv, off, SIA_WAVE);
            const int oi = __shfl_xor(bi, off, SIA_WAVE);
            if (ov > bv || (ov == bv && oi < bi)) { bv = ov; bi = oi; }
        }
        if (tid % SIA_WAVE == 0) { best_val[tid / SIA_WAVE] = bv; best_idx[tid / SIA_WAVE] = bi; }
        __syncthreads();
        if (tid == 0) {
            for (int w = 1; w < SAMPLE_THREADS / SIA_WAVE; ++w)
                if (best_val[w] > bv || (best_val[w] == bv && best_idx[w] < bi)) { bv = best_val[w]; bi = best_idx[w]; }
            out[r] = bi < vocab ? bi : 0;
        }
        return;
    }

    const int k = top_k[r];
    const float p = top_p[r];
    uint32_t cut = 0;  // keep tokens whose key >= cut

    float mx = -INFINITY;
    for (int i = tid; i < vocab; i += SAMPLE_THREADS) mx = fmaxf(mx, row[i] / T);
    mx = block_max(mx, fscratch);

    if (k > 0 && k < vocab) {  // key of the k-th largest value
        uint32_t t = 0;
        for (int bit = 31; bit >= 0; --bit) {
            const uint32_t cand = t | (1u << bit);
            int c = 0;
            for (int i = tid; i < vocab; i += SAMPLE_THREADS) c += ordered_key(row[i] / T) >= cand;
            if (block_sum_int(c, iscratch) >= k) t = cand;
        }
        cut = t;
    }
    if (p <= 0.f) {
        cut = ordered_key(mx);
    } else if (p < 1.f) {
        float z = 0.f;
        for (int i = tid; i < vocab; i += SAMPLE_THREADS) {
            const float x = row[i] / T;
            if (ordered_key(x) >= cut) z += expf(x - mx);
        }
        z = block_sum(z, fscratch);
        const float limit = p * z;
        // f(t) = [mass of kept tokens with key > t  <=  limit] is monotone in t; find the
        // largest t for which it is false, the cut is one above it.
        uint32_t t = 0;
        bool any_false = false;
        for (int bit = 31; bit >= 0; --bit) {
            const uint32_t cand = t | (1u << bit);
            float mass = 0.f;
            for (int i = tid; i < vocab; i += SAMPLE_THREADS) {
                const float x = row[i] / T;
                const uint32_t key = ordered_key(x);
                if (key >= cut && key > cand) mass += expf(x - mx);
            }
            mass = block_sum(mass, fscratch);
            if (mass > limit) { t = cand; any_false = true; }
        }
        if (!any_false) {  // is f(0) false?
            float mass = 0.f;
            for (int i = tid; i < vocab; i += SAMPLE_THREADS) {
                const float x = row[i] / T;
                const uint32_t key = ordered_key(x);
                if (key >= cut && key > 0u) mass += expf(x - mx);
            }
            any_false = block_sum(mass, fscratch) > limit;
        }
        const uint32_t p_cut = any_false ? t + 1u : 0u;
        cut = max(cut, p_cut);
    }

    // Inverse of the cumulative distribution, in index order, over contiguous chunks.
    const int chunk = (vocab + SAMPLE_THREADS - 1) / SAMPLE_THREADS;
    const int i0 = min(tid * chunk, vocab), i1 = min(i0 + chunk, vocab);
    float s = 0.f;
    for (int i = i0; i < i1; ++i) {
        const float x = row[i] / T;
        if (ordered_key(x) >= cut) s += expf(x - mx);
    }
    chunk_sum[tid] = s;
    __syncthreads();
    if (tid == 0) {
        float total = 0.f;
        for (int c = 0; c < SAMPLE_THREADS; ++c) total += chunk_sum[c];
        const float target = uniform[r] * total;
        float before = 0.f;
        int c = 0;
        for (; c < SAMPLE_THREADS - 1; ++c) {
            if (before + chunk_sum[c] > target) break;
            before += chunk_sum[c];
        }
        chosen_chunk = c;
        chosen_before = before;
        // target is kept in fscratch for the walking thread
        fscratch[0] = target;
    }
    __syncthreads();
    if (tid == chosen_chunk) {
        const float target = fscratch[0];
        float cum = chosen_before;
        int pick = -1, last_kept = -1;
        for (int i = i0; i < i1; ++i) {
            const float x = row[i] / T;
            if (ordered_key(x) >= cut) {
                cum += expf(x - mx);
                last_kept = i;
                if (cum > target) { pick = i; break; }
            }
        }
        if (pick < 0) pick = last_kept;
        if (pick < 0) {  // rounding left nothing in this chunk: the last kept token overall
            for (int i = vocab - 1; i >= 0; --i)
                if (ordered_key(row[i] / T) >= cut) { pick = i; break; }
        }
        out[r] = pick < 0 ? 0 : pick;
    }
}

// ---------------------------------------------------------------------------------------------------
// Argmax of every row (steps whose requests are all greedy), spread over the chip: ARGMAX_CHUNKS workgroups a
// row each reduce a contiguous piece of it, with 16-byte loads where the row length allows, to one (value,
// index) pair; a second kernel reduces a row's pairs.  Ties go to the lowest index, as in sample_kernel.
// ---------------------------------------------------------------------------------------------------
#define ARGMAX_CHUNKS 64
#define ARGMAX_THREADS 256

__device__ __forceinline__ void take_better(float& bv, int& bi, float v, int i) {
    if (v > bv || (v == bv && i < bi)) { bv = v; bi = i; }
}

__device__ __forceinline__ void block_argmax(float& bv, int& bi, float* vals, int* idxs) {
#pragma unroll
    for (int off = SIA_WAVE / 2; off > 0; off >>= 1) {
        const float ov = __shfl_xor(bv, off, SIA_WAVE);
        const int oi = __shfl_xor(bi, off, SIA_WAVE);
        take_better(bv, bi, ov, oi);
    }
    const int wave = threadIdx.x / SIA_WAVE, n_waves = blockDim.x / SIA_WAVE;
    if (threadIdx.x % SIA_WAVE == 0) { vals[wave] = bv; idxs[wave] = bi; }
    __syncthreads();
    if (threadIdx.x == 0)
        for (int w = 1; w < n_waves; ++w) take_better(bv, bi, vals[w], idxs[w]);
}

__global__ __launch_bounds__(ARGMAX_THREADS) void argmax_chunks_kernel(const float* __restrict__ logits, int vocab,
                                                                       float* __restrict__ ws_val,
                                                                       int* __restrict__ ws_idx) {
    __shared__ float vals[ARGMAX_THREADS / SIA_WAVE];
    __shared__ int idxs[ARGMAX_THREADS / SIA_WAVE];
    const int chunk = blockIdx.x, r = blockIdx.y;
    const float* row = logits + (size_t)r * vocab;
    float bv = -INFINITY;
    int bi = vocab;
    if (vocab % 4 == 0) {
        const int quads = vocab / 4, per = (quads + ARGMAX_CHUNKS - 1) / ARGMAX_CHUNKS;
        const int q_end = min(quads, (chunk + 1) * per);
        for (int q = chunk * per + threadIdx.x; q < q_end; q += ARGMAX_THREADS) {
            const float4 v = reinterpret_cast<const float4*>(row)[q];
            take_better(bv, bi, v.x, 4 * q);
            take_better(bv, bi, v.y, 4 * q + 1);
            take_better(bv, bi, v.z, 4 * q + 2);
            take_better(bv, bi, v.w, 4 * q + 3);
        }
    } else {
        const int per = (vocab + ARGMAX_CHUNKS - 1) / ARGMAX_CHUNKS;
        const int i_end = min(vocab, (chunk + 1) * per);
        for (int i = chunk * per + threadIdx.x; i < i_end; i += ARGMAX_THREADS) take_better(bv, bi, row[i], i);
    }
    block_argmax(bv, bi, vals, idxs);
    if (threadIdx.x == 0) {
        ws_val[r * ARGMAX_CHUNKS + chunk] = bv;
        ws_idx[r * ARGMAX_CHUNKS + chunk] = bi;
    }
}

__global__ __launch_bounds__(SIA_WAVE) void argmax_finish_kernel(const float* __restrict__ ws_val,
                                                                 const int* __restrict__ ws_idx,
                                                                 int* __restrict__ out, int vocab) {
    __shared__ float vals[1];
    __shared__ int idxs[1];
    const int r = blockIdx.x;
    float bv = -INFINITY;
    int bi = vocab;
    for (int c = threadIdx.x; c < ARGMAX_CHUNKS; c += SIA_WAVE)
        take_better(bv, bi, ws_val[r * ARGMAX_CHUNKS + c], ws_idx[r * ARGMAX_CHUNKS + c]);
    block_argmax(bv, bi, vals, idxs);
    if (threadIdx.x == 0) out[r] = bi < vocab ? bi : 0;
}

SIA_EXPORT int sia_argmax_workspace_per_row() { return ARGMAX_CHUNKS; }

// ws_val and ws_idx hold rows * sia_argmax_workspace_per_row() elements each.
SIA_EXPORT int sia_argmax(const float* logits, int* out, float* ws_val, int* ws_idx, int rows, int vocab,
                          hipStream_t stream) {
    if (rows <= 0) return 0;
    if (vocab <= 0 || rows > 65535) return SIA_BAD_ARGUMENT;
    hipLaunchKernelGGL(argmax_chunks_kernel, dim3(ARGMAX_CHUNKS, rows), dim3(ARGMAX_THREADS), 0, stream, logits,
                       vocab, ws_val, ws_idx);
    hipLaunchKernelGGL(argmax_finish_kernel, dim3(rows), dim3(SIA_WAVE), 0, stream, ws_val, ws_idx, out, vocab);
    return SIA_LAUNCH_CHECK();
}

SIA_EXPORT int sia_sample(const float* logits, const float* temperature, const int* top_k, const float* top_p,
                          const float* uniform, int* out, int rows, int vocab, hipStream_t stream) {
    if (rows <= 0) return 0;
    if (vocab <= 0) return SIA_BAD_ARGUMENT;
    hipLaunchKernelGGL(sample_kernel, dim3(rows), dim3(SAMPLE_THREADS), 0, stream, logits, temperature, top_k,
                       top_p, uniform, out, vocab);
    return SIA_LAUNCH_CHECK();
}
