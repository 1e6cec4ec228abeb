// Embedding gather, residual add + RMS norm, SwiGLU activation.
//
// These are bound by memory traffic or by launch latency.  The residual stream is float
// in both modes; rows are handled by one workgroup each, with vector accesses where the
// row length allows.
#include "common.h"

// ---------------------------------------------------------------------------------------
// Embedding: out[n, :] = float(table[ids[n], :])          (reference: ops/embedding.py:57-60)
// ---------------------------------------------------------------------------------------
template <typename T>
__global__ void embed_kernel(const int* __restrict__ ids, const T* __restrict__ table,
                             float* __restrict__ out, int hidden) {
    const int n = blockIdx.x;
    const T* src = table + (size_t)ids[n] * hidden;
    float* dst = out + (size_t)n * hidden;
    for (int i = threadIdx.x; i < hidden; i += blockDim.x) dst[i] = to_float(src[i]);
}

SIA_EXPORT int sia_embed(const int* ids, const void* table, float* out, int n_tokens, int hidden,
                         int table_dtype, hipStream_t stream) {
    if (n_tokens <= 0) return 0;
    dim3 grid(n_tokens), block(256);
    if (table_dtype == SIA_F32)
        hipLaunchKernelGGL(embed_kernel<float>, grid, block, 0, stream, ids, (const float*)table, out, hidden);
    else if (table_dtype == SIA_BF16)
        hipLaunchKernelGGL(embed_kernel<bf16_t>, grid, block, 0, stream, ids, (const bf16_t*)table, out, hidden);
    else
        return SIA_BAD_ARGUMENT;
    return SIA_LAUNCH_CHECK();
}

// ---------------------------------------------------------------------------------------
// Residual add + RMS norm  (reference: ops/rmsnorm.py:41-46, kernels/rmsnorm_kernel.py:105-113)
//
//   x = residual[row] + delta[row]            (float; delta may be absent)
//   y = x * rsqrt(mean(x^2) + eps) * w        (float, one rounding to the output type)
//
// rows == nullptr: every row r of the batch; x is written back into residual[r].
// rows != nullptr: out[i] comes from row rows[i]; residual is not written.
// The sum of squares is reduced in a fixed order that depends on the row length only.
// ---------------------------------------------------------------------------------------
template <typename T>
__global__ void add_rmsnorm_kernel(float* __restrict__ residual, const T* __restrict__ delta,
                                   const float* __restrict__ weight, T* __restrict__ out,
                                   const int* __restrict__ rows, int hidden, float eps) {
    __shared__ float scratch[16];
    const int i_out = blockIdx.x;
    const int row = rows ? rows[i_out] : i_out;
    float* res = residual + (size_t)row * hidden;
    const T* del = delta ? delta + (size_t)row * hidden : nullptr;
    T* dst = out + (size_t)i_out * hidden;

    float ss = 0.f;
    for (int i = threadIdx.x; i < hidden; i += blockDim.x) {
        float x = res[i];
        if (del) x += to_float(del[i]);
        if (!rows && del) res[i] = x;
        ss += x * x;
    }
    ss = block_sum(ss, scratch);
    const float inv = rsqrtf(ss / (float)hidden + eps);
    for (int i = threadIdx.x; i < hidden; i += blockDim.x) {
        float x = res[i];
        if (rows && del) x += to_float(del[i]);
        dst[i] = from_float<T>(x * inv * weight[i]);
    }
}

// The same for rows that one workgroup holds in registers (hidden % 8 == 0, hidden <= 8 * 1024): each
// thread takes 8 consecutive elements with 16- and 32-byte accesses, every input is read once and all
// loads (the gain's included) are issued before the first is used.
template <typename T>
__global__ void add_rmsnorm_row_kernel(float* __restrict__ residual, const T* __restrict__ delta,
                                       const float* __restrict__ weight, T* __restrict__ out,
                                       const int* __restrict__ rows, int hidden, float eps) {
    __shared__ float scratch[16];
    const int i_out = blockIdx.x;
    const int row = rows ? rows[i_out] : i_out;
    const int i0 = threadIdx.x * 8;
    const bool live = i0 < hidden;
    float x[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f}, w[8], d[8];
    if (live) {
        Vec8<float> vr, vw;
        Vec8<T> vd;
        vr.load(residual + (size_t)row * hidden + i0);
        vw.load(weight + i0);
        if (delta) vd.load(delta + (size_t)row * hidden + i0);
        vr.get(x);
        vw.get(w);
        if (delta) {
            vd.get(d);
#pragma unroll
            for (int i = 0; i < 8; ++i) x[i] += d[i];
            if (!rows) {
                vr.set(x);
                vr.store(residual + (size_t)row * hidden + i0);
            }
        }
    }
    float ss = 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i) ss += x[i] * x[i];
    ss = block_sum(ss, scratch);
    if (live) {
        const float inv = rsqrtf(ss / (float)hidden + eps);
#pragma unroll
        for (int i = 0; i < 8; ++i) x[i] = x[i] * inv * w[i];
        Vec8<T> vo;
        vo.set(x);
        vo.store(out + (size_t)i_out * hidden + i0);
    }
}

SIA_EXPORT int sia_add_rmsnorm(float* residual, const void* delta, const float* weight, void* out,
                               const int* rows, int n_out, int hidden, float eps, int dtype,
                               hipStream_t stream) {
    if (n_out <= 0) return 0;
    if (dtype != SIA_F32 && dtype != SIA_BF16) return SIA_BAD_ARGUMENT;
    dim3 grid(n_out);
    if (hidden % 8 == 0 && hidden <= 8 * 1024) {
        dim3 block(((hidden / 8 + SIA_WAVE - 1) / SIA_WAVE) * SIA_WAVE);
        if (dtype == SIA_F32)
            hipLaunchKernelGGL(add_rmsnorm_row_kernel<float>, grid, block, 0, stream, residual, (const float*)delta,
                               weight, (float*)out, rows, hidden, eps);
        else
            hipLaunchKernelGGL(add_rmsnorm_row_kernel<bf16_t>, grid, block, 0, stream, residual,
                               (const bf16_t*)delta, weight, (bf16_t*)out, rows, hidden, eps);
        return SIA_LAUNCH_CHECK();
    }
    dim3 block(hidden >= 2048 ? 512 : 256);
    if (dtype == SIA_F32)
        hipLaunchKernelGGL(add_rmsnorm_kernel<float>, grid, block, 0, stream, residual, (const float*)delta,
                           weight, (float*)out, rows, hidden, eps);
    else
        hipLaunchKernelGGL(add_rmsnorm_kernel<bf16_t>, grid, block, 0, stream, residual, (const bf16_t*)delta,
                           weight, (bf16_t*)out, rows, hidden, eps);
    return SIA_LAUNCH_CHECK();
}

// ---------------------------------------------------------------------------------------
// SwiGLU: out[n, i] = silu(gu[n, i]) * gu[n, I + i], silu(g) = g / (1 + exp(-g)), in float
// (reference: ops/mlp.py:117-128, kernels/swiglu_kernel.py:142-150)
// ---------------------------------------------------------------------------------------
template <typename T>
__global__ void swiglu_kernel(const T* __restrict__ gu, T* __restrict__ out, int inter) {
    const int n = blockIdx.y;
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= inter) return;
    const T* row = gu + (size_t)n * 2 * inter;
    const float g = to_float(row[i]);
    const float u = to_float(row[inter + i]);
    out[(size_t)n * inter + i] = from_float<T>(g / (1.f + expf(-g)) * u);
}

// Eight elements a thread, 16- or 32-byte accesses (inter % 8 == 0).
template <typename T>
__global__ void swiglu_vec_kernel(const T* __restrict__ gu, T* __restrict__ out, int inter) {
    const int n = blockIdx.y;
    const int i = (blockIdx.x * blockDim.x + threadIdx.x) * 8;
    if (i >= inter) return;
    const T* row = gu + (size_t)n * 2 * inter;
    Vec8<T> vg, vu;
    vg.load(row + i);
    vu.load(row + inter + i);
    float g[8], u[8];
    vg.get(g);
    vu.get(u);
#pragma unroll
    for (int j = 0; j < 8; ++j) g[j] = g[j] / (1.f + expf(-g[j])) * u[j];
    vg.set(g);
    vg.store(out + (size_t)n * inter + i);
}

SIA_EXPORT int sia_swiglu(const void* gu, void* out, int n_tokens, int inter, int dtype, hipStream_t stream) {
    if (n_tokens <= 0) return 0;
    if (n_tokens > 65535) return SIA_BAD_ARGUMENT;
    if (dtype != SIA_F32 && dtype != SIA_BF16) return SIA_BAD_ARGUMENT;
    if (inter % 8 == 0) {
        dim3 block(256), grid((inter / 8 + 255) / 256, n_tokens);
        if (dtype == SIA_F32)
            hipLaunchKernelGGL(swiglu_vec_kernel<float>, grid, block, 0, stream, (const float*)gu, (float*)out, inter);
        else
            hipLaunchKernelGGL(swiglu_vec_kernel<bf16_t>, grid, block, 0, stream, (const bf16_t*)gu, (bf16_t*)out, inter);
        return SIA_LAUNCH_CHECK();
    }
    dim3 block(256), grid((inter + 255) / 256, n_tokens);
    if (dtype == SIA_F32)
        hipLaunchKernelGGL(swiglu_kernel<float>, grid, block, 0, stream, (const float*)gu, (float*)out, inter);
    else
        hipLaunchKernelGGL(swiglu_kernel<bf16_t>, grid, block, 0, stream, (const bf16_t*)gu, (bf16_t*)out, inter);
    return SIA_LAUNCH_CHECK();
}

// ---------------------------------------------------------------------------------------
// Casts between the two element types (used where a float32-stored matrix meets bfloat16
// activations).
// ---------------------------------------------------------------------------------------
__global__ void cast_bf16_to_f32_kernel(const bf16_t* __restrict__ in, float* __restrict__ out, size_t n) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) out[i] = bf16_to_float(in[i]);
}
__global__ void cast_f32_to_bf16_kernel(const float* __restrict__ in, bf16_t* __restrict__ out, size_t n) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) out[i] = float_to_bf16(in[i]);
}

SIA_EXPORT int sia_cast(const void* in, void* out, long long n, int in_dtype, hipStream_t stream) {
    if (n <= 0) return 0;
    dim3 block(256), grid((unsigned)((n + 255) / 256));
    if (in_dtype == SIA_BF16)
        hipLaunchKernelGGL(cast_bf16_to_f32_kernel, grid, block, 0, stream, (const bf16_t*)in, (float*)out, (size_t)n);
    else if (in_dtype == SIA_F32)
        hipLaunchKernelGGL(cast_f32_to_bf16_kernel, grid, block, 0, stream, (const float*)in, (bf16_t*)out, (size_t)n);
    else
        return SIA_BAD_ARGUMENT;
    return SIA_LAUNCH_CHECK();
}

// out[m][k] = scaled[m][k] * rsqrt(sum_p partials[p][m] / width + eps): finishes the norm that a product with a
// residual epilogue left unfinished, for a consumer that cannot scale its own rows.
__global__ __launch_bounds__(256) void scale_rows_kernel(const bf16_t* __restrict__ scaled,
                                                         const float* __restrict__ partials, bf16_t* __restrict__ out,
                                                         int width, int n_partials, float eps) {
    __shared__ float sums[256];
    const int m = blockIdx.x;
    float ss = 0.f;
    for (int p = threadIdx.x; p < n_partials; p += 256) ss += partials[p * 16 + m];
    sums[threadIdx.x] = ss;
    __syncthreads();
    for (int half = 128; half > 0; half >>= 1) {
        if ((int)threadIdx.x < half) sums[threadIdx.x] += sums[threadIdx.x + half];
        __syncthreads();
    }
    const float rs = rsqrtf(sums[0] / (float)width + eps);
    for (int k = threadIdx.x; k < width; k += 256)
        out[(size_t)m * width + k] = float_to_bf16(bf16_to_float(scaled[(size_t)m * width + k]) * rs);
}

SIA_EXPORT int sia_scale_rows(const void* scaled, const float* partials, void* out, int rows, int width,
                              int n_partials, float eps, hipStream_t stream) {
    if (rows <= 0) return 0;
    if (rows > 16 || width <= 0 || n_partials <= 0) return SIA_BAD_ARGUMENT;
    hipLaunchKernelGGL(scale_rows_kernel, dim3(rows), dim3(256), 0, stream, (const bf16_t*)scaled, partials,
                       (bf16_t*)out, width, n_partials, eps);
    return SIA_LAUNCH_CHECK();
}

// dst[dst_rows[i]] = src[src_rows[i]]: token ids that a sampler has left on the device become the input of the
// next step without a trip through the host.
__global__ __launch_bounds__(256) void place_tokens_kernel(int* __restrict__ dst, const int* __restrict__ dst_rows,
                                                           const int* __restrict__ src,
                                                           const int* __restrict__ src_rows, int n) {
    const int i = blockIdx.x * 256 + threadIdx.x;
    if (i < n) dst[dst_rows[i]] = src[src_rows[i]];
}

SIA_EXPORT int sia_place_tokens(int* dst, const int* dst_rows, const int* src, const int* src_rows, int n,
                                hipStream_t stream) {
    if (n <= 0) return 0;
    if (!dst || !dst_rows || !src || !src_rows) return SIA_BAD_ARGUMENT;
    hipLaunchKernelGGL(place_tokens_kernel, dim3((n + 255) / 256), dim3(256), 0, stream, dst, dst_rows, src, src_rows,
                       n);
    return SIA_LAUNCH_CHECK();
}
