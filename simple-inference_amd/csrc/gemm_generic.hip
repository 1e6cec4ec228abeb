// Y[M, N] = X[M, K] * W[N, K]^T with float accumulation: the plain matrix product.
//
// This is the product of the 32-bit path (float operands, float fused multiply-adds, no
// reduced-precision matrix mode) and the fallback for shapes the fast bfloat16 kernels
// refuse.  Each output element is accumulated over k = 0 .. K-1 in that order, whatever
// M is, so a row's result does not depend on the other rows of a batch.
//
// 64 x 64 output tile per workgroup of 256 threads, 4 x 4 outputs per thread, K in steps
// of 16 staged through LDS.  Any M, N, K (edges are guarded).
#include "common.h"

#define GT 64   // tile edge
#define GK 16   // K step

template <typename TIn, typename TOut>
__global__ __launch_bounds__(256) void gemm_generic_kernel(const TIn* __restrict__ X, const TIn* __restrict__ W,
                                                           TOut* __restrict__ Y, int M, int N, int K) {
    __shared__ float xs[GK][GT + 4];
    __shared__ float ws[GK][GT + 4];
    const int tid = threadIdx.x;
    const int m0 = blockIdx.y * GT, n0 = blockIdx.x * GT;
    const int tm = (tid / 16) * 4, tn = (tid % 16) * 4;
    const int lr = tid / 4, lk = (tid % 4) * 4;  // this thread stages row lr, k offsets lk .. lk+3

    float acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = 0.f;

    for (int k0 = 0; k0 < K; k0 += GK) {
#pragma unroll
        for (int kk = 0; kk < 4; ++kk) {
            const int k = k0 + lk + kk;
            const int xm = m0 + lr, wn = n0 + lr;
            xs[lk + kk][lr] = (xm < M && k < K) ? to_float(X[(size_t)xm * K + k]) : 0.f;
            ws[lk + kk][lr] = (wn < N && k < K) ? to_float(W[(size_t)wn * K + k]) : 0.f;
        }
        __syncthreads();
#pragma unroll
        for (int kk = 0; kk < GK; ++kk) {
            float a[4], b[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) a[i] = xs[kk][tm + i];
#pragma unroll
            for (int j = 0; j < 4; ++j) b[j] = ws[kk][tn + j];
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], b[j], acc[i][j]);
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int m = m0 + tm + i;
        if (m >= M) continue;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int n = n0 + tn + j;
            if (n < N) Y[(size_t)m * N + n] = from_float<TOut>(acc[i][j]);
        }
    }
}

// in_dtype: element type of X and W.  out_float: 1 -> Y is float, 0 -> Y has in_dtype.
SIA_EXPORT int sia_gemm_generic(const void* X, const void* W, void* Y, int M, int N, int K, int in_dtype,
                                int out_float, hipStream_t stream) {
    if (M <= 0 || N <= 0) return 0;
    if (K <= 0) return SIA_BAD_ARGUMENT;
    dim3 grid((N + GT - 1) / GT, (M + GT - 1) / GT), block(256);
    if (grid.y > 65535) return SIA_BAD_ARGUMENT;
    if (in_dtype == SIA_F32)
        hipLaunchKernelGGL((gemm_generic_kernel<float, float>), grid, block, 0, stream, (const float*)X,
                           (const float*)W, (float*)Y, M, N, K);
    else if (in_dtype == SIA_BF16 && out_float)
        hipLaunchKernelGGL((gemm_generic_kernel<bf16_t, float>), grid, block, 0, stream, (const bf16_t*)X,
                           (const bf16_t*)W, (float*)Y, M, N, K);
    else if (in_dtype == SIA_BF16)
        hipLaunchKernelGGL((gemm_generic_kernel<bf16_t, bf16_t>), grid, block, 0, stream, (const bf16_t*)X,
                           (const bf16_t*)W, (bf16_t*)Y, M, N, K);
    else
        return SIA_BAD_ARGUMENT;
    return SIA_LAUNCH_CHECK();
}
