// Y[M, N] = X[M, K] * W[N, K]^T in bfloat16 with float accumulation, for few rows (M <= 16):
// the matrix products of a decode step, where every weight is read once and the time is the time
// to stream W from HBM.
//
// One workgroup of 8 waves per 16*RB rows of W.  The waves split K between them in interleaved
// chunks, so that the workgroup walks its rows front to back; their partial sums are added through
// LDS in wave order.  A wave's step covers 64 k of RB blocks of 16 rows with 2*RB MFMAs 16x16x32:
//   A = W[n0 + 16 rb + r][k0 + 16g .. + 15]   two 16-byte loads a lane, 128 contiguous bytes per row
//   B = X[r][same k]                           (rows r >= M are zero), loaded once for all RB blocks
// (an MFMA's k index only has to mean the same element in A and B, so lane group g may take the 16
// consecutive k that start at 16g and feed them to two MFMAs.)  X is small and comes from the
// caches; a large N takes RB = 4, so that X is fetched once per 64 rows of W.
//
// The result element (m, n) is summed over k in an order that depends on N and K only: a row's
// result does not depend on M or on the other rows.
#include "common.h"

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float floatx4;

constexpr int SK_WAVES = 8;
constexpr int SK_STEP = 64;  // k per step of one wave

__device__ __forceinline__ bf16x8 ld8(const bf16_t* p) {
    return __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(p));
}

enum SkinnyEpilogue { EPI_STORE = 0, EPI_SWIGLU = 1 };

// RB: blocks of 16 rows of W per workgroup, rb_stride rows apart; UNROLL: steps whose loads are in flight
// together.
//   EPI_STORE:   Y[m][n0 + 16 rb + n]  (TOut)
//   EPI_SWIGLU:  RB = 2, row block 0 is the gate and row block 1 (rb_stride = intermediate size) the up
//                projection: Y[m][n0 + n] = silu(gate) * up, in float, rounded once
template <typename TOut, int RB, int UNROLL, int EPI>
__global__ __launch_bounds__(SK_WAVES* SIA_WAVE) void gemm_skinny_kernel(const bf16_t* __restrict__ X,
                                                                        const bf16_t* __restrict__ W,
                                                                        TOut* __restrict__ Y, int M, int N, int K,
                                                                        int rb_stride) {
    __shared__ float part[SK_WAVES][RB][16][17];
    constexpr int CHUNK = SK_STEP * UNROLL;  // one wave's share of a round
    const int wave = threadIdx.x / SIA_WAVE, lane = threadIdx.x & 63, r = lane & 15, g = lane >> 4;
    const int n0 = blockIdx.x * 16 * (EPI == EPI_SWIGLU ? 1 : RB);
    const bf16_t* w_row = W + (size_t)(n0 + r) * K + g * 16;
    const bf16_t* x_row = X + (size_t)min(r, M - 1) * K + g * 16;
    const bool x_live = r < M;
    const bf16x8 zero = __builtin_bit_cast(bf16x8, make_uint4(0u, 0u, 0u, 0u));

    floatx4 acc[RB];
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) acc[rb] = floatx4{0.f, 0.f, 0.f, 0.f};
    for (int k0 = wave * CHUNK; k0 < K; k0 += SK_WAVES * CHUNK) {
        bf16x8 a[UNROLL][RB][2], b[UNROLL][2];
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) {
            const int k = k0 + u * SK_STEP;
            const bool in = k < K;  // K is a multiple of 64: a step is inside or outside as a whole
#pragma unroll
            for (int rb = 0; rb < RB; ++rb) {
                a[u][rb][0] = in ? ld8(w_row + (size_t)rb * rb_stride * K + k) : zero;
                a[u][rb][1] = in ? ld8(w_row + (size_t)rb * rb_stride * K + k + 8) : zero;
            }
            b[u][0] = (in && x_live) ? ld8(x_row + k) : zero;
            b[u][1] = (in && x_live) ? ld8(x_row + k + 8) : zero;
        }
#pragma unroll
        for (int u = 0; u < UNROLL; ++u)
#pragma unroll
            for (int rb = 0; rb < RB; ++rb) {
                acc[rb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[u][rb][0], b[u][0], acc[rb], 0, 0, 0);
                acc[rb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[u][rb][1], b[u][1], acc[rb], 0, 0, 0);
            }
    }
    // acc[rb][i] = partial Y[m = r][n = n0 + rb_stride rb + 4g + i]
#pragma unroll
    for (int rb = 0; rb < RB; ++rb)
#pragma unroll
        for (int i = 0; i < 4; ++i) part[wave][rb][r][g * 4 + i] = acc[rb][i];
    __syncthreads();
    if (EPI == EPI_SWIGLU) {
        const int m = threadIdx.x / 16, n = threadIdx.x % 16;
        if (threadIdx.x < 256 && m < M) {
            float gate = 0.f, up = 0.f;
#pragma unroll
            for (int w = 0; w < SK_WAVES; ++w) {
                gate += part[w][0][m][n];
                up += part[w][RB - 1][m][n];
            }
            Y[(size_t)m * N + n0 + n] = from_float<TOut>(gate / (1.f + expf(-gate)) * up);
        }
        return;
    }
    for (int idx = threadIdx.x; idx < RB * 256; idx += SK_WAVES * SIA_WAVE) {
        const int rb = idx / 256, m = (idx / 16) % 16, n = idx % 16;
        if (m < M) {
            float s = 0.f;
#pragma unroll
            for (int w = 0; w < SK_WAVES; ++w) s += part[w][rb][m][n];
            Y[(size_t)m * N + n0 + rb * rb_stride + n] = from_float<TOut>(s);
        }
    }
}

SIA_EXPORT int sia_gemm_skinny_max_rows() { return 16; }

template <typename TOut>
static void launch_skinny(const bf16_t* X, const bf16_t* W, TOut* Y, int M, int N, int K, hipStream_t stream) {
    dim3 block(SK_WAVES * SIA_WAVE);
    // 64 rows a workgroup when that still gives every compute unit a workgroup, else 16.
    if (N % 64 == 0 && N / 64 >= 256)
        hipLaunchKernelGGL((gemm_skinny_kernel<TOut, 4, 2, EPI_STORE>), dim3(N / 64), block, 0, stream, X, W, Y, M, N,
                           K, 16);
    else
        hipLaunchKernelGGL((gemm_skinny_kernel<TOut, 1, 4, EPI_STORE>), dim3(N / 16), block, 0, stream, X, W, Y, M, N,
                           K, 16);
}

// out_float: 1 -> Y is float, 0 -> bfloat16.  Needs M <= 16, N % 16 == 0, K % 64 == 0.
SIA_EXPORT int sia_gemm_skinny(const void* X, const void* W, void* Y, int M, int N, int K, int out_float,
                               hipStream_t stream) {
    if (M <= 0 || N <= 0) return 0;
    if (M > 16 || N % 16 || K % 64 || K <= 0) return SIA_BAD_ARGUMENT;
    if (out_float)
        launch_skinny<float>((const bf16_t*)X, (const bf16_t*)W, (float*)Y, M, N, K, stream);
    else
        launch_skinny<bf16_t>((const bf16_t*)X, (const bf16_t*)W, (bf16_t*)Y, M, N, K, stream);
    return SIA_LAUNCH_CHECK();
}

// Y[M, I] = silu(X Wg^T) * (X Wu^T) for W = [Wg; Wu] of 2 I rows.  Needs M <= 16, I % 16 == 0, K % 64 == 0.
SIA_EXPORT int sia_gemm_skinny_swiglu(const void* X, const void* W, void* Y, int M, int inter, int K,
                                      hipStream_t stream) {
    if (M <= 0 || inter <= 0) return 0;
    if (M > 16 || inter % 16 || K % 64 || K <= 0) return SIA_BAD_ARGUMENT;
    hipLaunchKernelGGL((gemm_skinny_kernel<bf16_t, 2, 2, EPI_SWIGLU>), dim3(inter / 16), dim3(SK_WAVES * SIA_WAVE), 0,
                       stream, (const bf16_t*)X, (const bf16_t*)W, (bf16_t*)Y, M, inter, K, inter);
    return SIA_LAUNCH_CHECK();
}
