// Y[M, N] = X[M, K] * W[N, K]^T in bfloat16 with float accumulation, for few rows (M <= 16):
// the matrix products of a decode step, where every weight is read once and the time is the time
// to stream W from HBM.
//
// One workgroup of 8 or 16 waves per 16*RB rows of W.  The waves split K between them in interleaved
// chunks, so that the workgroup walks its rows front to back; their partial sums are added through
// LDS in wave order.  A wave's step covers 64 k of RB blocks of 16 rows with 2*RB MFMAs 16x16x32:
//   A = W[n0 + 16 rb + r][k0 + 16g .. + 15]   two 16-byte loads a lane, 128 contiguous bytes per row
//   B = X[r][same k]                           (rows r >= M are zero), loaded once for all RB blocks
// (an MFMA's k index only has to mean the same element in A and B, so lane group g may take the 16
// consecutive k that start at 16g and feed them to two MFMAs.)  X is small and comes from the
// caches, once per workgroup: a workgroup takes as many row blocks (4, 2 or 1) as still leave some 160
// workgroups, which is what measurements of the decode shapes favour.
//
// The result element (m, n) is summed over k in an order that depends on N and K only: a row's
// result does not depend on M or on the other rows.
#include "common.h"

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float floatx4;

constexpr int SK_STEP = 64;  // k per step of one wave

__device__ __forceinline__ bf16x8 ld8(const bf16_t* p) {
    return __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(p));
}

enum SkinnyEpilogue { EPI_STORE = 0, EPI_SWIGLU = 1, EPI_ROPE = 2 };

// What the q/k/v product needs to rotate its result and to put keys and values into the cache pages.
struct RopeOut {
    const float* cos_table;      // [positions][head_dim / 2]
    const float* sin_table;
    const int* positions;        // [M]
    const int* seq_of_token;     // [M]
    const int* block_table;      // [sequences][table_width]
    bf16_t* k_pages;             // [page][kv_head][offset][dim]
    bf16_t* v_pages;             // [page][kv_head][dim][offset]
    int table_width, n_heads, n_kv, head_dim, page_size;
};

// RB: blocks of 16 rows of W per workgroup; WAVES: waves that split K; UNROLL: steps whose loads are in flight
// together.
//   EPI_STORE:   row block rb holds rows n0 + 16 rb ..: Y[m][n0 + 16 rb + n]  (TOut)
//   EPI_SWIGLU:  W = [gate; up] of N rows each; the first RB / 2 row blocks are gate rows n0 + 16 j .., the others
//                the up rows of the same columns: Y[m][n0 + 16 j + n] = silu(gate) * up, in float, rounded once
//   EPI_ROPE:    RB = 2, W = [q heads | k heads | v heads] of head_dim rows each; a workgroup owns 16 columns of
//                the first half of a head and the 16 that the rotation pairs them with (head_dim / 2 further).
//                q and k are rotated in float on the float sums (one rounding; the rotation kernel rotates the
//                rounded product, so the two paths differ by a rounding); q goes to Y, k and v into the pages.
template <typename TOut, int RB, int WAVES, int UNROLL, int EPI>
__global__ __launch_bounds__(WAVES* SIA_WAVE) void gemm_skinny_kernel(const bf16_t* __restrict__ X,
                                                                     const bf16_t* __restrict__ W,
                                                                     TOut* __restrict__ Y, int M, int N, int K,
                                                                     RopeOut rope) {
    __shared__ float part[WAVES][RB][16][17];
    constexpr int CHUNK = SK_STEP * UNROLL;  // one wave's share of a round
    constexpr int OUT_BLOCKS = EPI == EPI_SWIGLU ? RB / 2 : RB;  // 16-column blocks of Y per workgroup
    const int wave = threadIdx.x / SIA_WAVE, lane = threadIdx.x & 63, r = lane & 15, g = lane >> 4;
    const int rope_half = EPI == EPI_ROPE ? rope.head_dim / 2 : 0;
    const int rope_head = EPI == EPI_ROPE ? blockIdx.x / (rope_half / 16) : 0;       // which head of q, k, v
    const int rope_j0 = EPI == EPI_ROPE ? (blockIdx.x % (rope_half / 16)) * 16 : 0;  // first column within the half
    const int n0 = EPI == EPI_ROPE ? rope_head * rope.head_dim + rope_j0 : blockIdx.x * 16 * OUT_BLOCKS;
    const bf16_t* x_row = X + (size_t)min(r, M - 1) * K + g * 16;
    const bool x_live = r < M;
    const bf16x8 zero = __builtin_bit_cast(bf16x8, make_uint4(0u, 0u, 0u, 0u));
    const bf16_t* w_row[RB];
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) {
        // rb / OUT_BLOCKS: 0 gate (or all), 1 up; EPI_ROPE: the second row block is the rotation's partner
        const int row = EPI == EPI_ROPE ? n0 + rb * rope_half + r
                                        : n0 + (rb % OUT_BLOCKS) * 16 + (rb / OUT_BLOCKS) * N + r;
        w_row[rb] = W + (size_t)row * K + g * 16;
    }

    floatx4 acc[RB];
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) acc[rb] = floatx4{0.f, 0.f, 0.f, 0.f};
    for (int k0 = wave * CHUNK; k0 < K; k0 += WAVES * CHUNK) {
        bf16x8 a[UNROLL][RB][2], b[UNROLL][2];
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) {
            const int k = k0 + u * SK_STEP;
            const bool in = k < K;  // K is a multiple of 64: a step is inside or outside as a whole
#pragma unroll
            for (int rb = 0; rb < RB; ++rb) {
                a[u][rb][0] = in ? ld8(w_row[rb] + k) : zero;
                a[u][rb][1] = in ? ld8(w_row[rb] + k + 8) : zero;
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
    // acc[rb][i] = partial of row m = r, column 4g + i of row block rb
#pragma unroll
    for (int rb = 0; rb < RB; ++rb)
#pragma unroll
        for (int i = 0; i < 4; ++i) part[wave][rb][r][g * 4 + i] = acc[rb][i];
    __syncthreads();
    if (EPI == EPI_ROPE) {
        const int m = threadIdx.x / 16, n = threadIdx.x % 16;
        if (threadIdx.x >= 256 || m >= M) return;
        float a = 0.f, b = 0.f;  // columns j and j + half of the head
#pragma unroll
        for (int w = 0; w < WAVES; ++w) {
            a += part[w][0][m][n];
            b += part[w][1][m][n];
        }
        const int j = rope_j0 + n, pos = rope.positions[m];
        const bool is_v = rope_head >= rope.n_heads + rope.n_kv;
        if (!is_v) {
            const float c = rope.cos_table[(size_t)pos * rope_half + j], sn = rope.sin_table[(size_t)pos * rope_half + j];
            const float ra = a * c - b * sn, rb_ = b * c + a * sn;
            a = ra;
            b = rb_;
        }
        if (rope_head < rope.n_heads) {
            TOut* y = Y + (size_t)m * N + rope_head * rope.head_dim;
            y[j] = from_float<TOut>(a);
            y[j + rope_half] = from_float<TOut>(b);
            return;
        }
        const int page = rope.block_table[(size_t)rope.seq_of_token[m] * rope.table_width + pos / rope.page_size];
        if (page < 0) return;  // never for a token the step owns
        const int off = pos % rope.page_size, D = rope.head_dim, ps = rope.page_size;
        if (!is_v) {
            const int hk = rope_head - rope.n_heads;
            bf16_t* dst = rope.k_pages + (((size_t)page * rope.n_kv + hk) * ps + off) * D;
            dst[j] = float_to_bf16(a);
            dst[j + rope_half] = float_to_bf16(b);
        } else {
            const int hk = rope_head - rope.n_heads - rope.n_kv;
            bf16_t* dst = rope.v_pages + ((size_t)page * rope.n_kv + hk) * D * ps + off;
            dst[(size_t)j * ps] = float_to_bf16(a);
            dst[(size_t)(j + rope_half) * ps] = float_to_bf16(b);
        }
        return;
    }
    for (int idx = threadIdx.x; idx < OUT_BLOCKS * 256; idx += WAVES * SIA_WAVE) {
        const int j = idx / 256, m = (idx / 16) % 16, n = idx % 16;
        if (m >= M) continue;
        if (EPI == EPI_SWIGLU) {
            float gate = 0.f, up = 0.f;
#pragma unroll
            for (int w = 0; w < WAVES; ++w) {
                gate += part[w][j][m][n];
                up += part[w][OUT_BLOCKS + j][m][n];
            }
            Y[(size_t)m * N + n0 + j * 16 + n] = from_float<TOut>(gate / (1.f + expf(-gate)) * up);
        } else {
            float s = 0.f;
#pragma unroll
            for (int w = 0; w < WAVES; ++w) s += part[w][j][m][n];
            Y[(size_t)m * N + n0 + j * 16 + n] = from_float<TOut>(s);
        }
    }
}

SIA_EXPORT int sia_gemm_skinny_max_rows() { return 16; }

// Shapes measured on an MI355X at 1 to 16 rows (K 2,048 to 14,336): a workgroup should own as many rows of W as
// still leave some 160 workgroups (X is fetched once per workgroup); two row blocks go with 16 waves.
template <typename TOut>
static void launch_skinny(const bf16_t* X, const bf16_t* W, TOut* Y, int M, int N, int K, hipStream_t stream) {
#define LAUNCH(RB, WAVES, UNROLL)                                                                                \
    hipLaunchKernelGGL((gemm_skinny_kernel<TOut, RB, WAVES, UNROLL, EPI_STORE>), dim3(N / (16 * RB)),              \
                       dim3(WAVES * SIA_WAVE), 0, stream, X, W, Y, M, N, K, RopeOut{})
    if (N % 64 == 0 && N / 64 >= 160)
        LAUNCH(4, 8, 2);
    else if (N % 32 == 0 && N / 32 >= 160 && K >= 1024)
        LAUNCH(2, 16, 2);
    else if (M <= 4)
        LAUNCH(1, 8, 4);
    else
        LAUNCH(1, 8, 2);
#undef LAUNCH
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
    if (inter % 32 == 0 && inter / 32 >= 160 && K >= 1024 && M > 4)
        hipLaunchKernelGGL((gemm_skinny_kernel<bf16_t, 4, 16, 2, EPI_SWIGLU>), dim3(inter / 32), dim3(16 * SIA_WAVE), 0,
                           stream, (const bf16_t*)X, (const bf16_t*)W, (bf16_t*)Y, M, inter, K, RopeOut{});
    else
        hipLaunchKernelGGL((gemm_skinny_kernel<bf16_t, 2, 8, 2, EPI_SWIGLU>), dim3(inter / 16), dim3(8 * SIA_WAVE), 0,
                           stream, (const bf16_t*)X, (const bf16_t*)W, (bf16_t*)Y, M, inter, K, RopeOut{});
    return SIA_LAUNCH_CHECK();
}

// The q/k/v product of single-token steps with the rotation and the cache write in its epilogue:
// W = [q heads | k heads | v heads], head_dim % 32 == 0, every dim of a head rotates (tables of head_dim / 2 floats
// a position).  Rotated q goes to Y[M][(n_heads + 2 n_kv) head_dim] (its k and v columns are not written); rotated
// k and v go to the pages at each token's position.  Needs M <= 16, K % 64 == 0.
SIA_EXPORT int sia_gemm_skinny_rope(const void* X, const void* W, void* Y, int M, int K, const float* cos_table,
                                    const float* sin_table, const int* positions, const int* seq_of_token,
                                    const int* block_table, int table_width, void* k_pages, void* v_pages,
                                    int n_heads, int n_kv, int head_dim, int page_size, hipStream_t stream) {
    if (M <= 0) return 0;
    if (M > 16 || K % 64 || K <= 0 || head_dim % 32 || head_dim <= 0 || n_heads <= 0 || n_kv <= 0 || page_size <= 0 ||
        table_width <= 0 || !cos_table || !sin_table || !positions || !seq_of_token || !block_table || !k_pages ||
        !v_pages)
        return SIA_BAD_ARGUMENT;
    const int heads = n_heads + 2 * n_kv, N = heads * head_dim;
    const RopeOut rope{cos_table, sin_table, positions, seq_of_token, block_table, (bf16_t*)k_pages, (bf16_t*)v_pages,
                       table_width, n_heads, n_kv, head_dim, page_size};
    const dim3 grid(heads * (head_dim / 32));
    if (K >= 1024)
        hipLaunchKernelGGL((gemm_skinny_kernel<bf16_t, 2, 16, 2, EPI_ROPE>), grid, dim3(16 * SIA_WAVE), 0, stream,
                           (const bf16_t*)X, (const bf16_t*)W, (bf16_t*)Y, M, N, K, rope);
    else
        hipLaunchKernelGGL((gemm_skinny_kernel<bf16_t, 2, 8, 2, EPI_ROPE>), grid, dim3(8 * SIA_WAVE), 0, stream,
                           (const bf16_t*)X, (const bf16_t*)W, (bf16_t*)Y, M, N, K, rope);
    return SIA_LAUNCH_CHECK();
}
