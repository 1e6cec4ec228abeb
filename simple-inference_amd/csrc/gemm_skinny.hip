// Y[M, N] = X[M, K] * W[N, K]^T in bfloat16 with float accumulation, for few rows (M <= 16):
// the matrix products of a decode step, where every weight is read once and the time is the time
// to stream W from HBM.
//
// One workgroup of 8 or 16 waves per RB blocks of up to 16 rows of W.  K is cut into chunks of 128, and chunk c
// belongs to *share* c % 16: a share's chunks are summed front to back into one accumulator, and the 16 shares'
// sums are added as (s0 + s8) + (s1 + s9) + ... + (s7 + s15), left to right.  With 16 waves every wave has one
// share and the sums meet in LDS; with 8, wave w has shares w and w + 8 (chunks w, w + 8, w + 16, ... alternate
// between its two accumulators) and adds the two itself, so the workgroup still walks its rows front to back
// and needs half the LDS.  A wave's step covers 64 k of RB blocks of rows with 2*RB MFMAs 16x16x32:
//   A = W[row of lane r in block rb][k0 + 16g .. + 15]   two 16-byte loads a lane, 128 contiguous bytes per row
//   B = X[r][same k]                                     loaded once for all RB blocks
// (an MFMA's k index only has to mean the same element in A and B, so lane group g may take the 16
// consecutive k that start at 16g and feed them to two MFMAs.)  X is small and comes from the caches, once per
// workgroup.
//
// A compute unit streams its rows at a rate of its own, well below its share of what the memory delivers, so a
// product is as fast as the busiest compute unit: a block holds `bh` <= 16 rows, chosen on the host so that
// the workgroups come out as a whole number of rounds over the compute units (3,072 rows on 256 units: 256
// blocks of 12, not 192 of 16).  Lanes r >= bh load the block's last row again (the same cache lines, no further
// traffic) and rows m >= M of X the last live one; what the MFMAs make of them is never stored.
//
// The result element (m, n) is summed over k in an order that depends on K only, not on M, the other rows,
// the number of waves, the row blocks of a workgroup or their height: whichever shape a launch takes, a row's
// result is the same bit for bit.
#include "common.h"

#include <initializer_list>

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float floatx4;

constexpr int SK_STEP = 64;    // k per step of one wave
constexpr int SK_CHUNK = 128;  // k per chunk: two steps
constexpr int SK_SHARES = 16;  // chunk c is summed into share c % 16

__device__ __forceinline__ bf16x8 ld8(const bf16_t* p) {
    return __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(p));
}

enum SkinnyEpilogue { EPI_STORE = 0, EPI_SWIGLU = 1, EPI_ROPE = 2, EPI_RESIDUAL = 3 };

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

// The product adds its result into the float residual and leaves what the norm after it needs.
struct ResidualOut {
    float* residual;      // [M][N], updated in place
    const float* gain;    // [N], the norm's weight
    bf16_t* scaled;       // [M][N] = residual * gain, not yet divided by the row's root mean square
    float* partials;      // [column blocks][16]: sum over a block's columns of residual^2, by row
};

// X is such a `scaled` matrix: row m of the result is to be multiplied by rsqrt(sum_p partials[p][m] / K + eps).
struct RowScale {
    const float* partials;
    int n_partials;
    float eps;
};

struct Epilogue {
    RopeOut rope;
    ResidualOut res;
    RowScale scale;
};

// RB: blocks of bh rows of W per workgroup; WAVES: 8 or 16 waves that split K.
//   EPI_STORE:   row block rb holds bh rows of W and gives as many columns of Y (TOut)
//   EPI_SWIGLU:  W = [gate; up] of N rows each; the first RB / 2 row blocks are gate rows, the others the up rows of
//                the same columns: Y = silu(gate) * up, in float, rounded once
//   EPI_ROPE:    RB = 2, W = [q heads | k heads | v heads] of head_dim rows each; a workgroup owns 16 columns of
//                the first half of a head and the 16 that the rotation pairs them with (head_dim / 2 further).
//                q and k are rotated in float on the float sums (one rounding; the rotation kernel rotates the
//                rounded product, so the two paths differ by a rounding); q goes to Y, k and v into the pages.
//   EPI_RESIDUAL: the result, rounded as EPI_STORE rounds it, is added to the float residual; Y is not written.
//                RMSNorm(x) W^T = rsqrt(mean x^2 + eps) * ((x * gain) W^T): the kernel leaves x * gain and the sums
//                of squares of its own column blocks, and the product after it (SCALED) adds those up, in an
//                order that depends on their number only, and scales its rows: no kernel of its own for the norm.
// Output columns come in *units*: a column of Y (EPI_STORE, EPI_RESIDUAL, EPI_SWIGLU, where unit u needs row u of
// the gate half and row u of the up half of W), or a pair of columns that the rotation mixes (EPI_ROPE: unit u is
// column u % (head_dim / 2) of head u / (head_dim / 2) together with the column head_dim / 2 further).  A workgroup
// owns UNIT_BLOCKS blocks of bh consecutive units from blockIdx.x * UNIT_BLOCKS * bh on.
// TILED: W is not [N][K] but a copy laid out for this cut, so that every load instruction of a wave reads one
// run of memory: [block of bh rows][step of 64 k][half of a lane's 16 k][row][lane group][8 k] (see
// sia_gemm_skinny_tiled_weights).  The same elements meet in the same products, so no bit changes.
template <typename TOut, int RB, int WAVES, int EPI, bool SCALED, bool TILED = false>
__global__ __launch_bounds__(WAVES* SIA_WAVE) void gemm_skinny_kernel(const bf16_t* __restrict__ X,
                                                                     const bf16_t* __restrict__ W,
                                                                     TOut* __restrict__ Y, int M, int N, int K,
                                                                     int bh, const Epilogue ep) {
    static_assert(WAVES == 8 || WAVES == 16, "8 or 16 waves share the 16 shares of K");
    static_assert(EPI != EPI_ROPE || RB == 2, "the rotation pairs two row blocks");
    static_assert(EPI != EPI_SWIGLU || RB % 2 == 0, "gate and up rows come in equal numbers");
    constexpr int SPW = SK_SHARES / WAVES;  // shares per wave
    constexpr int UNIT_BLOCKS = EPI == EPI_SWIGLU ? RB / 2 : EPI == EPI_ROPE ? 1 : RB;
    __shared__ float part[WAVES][RB][16][17];
    __shared__ float squares[SK_SHARES][16];
    const RopeOut& rope = ep.rope;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / SIA_WAVE);  // a scalar, and the compiler knows
    const int lane = threadIdx.x & 63, r = lane & 15, g = lane >> 4;
    const int rope_half = EPI == EPI_ROPE ? rope.head_dim / 2 : 0;
    const int units = EPI == EPI_ROPE ? (rope.n_heads + 2 * rope.n_kv) * rope_half : N;
    const int u0 = blockIdx.x * UNIT_BLOCKS * bh;
    // the unit of place n of unit block jb; places beyond the block or beyond the last unit repeat a unit before
    auto unit_at = [&](int jb, int n) { return min(u0 + jb * bh + min(n, bh - 1), units - 1); };
    auto is_live = [&](int jb, int n) { return n < bh && u0 + jb * bh + n < units; };
    const bf16_t* x_row = X + (size_t)min(r, M - 1) * K + g * 16;
    const bf16_t* w_row[RB];
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) {
        int row;
        if (EPI == EPI_ROPE) {  // the second row block holds the rotation's partners
            const int u = unit_at(0, r);
            row = (u / rope_half) * rope.head_dim + u % rope_half + rb * rope_half;
        } else {  // rb / UNIT_BLOCKS: 0 gate (or all), 1 up
            row = unit_at(rb % UNIT_BLOCKS, r) + (rb / UNIT_BLOCKS) * N;
        }
        w_row[rb] = W + (size_t)row * K + g * 16;
        if (TILED)  // the block's tiles: (step, half) apart by bh * 32 elements, this lane's piece inside a tile
            w_row[rb] = W + (size_t)(blockIdx.x * RB + rb) * (K / SK_STEP) * 2 * bh * 32 + (min(r, bh - 1) * 4 + g) * 8;
    }
    static_assert(!TILED || EPI == EPI_STORE || EPI == EPI_RESIDUAL, "tiled weights: a row block is a block of columns");

    // requested before the weights, used after them.  The sums of squares of a row are added up the way the
    // products are: 64 runners (16 shares of 4 lane groups), runner l taking partials l, l + 64, ...
    constexpr int SQ_RUNNERS = SK_SHARES * 4;
    const int sq_m = lane & 15;
    float sq[SPW][4];
    if (SCALED) {
#pragma unroll
        for (int j = 0; j < SPW; ++j)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int p = (wave + j * WAVES) * 4 + (lane >> 4) + i * SQ_RUNNERS;
                sq[j][i] = p < ep.scale.n_partials ? ep.scale.partials[p * 16 + sq_m] : 0.f;
            }
    }
    constexpr int RES_ITER = (RB * 256 + WAVES * SIA_WAVE - 1) / (WAVES * SIA_WAVE);
    float res_old[RES_ITER], res_gain[RES_ITER];
    if (EPI == EPI_RESIDUAL) {
#pragma unroll
        for (int it = 0; it < RES_ITER; ++it) {
            const int idx = threadIdx.x + it * WAVES * SIA_WAVE;
            const int j = idx / 256, m = (idx / 16) % 16, n = idx % 16;
            const bool live = idx < RB * 256 && m < M && is_live(j, n);
            res_old[it] = live ? ep.res.residual[(size_t)m * N + u0 + j * bh + n] : 0.f;
            res_gain[it] = live ? ep.res.gain[u0 + j * bh + n] : 0.f;
        }
    }

    // acc[j] belongs to share wave + j * WAVES.  This wave's t-th chunk is chunk wave + t * WAVES, of share
    // (wave + t * WAVES) % 16 = wave + (t % SPW) * WAVES, so it goes into accumulator t % SPW; the chunks are
    // taken in order of t, which is each share's own order.  (Loading a second group of chunks into registers of
    // their own while the first is multiplied was measured and changes nothing: enough waves are in flight.)
    floatx4 acc[SPW][RB];
#pragma unroll
    for (int j = 0; j < SPW; ++j)
#pragma unroll
        for (int rb = 0; rb < RB; ++rb) acc[j][rb] = floatx4{0.f, 0.f, 0.f, 0.f};
    constexpr int HOP = WAVES * SK_CHUNK;  // from one chunk of the wave to its next
    for (int k0 = wave * SK_CHUNK; k0 < K; k0 += SPW * HOP) {
#pragma unroll
        for (int j = 0; j < SPW; ++j) {
            // k is the same in all lanes of the wave (a scalar): a step outside K is skipped by a branch of the
            // wave, not by a mask of lanes.  K is a multiple of 64, so a step is inside or outside as a whole.
            const int k = k0 + j * HOP;
            bf16x8 a[2][RB][2], b[2][2];
#pragma unroll
            for (int u = 0; u < 2; ++u)
                if (k + u * SK_STEP < K) {
#pragma unroll
                    for (int rb = 0; rb < RB; ++rb) {
                        if (TILED) {
                            const size_t tile = (size_t)((k / SK_STEP + u) * 2) * bh * 32;
                            a[u][rb][0] = ld8(w_row[rb] + tile);
                            a[u][rb][1] = ld8(w_row[rb] + tile + bh * 32);
                        } else {
                            a[u][rb][0] = ld8(w_row[rb] + k + u * SK_STEP);
                            a[u][rb][1] = ld8(w_row[rb] + k + u * SK_STEP + 8);
                        }
                    }
                    b[u][0] = ld8(x_row + k + u * SK_STEP);
                    b[u][1] = ld8(x_row + k + u * SK_STEP + 8);
                }
#pragma unroll
            for (int u = 0; u < 2; ++u)
                if (k + u * SK_STEP < K) {
#pragma unroll
                    for (int rb = 0; rb < RB; ++rb) {
                        acc[j][rb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[u][rb][0], b[u][0], acc[j][rb], 0, 0, 0);
                        acc[j][rb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[u][rb][1], b[u][1], acc[j][rb], 0, 0, 0);
                    }
                }
        }
    }
    // acc[j][rb][i] = share wave + j * WAVES of row m = r, column 4g + i of row block rb
#pragma unroll
    for (int rb = 0; rb < RB; ++rb)
#pragma unroll
        for (int i = 0; i < 4; ++i)
            part[wave][rb][r][g * 4 + i] = SPW == 2 ? acc[0][rb][i] + acc[SPW - 1][rb][i] : acc[0][rb][i];
    // the sum over all of k of element (j, m, n): pairs of shares s and s + 8, then the pairs left to right
    auto total = [&](int j, int m, int n) -> float {
        float s = 0.f;
#pragma unroll
        for (int w = 0; w < 8; ++w) s += WAVES == 16 ? part[w][j][m][n] + part[w + 8][j][m][n] : part[w][j][m][n];
        return s;
    };
    if (SCALED) {
#pragma unroll
        for (int j = 0; j < SPW; ++j) {
            float ss = (sq[j][0] + sq[j][1]) + (sq[j][2] + sq[j][3]);
            for (int p = (wave + j * WAVES) * 4 + (lane >> 4) + 4 * SQ_RUNNERS; p < ep.scale.n_partials; p += SQ_RUNNERS)
                ss += ep.scale.partials[p * 16 + sq_m];
            ss += __shfl_xor(ss, 16);
            ss += __shfl_xor(ss, 32);
            if (lane < 16) squares[wave + j * WAVES][lane] = ss;
        }
    }
    __syncthreads();
    // the row's scale: every thread that finishes an element of row m adds the waves' sums in the same order
    auto row_scale = [&](int m) -> float {
        if (!SCALED) return 1.f;
        float ss = 0.f;
#pragma unroll
        for (int w = 0; w < SK_SHARES; ++w) ss += squares[w][m];
        return rsqrtf(ss / (float)K + ep.scale.eps);
    };
    if (EPI == EPI_ROPE) {
        const int m = threadIdx.x / 16, n = threadIdx.x % 16;
        if (threadIdx.x >= 256 || m >= M || !is_live(0, n)) return;
        float a = total(0, m, n), b = total(1, m, n);  // columns j and j + half of the head
        const float rs = row_scale(m);
        a *= rs;
        b *= rs;
        const int u = u0 + n, head = u / rope_half, j = u % rope_half, pos = rope.positions[m];
        const bool is_v = head >= rope.n_heads + rope.n_kv;
        if (!is_v) {
            const float c = rope.cos_table[(size_t)pos * rope_half + j], sn = rope.sin_table[(size_t)pos * rope_half + j];
            const float ra = a * c - b * sn, rb_ = b * c + a * sn;
            a = ra;
            b = rb_;
        }
        if (head < rope.n_heads) {
            TOut* y = Y + (size_t)m * N + head * rope.head_dim;
            y[j] = from_float<TOut>(a);
            y[j + rope_half] = from_float<TOut>(b);
            return;
        }
        const int page = rope.block_table[(size_t)rope.seq_of_token[m] * rope.table_width + pos / rope.page_size];
        if (page < 0) return;  // never for a token the step owns
        const int off = pos % rope.page_size, D = rope.head_dim, ps = rope.page_size;
        if (!is_v) {
            const int hk = head - rope.n_heads;
            bf16_t* dst = rope.k_pages + (((size_t)page * rope.n_kv + hk) * ps + off) * D;
            dst[j] = float_to_bf16(a);
            dst[j + rope_half] = float_to_bf16(b);
        } else {
            const int hk = head - rope.n_heads - rope.n_kv;
            bf16_t* dst = rope.v_pages + ((size_t)page * rope.n_kv + hk) * D * ps + off;
            dst[(size_t)j * ps] = float_to_bf16(a);
            dst[(size_t)(j + rope_half) * ps] = float_to_bf16(b);
        }
        return;
    }
    if (EPI == EPI_RESIDUAL) {
#pragma unroll
        for (int it = 0; it < RES_ITER; ++it) {
            const int idx = threadIdx.x + it * WAVES * SIA_WAVE;
            const int j = idx / 256, m = (idx / 16) % 16, n = idx % 16;
            if (idx >= RB * 256 || m >= M) continue;  // a whole 16-lane group leaves or stays
            const bool live = is_live(j, n);
            float x = 0.f;
            if (live) {
                x = res_old[it] + bf16_to_float(float_to_bf16(total(j, m, n) * row_scale(m)));
                const size_t at = (size_t)m * N + u0 + j * bh + n;
                ep.res.residual[at] = x;
                ep.res.scaled[at] = float_to_bf16(x * res_gain[it]);
            }
            float xx = x * x;
            xx += __shfl_xor(xx, 1);
            xx += __shfl_xor(xx, 2);
            xx += __shfl_xor(xx, 4);
            xx += __shfl_xor(xx, 8);
            if (n == 0) ep.res.partials[(blockIdx.x * RB + j) * 16 + m] = xx;  // 0 for a block beyond the last column
        }
        return;
    }
    for (int idx = threadIdx.x; idx < UNIT_BLOCKS * 256; idx += WAVES * SIA_WAVE) {
        const int j = idx / 256, m = (idx / 16) % 16, n = idx % 16;
        if (m >= M || !is_live(j, n)) continue;
        const float rs = row_scale(m);
        TOut* y = Y + (size_t)m * N + u0 + j * bh + n;
        if (EPI == EPI_SWIGLU) {
            float gate = total(j, m, n), up = total(UNIT_BLOCKS + j, m, n);
            gate *= rs;
            up *= rs;
            *y = from_float<TOut>(gate / (1.f + expf(-gate)) * up);
        } else {
            *y = from_float<TOut>(total(j, m, n) * rs);
        }
    }
}

SIA_EXPORT int sia_gemm_skinny_max_rows() { return 16; }

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

// How a product is cut into workgroups: `unit_blocks` blocks of `bh` units each, `grid` workgroups.
struct Cut {
    int unit_blocks, bh, grid;
    long long cost;  // rows of W the busiest compute unit streams, if workgroups ran in rounds over the units
};

// The block height for workgroups of `unit_blocks` blocks (each unit costs `rows_per_unit` rows of W): 16 when the
// workgroups are many; else the height from 8 to 16 that gives the busiest compute unit the least to stream.
static Cut cut_for(int units, int unit_blocks, int rows_per_unit) {
    const int cus = compute_units();
    auto with = [&](int bh) {
        const int grid = (units + unit_blocks * bh - 1) / (unit_blocks * bh);
        return Cut{unit_blocks, bh, grid, (long long)((grid + cus - 1) / cus) * bh * unit_blocks * rows_per_unit};
    };
    Cut best = with(16);
    if (best.grid > 2 * cus) return best;
    for (int bh = 15; bh >= 8; --bh) {
        const Cut c = with(bh);
        if (c.cost < best.cost) best = c;
    }
    return best;
}

// Of the cuts an epilogue has kernels for, the cheapest; of equals the one with the higher blocks (fewer lanes that
// repeat a row), then the one with more blocks per workgroup (fewer workgroups fetch X).
static Cut cheapest(int units, int rows_per_unit, std::initializer_list<int> unit_blocks) {
    Cut best{0, 0, 0, 0};
    for (int ub : unit_blocks) {
        const Cut c = cut_for(units, ub, rows_per_unit);
        if (!best.grid || c.cost < best.cost || (c.cost == best.cost && c.bh > best.bh)) best = c;
    }
    return best;
}

template <typename TOut, int EPI>
static void launch_skinny(const bf16_t* X, const bf16_t* W, TOut* Y, int M, int N, int K, const Epilogue& ep,
                          hipStream_t stream) {
    const Cut cut = cheapest(N, 1, {4, 2, 1});
#define LAUNCH(RB, WAVES)                                                                                 \
    hipLaunchKernelGGL((gemm_skinny_kernel<TOut, RB, WAVES, EPI, false>), dim3(cut.grid),                  \
                       dim3(WAVES * SIA_WAVE), 0, stream, X, W, Y, M, N, K, cut.bh, ep)
    if (cut.unit_blocks == 4)
        LAUNCH(4, 8);
    else if (cut.unit_blocks == 2)
        LAUNCH(2, 16);
    else
        LAUNCH(1, 8);
#undef LAUNCH
}

// out_float: 1 -> Y is float, 0 -> bfloat16.  Needs M <= 16, K % 64 == 0.
SIA_EXPORT int sia_gemm_skinny(const void* X, const void* W, void* Y, int M, int N, int K, int out_float,
                               hipStream_t stream) {
    if (M <= 0 || N <= 0) return 0;
    if (M > 16 || K % 64 || K <= 0) return SIA_BAD_ARGUMENT;
    if (out_float)
        launch_skinny<float, EPI_STORE>((const bf16_t*)X, (const bf16_t*)W, (float*)Y, M, N, K, Epilogue{}, stream);
    else
        launch_skinny<bf16_t, EPI_STORE>((const bf16_t*)X, (const bf16_t*)W, (bf16_t*)Y, M, N, K, Epilogue{}, stream);
    return SIA_LAUNCH_CHECK();
}

// Blocks of columns whose sums of squares sia_gemm_skinny_residual leaves for a result of N columns.
SIA_EXPORT int sia_gemm_skinny_residual_blocks(int N) {
    if (N <= 0) return 0;
    const Cut cut = cheapest(N, 1, {4, 2, 1});
    return cut.grid * cut.unit_blocks;
}

// residual[M, N] += round_bf16(X W^T); scaled = residual * gain (bfloat16); partials[blocks][16] = sums of squares of
// the residual over blocks of columns, by row (rows >= M are not written), blocks = sia_gemm_skinny_residual_blocks(N).
// Needs M <= 16, K % 64 == 0.
SIA_EXPORT int sia_gemm_skinny_residual(const void* X, const void* W, int M, int N, int K, float* residual,
                                        const float* gain, void* scaled, float* partials, hipStream_t stream) {
    if (M <= 0 || N <= 0) return 0;
    if (M > 16 || K % 64 || K <= 0 || !residual || !gain || !scaled || !partials) return SIA_BAD_ARGUMENT;
    Epilogue ep{};
    ep.res = ResidualOut{residual, gain, (bf16_t*)scaled, partials};
    launch_skinny<bf16_t, EPI_RESIDUAL>((const bf16_t*)X, (const bf16_t*)W, (bf16_t*)nullptr, M, N, K, ep, stream);
    return SIA_LAUNCH_CHECK();
}

// The tiled copy of W[N][K] that sia_gemm_skinny_residual_tiled reads: sia_gemm_skinny_tile_height(N) rows a block
// (0: this N is cut into workgroups of several blocks, which have no tiled form), blocks = ceil(N / height), the
// last block's missing rows repeating row N - 1; elements [block][K / 64][2][height][4][8], where element
// (b, s, h, r, g, e) is W[b * height + r][64 s + 16 g + 8 h + e].
SIA_EXPORT int sia_gemm_skinny_tile_height(int N) {
    if (N <= 0) return 0;
    const Cut cut = cheapest(N, 1, {4, 2, 1});
    return cut.unit_blocks == 1 ? cut.bh : 0;
}

SIA_EXPORT int sia_gemm_skinny_residual_tiled(const void* X, const void* W_tiled, int M, int N, int K, float* residual,
                                              const float* gain, void* scaled, float* partials, hipStream_t stream) {
    if (M <= 0 || N <= 0) return 0;
    if (M > 16 || K % 64 || K <= 0 || !residual || !gain || !scaled || !partials) return SIA_BAD_ARGUMENT;
    const Cut cut = cheapest(N, 1, {4, 2, 1});
    if (cut.unit_blocks != 1) return SIA_BAD_ARGUMENT;
    Epilogue ep{};
    ep.res = ResidualOut{residual, gain, (bf16_t*)scaled, partials};
    hipLaunchKernelGGL((gemm_skinny_kernel<bf16_t, 1, 8, EPI_RESIDUAL, false, true>), dim3(cut.grid), dim3(8 * SIA_WAVE), 0,
                       stream, (const bf16_t*)X, (const bf16_t*)W_tiled, (bf16_t*)nullptr, M, N, K, cut.bh, ep);
    return SIA_LAUNCH_CHECK();
}

// Y[M, I] = silu(X Wg^T) * (X Wu^T) for W = [Wg; Wu] of 2 I rows.  Needs M <= 16, K % 64 == 0.
// With `partials` (else null) X is a `scaled` matrix of sia_gemm_skinny_residual and the rows are divided by their
// root mean square first.
SIA_EXPORT int sia_gemm_skinny_swiglu(const void* X, const void* W, void* Y, int M, int inter, int K,
                                      const float* partials, int n_partials, float eps, hipStream_t stream) {
    if (M <= 0 || inter <= 0) return 0;
    if (M > 16 || K % 64 || K <= 0 || (partials && n_partials <= 0)) return SIA_BAD_ARGUMENT;
    Epilogue ep{};
    ep.scale = RowScale{partials, n_partials, eps};
    const Cut cut = cheapest(inter, 2, {2, 1});
#define LAUNCH(RB, WAVES, SCALED)                                                                                  \
    hipLaunchKernelGGL((gemm_skinny_kernel<bf16_t, RB, WAVES, EPI_SWIGLU, SCALED>), dim3(cut.grid),              \
                       dim3(WAVES * SIA_WAVE), 0, stream, (const bf16_t*)X, (const bf16_t*)W, (bf16_t*)Y, M, inter, \
                       K, cut.bh, ep)
    if (cut.unit_blocks == 2 && partials)
        LAUNCH(4, 16, true);
    else if (cut.unit_blocks == 2)
        LAUNCH(4, 16, false);
    else if (partials)
        LAUNCH(2, 8, true);
    else
        LAUNCH(2, 8, false);
#undef LAUNCH
    return SIA_LAUNCH_CHECK();
}

// The q/k/v product of single-token steps with the rotation and the cache write in its epilogue:
// W = [q heads | k heads | v heads], head_dim even, every dim of a head rotates (tables of head_dim / 2 floats
// a position).  Rotated q goes to Y[M][(n_heads + 2 n_kv) head_dim] (its k and v columns are not written); rotated
// k and v go to the pages at each token's position.  Needs M <= 16, K % 64 == 0.  `partials` as above.
SIA_EXPORT int sia_gemm_skinny_rope(const void* X, const void* W, void* Y, int M, int K, const float* cos_table,
                                    const float* sin_table, const int* positions, const int* seq_of_token,
                                    const int* block_table, int table_width, void* k_pages, void* v_pages,
                                    int n_heads, int n_kv, int head_dim, int page_size, const float* partials,
                                    int n_partials, float eps, hipStream_t stream) {
    if (M <= 0) return 0;
    if (M > 16 || K % 64 || K <= 0 || head_dim % 2 || head_dim <= 0 || n_heads <= 0 || n_kv <= 0 || page_size <= 0 ||
        table_width <= 0 || !cos_table || !sin_table || !positions || !seq_of_token || !block_table || !k_pages ||
        !v_pages || (partials && n_partials <= 0))
        return SIA_BAD_ARGUMENT;
    const int heads = n_heads + 2 * n_kv, N = heads * head_dim;
    Epilogue ep{};
    ep.rope = RopeOut{cos_table, sin_table, positions, seq_of_token, block_table, (bf16_t*)k_pages, (bf16_t*)v_pages,
                      table_width, n_heads, n_kv, head_dim, page_size};
    ep.scale = RowScale{partials, n_partials, eps};
    const Cut cut = cut_for(heads * (head_dim / 2), 1, 2);
#define LAUNCH(WAVES, SCALED)                                                                              \
    hipLaunchKernelGGL((gemm_skinny_kernel<bf16_t, 2, WAVES, EPI_ROPE, SCALED>), dim3(cut.grid),            \
                       dim3(WAVES * SIA_WAVE), 0, stream, (const bf16_t*)X, (const bf16_t*)W, (bf16_t*)Y, M, N, K,  \
                       cut.bh, ep)
    if (K >= 1024 && partials)
        LAUNCH(16, true);
    else if (K >= 1024)
        LAUNCH(16, false);
    else if (partials)
        LAUNCH(8, true);
    else
        LAUNCH(8, false);
#undef LAUNCH
    return SIA_LAUNCH_CHECK();
}
