// What a plain streaming read reaches on this card: the ceiling that the decode step's weight and cache reads are
// priced against, beside the published figure.
//
// Every workgroup takes pieces of 32 KiB in turn (a grid stride of pieces), 16 bytes a lane and eight loads in
// flight, and folds what it reads into one word, which is written only if it has a value that data does not take
// in practice, so that the loads cannot be dropped and nothing is written.
#include "common.h"

constexpr size_t BW_PIECE = 8 * 256;  // 16-byte words of a piece

__global__ __launch_bounds__(256) void stream_read_kernel(const uint4* __restrict__ src, size_t n_pieces,
                                                          unsigned* __restrict__ sink) {
    unsigned fold = 0;
    for (size_t piece = blockIdx.x; piece < n_pieces; piece += gridDim.x) {
        const uint4* p = src + piece * BW_PIECE + threadIdx.x;
        uint4 v[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) v[j] = p[j * 256];
#pragma unroll
        for (int j = 0; j < 8; ++j) fold ^= v[j].x ^ v[j].y ^ v[j].z ^ v[j].w;
    }
    if (fold == 0x9e3779b9u) sink[0] = fold;
}

// Reads `bytes` bytes (a multiple of 32 KiB) at src once.  sink: one word of device memory.
SIA_EXPORT int sia_stream_read(const void* src, long long bytes, void* sink, hipStream_t stream) {
    if (bytes <= 0) return 0;
    if (bytes % (long long)(BW_PIECE * 16) || !src || !sink) return SIA_BAD_ARGUMENT;
    int device = 0, cus = 256;
    if (hipGetDevice(&device) == hipSuccess) {
        int n = 0;
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, device) == hipSuccess && n > 0) cus = n;
    }
    hipLaunchKernelGGL(stream_read_kernel, dim3(cus * 8), dim3(256), 0, stream, (const uint4*)src,
                       (size_t)(bytes / (long long)(BW_PIECE * 16)), (unsigned*)sink);
    return SIA_LAUNCH_CHECK();
}
