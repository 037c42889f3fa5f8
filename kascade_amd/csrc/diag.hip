// Diagnostic read kernels: what the device delivers for the two access patterns of the decode
// path with no arithmetic attached -- a streaming read (dense decode) and a gather of whole
// 256-byte rows through an index list (reuse decode).  Used by the benchmark to put the decode
// kernels' GB/s next to what a plain kernel reaches; they compute nothing that is kept.
#include "diag.h"

namespace kascade {

namespace {

constexpr int kUnroll = 8;

// 16 bytes per lane, kUnroll independent non-temporal loads in flight per lane, grid-stride.
__global__ __launch_bounds__(256) void diag_stream_read_kernel(const uint4_t* __restrict__ src, long long n16,
                                                               uint4_t* __restrict__ sink) {
    const long long tid = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    const long long stride = (long long)gridDim.x * blockDim.x;
    uint4_t acc = {0, 0, 0, 0};
    long long i = tid;
    for (; i + (kUnroll - 1) * stride < n16; i += kUnroll * stride) {
        uint4_t v[kUnroll];
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) v[u] = __builtin_nontemporal_load(src + i + u * stride);
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) acc ^= v[u];
    }
    for (; i < n16; i += stride) acc ^= src[i];
    if (acc[0] == 0x12345678u && acc[1] == 0x9abcdef0u) sink[0] = acc;   // keeps the loads alive
}

// One 256-byte row per 16 lanes (16 rows per workgroup instruction), rows taken from a contiguous
// piece of the index list per workgroup; optionally the same row of a second array (K and V).
template <bool TWO>
__global__ __launch_bounds__(256) void diag_gather_rows_kernel(const char* __restrict__ a0, const char* __restrict__ a1,
                                                               const int* __restrict__ rows, long long n_rows,
                                                               int rows_per_block, long long row_stride_bytes,
                                                               uint4_t* __restrict__ sink) {
    const long long first = (long long)blockIdx.x * rows_per_block;
    const int dl = threadIdx.x & 15, rg = threadIdx.x >> 4;
    uint4_t acc = {0, 0, 0, 0};
    for (int r0 = 0; r0 < rows_per_block; r0 += 16 * kUnroll) {
        uint4_t v[kUnroll][2];
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
            const long long pos = min(first + r0 + u * 16 + rg, n_rows - 1);
            const long long off = (long long)rows[pos] * row_stride_bytes + dl * 16;
            v[u][0] = __builtin_nontemporal_load(reinterpret_cast<const uint4_t*>(a0 + off));
            v[u][1] = TWO ? __builtin_nontemporal_load(reinterpret_cast<const uint4_t*>(a1 + off)) : uint4_t{0, 0, 0, 0};
        }
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) acc ^= v[u][0] ^ v[u][1];
    }
    if (acc[0] == 0x12345678u && acc[1] == 0x9abcdef0u) sink[0] = acc;
}

}  // namespace

hipError_t launch_diag_stream_read(const void* src, long long bytes, void* sink, int blocks, hipStream_t stream) {
    hipLaunchKernelGGL(diag_stream_read_kernel, dim3(blocks), dim3(256), 0, stream,
                       static_cast<const uint4_t*>(src), bytes / 16, static_cast<uint4_t*>(sink));
    return hipGetLastError();
}

hipError_t launch_diag_gather_rows(const void* a0, const void* a1, const int* rows, long long n_rows,
                                   int rows_per_block, long long row_stride_bytes, void* sink,
                                   hipStream_t stream) {
    const int blocks = (int)((n_rows + rows_per_block - 1) / rows_per_block);
    if (a1)
        hipLaunchKernelGGL(diag_gather_rows_kernel<true>, dim3(blocks), dim3(256), 0, stream,
                           static_cast<const char*>(a0), static_cast<const char*>(a1), rows, n_rows,
                           rows_per_block, row_stride_bytes, static_cast<uint4_t*>(sink));
    else
        hipLaunchKernelGGL(diag_gather_rows_kernel<false>, dim3(blocks), dim3(256), 0, stream,
                           static_cast<const char*>(a0), static_cast<const char*>(a0), rows, n_rows,
                           rows_per_block, row_stride_bytes, static_cast<uint4_t*>(sink));
    return hipGetLastError();
}

}  // namespace kascade
