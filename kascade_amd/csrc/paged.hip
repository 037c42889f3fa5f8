// Paged KV-cache append: scatter the new tokens' K/V rows into their page slots.
// One 16-byte chunk per thread; grid covers B * n_new * G * 16 chunks for K and V.
#include "paged.h"

namespace kascade {

namespace {

__global__ __launch_bounds__(256) void paged_kv_append_kernel(
    half_t* __restrict__ Kp, half_t* __restrict__ Vp, const half_t* __restrict__ k_new,
    const half_t* __restrict__ v_new, const int* __restrict__ start_pos,
    const int* __restrict__ block_table, int batch, int n_new, int max_pages, int page_shift,
    long long sb, long long sl, long long sh) {
    const long long total = (long long)batch * n_new * kGroups * 16;
    const long long c = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (c >= total) return;
    const int col = (int)(c & 15);
    const int g = (int)((c >> 4) % kGroups);
    const long long bt = c / (16 * kGroups);
    const int t = (int)(bt % n_new);
    const int b = (int)(bt / n_new);
    const int tok = start_pos[b] + t;
    const int pg = block_table[(long long)b * max_pages + (tok >> page_shift)];
    const long long row = ((long long)pg << page_shift) + (tok & ((1 << page_shift) - 1));
    const long long dst = (row * kGroups + g) * kDim + col * 8;
    const long long src = b * sb + t * sl + g * sh + col * 8;
    *reinterpret_cast<uint4_t*>(Kp + dst) = ld_global_16(k_new + src);
    *reinterpret_cast<uint4_t*>(Vp + dst) = ld_global_16(v_new + src);
}

}  // namespace

hipError_t launch_paged_kv_append(half_t* Kp, half_t* Vp, const half_t* k_new, const half_t* v_new,
                                  const int* start_pos, const int* block_table, int batch,
                                  int n_new, int max_pages, int page_shift, long long sb,
                                  long long sl, long long sh, hipStream_t stream) {
    const long long total = (long long)batch * n_new * kGroups * 16;
    if (total == 0) return hipSuccess;
    dim3 grid((unsigned)((total + 255) / 256)), block(256);
    hipLaunchKernelGGL(paged_kv_append_kernel, grid, block, 0, stream, Kp, Vp, k_new, v_new,
                       start_pos, block_table, batch, n_new, max_pages, page_shift, sb, sl, sh);
    return hipGetLastError();
}

}  // namespace kascade
