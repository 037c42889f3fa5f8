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

// Per (sequence, KV head) row of a ragged decode step: how many pooled scores are valid and how
// many of them the selection keeps, n(b) = 128*ceil(floor(percent*len_b/100)/128), optionally
// after adding `advance` to every length in place (the step's new token).
__global__ __launch_bounds__(256) void decode_budgets_kernel(int* __restrict__ seqlens, int advance,
                                                             float percent, int batch,
                                                             int* __restrict__ valid_rows,
                                                             int* __restrict__ n_sel_rows) {
    // a single workgroup: the barrier puts the in-place update after every read of a length
    for (int i = threadIdx.x; i < batch * kGroups; i += blockDim.x) {
        const int len = seqlens[i / kGroups] + advance;
        const long long fl = (long long)floor((double)percent * (double)len / 100.0);
        if (valid_rows) valid_rows[i] = len;
        if (n_sel_rows) n_sel_rows[i] = (int)(((fl + 127) / 128) * 128);
    }
    __syncthreads();
    if (advance != 0)
        for (int b = threadIdx.x; b < batch; b += blockDim.x) seqlens[b] += advance;
}

}  // namespace

hipError_t launch_decode_budgets(int* seqlens, int advance, float percent, int batch, int* valid_rows,
                                 int* n_sel_rows, hipStream_t stream) {
    hipLaunchKernelGGL(decode_budgets_kernel, dim3(1), dim3(256), 0, stream, seqlens, advance, percent,
                       batch, valid_rows, n_sel_rows);
    return hipGetLastError();
}

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
