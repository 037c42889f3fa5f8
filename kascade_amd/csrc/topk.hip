// Exact per-row top-n selection over fp16 scores (radix select on the 16-bit
// order-preserving key), one 1024-thread workgroup per row:
//   pass 1  LDS histogram of the high 11 key bits, suffix scan -> threshold bin
//   pass 2  LDS histogram of the low 5 bits inside that bin -> exact threshold
//           key T and the number r of entries equal to T that still fit
//   pass 3  ordered compaction: entries > T and the first r entries == T, written
//           in ascending index order (deterministic, ties to the lower index)
// The row is streamed from L2/HBM three times as 16-byte loads.
#include "topk.h"

namespace kascade {

namespace {

constexpr int kThreads = 1024;
constexpr int kWaves = kThreads / 64;
constexpr int kChunk = kThreads * 8;
constexpr int kBins1 = 2048;

__device__ __forceinline__ uint32_t order_key(uint16_t bits) {
    // monotone map fp16 -> u16: negatives below positives, -inf lowest finite order
    return (bits & 0x8000u) ? (uint32_t)(uint16_t)~bits : (uint32_t)(bits | 0x8000u);
}

// Loads entries [base, base+8) of a row as order keys; entries >= len get key 0xFFFFFFFF
// marker "absent" through the valid mask.
__device__ __forceinline__ int load_keys(const uint16_t* __restrict__ src, bool aligned, int base,
                                         int len, uint32_t keys[8]) {
    int nvalid = min(8, len - base);
    if (aligned && nvalid == 8) {
        uint4_t v = *reinterpret_cast<const uint4_t*>(src + base);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            keys[2 * e] = order_key((uint16_t)(v[e] & 0xFFFFu));
            keys[2 * e + 1] = order_key((uint16_t)(v[e] >> 16));
        }
    } else {
#pragma unroll
        for (int e = 0; e < 8; ++e) keys[e] = (e < nvalid) ? order_key(src[base + e]) : 0u;
    }
    return nvalid;
}

// Exclusive prefix sum over the 1024 threads of the block; *total receives the block sum.
__device__ __forceinline__ uint32_t block_excl_scan(uint32_t v, uint32_t* s_wave, uint32_t* total) {
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    uint32_t inc = v;
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
        uint32_t t = __shfl_up(inc, o);
        if (lane >= o) inc += t;
    }
    if (lane == 63) s_wave[wave] = inc;
    __syncthreads();
    uint32_t before = 0, all = 0;
#pragma unroll
    for (int w = 0; w < kWaves; ++w) {
        uint32_t t = s_wave[w];
        if (w < wave) before += t;
        all += t;
    }
    __syncthreads();
    *total = all;
    return before + inc - v;
}

__global__ __launch_bounds__(kThreads) void topk_select_kernel(
    const uint16_t* __restrict__ scores, int* __restrict__ out, long long row_stride,
    int uniform_len, const int* __restrict__ valid_len, const int* __restrict__ n_sel, int period,
    int k, int fill) {
    __shared__ uint32_t s_hist[kBins1];
    __shared__ uint32_t s_hist2[32];
    __shared__ uint32_t s_wave[kWaves];
    __shared__ uint32_t s_sel[4];  // b1, cum_above, T, r

    const int tid = threadIdx.x;
    const long long row = blockIdx.x;
    const int pr = (int)(row % period);
    const int len = valid_len ? valid_len[pr] : uniform_len;
    int n = n_sel ? n_sel[pr] : k;
    n = max(0, min(n, k));
    const uint16_t* src = scores + row * row_stride;
    int* dst = out + row * (long long)k;

    if (len <= n || n == 0) {
        for (int i = tid; i < k; i += kThreads) dst[i] = (i < n) ? i : fill;
        return;
    }
    const bool aligned = ((reinterpret_cast<uintptr_t>(src) & 15) == 0);

    // ---- pass 1: coarse histogram ----
    for (int i = tid; i < kBins1; i += kThreads) s_hist[i] = 0;
    if (tid < 32) s_hist2[tid] = 0;
    __syncthreads();
    for (int base = tid * 8; base < len; base += kChunk) {
        uint32_t keys[8];
        int nv = load_keys(src, aligned, base, len, keys);
#pragma unroll
        for (int e = 0; e < 8; ++e)
            if (e < nv) atomicAdd(&s_hist[keys[e] >> 5], 1u);
    }
    __syncthreads();
    {
        // thread t owns bins 2047-2t and 2046-2t (descending order)
        const int rb0 = kBins1 - 1 - 2 * tid;
        const uint32_t c0 = s_hist[rb0], c1 = s_hist[rb0 - 1];
        uint32_t total;
        const uint32_t above0 = block_excl_scan(c0 + c1, s_wave, &total);
        const uint32_t above1 = above0 + c0;
        const uint32_t un = (uint32_t)n;
        if (above0 < un && un <= above0 + c0) {
            s_sel[0] = rb0;
            s_sel[1] = above0;
        } else if (above1 < un && un <= above1 + c1) {
            s_sel[0] = rb0 - 1;
            s_sel[1] = above1;
        }
    }
    __syncthreads();
    const uint32_t b1 = s_sel[0];
    const uint32_t cum_above = s_sel[1];

    // ---- pass 2: fine histogram inside the threshold bin ----
    for (int base = tid * 8; base < len; base += kChunk) {
        uint32_t keys[8];
        int nv = load_keys(src, aligned, base, len, keys);
#pragma unroll
        for (int e = 0; e < 8; ++e)
            if (e < nv && (keys[e] >> 5) == b1) atomicAdd(&s_hist2[keys[e] & 31u], 1u);
    }
    __syncthreads();
    if (tid == 0) {
        uint32_t above = cum_above;
        int b2 = 31;
        for (; b2 > 0; --b2) {
            uint32_t c = s_hist2[b2];
            if (above + c >= (uint32_t)n) break;
            above += c;
        }
        s_sel[2] = (b1 << 5) | (uint32_t)b2;
        s_sel[3] = (uint32_t)n - above;  // entries equal to T to take
    }
    __syncthreads();
    const uint32_t T = s_sel[2];
    const uint32_t r = s_sel[3];

    // ---- pass 3: ordered compaction ----
    uint32_t gt_base = 0, eq_base = 0;
    for (int cbase = 0; cbase < len; cbase += kChunk) {
        const int base = cbase + tid * 8;
        uint32_t keys[8];
        int nv = (base < len) ? load_keys(src, aligned, base, len, keys) : 0;
        uint32_t gt = 0, eq = 0;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            if (e < nv) {
                gt += (keys[e] > T);
                eq += (keys[e] == T);
            }
        }
        uint32_t total;
        const uint32_t ex = block_excl_scan(gt | (eq << 16), s_wave, &total);
        uint32_t my_gt = gt_base + (ex & 0xFFFFu);
        uint32_t my_eq = eq_base + (ex >> 16);
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            if (e < nv) {
                if (keys[e] > T) {
                    dst[my_gt + min(my_eq, r)] = base + e;
                    ++my_gt;
                } else if (keys[e] == T) {
                    if (my_eq < r) dst[my_gt + my_eq] = base + e;
                    ++my_eq;
                }
            }
        }
        gt_base += total & 0xFFFFu;
        eq_base += total >> 16;
    }
    for (int i = n + tid; i < k; i += kThreads) dst[i] = fill;
}

}  // namespace

hipError_t launch_topk(const half_t* scores, int* out_idx, int rows, long long row_stride,
                       int uniform_len, const int* valid_len, const int* n_sel, int period, int k,
                       int fill, hipStream_t stream) {
    if (rows == 0) return hipSuccess;
    hipLaunchKernelGGL(topk_select_kernel, dim3(rows), dim3(kThreads), 0, stream,
                       reinterpret_cast<const uint16_t*>(scores), out_idx, row_stride, uniform_len,
                       valid_len, n_sel, period, k, fill);
    return hipGetLastError();
}

}  // namespace kascade
