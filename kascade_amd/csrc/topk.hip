// Exact per-row top-n selection over fp16 scores (radix select on the 16-bit
// order-preserving key), one 1024-thread workgroup per row:
//   pass 1  LDS histogram of the high 11 key bits, suffix scan -> threshold bin
//   pass 2  LDS histogram of the low 5 bits inside that bin -> exact threshold
//           key T and the number r of entries equal to T that still fit
//   pass 3  ordered compaction: entries > T and the first r entries == T, written
//           in ascending index order (deterministic, ties to the lower index)
// The row is streamed from L2/HBM three times as 16-byte loads.
#include "topk.h"

#include <type_traits>

#include "prefill.h"   // launch_translate_indices

namespace kascade {

namespace {

constexpr int kThreads = 1024;
constexpr int kWaves = kThreads / 64;
constexpr int kChunk = kThreads * 8;
constexpr int kBins1 = 2048;
}  // namespace
constexpr int kSplitMinLen = 65537;   // longer than a workgroup's registers hold: multi-workgroup path
constexpr int kSplitMaxRows = 4096;   // workspace is 8 KB per row for the coarse histogram
namespace {

// Optional second output: every selected position translated to its row of a paged cache
// (block_table[sequence][pos / page] * page + pos % page), sequence = row / rows_per_seq.  What the
// gather kernels of the reuse layers read, produced here so that no separate launch is needed.
struct RowsOut {
    int* rows;               // [rows, k] or null
    const int* block_table;  // [sequences, max_pages]
    int max_pages;
    int page_shift;
    int rows_per_seq;
};

__device__ __forceinline__ int to_cache_row(const RowsOut& ro, long long row, int pos) {
    const int* bt = ro.block_table + (row / ro.rows_per_seq) * ro.max_pages;
    pos = max(0, min(pos, (ro.max_pages << ro.page_shift) - 1));
    return (bt[pos >> ro.page_shift] << ro.page_shift) + (pos & ((1 << ro.page_shift) - 1));
}

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

// Inclusive prefix sum over the 64 lanes of a wavefront in six DPP additions: four shifts within
// the rows of 16 lanes, then the last lane of row 0 / 2 added to row 1 / 3 and lane 31 to the
// upper half.
__device__ __forceinline__ uint32_t wave_incl_scan(uint32_t v) {
    v += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x111, 0xF, 0xF, false);   // row_shr:1
    v += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x112, 0xF, 0xF, false);   // row_shr:2
    v += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x114, 0xF, 0xF, false);   // row_shr:4
    v += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x118, 0xF, 0xF, false);   // row_shr:8
    v += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x142, 0xA, 0xF, false);   // row_bcast:15 -> rows 1, 3
    v += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x143, 0xC, 0xF, false);   // row_bcast:31 -> rows 2, 3
    return v;
}

// Packed 16-bit operations on the two halves of a word.  Written as instructions: the compiler
// otherwise turns min(sat(a - b), 1) into two compares, two selects and a byte permute.
__device__ __forceinline__ uint32_t pk_sub_sat_u16(uint32_t a, uint32_t b) {
    uint32_t r;
    asm("v_pk_sub_u16 %0, %1, %2 clamp" : "=v"(r) : "v"(a), "v"(b));
    return r;
}
__device__ __forceinline__ uint32_t pk_min_u16(uint32_t a, uint32_t b) {
    uint32_t r;
    asm("v_pk_min_u16 %0, %1, %2" : "=v"(r) : "v"(a), "v"(b));
    return r;
}
__device__ __forceinline__ uint32_t pk_max_u16(uint32_t a, uint32_t b) {
    uint32_t r;
    asm("v_pk_max_u16 %0, %1, %2" : "=v"(r) : "v"(a), "v"(b));
    return r;
}
// arithmetic shift right by 15 of both halves: 0xFFFF where a half is negative as int16, else 0
__device__ __forceinline__ uint32_t pk_sign_mask_i16(uint32_t a) {
    uint32_t r;
    asm("v_pk_ashrrev_i16 %0, %1, %2" : "=v"(r) : "v"(0x000F000Fu), "v"(a));
    return r;
}
__device__ __forceinline__ uint32_t pk_add_u16(uint32_t a, uint32_t b) {
    uint32_t r;
    asm("v_pk_add_u16 %0, %1, %2" : "=v"(r) : "v"(a), "v"(b));
    return r;
}

// Exclusive prefix sum over the 1024 threads of the block; *total receives the block sum.
__device__ __forceinline__ uint32_t block_excl_scan(uint32_t v, uint32_t* s_wave, uint32_t* total) {
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const uint32_t inc = wave_incl_scan(v);
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
    int k, int fill, RowsOut ro) {
    __shared__ uint32_t s_hist[kBins1];
    __shared__ uint32_t s_hist2[32];
    __shared__ uint32_t s_wave[kWaves];
    __shared__ uint32_t s_sel[4];  // b1, cum_above, T, r

    const int tid = threadIdx.x;
    const long long row = blockIdx.x;
    const int pr = (int)(row % period);
    const int len = valid_len ? min(valid_len[pr], uniform_len) : uniform_len;
    int n = n_sel ? n_sel[pr] : k;
    n = max(0, min(n, k));
    const uint16_t* src = scores + row * row_stride;
    int* dst = out + row * (long long)k;
    int* rdst = ro.rows ? ro.rows + row * (long long)k : nullptr;
    auto put = [&](int slot, int pos) {
        dst[slot] = pos;
        if (rdst) rdst[slot] = to_cache_row(ro, row, pos);
    };

    if (len <= n || n == 0) {
        for (int i = tid; i < k; i += kThreads) put(i, (i < n) ? i : fill);
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
                    put(my_gt + min(my_eq, r), base + e);
                    ++my_gt;
                } else if (keys[e] == T) {
                    if (my_eq < r) put(my_gt + my_eq, base + e);
                    ++my_eq;
                }
            }
        }
        gt_base += total & 0xFFFFu;
        eq_base += total >> 16;
    }
    for (int i = n + tid; i < k; i += kThreads) put(i, fill);
}


// The same selection with the row held in registers: every thread loads its share of the row
// once (MAXC 16-byte loads in flight, instead of one per pass and chunk with its latency
// exposed), turns it into packed order keys once, and the three passes run on registers.  With
// 16 to 64 entries per thread and eight wavefronts per SIMD the kernel is bound by the
// instructions spent per entry, so the per-entry work is kept to a few instructions:
//  * Real entries carry keys >= 1 (the two lowest negative NaN patterns share key 1) and the
//    slots past the end of the row key 0, so the threshold key T is >= 1 and no count needs a
//    validity test: a slot past the end is neither above T nor equal to it.
//  * The coarse histogram is kept in kCopies copies selected by the lane number, which spreads
//    the same-address conflicts of the LDS atomics (pooled softmax scores crowd into a few
//    exponent bins).  The bin of +0 and the 31 smallest subnormals, where pooled probabilities
//    underflow to by the thousand, is not counted at all: its count is the row length minus the
//    sum of the others.
//  * The fine histogram tests both halves of a word against the threshold bin at once; the counts
//    above / equal to T are sums of min(sat(key - (T-1)), 2) over packed halves.
//  * The compaction computes every (chunk, thread) offset with two barriers in all (per-chunk
//    wavefront scans, then one scan over the chunk x wavefront totals), and stages the selected
//    indices in LDS in their final order, so that the row's list leaves as full-width stores.
// The tensor must start 16-byte aligned (its rows need not) and a row, with the up to 7 slots
// between the boundary before it and its start, must fit MAXC*8192 slots (MAXC = 16: 131072, 64
// registers of row data per thread, still one workgroup of 1024 threads per CU).
template <int MAXC>
__global__ __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(MAXC <= 4 ? 8 : 4)))
void topk_select_reg_kernel(
    const uint16_t* __restrict__ scores, int* __restrict__ out, long long row_stride,
    int uniform_len, const int* __restrict__ valid_len, const int* __restrict__ n_sel, int period,
    int k, int fill, RowsOut ro) {
    constexpr int kCopies = 4;
    constexpr int kStage = kBins1 * kCopies;       // selected indices staged in the histogram's LDS
    constexpr uint32_t kOne = 0x00010001u, kTwo = 0x00020002u;
    constexpr uint32_t kZeroKey = 0x8000u;         // order key of +0
    constexpr uint32_t kSkipBin = kZeroKey >> 5;   // coarse bin of +0: counted by subtraction
    __shared__ __attribute__((aligned(16))) uint32_t s_hist[kBins1 * kCopies];
    __shared__ uint32_t s_hist2[32];
    __shared__ uint32_t s_wave[kWaves];
    __shared__ uint32_t s_tot[MAXC * kWaves];      // pass 3: totals per (chunk, wavefront), packed
    __shared__ uint32_t s_pgt[MAXC * kWaves];      // pass 3: exclusive prefixes of the counts above T
    __shared__ uint32_t s_peq[MAXC * kWaves];      // ... and of the counts equal to T
    __shared__ uint32_t s_sel[4];  // b1, cum_above, T, r
    // pass 3: the wavefront scans of the per-thread counts; in registers up to 8 chunks, beyond
    // that the row itself fills the register file
    constexpr bool kExwInLds = MAXC > 8;
    __shared__ uint32_t s_exw[kExwInLds ? MAXC * kThreads : 1];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const long long row = blockIdx.x;
    const int pr = (int)(row % period);
    const int len = valid_len ? min(valid_len[pr], uniform_len) : uniform_len;
    int n = n_sel ? n_sel[pr] : k;
    n = max(0, min(n, k));
    // A row that does not start on a 16-byte boundary (a row stride that is no multiple of 8) is
    // read from the boundary before it: `lead` slots in front of the row count as absent, like
    // the slots past its end, and every position below is taken in these shifted coordinates
    // (the tensor itself starts on a boundary, so the slots in front belong to the row before).
    const uint16_t* row_src = scores + row * row_stride;
    const int lead = (int)((reinterpret_cast<uintptr_t>(row_src) & 15) >> 1);
    const uint16_t* src = row_src - lead;
    const int row_len = len;            // entries of the row itself
    int* dst = out + row * (long long)k;
    int* rdst = ro.rows ? ro.rows + row * (long long)k : nullptr;
    auto put = [&](int slot, int pos) {
        dst[slot] = pos;
        if (rdst) rdst[slot] = to_cache_row(ro, row, pos);
    };

    if (row_len <= n || n == 0) {
        for (int i = tid; i < k; i += kThreads) put(i, (i < n) ? i : fill);
        return;
    }
    const int slots = row_len + lead;   // the row in shifted coordinates: [lead, slots)
    const int nchunks = (slots + kChunk - 1) / kChunk;   // <= MAXC (host)

    // ---- the row: chunk c, slots [c*8192 + 8*tid, +8) as packed order keys ----
    uint4_t data[MAXC];
    // slots of chunk c that lie before the row's end (recomputed where needed: an array of them
    // would cost MAXC registers), and the absent slots in front (only the first thread has any)
    auto nv_of = [&](int c) { return max(0, min(8, slots - (c * kChunk + tid * 8))); };
    auto lead_of = [&](int c) { return (c == 0 && tid == 0) ? lead : 0; };
    // Every thread loads 16 bytes per chunk without a branch around the load, so that the loads
    // are in flight together: where the chunk's share lies past the end of the row the address
    // is pulled back inside it and the data replaced below.
    const int last_full = max(slots - 8, 0) & ~7;
#pragma unroll
    for (int c = 0; c < MAXC; ++c) {
        data[c] = uint4_t{0, 0, 0, 0};
        if (slots >= 8)   // uniform
            data[c] = *reinterpret_cast<const uint4_t*>(src + min(c * kChunk + tid * 8, last_full));
    }
#pragma unroll
    for (int c = 0; c < MAXC; ++c) {
        const int base = c * kChunk + tid * 8;
        const int nvc = nv_of(c);
        const int ldc = lead_of(c);
        uint4_t raw = data[c];
        if (nvc == 8 && ldc == 0) {
            // order_key on both halves at once: negative values flip every bit, others the sign
            // bit; then at least 1
#pragma unroll
            for (int j = 0; j < 4; ++j)
                raw[j] = pk_max_u16(raw[j] ^ (pk_sign_mask_i16(raw[j]) | 0x80008000u), kOne);
        } else {   // the thread at the end of the row, and every thread beyond it
            uint32_t w[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const uint32_t lo = (2 * e < nvc && 2 * e >= ldc) ? max(order_key(src[base + 2 * e]), 1u) : 0u;
                const uint32_t hi = (2 * e + 1 < nvc && 2 * e + 1 >= ldc) ? max(order_key(src[base + 2 * e + 1]), 1u) : 0u;
                w[e] = lo | (hi << 16);
            }
            raw = uint4_t{w[0], w[1], w[2], w[3]};
        }
        data[c] = raw;
    }

    // ---- pass 1: coarse histogram ----
    {
        const uint4_t z = {0, 0, 0, 0};
#pragma unroll
        for (int i = 0; i < kBins1 * kCopies / (4 * kThreads); ++i)
            *reinterpret_cast<uint4_t*>(&s_hist[(i * kThreads + tid) * 4]) = z;
    }
    if (tid < 32) s_hist2[tid] = 0;
    __syncthreads();
    const uint32_t copy = tid & (kCopies - 1);
    auto count1 = [&](uint32_t key) {
        const uint32_t bin = key >> 5;
        if (bin != kSkipBin) atomicAdd(&s_hist[bin * kCopies + copy], 1u);
    };
#pragma unroll
    for (int c = 0; c < MAXC; ++c) {
        if (c < nchunks) {
            const int nvc = nv_of(c);
            const int ldc = lead_of(c);
            if (nvc == 8 && ldc == 0) {
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    count1(data[c][j] & 0xFFFFu);
                    count1(data[c][j] >> 16);
                }
            } else if (nvc > 0) {
#pragma unroll
                for (int e = 0; e < 8; ++e)
                    if (e < nvc && e >= ldc) count1((e & 1) ? (data[c][e >> 1] >> 16) : (data[c][e >> 1] & 0xFFFFu));
            }
        }
    }
    __syncthreads();
    {
        // thread t owns bins 2047-2t and 2046-2t (descending order); the uncounted bin is the
        // lower bin of its owner
        const int rb0 = kBins1 - 1 - 2 * tid;
        constexpr int kSkipOwner = (kBins1 - 2 - (int)kSkipBin) / 2;
        static_assert(kBins1 - 2 - 2 * kSkipOwner == (int)kSkipBin, "the uncounted bin must be a lower bin");
        const uint4_t h0 = *reinterpret_cast<const uint4_t*>(&s_hist[rb0 * kCopies]);
        const uint4_t h1 = *reinterpret_cast<const uint4_t*>(&s_hist[(rb0 - 1) * kCopies]);
        const uint32_t c0 = h0[0] + h0[1] + h0[2] + h0[3];
        uint32_t c1 = h1[0] + h1[1] + h1[2] + h1[3];
        uint32_t total;
        uint32_t above0 = block_excl_scan(c0 + c1, s_wave, &total);
        const uint32_t skipped = (uint32_t)row_len - total;
        if (tid == kSkipOwner) c1 += skipped;
        if (tid > kSkipOwner) above0 += skipped;
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
    if (b1 != kSkipBin) {
        // few entries match: test both halves of a word at once, then a branch
        const uint32_t bb = (b1 << 5) | (b1 << 21);
#pragma unroll
        for (int c = 0; c < MAXC; ++c) {
            if (c < nchunks) {
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const uint32_t w = data[c][j];
                    const uint32_t x = (w ^ bb) & 0xFFE0FFE0u;   // a half is 0 iff its key lies in the bin
                    if (pk_min_u16(x, kOne) != kOne) {
                        if ((x & 0xFFFFu) == 0) atomicAdd(&s_hist2[w & 31u], 1u);
                        if ((x >> 16) == 0) atomicAdd(&s_hist2[(w >> 16) & 31u], 1u);
                    }
                }
            }
        }
    } else {
        // The threshold lies among +0 and the smallest subnormals: that many atomics on one
        // address would serialise, so each wavefront counts its zeros with a ballot.
        uint32_t zeros = 0;                        // wavefront-uniform
#pragma unroll
        for (int c = 0; c < MAXC; ++c) {
            if (c < nchunks) {
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    const uint32_t w = data[c][e >> 1];
                    const uint32_t key = (e & 1) ? (w >> 16) : (w & 0xFFFFu);
                    const bool zero = key == kZeroKey;
                    zeros += (uint32_t)__popcll(__ballot(zero));
                    if ((key >> 5) == b1 && !zero) atomicAdd(&s_hist2[key & 31u], 1u);
                }
            }
        }
        if (lane == 0 && zeros) atomicAdd(&s_hist2[kZeroKey & 31u], zeros);
    }
    __syncthreads();
    if (tid < 64) {
        // suffix sums of the 32 fine bins, top bin first; the threshold is the first bin whose
        // running count reaches n
        const uint32_t c = (lane < 32) ? s_hist2[31 - lane] : 0u;
        const uint32_t v = wave_incl_scan(c);
        const uint32_t above = cum_above + v - c;             // entries in finer bins above this one
        const bool hit = lane < 32 && above < (uint32_t)n && (uint32_t)n <= above + c;
        // bin 0 takes what is left when no finer bin reaches n (cannot happen for a consistent
        // histogram; kept so that s_sel is always written)
        const unsigned long long m = __ballot(hit);
        const int first = m ? __ffsll((long long)m) - 1 : 31;
        if (lane == first) {
            s_sel[2] = max((b1 << 5) | (uint32_t)(31 - first), 1u);
            s_sel[3] = (uint32_t)n - above;  // entries equal to T to take
        }
    }
    __syncthreads();
    const uint32_t T = s_sel[2];
    const uint32_t r = s_sel[3];
    const uint32_t tm1 = (T - 1u) | ((T - 1u) << 16);   // T >= 1

    // ---- pass 3: ordered compaction (index order = chunk, then thread, then element) ----
    // code of a half: min(sat(key - (T-1)), 2) = 0 below T, 1 equal to T, 2 above T
    // counts of one (chunk, thread): entries above T in the low half, equal to T in the high half
    uint32_t exw[kExwInLds ? 1 : MAXC];   // exclusive scan of the counts over the wavefront
#pragma unroll
    for (int c = 0; c < MAXC; ++c) {
        uint32_t cnt = 0;
        if (c < nchunks) {
            uint32_t sum = 0, ties = 0;   // per half: sum of the codes (<= 8), number of ones (<= 4)
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const uint32_t code = pk_min_u16(pk_sub_sat_u16(data[c][j], tm1), kTwo);
                sum = pk_add_u16(sum, code);
                ties = pk_add_u16(ties, code & kOne);
            }
            const uint32_t s2 = (sum & 0xFFFFu) + (sum >> 16);     // ties + 2 * above
            const uint32_t eq = (ties & 0xFFFFu) + (ties >> 16);
            cnt = ((s2 - eq) >> 1) | (eq << 16);
        }
        const uint32_t v = wave_incl_scan(cnt);
        if (kExwInLds) s_exw[c * kThreads + tid] = v - cnt;
        else exw[c] = v - cnt;
        if (lane == 63) s_tot[c * kWaves + wave] = v;
    }
    __syncthreads();
    if (wave == 0) {
        // exclusive prefixes over the MAXC*16 (chunk, wavefront) totals, chunk-major, 64 per step.
        // A wavefront's totals fit the packed halves (at most 512 entries each); the prefixes over
        // a row of more than 65536 entries do not, so they are kept apart.
        uint32_t carry_gt = 0, carry_eq = 0;
#pragma unroll
        for (int i0 = 0; i0 < MAXC * kWaves; i0 += 64) {
            const uint32_t x = s_tot[i0 + lane];
            const uint32_t xg = x & 0xFFFFu, xe = x >> 16;
            const uint32_t vg = wave_incl_scan(xg), ve = wave_incl_scan(xe);
            s_pgt[i0 + lane] = carry_gt + vg - xg;
            s_peq[i0 + lane] = carry_eq + ve - xe;
            carry_gt += (uint32_t)__builtin_amdgcn_readlane((int)vg, 63);
            carry_eq += (uint32_t)__builtin_amdgcn_readlane((int)ve, 63);
        }
    }
    __syncthreads();
    // The selected indices are staged in LDS in their final order, kStage positions per round (one
    // round unless n > kStage), and leave as full-width stores.
    int* stage = reinterpret_cast<int*>(s_hist);
    for (uint32_t lo = 0; lo < (uint32_t)n; lo += kStage) {
        auto emit = [&](uint32_t pos, int idx) {
            if (pos - lo < (uint32_t)kStage) stage[pos - lo] = idx;
        };
        // opaque copy: the codes are recomputed per round instead of being kept in registers
        // across rounds (a second workgroup per CU needs the kernel within 64 registers)
        uint32_t tm1_r = tm1;
        asm volatile("" : "+v"(tm1_r));
#pragma unroll
        for (int c = 0; c < MAXC; ++c) {
            // with 16 chunks the row fills the registers: keep the chunks' LDS reads from
            // being moved ahead of the earlier chunks' work
            if (kExwInLds) __builtin_amdgcn_sched_barrier(0);
            if (c < nchunks) {
                const uint32_t ex = kExwInLds ? s_exw[c * kThreads + tid] : exw[c];
                uint32_t my_eq = s_peq[c * kWaves + wave] + (ex >> 16);
                // where the next selected entry goes: after the earlier ones above T and the
                // earlier ties taken
                uint32_t pos = s_pgt[c * kWaves + wave] + (ex & 0xFFFFu) + min(my_eq, r);
                const int base = c * kChunk + tid * 8 - lead;   // back to positions of the row
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const uint32_t code = pk_min_u16(pk_sub_sat_u16(data[c][j], tm1_r), kTwo);
                    if ((code & kOne) == 0) {           // no tie in this word: the common case
                        if (code & 0xFFFFu) emit(pos++, base + 2 * j);
                        if (code >> 16) emit(pos++, base + 2 * j + 1);
                    } else {
#pragma unroll
                        for (int h = 0; h < 2; ++h) {
                            const uint32_t ch = h ? (code >> 16) : (code & 0xFFFFu);
                            if (ch == 2u) {
                                emit(pos++, base + 2 * j + h);
                            } else if (ch == 1u) {
                                if (my_eq < r) emit(pos++, base + 2 * j + h);
                                ++my_eq;
                            }
                        }
                    }
                }
            }
        }
        __syncthreads();
        // this round's slots; the last round also fills the slots from n to k
        const int hi = (lo + kStage >= (uint32_t)n) ? k : (int)(lo + kStage);
        // k is a multiple of 4 for every budget the library produces; otherwise element stores
        if ((k & 3) == 0 && (reinterpret_cast<uintptr_t>(out) & 15) == 0) {
            for (int i = (int)lo + tid * 4; i < hi; i += kThreads * 4) {
                int4 v;
                v.x = (i + 0 < n) ? stage[i + 0 - lo] : fill;
                v.y = (i + 1 < n) ? stage[i + 1 - lo] : fill;
                v.z = (i + 2 < n) ? stage[i + 2 - lo] : fill;
                v.w = (i + 3 < n) ? stage[i + 3 - lo] : fill;
                *reinterpret_cast<int4*>(dst + i) = v;
                if (rdst) {   // k % 4 == 0 here; the rows tensor has the layout of the index tensor
                    int4 w;
                    w.x = to_cache_row(ro, row, v.x);
                    w.y = to_cache_row(ro, row, v.y);
                    w.z = to_cache_row(ro, row, v.z);
                    w.w = to_cache_row(ro, row, v.w);
                    if ((reinterpret_cast<uintptr_t>(ro.rows) & 15) == 0) {
                        *reinterpret_cast<int4*>(rdst + i) = w;
                    } else {
                        rdst[i] = w.x; rdst[i + 1] = w.y; rdst[i + 2] = w.z; rdst[i + 3] = w.w;
                    }
                }
            }
        } else {
            for (int i = (int)lo + tid; i < hi; i += kThreads) put(i, (i < n) ? stage[i - lo] : fill);
        }
        __syncthreads();   // the stage is free for the next round
    }
}


// --------------------------------------------------------------------------
// Long rows: the same radix select spread over several workgroups per row.
// Every workgroup owns one chunk of kSplitChunk entries of one row and holds it in registers
// (kSplitU 16-byte loads per thread, all in flight at once); per-row state lives in a
// caller-provided workspace:
//   hist1  [rows][2048]           coarse histogram (atomically merged)
//   arrive [rows][2]              workgroups of the row that have finished pass 1 / pass 2
//   sel    [rows][8]              {mode, b1, cum_above, T, r, n, len}
//   cinfo  [rows][chunks][34]     per chunk: fine histogram of bin b1 (32) and the
//                                 number of entries in bins above b1
//   coff   [rows][chunks][2]      per chunk: selected-greater / equal counts before it
// Launch sequence: zero -> hist1 -> [scan1] -> hist2 -> [scan2] -> write.  With few workgroups
// (a handful of very long rows: decode) the scan over a row's merged histogram is done by the
// row's last workgroup to finish its pass (FUSED: an arrival counter per row), which saves the
// two small launches; what one workgroup leaves for another of the same launch goes through
// device-coherent atomics, stores and loads.  With thousands of rows (prefill) the counter's
// round trip at the end of every workgroup costs more than the launches, so the scans stay
// kernels of their own.
// --------------------------------------------------------------------------
constexpr int kSplitU = 4;
constexpr int kSplitChunk = kSplitU * kChunk;   // 32768 entries per workgroup
constexpr int kSelWords = 8;
constexpr int kInfoWords = 34;
constexpr int kHistCopies = 4;
constexpr long long kSplitFusedMax = 2048;   // workgroups up to which the scans are fused into the passes

struct SplitWs {
    uint32_t* hist1;
    uint32_t* arrive;
    uint32_t* sel;
    uint32_t* cinfo;
    uint32_t* coff;
};

__device__ __forceinline__ uint32_t load_device_u32(const uint32_t* p) {
    return __hip_atomic_load(const_cast<uint32_t*>(p), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void store_device_u32(uint32_t* p, uint32_t v) {
    __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

__device__ __forceinline__ void row_params(const int* valid_len, const int* n_sel, int period,
                                           int uniform_len, int k, long long row, int& len, int& n) {
    const int pr = (int)(row % period);
    len = valid_len ? min(valid_len[pr], uniform_len) : uniform_len;
    n = n_sel ? n_sel[pr] : k;
    n = max(0, min(n, k));
}

// The chunk [c0, c1) of a row as order keys: thread t holds entries c0 + u*8192 + 8t .. +8 for
// u = 0..kSplitU-1 (every load instruction covers consecutive 16-byte pieces).
__device__ __forceinline__ void load_chunk(const uint16_t* __restrict__ src, bool aligned, int c0, int c1,
                                           uint32_t (&keys)[kSplitU][8], int (&nv)[kSplitU]) {
#pragma unroll
    for (int u = 0; u < kSplitU; ++u) {
        const int base = c0 + u * kChunk + (int)threadIdx.x * 8;
        nv[u] = 0;
        if (base < c1) nv[u] = load_keys(src, aligned, base, c1, keys[u]);
    }
}

// True in every thread of the row's last workgroup to get here (all of the row's `expected`
// workgroups call it once per pass).  The caller's device-coherent stores and atomics are
// waited for before the workgroup counts itself in.
__device__ __forceinline__ bool last_of_row(uint32_t* counter, int expected, int* s_flag) {
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    if (threadIdx.x == 0) {
        const uint32_t arrived = __hip_atomic_fetch_add(counter, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        *s_flag = (arrived == (uint32_t)(expected - 1));
    }
    __syncthreads();
    return *s_flag != 0;
}

__global__ __launch_bounds__(256) void topk_zero_kernel(uint32_t* p, long long n) {
    long long i = (long long)blockIdx.x * 256 + threadIdx.x;
    if (i < n) p[i] = 0;
}

// The bin that holds the n-th largest entry of a row whose coarse histogram is complete (all
// 1024 threads of a workgroup).
__device__ __forceinline__ void split_scan1(const uint32_t* gh, uint32_t* sel, int n, int len, uint32_t* s_wave) {
    const int tid = threadIdx.x;
    const int rb0 = kBins1 - 1 - 2 * tid;   // this thread's bins, in descending order
    const uint32_t h0 = load_device_u32(gh + rb0), h1 = load_device_u32(gh + rb0 - 1);
    uint32_t total;
    const uint32_t above0 = block_excl_scan(h0 + h1, s_wave, &total);
    const uint32_t above1 = above0 + h0;
    const uint32_t un = (uint32_t)n;
    if (above0 < un && un <= above0 + h0) {
        sel[1] = rb0; sel[2] = above0;
    } else if (above1 < un && un <= above1 + h1) {
        sel[1] = rb0 - 1; sel[2] = above1;
    }
    if (tid == 0) { sel[0] = 1; sel[5] = (uint32_t)n; sel[6] = (uint32_t)len; }
}

template <bool FUSED>
__global__ __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(8))) void topk_split_hist1_kernel(
    const uint16_t* __restrict__ scores, long long row_stride, int uniform_len,
    const int* __restrict__ valid_len, const int* __restrict__ n_sel, int period, int k, SplitWs ws) {
    __shared__ uint32_t s_hist[kHistCopies][kBins1];
    __shared__ uint32_t s_wave[kWaves];
    __shared__ int s_flag;
    const int tid = threadIdx.x;
    const long long row = blockIdx.y;
    int len, n;
    row_params(valid_len, n_sel, period, uniform_len, k, row, len, n);
    uint32_t* sel = ws.sel + row * kSelWords;
    if (len <= n || n == 0) {   // nothing to select: the write pass lists the row's head
        if (FUSED && blockIdx.x == 0 && tid == 0) { sel[0] = 0; sel[5] = (uint32_t)n; sel[6] = (uint32_t)len; }
        return;
    }
    const int c0 = blockIdx.x * kSplitChunk;
    if (c0 >= len) return;
    const int c1 = min(len, c0 + kSplitChunk);
    const uint16_t* src = scores + row * row_stride;
    const bool aligned = ((reinterpret_cast<uintptr_t>(src) & 15) == 0);
    uint32_t keys[kSplitU][8];
    int nv[kSplitU];
    load_chunk(src, aligned, c0, c1, keys, nv);
    for (int i = tid; i < kHistCopies * kBins1; i += kThreads) (&s_hist[0][0])[i] = 0;
    __syncthreads();
    // +0 (pooled probabilities underflow to it by the thousand) is not counted: its number is
    // the chunk's length minus the sum of the others.  The other entries go to one of four
    // copies of the histogram, chosen by the lane, which spreads the crowded bins.
    uint32_t* mine = s_hist[tid & (kHistCopies - 1)];
    uint32_t counted = 0;
#pragma unroll
    for (int u = 0; u < kSplitU; ++u)
#pragma unroll
        for (int e = 0; e < 8; ++e)
            if (e < nv[u] && keys[u][e] != 0x8000u) {
                atomicAdd(&mine[keys[u][e] >> 5], 1u);
                ++counted;
            }
#pragma unroll
    for (int o = 32; o >= 1; o >>= 1) counted += __shfl_xor(counted, o);
    if ((tid & 63) == 0) s_wave[tid >> 6] = counted;
    __syncthreads();
    uint32_t* gh = ws.hist1 + row * kBins1;
    for (int i = tid; i < kBins1; i += kThreads) {
        uint32_t c = 0;
#pragma unroll
        for (int j = 0; j < kHistCopies; ++j) c += s_hist[j][i];
        if (i == (int)(0x8000u >> 5)) {
            uint32_t all = 0;
#pragma unroll
            for (int w = 0; w < kWaves; ++w) all += s_wave[w];
            c += (uint32_t)(c1 - c0) - all;
        }
        if (c) atomicAdd(&gh[i], c);
    }
    if (!FUSED) return;
    const int nchunks = (len + kSplitChunk - 1) / kSplitChunk;
    if (!last_of_row(ws.arrive + 2 * row, nchunks, &s_flag)) return;
    split_scan1(gh, sel, n, len, s_wave);
}

__global__ __launch_bounds__(kThreads) void topk_split_scan1_kernel(
    int uniform_len, const int* __restrict__ valid_len, const int* __restrict__ n_sel, int period,
    int k, SplitWs ws) {
    __shared__ uint32_t s_wave[kWaves];
    const long long row = blockIdx.x;
    int len, n;
    row_params(valid_len, n_sel, period, uniform_len, k, row, len, n);
    uint32_t* sel = ws.sel + row * kSelWords;
    if (len <= n || n == 0) {
        if (threadIdx.x == 0) { sel[0] = 0; sel[5] = (uint32_t)n; sel[6] = (uint32_t)len; }
        return;
    }
    split_scan1(ws.hist1 + row * kBins1, sel, n, len, s_wave);
}

// From the chunks' fine histograms of a row: the threshold key T, the number r of entries equal
// to T that still fit, and every chunk's offsets into the output.  One wavefront, lane c for
// chunk c (64 chunks per round).
__device__ __forceinline__ void split_scan2(uint32_t* sel, const uint32_t* rinfo, uint32_t* off, int nchunks) {
    const int lane = threadIdx.x & 63;
    const uint32_t n = sel[5], b1 = sel[1];
    uint32_t h[32];
#pragma unroll
    for (int j = 0; j < 32; ++j) h[j] = 0;
    for (int cb = 0; cb < nchunks; cb += 64) {
        const int c = cb + lane;
        if (c < nchunks) {
#pragma unroll
            for (int j = 0; j < 32; ++j) h[j] += load_device_u32(rinfo + c * kInfoWords + j);
        }
    }
#pragma unroll
    for (int j = 0; j < 32; ++j)
#pragma unroll
        for (int o = 32; o >= 1; o >>= 1) h[j] += __shfl_xor(h[j], o);
    // the fine bin of the n-th largest entry, from the top (bin 0 takes whatever is left)
    uint32_t above = sel[2];
    int b2 = 0;
    bool found = false;
#pragma unroll
    for (int j = 31; j >= 1; --j) {
        if (!found) {
            if (above + h[j] >= n) { found = true; b2 = j; }
            else above += h[j];
        }
    }
    const uint32_t r = n - above;
    if (lane == 0) { sel[3] = (b1 << 5) | (uint32_t)b2; sel[4] = r; }
    // per-chunk counts of entries above T and equal to T, and their exclusive prefixes
    uint32_t gt_run = 0, eq_run = 0;
    for (int cb = 0; cb < nchunks; cb += 64) {
        const int c = cb + lane;
        uint32_t gt = 0, eq = 0;
        if (c < nchunks) {
            gt = load_device_u32(rinfo + c * kInfoWords + 32);
#pragma unroll
            for (int j = 0; j < 32; ++j) {
                const uint32_t v = load_device_u32(rinfo + c * kInfoWords + j);
                gt += (j > b2) ? v : 0u;
                eq += (j == b2) ? v : 0u;
            }
        }
        const uint32_t gi = wave_incl_scan(gt), ei = wave_incl_scan(eq);
        if (c < nchunks) { off[2 * c] = gt_run + gi - gt; off[2 * c + 1] = eq_run + ei - eq; }
        gt_run += __shfl(gi, 63);
        eq_run += __shfl(ei, 63);
    }
}

// Pass 2 of a chunk: the fine histogram of the threshold bin and the count of entries above it.
// The chunk's loads are issued for the row's full width before the row's state (its length,
// the threshold bin) has arrived, and cut down to the length afterwards.
template <bool FUSED>
__global__ __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(8))) void topk_split_hist2_kernel(
    const uint16_t* __restrict__ scores, long long row_stride, int uniform_len, int max_chunks, SplitWs ws) {
    __shared__ uint32_t s_hist2[32];
    __shared__ uint32_t s_gt1;
    __shared__ int s_flag;
    const int tid = threadIdx.x, lane = tid & 63;
    const long long row = blockIdx.y;
    uint32_t* sel = ws.sel + row * kSelWords;
    const int c0 = blockIdx.x * kSplitChunk;
    if (c0 >= uniform_len) return;
    const uint16_t* src = scores + row * row_stride;
    const bool aligned = ((reinterpret_cast<uintptr_t>(src) & 15) == 0);
    uint32_t keys[kSplitU][8];
    int nv[kSplitU];
    load_chunk(src, aligned, c0, min(uniform_len, c0 + kSplitChunk), keys, nv);
    const int len = (int)sel[6];
    if (sel[0] == 0 || c0 >= len) return;
    const uint32_t b1 = sel[1];
#pragma unroll
    for (int u = 0; u < kSplitU; ++u) nv[u] = max(0, min(nv[u], len - (c0 + u * kChunk + tid * 8)));
    if (tid < 32) s_hist2[tid] = 0;
    if (tid == 32) s_gt1 = 0;
    __syncthreads();
    uint32_t gt1 = 0, zeros = 0;
    const bool zero_bin = b1 == (0x8000u >> 5);   // uniform: the threshold lies among +0 and the smallest subnormals
#pragma unroll
    for (int u = 0; u < kSplitU; ++u)
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const bool in = e < nv[u];
            const uint32_t hb = keys[u][e] >> 5;
            if (zero_bin) {   // that many atomics on one address would serialise: a ballot per wavefront
                const bool zero = in && keys[u][e] == 0x8000u;
                zeros += (uint32_t)__popcll(__ballot(zero));
                if (in && !zero && hb == b1) atomicAdd(&s_hist2[keys[u][e] & 31u], 1u);
            } else if (in && hb == b1) {
                atomicAdd(&s_hist2[keys[u][e] & 31u], 1u);
            }
            gt1 += (in && hb > b1);
        }
#pragma unroll
    for (int o = 32; o >= 1; o >>= 1) gt1 += __shfl_xor(gt1, o);
    if (lane == 0 && gt1) atomicAdd(&s_gt1, gt1);
    if (lane == 0 && zeros) atomicAdd(&s_hist2[0], zeros);   // +0 is entry 0 of its bin
    __syncthreads();
    uint32_t* info = ws.cinfo + (row * max_chunks + blockIdx.x) * kInfoWords;
    if (tid < 32) store_device_u32(info + tid, s_hist2[tid]);
    if (tid == 32) store_device_u32(info + 32, s_gt1);
    if (!FUSED) return;
    const int nchunks = (len + kSplitChunk - 1) / kSplitChunk;
    if (!last_of_row(ws.arrive + 2 * row + 1, nchunks, &s_flag)) return;
    if (tid >= 64) return;
    split_scan2(sel, ws.cinfo + row * max_chunks * kInfoWords, ws.coff + row * max_chunks * 2, nchunks);
}

__global__ __launch_bounds__(64) void topk_split_scan2_kernel(int max_chunks, SplitWs ws) {
    const long long row = blockIdx.x;
    uint32_t* sel = ws.sel + row * kSelWords;
    if (sel[0] == 0) return;
    const int nchunks = ((int)sel[6] + kSplitChunk - 1) / kSplitChunk;
    split_scan2(sel, ws.cinfo + row * max_chunks * kInfoWords, ws.coff + row * max_chunks * 2, nchunks);
}

__global__ __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(8))) void topk_split_write_kernel(
    const uint16_t* __restrict__ scores, int* __restrict__ out, long long row_stride, int uniform_len,
    int k, int fill, int max_chunks, SplitWs ws, RowsOut ro) {
    static_assert(kSplitU * kWaves == 64, "one wavefront scans the (load, wavefront) totals");
    __shared__ uint32_t s_tot[kSplitU * kWaves];
    __shared__ uint32_t s_pre[kSplitU * kWaves];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const long long row = blockIdx.y;
    const uint32_t* sel = ws.sel + row * kSelWords;
    const int c0 = blockIdx.x * kSplitChunk;
    const uint16_t* src = scores + row * row_stride;
    const bool aligned = ((reinterpret_cast<uintptr_t>(src) & 15) == 0);
    // the chunk's loads go out before the row's state has arrived (cut down to its length below)
    uint32_t keys[kSplitU][8];
    int nv[kSplitU];
    load_chunk(src, aligned, c0, min(uniform_len, c0 + kSplitChunk), keys, nv);
    const int len = (int)sel[6];
    const int n = (int)sel[5];
    int* dst = out + row * (long long)k;
    int* rdst = ro.rows ? ro.rows + row * (long long)k : nullptr;
    auto put = [&](int slot, int pos) {
        dst[slot] = pos;
        if (rdst) rdst[slot] = to_cache_row(ro, row, pos);
    };
    if (blockIdx.x == 0) {
        if (sel[0] == 0) {
            for (int i = tid; i < k; i += kThreads) put(i, (i < n) ? i : fill);
            return;
        }
        for (int i = n + tid; i < k; i += kThreads) put(i, fill);
    }
    if (sel[0] == 0 || c0 >= len) return;
    const uint32_t T = sel[3];
    const uint32_t r = sel[4];
    const uint32_t* off = ws.coff + (row * max_chunks + blockIdx.x) * 2;
    const uint32_t gt_base = off[0], eq_base = off[1];
#pragma unroll
    for (int u = 0; u < kSplitU; ++u) nv[u] = max(0, min(nv[u], len - (c0 + u * kChunk + tid * 8)));
    // counts above / equal to T per (load, thread), packed; position order is (load, thread, entry)
    uint32_t cnt[kSplitU], inc[kSplitU];
#pragma unroll
    for (int u = 0; u < kSplitU; ++u) {
        uint32_t gt = 0, eq = 0;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            if (e < nv[u]) {
                gt += (keys[u][e] > T);
                eq += (keys[u][e] == T);
            }
        }
        cnt[u] = gt | (eq << 16);
        inc[u] = wave_incl_scan(cnt[u]);
        if (lane == 63) s_tot[u * kWaves + wave] = inc[u];
    }
    __syncthreads();
    if (wave == 0) {
        const uint32_t t = s_tot[lane];
        s_pre[lane] = wave_incl_scan(t) - t;
    }
    __syncthreads();
#pragma unroll
    for (int u = 0; u < kSplitU; ++u) {
        const uint32_t ex = s_pre[u * kWaves + wave] + inc[u] - cnt[u];
        uint32_t my_gt = gt_base + (ex & 0xFFFFu);
        uint32_t my_eq = eq_base + (ex >> 16);
        const int base = c0 + u * kChunk + tid * 8;
        // stores straight from the threads: staging the chunk's list in LDS for full-width stores
        // was measured slower (its two extra barriers cost more than the narrow stores)
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            if (e < nv[u]) {
                if (keys[u][e] > T) {
                    put(my_gt + min(my_eq, r), base + e);
                    ++my_gt;
                } else if (keys[u][e] == T) {
                    if (my_eq < r) put(my_gt + my_eq, base + e);
                    ++my_eq;
                }
            }
        }
    }
}

SplitWs carve_ws(void* workspace, int rows, int max_chunks) {
    SplitWs ws;
    uint32_t* p = reinterpret_cast<uint32_t*>(workspace);
    ws.hist1 = p;  p += (size_t)rows * kBins1;
    ws.arrive = p; p += (size_t)rows * 2;       // right behind hist1: one launch zeroes both
    ws.sel = p;    p += (size_t)rows * kSelWords;
    ws.cinfo = p;  p += (size_t)rows * max_chunks * kInfoWords;
    ws.coff = p;
    return ws;
}


// ---------------------------------------------------------------- rows ordered by score
// Reorders the first n entries of every row's position list by descending score, equal scores by
// ascending position: the order of torch.topk(...).indices.  A radix sort on the 16-bit order key
// in two stable passes (low byte, then high byte), one workgroup per row.  The keys are gathered
// once (the only dependent loads), then keys and positions move together between two buffers: in
// LDS for lists of up to kSortLdsEntries entries, in the caller's workspace for longer ones.  A
// wavefront owns a contiguous share of the list and walks it 64 entries at a time, the next
// step's entries already in flight; the lanes that hold the same digit find each other with
// eight ballots, so every entry's place follows from counters per (wavefront, digit) in LDS: no
// atomics, nothing depends on timing, and the input order (ascending position) survives among
// equal scores.
constexpr int kSortLdsEntries = 4096;

// lanes of the wavefront that are valid and hold the same 8-bit digit as this lane
__device__ __forceinline__ uint64_t digit_peers(uint32_t d, bool valid) {
    uint64_t peers = __ballot(valid);
#pragma unroll
    for (int b = 0; b < 8; ++b) {
        const bool bit = (d >> b) & 1u;
        const uint64_t set = __ballot(bit);
        peers &= bit ? set : ~set;
    }
    return valid ? peers : 0ull;
}

template <int WAVES, int LDS_N>
__global__ __launch_bounds__(WAVES * 64) void topk_sort_rows_kernel(
    const uint16_t* __restrict__ scores, int* __restrict__ idx, int* __restrict__ ws_pos,
    uint16_t* __restrict__ ws_keys, long long row_stride, int uniform_len,
    const int* __restrict__ valid_len, int period, int k) {
    constexpr int kT = WAVES * 64;
    static_assert(kT >= 256, "one thread per digit in the offset step");
    __shared__ uint32_t s_cnt[WAVES][256];
    __shared__ uint32_t s_wsum[4];
    __shared__ int s_pos[LDS_N > 0 ? 2 * LDS_N : 1];
    __shared__ uint16_t s_key[LDS_N > 0 ? 2 * LDS_N : 2];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const long long row = blockIdx.x;
    const int len = valid_len ? min(valid_len[(int)(row % period)], uniform_len) : uniform_len;
    const int n = max(0, min(k, len));   // entries beyond n name positions past the row's end: they stay
    if (n <= 1) return;
    const uint16_t* src = scores + row * row_stride;
    int* first = idx + row * (long long)k;
    int *pos_a, *pos_b;
    uint16_t *key_a, *key_b;
    if constexpr (LDS_N > 0) {
        pos_a = s_pos; pos_b = s_pos + LDS_N; key_a = s_key; key_b = s_key + LDS_N;
    } else {
        pos_a = first; pos_b = ws_pos + row * (long long)k;
        key_a = ws_keys + row * 2ll * k; key_b = key_a + k;
    }
    for (int i = tid; i < n; i += kT) {
        const int pos = first[i];
        if constexpr (LDS_N > 0) pos_a[i] = pos;
        key_a[i] = (uint16_t)order_key(src[pos]);
    }
    __syncthreads();

    const int seg = (n + kT - 1) / kT * 64;
    const int s0 = min(n, wave * seg), s1 = min(n, s0 + seg);
    const uint64_t below = (1ull << lane) - 1ull;
    volatile uint32_t* mine = s_cnt[wave];

    for (int pass = 0; pass < 2; ++pass) {
        const int* from_pos = pass ? pos_b : pos_a;
        const uint16_t* from_key = pass ? key_b : key_a;
        int* to_pos = pass ? first : pos_b;
        const int shift = 8 * pass;
        for (int i = tid; i < WAVES * 256; i += kT) (&s_cnt[0][0])[i] = 0;
        __syncthreads();
        // how many entries of each digit this wavefront's share holds
        {
            bool valid = s0 + lane < s1;
            uint32_t key = valid ? from_key[s0 + lane] : 0u;
            for (int base = s0; base < s1; base += 64) {
                const bool nvalid = base + 64 + lane < s1;
                const uint32_t nkey = nvalid ? from_key[base + 64 + lane] : 0u;
                const uint32_t d = (key >> shift) & 255u;
                const uint64_t peers = digit_peers(d, valid);
                if (valid && (peers & below) == 0) mine[d] += (uint32_t)__popcll(peers);
                valid = nvalid; key = nkey;
            }
        }
        __syncthreads();
        // thread t < 256 owns digit 255 - t: the entries with a larger digit come first, then the
        // earlier shares' entries of the same digit
        {
            const int d = 255 - (tid & 255);
            uint32_t c[WAVES], total = 0;
            if (tid < 256) {
#pragma unroll
                for (int w = 0; w < WAVES; ++w) { c[w] = s_cnt[w][d]; total += c[w]; }
            }
            const uint32_t inc = wave_incl_scan(total);
            if (tid < 256 && lane == 63) s_wsum[wave] = inc;
            __syncthreads();
            if (tid < 256) {
                uint32_t start = inc - total;
#pragma unroll
                for (int w = 0; w < 4; ++w) if (w < wave) start += s_wsum[w];
#pragma unroll
                for (int w = 0; w < WAVES; ++w) { s_cnt[w][d] = start; start += c[w]; }
            }
        }
        __syncthreads();
        // place: the counter of a digit is read by all its lanes, then advanced by the first of them
        {
            bool valid = s0 + lane < s1;
            int pos = valid ? from_pos[s0 + lane] : 0;
            uint32_t key = valid ? from_key[s0 + lane] : 0u;
            for (int base = s0; base < s1; base += 64) {
                const bool nvalid = base + 64 + lane < s1;
                const int npos = nvalid ? from_pos[base + 64 + lane] : 0;
                const uint32_t nkey = nvalid ? from_key[base + 64 + lane] : 0u;
                const uint32_t d = (key >> shift) & 255u;
                const uint64_t peers = digit_peers(d, valid);
                const uint32_t rank = (uint32_t)__popcll(peers & below);
                const uint32_t at = valid ? mine[d] : 0u;
                if (valid && rank == 0) mine[d] = at + (uint32_t)__popcll(peers);
                if (valid) {
                    to_pos[at + rank] = pos;
                    if (pass == 0) key_b[at + rank] = (uint16_t)key;
                }
                valid = nvalid; pos = npos; key = nkey;
            }
        }
        __syncthreads();   // the second pass reads what other wavefronts placed
    }
}

}  // namespace

int topk_max_register_row() { return 16 * kChunk; }

long long topk_split_workspace_bytes(int rows, long long row_len) {
    if (row_len < kSplitMinLen || rows > kSplitMaxRows) return 0;
    const long long chunks = (row_len + kSplitChunk - 1) / kSplitChunk;
    return 4ll * rows * (kBins1 + 2 + kSelWords + chunks * (kInfoWords + 2));
}

namespace {
RowsOut rows_out(const TopkRows* tr) {
    RowsOut ro{};
    if (tr && tr->out_rows) {
        ro.rows = tr->out_rows; ro.block_table = tr->block_table; ro.max_pages = tr->max_pages;
        ro.page_shift = tr->page_shift; ro.rows_per_seq = tr->rows_per_seq;
    }
    return ro;
}
}  // namespace

hipError_t launch_topk_split(const half_t* scores, int* out_idx, int rows, long long row_stride,
                             int max_len, int uniform_len, const int* valid_len, const int* n_sel,
                             int period, int k, int fill, void* workspace, const TopkRows* tr,
                             hipStream_t stream) {
    if (rows == 0) return hipSuccess;
    // The chunk workgroups write their selections to scattered slots, where a block-table lookup
    // per element would sit in the middle of the compaction (+40 us on four rows of 131072 to
    // 524288 entries); the long-row path translates in a launch of its own at the end instead.
    const RowsOut ro{};
    const int max_chunks = (max_len + kSplitChunk - 1) / kSplitChunk;
    SplitWs ws = carve_ws(workspace, rows, max_chunks);
    const uint16_t* src = reinterpret_cast<const uint16_t*>(scores);
    const long long nz = (long long)rows * (kBins1 + 2);   // histograms and arrival counters
    hipLaunchKernelGGL(topk_zero_kernel, dim3((unsigned)((nz + 255) / 256)), dim3(256), 0, stream,
                       ws.hist1, nz);
    dim3 grid(max_chunks, rows);
    // few workgroups: the scans ride on the histogram passes; many: launches of their own
    const bool fused = (long long)rows * max_chunks <= kSplitFusedMax;
    if (fused) {
        hipLaunchKernelGGL(topk_split_hist1_kernel<true>, grid, dim3(kThreads), 0, stream, src, row_stride,
                           uniform_len, valid_len, n_sel, period, k, ws);
        hipLaunchKernelGGL(topk_split_hist2_kernel<true>, grid, dim3(kThreads), 0, stream, src, row_stride,
                           uniform_len, max_chunks, ws);
    } else {
        hipLaunchKernelGGL(topk_split_hist1_kernel<false>, grid, dim3(kThreads), 0, stream, src, row_stride,
                           uniform_len, valid_len, n_sel, period, k, ws);
        hipLaunchKernelGGL(topk_split_scan1_kernel, dim3(rows), dim3(kThreads), 0, stream, uniform_len,
                           valid_len, n_sel, period, k, ws);
        hipLaunchKernelGGL(topk_split_hist2_kernel<false>, grid, dim3(kThreads), 0, stream, src, row_stride,
                           uniform_len, max_chunks, ws);
        hipLaunchKernelGGL(topk_split_scan2_kernel, dim3(rows), dim3(64), 0, stream, max_chunks, ws);
    }
    hipLaunchKernelGGL(topk_split_write_kernel, grid, dim3(kThreads), 0, stream, src, out_idx,
                       row_stride, uniform_len, k, fill, max_chunks, ws, ro);
    if (tr && tr->out_rows)
        return launch_translate_indices(out_idx, tr->out_rows, tr->block_table, rows / tr->rows_per_seq,
                                        (long long)tr->rows_per_seq * k, tr->max_pages, tr->page_shift,
                                        tr->max_pages << tr->page_shift, stream);
    return hipGetLastError();
}

hipError_t launch_topk(const half_t* scores, int* out_idx, int rows, long long row_stride,
                       int uniform_len, const int* valid_len, const int* n_sel, int period, int k,
                       int fill, const TopkRows* tr, hipStream_t stream) {
    if (rows == 0) return hipSuccess;
    const RowsOut ro = rows_out(tr);
    const uint16_t* src = reinterpret_cast<const uint16_t*>(scores);
    // rows of a tensor that starts 16-byte aligned and that fit the register file of a workgroup
    // are selected from registers (rows that start off a boundary bring up to 7 slots in front);
    // anything else streams the row three times
    const bool aligned_rows = (reinterpret_cast<uintptr_t>(scores) & 15) == 0;
    const int slots = uniform_len + (row_stride % 8 != 0 ? 7 : 0);
    if (aligned_rows && slots <= 4 * kChunk)
        hipLaunchKernelGGL(topk_select_reg_kernel<4>, dim3(rows), dim3(kThreads), 0, stream, src, out_idx,
                           row_stride, uniform_len, valid_len, n_sel, period, k, fill, ro);
    else if (aligned_rows && slots <= 8 * kChunk)
        hipLaunchKernelGGL(topk_select_reg_kernel<8>, dim3(rows), dim3(kThreads), 0, stream, src, out_idx,
                           row_stride, uniform_len, valid_len, n_sel, period, k, fill, ro);
    else if (aligned_rows && slots <= 16 * kChunk)
        hipLaunchKernelGGL(topk_select_reg_kernel<16>, dim3(rows), dim3(kThreads), 0, stream, src, out_idx,
                           row_stride, uniform_len, valid_len, n_sel, period, k, fill, ro);
    else
        hipLaunchKernelGGL(topk_select_kernel, dim3(rows), dim3(kThreads), 0, stream, src, out_idx,
                           row_stride, uniform_len, valid_len, n_sel, period, k, fill, ro);
    return hipGetLastError();
}

long long topk_sort_workspace_bytes(int rows, int k) {
    return k <= kSortLdsEntries ? 0 : 8ll * rows * k;   // positions (4 bytes) and two key buffers (2 + 2)
}

hipError_t launch_topk_sort_rows(const half_t* scores, int* idx, void* workspace, int rows,
                                 long long row_stride, int uniform_len, const int* valid_len,
                                 int period, int k, hipStream_t stream) {
    if (rows == 0) return hipSuccess;
    const uint16_t* src = reinterpret_cast<const uint16_t*>(scores);
    if (k <= kSortLdsEntries) {
        hipLaunchKernelGGL((topk_sort_rows_kernel<4, kSortLdsEntries>), dim3(rows), dim3(256), 0, stream, src, idx,
                           (int*)nullptr, (uint16_t*)nullptr, row_stride, uniform_len, valid_len, period, k);
    } else {
        int* ws_pos = static_cast<int*>(workspace);
        uint16_t* ws_keys = reinterpret_cast<uint16_t*>(ws_pos + (long long)rows * k);
        hipLaunchKernelGGL((topk_sort_rows_kernel<16, 0>), dim3(rows), dim3(1024), 0, stream, src, idx, ws_pos,
                           ws_keys, row_stride, uniform_len, valid_len, period, k);
    }
    return hipGetLastError();
}

}  // namespace kascade
