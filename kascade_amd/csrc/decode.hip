// Decode-step attention kernels for gfx950: bandwidth-bound split-K streaming of
// K/V rows (gathered through a top-k index list, or dense), log-sum merge, and
// pooled post-softmax scores for anchor layers.
//
// Work decomposition (one launch = all sequences, KV heads and splits):
//   grid  (num_split, G, B), 256 threads = 4 wavefronts.
//   A wavefront is four row-groups of 16 lanes; lane d-slice dl = lane%16 owns
//   halves [8*dl, 8*dl+8) of every row it touches, so one 16-byte load per lane
//   fetches four complete 256-byte K (or V) rows per wavefront instruction.
//   Each row-group keeps an independent online-softmax state (max, sum, 4x8
//   output accumulators per lane); the 16 states of a workgroup are merged once
//   at the end, the splits by the combine kernel.
//   q.k dot products run on v_dot2_f32_f16 + a 4-step DPP row reduction; p.v on
//   fp32 FMAs.  2 flop/byte is far below the machine balance, so no MFMA here.
#include "decode.h"

#include <type_traits>

namespace kascade {

namespace {

constexpr int kThreads = 256;
// The instruction scheduler otherwise sinks every prefetch load down to its first use (to save
// registers), which serialises load -> wait -> use and removes all memory-level parallelism.
#define KASCADE_SCHED_FENCE() __builtin_amdgcn_sched_barrier(0)
#ifndef KASCADE_DECODE_UNROLL
#define KASCADE_DECODE_UNROLL 4
#endif
#ifndef KASCADE_GATHER_MFMA
#define KASCADE_GATHER_MFMA 1
#endif
#ifndef KASCADE_DENSE_MFMA
#define KASCADE_DENSE_MFMA 1
#endif
constexpr int kUnroll = KASCADE_DECODE_UNROLL;  // rows per row-group per iteration
constexpr int kRowsPerIter = 16 * kUnroll;    // rows per workgroup iteration (128)
constexpr int kScoreBatches = 16;             // batches between two score flushes (anchor mode)
constexpr int kStripRows = 16 * kScoreBatches;  // rows a wavefront owns per super-iteration
constexpr int kSubChunk = 2048;               // rows whose physical ids are staged in LDS at once
// Raw scores travel from the anchor pass to the pooling kernel in a compact form: per head a row of
// scores_stride floats holds, in its first half, one 16-bit code per token and, behind them, one
// fp32 reference per granule of 64 tokens (the granule's largest scaled score, log2 domain).
// code = round((reference - score*scale) * 2048), i.e. steps of 2^-11 in the exponent: the
// probability recovered from it is within 1.7e-4 (a third of an fp16 step) of the exact one, and
// a code of 65534 steps (2^-32 of the granule's maximum, itself at most the row's log-sum) is far
// below what survives the pooled sum's fp16 rounding.  65535 marks a masked position.  Splits
// start at multiples of 64 tokens, so a granule belongs to one workgroup.  Half the bytes of fp32
// scores: their write-back to HBM, interleaved with the K stream, costs several times its size.
constexpr float kScoreSteps = 2048.f;
constexpr uint32_t kScoreNone = 65535u;

// Device-coherent accesses (relaxed atomics at agent scope) for data that one workgroup writes
// and another workgroup of the same launch reads.
__device__ __forceinline__ void store_device(float* p, float v) {
    __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void store_device2(float* p, float a, float b) {
    union { float f[2]; unsigned long long u; } x;
    x.f[0] = a; x.f[1] = b;
    __hip_atomic_store(reinterpret_cast<unsigned long long*>(p), x.u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ float load_device(const float* p) {
    return __hip_atomic_load(const_cast<float*>(p), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ float2 load_device2(const float* p) {
    union { float f[2]; unsigned long long u; } x;
    x.u = __hip_atomic_load(reinterpret_cast<unsigned long long*>(const_cast<float*>(p)), __ATOMIC_RELAXED,
                            __HIP_MEMORY_SCOPE_AGENT);
    return make_float2(x.f[0], x.f[1]);
}

struct alignas(16) MergeState {  // one per wavefront after the in-wave merge
    float m[kGroupSize];
    float l[kGroupSize];
    float acc[kGroupSize][kDim];
};

template <bool GATHER, bool WITH_V, bool WRITE_SCORES>
__global__ __launch_bounds__(WRITE_SCORES ? kThreads + 64 : kThreads) __attribute__((amdgpu_waves_per_eu(3)))
void decode_split_kernel(DecodeParams p) {
    __shared__ int s_row[GATHER ? kSubChunk : 1];
    __shared__ MergeState s_merge[4];
    __shared__ int s_last;
    __shared__ int s_found;   // gather mode: sub-chunk whose index list names the newest token
    // anchor mode: two buffers of four wavefront strips (4 heads x kStripRows raw scores)
    __shared__ __attribute__((aligned(16))) float s_sc[WRITE_SCORES ? 2 : 1][WRITE_SCORES ? 4 : 1][kGroupSize][WRITE_SCORES ? kStripRows : 4];
    // anchor pass without output: per wavefront one tile of 16 K rows on its way into the matrix layout
    constexpr int kKtStride = 136;   // halves per K row (128 + 8): rows 272 bytes apart
    constexpr int kVtStride = 144;   // halves per V row: 288 bytes, conflict-free for the transposing reads
    constexpr bool kGatherMfma = GATHER && (KASCADE_GATHER_MFMA != 0);
    constexpr bool kDenseMfma = !GATHER && ((!WITH_V && WRITE_SCORES) || (KASCADE_DENSE_MFMA != 0));
    constexpr bool kTiles = kDenseMfma || kGatherMfma;
    constexpr bool kTilesV = kTiles && WITH_V;
    __shared__ __attribute__((aligned(16))) half_t s_kt[kTiles ? 4 : 1][kTiles ? 16 * kKtStride : 8];
    __shared__ __attribute__((aligned(16))) half_t s_vt[kTilesV ? 4 : 1][kTilesV ? 16 * kVtStride : 8];

    const int g = blockIdx.x;       // the 8 KV heads of one token range are adjacent in dispatch order
    const int split = blockIdx.y;
    const int b = blockIdx.z;
    const int tid = threadIdx.x;
    const int wave = tid >> 6;
    const int lane = tid & 63;
    const int rg = lane >> 4;   // row group within the wavefront
    const int dl = lane & 15;   // 16-byte slice of the 256-byte row

    int seqlen = p.seqlens ? p.seqlens[b] : p.kv_stride_tokens;
    // a length beyond what the block table covers must not index past the table
    if (p.block_table) seqlen = min(seqlen, p.max_pages << p.page_shift);
    seqlen = max(seqlen, 0);
    int n;  // rows this (b, g) pair attends to
    if (GATHER) {
        if (p.topk_percent > 0.f) {
            long long fl = (long long)floor((double)p.topk_percent * (double)seqlen / 100.0);
            n = (int)(((fl + 127) / 128) * 128);
        } else {
            n = p.topk;
        }
        n = min(n, p.topk);
        if (p.seqlens) n = min(n, seqlen);   // never more rows than the sequence holds
    } else {
        n = seqlen;
    }
    // contiguous range of this split; every split covers rows_per_split rows, sequences
    // shorter than num_split*rows_per_split leave their last splits empty
    const long long r0l = (long long)split * p.rows_per_split;
    const int r0 = (int)min((long long)n, r0l);
    const int r1 = (int)min((long long)n, r0l + p.rows_per_split);

    // Fused append.  With k_new/v_new the K/V rows of the newest token (position seqlen-1)
    // arrive beside the cache and have to end up in it.  A workgroup that is going to read that
    // row writes it first and waits for its own stores at a barrier; what other workgroups write
    // there is the same bytes.  `write_newest` is uniform over the workgroup.
    const int newest = seqlen - 1;
    auto write_newest = [&]() {
        if (tid < 32) {
            const int part = tid >> 4, c = tid & 15;
            size_t off;
            if (p.block_table) {
                const int pg = p.block_table[(size_t)b * p.max_pages + (newest >> p.page_shift)];
                const int row = (pg << p.page_shift) + (newest & ((1 << p.page_shift) - 1));
                off = (size_t)row * (kGroups * kDim) + (size_t)g * kDim + c * 8;
            } else {
                off = (size_t)b * p.kv_stride_b + (size_t)g * p.kv_stride_h + (size_t)newest * p.kv_stride_l + c * 8;
            }
            const half_t* src = (part ? p.v_new : p.k_new) + ((size_t)b * kGroups + g) * kDim + c * 8;
            half_t* dst = (part ? p.v_cache : p.k_cache) + off;
            *reinterpret_cast<uint4_t*>(dst) = ld_global_16(src);
        }
    };
    if (p.k_new != nullptr && newest >= 0) {
        if (!GATHER) {
            if (newest >= r0 && newest < r1) {   // the split that streams the newest row
                write_newest();
                __syncthreads();
            }
        } else if (split == 0) {
            write_newest();   // lists that do not name the newest token still leave it cached
        }
    }
    if (GATHER && tid == 0) s_found = -1;

    // q fragments: 4 heads x 8 halves of this lane's d-slice
    Pack16 qf[kGroupSize];
#pragma unroll
    for (int h = 0; h < kGroupSize; ++h)
        qf[h].u = ld_global_16(p.Q + ((size_t)b * kHeads + g * kGroupSize + h) * kDim + dl * 8);

    float m[kGroupSize], l[kGroupSize], acc[kGroupSize][8];
#pragma unroll
    for (int h = 0; h < kGroupSize; ++h) {
        m[h] = -INFINITY;
        l[h] = 0.f;
#pragma unroll
        for (int d = 0; d < 8; ++d) acc[h][d] = 0.f;
    }

    const int* idx_row = nullptr;
    if (GATHER) idx_row = p.idx + ((size_t)b * kGroups + p.head_map[g]) * p.topk;
    const int page_mask = (1 << p.page_shift) - 1;
    // Element offset of (token row r, this head, this lane's slice): paged rows are physical rows
    // of [P*page,G,D]; without a table rows are token numbers of sequence b behind the caller's
    // (batch, token, head) strides, so a head-major cache is read in place.
    const size_t head_off = (size_t)g * kDim + dl * 8;
    const size_t strided_off = (size_t)b * p.kv_stride_b + (size_t)g * p.kv_stride_h + dl * 8;
    const unsigned stride_l = p.kv_stride_l;

    struct Batch {
        Pack16 k[kUnroll];
        Pack16 v[kUnroll];
    };
    // A wavefront covers 4*kUnroll consecutive rows of an iteration: row = it + wave*4U + u*4 + rg.
    // `rows` are physical row numbers (page*page_size + slot, or b*stride + token).
    auto issue_loads = [&](auto paged_tag, const int (&rows)[kUnroll], Batch& bt) {
        constexpr bool PAGED = decltype(paged_tag)::value;
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
            const size_t off = PAGED ? (size_t)rows[u] * (kGroups * kDim) + head_off
                                     : (size_t)(unsigned)rows[u] * stride_l + strided_off;
            // every K/V row is read once per launch: non-temporal loads keep the stream from
            // displacing what the launch does want cached (index lists, block table, the raw
            // scores an anchor pass writes for the kernels that follow) -- measured -12 % on the
            // gather, -7 % on the anchor passes
            bt.k[u].u = __builtin_nontemporal_load(reinterpret_cast<const uint4_t*>(p.K + off));
            if (WITH_V) bt.v[u].u = __builtin_nontemporal_load(reinterpret_cast<const uint4_t*>(p.V + off));
        }
    };
    // Straight-line on purpose (no early exit, loads never skipped): a branch between issuing
    // a batch and consuming it makes the compiler wait for every outstanding load.
    // rbase: first row (relative to c0) of this lane's row-group in the batch, rows rbase + 4u.
    auto compute_batch = [&](int rbase, int cn, int c0, int phase, int buf, const Batch& bt) {
        float s[kUnroll][kGroupSize];
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
            const bool valid = (rbase + u * 4) < cn;
#pragma unroll
            for (int h = 0; h < kGroupSize; ++h) {
                float d = dot8(bt.k[u], qf[h], 0.f);
                d = row16_sum(d);
                s[u][h] = valid ? d : -INFINITY;
            }
        }
        if (WRITE_SCORES) {
            // Raw scores are parked in LDS strips (per wavefront: 4 heads x kStripRows tokens)
            // and written to HBM by a fifth wavefront that streams nothing.  A store issued by
            // a streaming wavefront costs it dearly: loads and stores complete in order on one
            // counter, so every younger K/V load is held back until the store is acknowledged.
            static_assert(!WRITE_SCORES || kUnroll == 4, "score staging assumes 4 rows per row-group");
            const int usel = dl & 3, hsel = dl >> 2;
            float w[kGroupSize];
#pragma unroll
            for (int h = 0; h < kGroupSize; ++h) {
                w[h] = s[0][h];
#pragma unroll
                for (int u = 1; u < kUnroll; ++u) w[h] = (usel == u) ? s[u][h] : w[h];
            }
            float val = w[0];
#pragma unroll
            for (int h = 1; h < kGroupSize; ++h) val = (hsel == h) ? w[h] : val;
            s_sc[buf][wave][hsel][phase * 16 + usel * 4 + rg] = val;
        }
#pragma unroll
        for (int h = 0; h < kGroupSize; ++h) {
            float mx = m[h];
#pragma unroll
            for (int u = 0; u < kUnroll; ++u) mx = fmaxf(mx, s[u][h]);
            const float mref = (mx == -INFINITY) ? 0.f : mx * kScaleLog2;
            const float corr = fast_exp2(m[h] * kScaleLog2 - mref);  // m=-inf -> 0
            m[h] = mx;
            float ps[kUnroll];
            float sum = 0.f;
#pragma unroll
            for (int u = 0; u < kUnroll; ++u) {
                ps[u] = fast_exp2(s[u][h] * kScaleLog2 - mref);
                sum += ps[u];
            }
            l[h] = l[h] * corr + sum;
            if (WITH_V) {
#pragma unroll
                for (int d = 0; d < 8; ++d) {
                    float a = acc[h][d] * corr;
#pragma unroll
                    for (int u = 0; u < kUnroll; ++u) a = fmaf(ps[u], (float)bt.v[u].h[d], a);
                    acc[h][d] = a;
                }
            }
        }
    };

    // Writer wavefront of the anchor passes: stores the four strips of super-iteration `sup`
    // (buffer sup & 1) in the compact score format (see kScoreSteps): per instruction one
    // (strip, head) row of 256 tokens, 16 lanes per granule of 64 tokens, four tokens per lane;
    // 128 contiguous bytes per granule plus its reference value.
    auto flush_scores = [&](int sup) {
        const int cn = r1 - r0;
        constexpr int kVecPerStrip = kGroupSize * kStripRows / 4;   // float4 per strip
#pragma unroll 4
        for (int i = 0; i < 4 * kVecPerStrip / 64; ++i) {
            const int idx = i * 64 + lane;
            const int w = idx / kVecPerStrip, rem = idx % kVecPerStrip;
            const int h = rem / (kStripRows / 4), t4 = (rem % (kStripRows / 4)) * 4;
            float4_t v = *reinterpret_cast<const float4_t*>(&s_sc[sup & 1][w][h][t4]);
            const int r = sup * (4 * kStripRows) + w * kStripRows + t4;
#pragma unroll
            for (int e = 0; e < 4; ++e)      // strip positions past the range were never filled
                v[e] = (r + e < cn) ? v[e] : -INFINITY;
            const float mx = row16_max(fmaxf(fmaxf(v[0], v[1]), fmaxf(v[2], v[3])));
            const float base = (mx == -INFINITY) ? 0.f : mx;
            uint32_t q[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const float d = (base - v[e]) * (kScaleLog2 * kScoreSteps);      // >= 0, +inf if masked
                q[e] = (v[e] == -INFINITY) ? kScoreNone : (uint32_t)fminf(rintf(d), (float)(kScoreNone - 1));
            }
            float* row = p.scores + ((size_t)b * kHeads + g * kGroupSize + h) * p.scores_stride;
            uint16_t* dst = reinterpret_cast<uint16_t*>(row) + r0 + r;
            if (r + 3 < cn) {
                *reinterpret_cast<uint2*>(dst) = make_uint2(q[0] | (q[1] << 16), q[2] | (q[3] << 16));
            } else {
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    if (r + e < cn) dst[e] = (uint16_t)q[e];
            }
            if ((lane & 15) == 0 && r < cn) row[p.scores_stride / 2 + ((r0 + r) >> 6)] = base * kScaleLog2;
        }
    };

    if constexpr (kGatherMfma) {
        // Gathered rows on the matrix unit.  Tiles of 16 rows per wavefront: rows are loaded as
        // 16 lanes x 16 bytes each (four rows per instruction, K and V), pass through
        // wavefront-private LDS tiles, and S^T = K Q^T (16 keys x 4 of 16 columns, contraction
        // over d, v_mfma_f32_16x16x32_f16) leaves every lane with four keys of one column: the
        // B-operand layout of O^T += V^T P^T (v_mfma_f32_16x16x16_f16, contraction over the 16
        // keys), whose A operand comes out of the row-major V tile through the transposing LDS
        // read.  One running maximum per column (two cross-lane exchanges per tile); ~10 vector
        // instructions per row instead of ~110.
        const int col = lane & 15, dq = lane >> 4;
        half8_t qb[4];
#pragma unroll
        for (int st = 0; st < 4; ++st) {
            Pack16 t;
            t.u = ld_global_16(p.Q + ((size_t)b * kHeads + g * kGroupSize + (col & 3)) * kDim + 32 * st + 8 * dq);
            if (col >= kGroupSize) t.u = uint4_t{0, 0, 0, 0};
            qb[st] = t.h8;
        }
        float mcol = -INFINITY, lcol = 0.f;
        float4_t oacc[8];
#pragma unroll
        for (int blk = 0; blk < 8; ++blk) oacc[blk] = float4_t{0.f, 0.f, 0.f, 0.f};
        half_t* kt = &s_kt[wave][0];
        half_t* vt = &s_vt[wave][0];
        struct Tile {
            uint4_t k[4], v[4];
        };
        auto run = [&](auto paged_tag) {
        constexpr bool PAGED = decltype(paged_tag)::value;
        for (int c0 = r0; c0 < r1; c0 += kSubChunk) {
            const int cn = min(kSubChunk, r1 - c0);
            __syncthreads();
            for (int i = tid; i < cn; i += kThreads) {
                int tok = idx_row[c0 + i];
                tok = max(0, min(tok, seqlen - 1));   // a corrupt index must not leave the sequence
                if (tok == newest) s_found = c0;
                int row;
                if (p.block_table) {
                    int pg = p.block_table[(size_t)b * p.max_pages + (tok >> p.page_shift)];
                    row = (pg << p.page_shift) + (tok & page_mask);
                } else {
                    row = tok;
                }
                s_row[i] = row;
            }
            __syncthreads();
            if (p.k_new != nullptr && s_found == c0) {   // c0 differs per sub-chunk: no reset needed
                write_newest();
                __syncthreads();
            }
            // tile t: rows [16t, 16t+16) of the sub-chunk; lane (dq, col) loads chunk col of rows 4i + dq
            auto issue = [&](int t, Tile& tb) {
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const int row = s_row[min(16 * t + 4 * i + dq, cn - 1)];   // past the end: clamped, masked later
                    const size_t off = PAGED ? ((size_t)row * kGroups + g) * kDim + 8 * col
                                             : (size_t)b * p.kv_stride_b + (size_t)g * p.kv_stride_h +
                                                   (size_t)(unsigned)row * stride_l + 8 * col;
                    tb.k[i] = __builtin_nontemporal_load(reinterpret_cast<const uint4_t*>(p.K + off));
                    tb.v[i] = __builtin_nontemporal_load(reinterpret_cast<const uint4_t*>(p.V + off));
                }
            };
            auto compute = [&](int t, const Tile& tb) {
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    *reinterpret_cast<uint4_t*>(&kt[(4 * i + dq) * kKtStride + 8 * col]) = tb.k[i];
                    *reinterpret_cast<uint4_t*>(&vt[(4 * i + dq) * kVtStride + 8 * col]) = tb.v[i];
                }
                __builtin_amdgcn_wave_barrier();   // the reads below are other lanes' writes (same wavefront: in order)
                float4_t sc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int st = 0; st < 4; ++st) {
                    const half8_t a = *reinterpret_cast<const half8_t*>(&kt[col * kKtStride + 32 * st + 8 * dq]);
                    sc = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, qb[st], sc, 0, 0, 0);
                }
                // sc[e] = q_col . k of row 16t + 4*dq + e
                const int key0 = 16 * t + 4 * dq;
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    if (key0 + e >= cn) sc[e] = -INFINITY;
                float mx = fmaxf(fmaxf(sc[0], sc[1]), fmaxf(sc[2], sc[3]));
                mx = fmaxf(mx, __shfl_xor(mx, 16));
                mx = fmaxf(mx, __shfl_xor(mx, 32));
                mx = fmaxf(mx, mcol);
                const float mref = (mx == -INFINITY) ? 0.f : mx * kScaleLog2;
                const float corr = fast_exp2(mcol * kScaleLog2 - mref);
                mcol = mx;
                float pe[4];
                float sum = 0.f;
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    pe[e] = fast_exp2(sc[e] * kScaleLog2 - mref);
                    sum += pe[e];
                }
                lcol = lcol * corr + sum;
                if (__any(corr != 1.f)) {
#pragma unroll
                    for (int blk = 0; blk < 8; ++blk) oacc[blk] *= corr;
                }
                const half4_t pb = {(half_t)pe[0], (half_t)pe[1], (half_t)pe[2], (half_t)pe[3]};
                typedef short short4_t __attribute__((ext_vector_type(4)));
                // lane (dq, col) points at V[row 4dq + col/4][16blk + 4(col%4), +4) and receives
                // V[rows 4dq .. 4dq+3][16blk + col]
                const half_t* vp = &vt[(4 * dq + (col >> 2)) * kVtStride + 4 * (col & 3)];
#pragma unroll
                for (int blk = 0; blk < 8; ++blk) {
                    const short4_t raw = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                        (__attribute__((address_space(3))) short4_t*)(vp + 16 * blk));
                    oacc[blk] = __builtin_amdgcn_mfma_f32_16x16x16f16(__builtin_bit_cast(half4_t, raw), pb, oacc[blk], 0, 0, 0);
                }
                __builtin_amdgcn_wave_barrier();
            };
            const int ntiles = (cn + 15) / 16;
            Tile ta, tb;
            issue(wave, ta);
            for (int t = wave; t < ntiles; t += 8) {
                issue(t + 4, tb);
                KASCADE_SCHED_FENCE();
                compute(t, ta);
                KASCADE_SCHED_FENCE();
                issue(t + 8, ta);
                KASCADE_SCHED_FENCE();
                compute(t + 4, tb);
                KASCADE_SCHED_FENCE();
            }
        }
        };
        if (p.block_table) run(std::true_type{}); else run(std::false_type{});
        lcol += __shfl_xor(lcol, 16);
        lcol += __shfl_xor(lcol, 32);
        if (col < kGroupSize) {
            if (dq == 0) {
                s_merge[wave].m[col] = mcol;
                s_merge[wave].l[col] = lcol;
            }
#pragma unroll
            for (int blk = 0; blk < 8; ++blk)
                *reinterpret_cast<float4_t*>(&s_merge[wave].acc[col][16 * blk + 4 * dq]) = oacc[blk];
        }
    } else if constexpr (GATHER) {
        // Index list -> block table -> physical row, staged in LDS one sub-chunk at a time.
        auto run = [&](auto paged_tag) {
        for (int c0 = r0; c0 < r1; c0 += kSubChunk) {
            const int cn = min(kSubChunk, r1 - c0);
            __syncthreads();
            for (int i = tid; i < cn; i += kThreads) {
                int tok = idx_row[c0 + i];
                tok = max(0, min(tok, seqlen - 1));   // a corrupt index must not leave the sequence
                if (tok == newest) s_found = c0;
                int row;
                if (p.block_table) {
                    int pg = p.block_table[(size_t)b * p.max_pages + (tok >> p.page_shift)];
                    row = (pg << p.page_shift) + (tok & page_mask);
                } else {
                    row = tok;
                }
                s_row[i] = row;
            }
            __syncthreads();
            if (p.k_new != nullptr && s_found == c0) {   // c0 differs per sub-chunk: no reset needed
                write_newest();
                __syncthreads();
            }
            auto staged_rows = [&](int it, int (&rows)[kUnroll]) {
                const int rbase = it + wave * (4 * kUnroll) + rg;
#pragma unroll
                for (int u = 0; u < kUnroll; ++u) rows[u] = s_row[min(rbase + u * 4, cn - 1)];
            };
            // software pipeline: the loads of iteration i+1 are in flight while iteration i computes
            Batch ba, bb;
            int rows[kUnroll];
            staged_rows(0, rows);
            issue_loads(paged_tag, rows, ba);
            for (int it = 0; it < cn; it += 2 * kRowsPerIter) {
                staged_rows(it + kRowsPerIter, rows);      // rows past the end are clamped and masked
                issue_loads(paged_tag, rows, bb);
                KASCADE_SCHED_FENCE();
                compute_batch(it + wave * (4 * kUnroll) + rg, cn, c0, 0, 0, ba);
                KASCADE_SCHED_FENCE();
                staged_rows(it + 2 * kRowsPerIter, rows);
                issue_loads(paged_tag, rows, ba);
                KASCADE_SCHED_FENCE();
                compute_batch(it + kRowsPerIter + wave * (4 * kUnroll) + rg, cn, c0, 0, 0, bb);
                KASCADE_SCHED_FENCE();
            }
        }
        };
        if (p.block_table) run(std::true_type{}); else run(std::false_type{});
    } else if constexpr (kDenseMfma) {
        // Token ranges (dense baseline, anchor passes) on the matrix unit, tile for tile like the
        // gathered rows above.  A wavefront owns 256 consecutive tokens of every 1024 (the strips
        // whose raw scores the anchor passes park in LDS for the writer wavefront) and walks them
        // in tiles of 16.  Without V (anchor pass that produces no output) a lane only needs the
        // log-sum of its own keys, four tiles are in flight and nothing crosses lanes until the
        // end; with V two tiles (K and V) are in flight.
        const int cn = r1 - r0;
        const int* bt_row = p.block_table ? p.block_table + (size_t)b * p.max_pages : nullptr;
        const int col = lane & 15, dq = lane >> 4;
        half8_t qb[4];
#pragma unroll
        for (int st = 0; st < 4; ++st) {
            Pack16 t;
            t.u = ld_global_16(p.Q + ((size_t)b * kHeads + g * kGroupSize + (col & 3)) * kDim + 32 * st + 8 * dq);
            if (col >= kGroupSize) t.u = uint4_t{0, 0, 0, 0};
            qb[st] = t.h8;
        }
        float mcol = -INFINITY, lcol = 0.f;   // running max / sum (with V: one max per column)
        float4_t oacc[WITH_V ? 8 : 1];
#pragma unroll
        for (int blk = 0; blk < (WITH_V ? 8 : 1); ++blk) oacc[blk] = float4_t{0.f, 0.f, 0.f, 0.f};
        struct Tile {
            uint4_t k[4];
            uint4_t v[WITH_V ? 4 : 1];
        };
        constexpr int kDepth = WITH_V ? 2 : 4;
        auto run = [&](auto paged_tag) {
        constexpr bool PAGED = decltype(paged_tag)::value;
        constexpr int kTilesPerStrip = kStripRows / 16;
        // tile k of this wavefront: 16 keys from row (k / 16) * 1024 + wave * 256 + (k % 16) * 16
        auto tile_row = [&](int k) { return (k / kTilesPerStrip) * (4 * kStripRows) + wave * kStripRows + (k % kTilesPerStrip) * 16; };
        // loads: lane (dq, col) takes chunk col of rows 4i + dq of the tile; past the end: clamped, masked later
        auto tok_of = [&](int k, int i) { return min(r0 + tile_row(k) + 4 * i + dq, r1 - 1); };
        auto fetch_pages = [&](int k, int (&pg)[4]) {
#pragma unroll
            for (int i = 0; i < 4; ++i) pg[i] = PAGED ? bt_row[tok_of(k, i) >> p.page_shift] : 0;
        };
        auto issue = [&](int k, const int (&pg)[4], Tile& tb) {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int tok = tok_of(k, i);
                const size_t off = PAGED ? ((size_t)((pg[i] << p.page_shift) + (tok & page_mask)) * kGroups + g) * kDim + 8 * col
                                         : (size_t)b * p.kv_stride_b + (size_t)g * p.kv_stride_h +
                                               (size_t)(unsigned)tok * stride_l + 8 * col;
                tb.k[i] = __builtin_nontemporal_load(reinterpret_cast<const uint4_t*>(p.K + off));
                if (WITH_V) tb.v[i] = __builtin_nontemporal_load(reinterpret_cast<const uint4_t*>(p.V + off));
            }
        };
        half_t* kt = &s_kt[wave < 4 ? wave : 0][0];
        half_t* vt = &s_vt[wave < 4 ? wave : 0][0];
        auto compute = [&](int k, const Tile& tb) {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                *reinterpret_cast<uint4_t*>(&kt[(4 * i + dq) * kKtStride + 8 * col]) = tb.k[i];
                if (WITH_V) *reinterpret_cast<uint4_t*>(&vt[(4 * i + dq) * kVtStride + 8 * col]) = tb.v[i];
            }
            __builtin_amdgcn_wave_barrier();   // the reads below are other lanes' writes (same wavefront: in order)
            float4_t sc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int st = 0; st < 4; ++st) {
                const half8_t a = *reinterpret_cast<const half8_t*>(&kt[col * kKtStride + 32 * st + 8 * dq]);
                sc = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, qb[st], sc, 0, 0, 0);
            }
            // sc[e] = q_col . k of key tile_row(k) + 4*dq + e
            const int key0 = tile_row(k) + 4 * dq;
#pragma unroll
            for (int e = 0; e < 4; ++e)
                if (key0 + e >= cn) sc[e] = -INFINITY;
            if (WRITE_SCORES) {
                if (col < kGroupSize)
                    *reinterpret_cast<float4_t*>(&s_sc[(k / kTilesPerStrip) & 1][wave][col][(k % kTilesPerStrip) * 16 + 4 * dq]) = sc;
            }
            float mx = fmaxf(fmaxf(sc[0], sc[1]), fmaxf(sc[2], sc[3]));
            if (WITH_V) {   // the second product needs one reference per column
                mx = fmaxf(mx, __shfl_xor(mx, 16));
                mx = fmaxf(mx, __shfl_xor(mx, 32));
            }
            mx = fmaxf(mx, mcol);
            const float mref = (mx == -INFINITY) ? 0.f : mx * kScaleLog2;
            const float corr = fast_exp2(mcol * kScaleLog2 - mref);
            mcol = mx;
            float pe[4];
            float sum = 0.f;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                pe[e] = fast_exp2(sc[e] * kScaleLog2 - mref);
                sum += pe[e];
            }
            lcol = lcol * corr + sum;
            if (WITH_V) {
                if (__any(corr != 1.f)) {
#pragma unroll
                    for (int blk = 0; blk < 8; ++blk) oacc[blk] *= corr;
                }
                const half4_t pb = {(half_t)pe[0], (half_t)pe[1], (half_t)pe[2], (half_t)pe[3]};
                typedef short short4_t __attribute__((ext_vector_type(4)));
                // lane (dq, col) points at V[row 4dq + col/4][16blk + 4(col%4), +4) and receives
                // V[rows 4dq .. 4dq+3][16blk + col]
                const half_t* vp = &vt[(4 * dq + (col >> 2)) * kVtStride + 4 * (col & 3)];
#pragma unroll
                for (int blk = 0; blk < 8; ++blk) {
                    const short4_t raw = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                        (__attribute__((address_space(3))) short4_t*)(vp + 16 * blk));
                    oacc[blk] = __builtin_amdgcn_mfma_f32_16x16x16f16(__builtin_bit_cast(half4_t, raw), pb, oacc[blk], 0, 0, 0);
                }
            }
            __builtin_amdgcn_wave_barrier();
        };
        if (cn > 0) {
            const int nsup = (cn + 4 * kStripRows - 1) / (4 * kStripRows);
            if (WRITE_SCORES && wave == 4) {
                for (int sup = 0; sup < nsup; ++sup) {
                    __syncthreads();
                    flush_scores(sup);
                }
            } else {
                // kDepth tiles in flight per wavefront (16 KB); page numbers one round further ahead
                const int ntile = nsup * kTilesPerStrip;
                Tile buf[kDepth];
                int pgn[kDepth][4];
#pragma unroll
                for (int j = 0; j < kDepth; ++j) {
                    fetch_pages(j, pgn[j]);
                    issue(j, pgn[j], buf[j]);
                }
#pragma unroll
                for (int j = 0; j < kDepth; ++j) fetch_pages(kDepth + j, pgn[j]);
                for (int k = 0; k < ntile; k += kDepth) {
#pragma unroll
                    for (int j = 0; j < kDepth; ++j) {
                        compute(k + j, buf[j]);
                        KASCADE_SCHED_FENCE();
                        issue(k + kDepth + j, pgn[j], buf[j]);      // past the last tile: clamped rows, never used
                        fetch_pages(k + 2 * kDepth + j, pgn[j]);
                        KASCADE_SCHED_FENCE();
                    }
                    if (WRITE_SCORES && (k + kDepth) % kTilesPerStrip == 0)
                        __syncthreads();   // a strip is complete: hand it to the writer
                }
            }
        }
        };
        if (bt_row) run(std::true_type{}); else run(std::false_type{});
        if (WITH_V) {   // one reference per column: the partial sums just add
            lcol += __shfl_xor(lcol, 16);
            lcol += __shfl_xor(lcol, 32);
        } else {        // the four key subsets of a column (lanes col, col+16, col+32, col+48) have their own
#pragma unroll
            for (int sh = 16; sh <= 32; sh <<= 1) {
                const float mo = __shfl_xor(mcol, sh), lo = __shfl_xor(lcol, sh);
                const float mx = fmaxf(mcol, mo);
                const float mref = (mx == -INFINITY) ? 0.f : mx * kScaleLog2;
                lcol = lcol * fast_exp2(mcol * kScaleLog2 - mref) + lo * fast_exp2(mo * kScaleLog2 - mref);
                mcol = mx;
            }
        }
        if (wave < 4 && col < kGroupSize) {
            if (dq == 0) {
                s_merge[wave].m[col] = mcol;
                s_merge[wave].l[col] = lcol;
            }
            if (WITH_V) {
#pragma unroll
                for (int blk = 0; blk < 8; ++blk)
                    *reinterpret_cast<float4_t*>(&s_merge[wave].acc[col][16 * blk + 4 * dq]) = oacc[blk];
            }
        }
    } else {
        // Dense range [r0, r1): no staging and no barriers.  Three-stage pipeline: block-table
        // entries two iterations ahead, K/V rows one iteration ahead, arithmetic on the current.
        const int cn = r1 - r0;
        const int* bt_row = p.block_table ? p.block_table + (size_t)b * p.max_pages : nullptr;
        // A wavefront owns kStripRows consecutive rows of every super-iteration of
        // 4*kStripRows rows and walks them in kScoreBatches batches of 16 (batch number
        // q = it / kRowsPerIter, phase q % kScoreBatches).
        auto rbase_of = [&](int it) {
            const int q = it / kRowsPerIter;
            return (q / kScoreBatches) * (4 * kStripRows) + wave * kStripRows + (q % kScoreBatches) * 16 + rg;
        };
        auto tok_of = [&](int it, int u) { return min(r0 + rbase_of(it) + u * 4, r1 - 1); };
        // The paged / contiguous choice is hoisted out of the loop as a compile-time tag: a
        // per-load "table ? table[i] : 0" turns into a branch whose join waits for every load
        // in flight.
        auto run = [&](auto paged_tag) {
        constexpr bool PAGED = decltype(paged_tag)::value;
        auto fetch_pages = [&](int it, int (&pg)[kUnroll]) {
#pragma unroll
            for (int u = 0; u < kUnroll; ++u) pg[u] = PAGED ? bt_row[tok_of(it, u) >> p.page_shift] : 0;
        };
        auto rows_of = [&](int it, const int (&pg)[kUnroll], int (&rows)[kUnroll]) {
#pragma unroll
            for (int u = 0; u < kUnroll; ++u) {
                const int tok = tok_of(it, u);
                rows[u] = PAGED ? (pg[u] << p.page_shift) + (tok & page_mask) : tok;
            }
        };
        if (cn > 0) {
            // Block-table entries are fetched *before* the K/V loads of the preceding batch in
            // program order: loads complete in order, so waiting for a younger table entry would
            // otherwise drain the K/V loads in flight.
            Batch ba, bb;
            int pga[kUnroll], pgb[kUnroll], rows[kUnroll];
            fetch_pages(0, pga);
            rows_of(0, pga, rows);
            issue_loads(paged_tag, rows, ba);
            fetch_pages(kRowsPerIter, pgb);
            // every wavefront runs the same number of batches: enough for the longest strip
            const int full = cn / (4 * kStripRows), rem = cn - full * (4 * kStripRows);
            const int nbatch = full * kScoreBatches + min(kScoreBatches, (rem + 15) / 16);
            const int it_end = ((nbatch + 1) & ~1) * kRowsPerIter;   // the loop body handles two batches
            if (WRITE_SCORES && wave == 4) {
                // one barrier per super-iteration, matched by the streaming wavefronts below
                const int nsup = (it_end / kRowsPerIter + kScoreBatches - 1) / kScoreBatches;
                for (int sup = 0; sup < nsup; ++sup) {
                    __syncthreads();
                    flush_scores(sup);
                }
            } else {
            for (int it = 0; it < it_end; it += 2 * kRowsPerIter) {
                const int q = it / kRowsPerIter;
                fetch_pages(it + 2 * kRowsPerIter, pga);   // tokens past the end are clamped and masked
                rows_of(it + kRowsPerIter, pgb, rows);
                issue_loads(paged_tag, rows, bb);
                KASCADE_SCHED_FENCE();
                compute_batch(rbase_of(it), cn, r0, q % kScoreBatches, (q / kScoreBatches) & 1, ba);
                KASCADE_SCHED_FENCE();
                fetch_pages(it + 3 * kRowsPerIter, pgb);
                rows_of(it + 2 * kRowsPerIter, pga, rows);
                issue_loads(paged_tag, rows, ba);
                KASCADE_SCHED_FENCE();
                compute_batch(rbase_of(it + kRowsPerIter), cn, r0, (q + 1) % kScoreBatches, (q / kScoreBatches) & 1, bb);
                KASCADE_SCHED_FENCE();
                if (WRITE_SCORES && ((q + 2) % kScoreBatches == 0 || it + 2 * kRowsPerIter >= it_end))
                    __syncthreads();   // strips of this super-iteration are complete: hand them to the writer
            }
            }
        }
        };
        if (bt_row) run(std::true_type{}); else run(std::false_type{});
    }

    // ---- merge the four row-groups of the wavefront (lanes l, l^16, l^32) ----
    if constexpr (!kDenseMfma && !kGatherMfma) {
#pragma unroll
    for (int h = 0; h < kGroupSize; ++h) {
#pragma unroll
        for (int sh = 16; sh <= 32; sh <<= 1) {
            float mo = __shfl_xor(m[h], sh);
            float lo = __shfl_xor(l[h], sh);
            float mx = fmaxf(m[h], mo);
            float mref = (mx == -INFINITY) ? 0.f : mx * kScaleLog2;
            float ca = fast_exp2(m[h] * kScaleLog2 - mref);
            float cb = fast_exp2(mo * kScaleLog2 - mref);
            l[h] = l[h] * ca + lo * cb;
            if (WITH_V) {
#pragma unroll
                for (int d = 0; d < 8; ++d) {
                    float ao = __shfl_xor(acc[h][d], sh);
                    acc[h][d] = acc[h][d] * ca + ao * cb;
                }
            }
            m[h] = mx;
        }
    }
    if (rg == 0 && wave < 4) {   // the writer wavefront of the anchor variants holds no state
#pragma unroll
        for (int h = 0; h < kGroupSize; ++h) {
            if (dl == 0) {
                s_merge[wave].m[h] = m[h];
                s_merge[wave].l[h] = l[h];
            }
            if (WITH_V) {
#pragma unroll
                for (int d = 0; d < 8; ++d) s_merge[wave].acc[h][dl * 8 + d] = acc[h][d];
            }
        }
    }
    }
    __syncthreads();
    // ---- merge the four wavefronts; thread -> (head, two d's) ----
    if (tid < kThreads) {
        const int h = tid >> 6;
        const int d0 = (tid & 63) * 2;
        float mx = -INFINITY;
#pragma unroll
        for (int w = 0; w < 4; ++w) mx = fmaxf(mx, s_merge[w].m[h]);
        const float mref = (mx == -INFINITY) ? 0.f : mx * kScaleLog2;
        float L = 0.f, o0 = 0.f, o1 = 0.f;
#pragma unroll
        for (int w = 0; w < 4; ++w) {
            float c = fast_exp2(s_merge[w].m[h] * kScaleLog2 - mref);
            L += s_merge[w].l[h] * c;
            if (WITH_V) {
                o0 += s_merge[w].acc[h][d0] * c;
                o1 += s_merge[w].acc[h][d0 + 1] * c;
            }
        }
        const size_t ph = ((size_t)b * kHeads + g * kGroupSize + h) * p.num_split + split;
        const float lse_part = (L > 0.f) ? (fast_log2(L) + mref) : -INFINITY;
        const float inv = (L > 0.f) ? 1.f / L : 0.f;
        if (p.counters == nullptr) {
            if ((tid & 63) == 0) p.glse[ph] = lse_part;
            if (WITH_V) *reinterpret_cast<float2*>(p.opart + ph * kDim + d0) = make_float2(o0 * inv, o1 * inv);
        } else {
            // read by another workgroup of this launch: device-coherent stores
            if ((tid & 63) == 0) store_device(p.glse + ph, lse_part);
            if (WITH_V) store_device2(p.opart + ph * kDim + d0, o0 * inv, o1 * inv);
        }
    }
    // ---- fused combine: the last workgroup of (b, g) to arrive merges the splits ----
    // The partial results above are written through to device-coherent memory and the barrier
    // waits for those stores before thread 0 counts this workgroup in; the merging workgroup
    // reads them back with device-coherent loads.  No device-wide fence is involved: one per
    // workgroup would write back and invalidate the L2 that the K/V stream lives in.
    if (p.counters == nullptr) return;
    __syncthreads();
    if (tid == 0) {
        const int arrived = __hip_atomic_fetch_add(&p.counters[b * kGroups + g], 1, __ATOMIC_RELAXED,
                                                   __HIP_MEMORY_SCOPE_AGENT);
        s_last = (arrived == p.num_split - 1);
    }
    __syncthreads();
    if (!s_last) return;
    if (tid == 0)   // ready for the next launch
        __hip_atomic_store(&p.counters[b * kGroups + g], 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (tid < kThreads) {
        // wavefront -> head; lanes over the splits for the reductions, then two d's per lane
        const int head = g * kGroupSize + wave;
        const int ns = p.num_split;
        const size_t base = ((size_t)b * kHeads + head) * ns;
        const float* gl = p.glse + base;
        const float* op = p.opart + base * kDim + lane * 2;
        // the first partial outputs are requested together with the log-sums, so that short
        // split lists cost one trip to memory, not two
        constexpr int kEarly = 16;
        float2 xe[kEarly];
        if (WITH_V) {
#pragma unroll
            for (int j = 0; j < kEarly; ++j) xe[j] = load_device2(op + (size_t)min(j, ns - 1) * kDim);
        }
        const float g0 = (lane < ns) ? load_device(gl + lane) : -INFINITY;   // splits [0, 64)
        float mx = g0;
        for (int s = lane + 64; s < ns; s += 64) mx = fmaxf(mx, load_device(gl + s));
#pragma unroll
        for (int o = 32; o >= 1; o >>= 1) mx = fmaxf(mx, __shfl_xor(mx, o));
        const float mref = (mx == -INFINITY) ? 0.f : mx;
        float sum = fast_exp2(g0 - mref);
        for (int s = lane + 64; s < ns; s += 64) sum += fast_exp2(load_device(gl + s) - mref);
#pragma unroll
        for (int o = 32; o >= 1; o >>= 1) sum += __shfl_xor(sum, o);
        const float lse = (sum > 0.f) ? fast_log2(sum) + mref : -INFINITY;
        if (p.row_sums && lane == 0) p.row_sums[(size_t)b * kHeads + head] = lse;
        if (WITH_V) {
            const float lref = (lse == -INFINITY) ? 0.f : lse;
            float o0 = 0.f, o1 = 0.f;
            float wl = fast_exp2(g0 - lref);   // 0 in lanes beyond the split count
#pragma unroll
            for (int j = 0; j < kEarly; ++j) {
                const float w = __shfl(wl, j);
                o0 += w * xe[j].x;
                o1 += w * xe[j].y;
            }
            for (int s0 = 0; s0 < ns; s0 += 64) {
                if (s0 > 0) wl = (s0 + lane < ns) ? fast_exp2(load_device(gl + s0 + lane) - lref) : 0.f;
                const int cnt = min(64, ns - s0);
#pragma unroll 8
                for (int j = (s0 == 0 ? kEarly : 0); j < cnt; ++j) {
                    const float w = __shfl(wl, j);
                    const float2 x = load_device2(op + (size_t)(s0 + j) * kDim);
                    o0 += w * x.x;
                    o1 += w * x.y;
                }
            }
            half2_t o = {(half_t)o0, (half_t)o1};
            *reinterpret_cast<half2_t*>(p.out + ((size_t)b * kHeads + head) * kDim + lane * 2) = o;
        }
    }
}

// Merge the per-split log-sums (and partial outputs) of one (b, head).
// grid (H, B), 128 threads: the splits are spread over the threads for the two reductions,
// then thread d accumulates output dimension d with the weights staged in LDS.
constexpr int kCombineLds = 512;   // splits whose weights fit the LDS buffer

__device__ __forceinline__ float combine_reduce(float x, bool is_max, float* s_red) {
#pragma unroll
    for (int o = 32; o >= 1; o >>= 1) {
        const float y = __shfl_xor(x, o);
        x = is_max ? fmaxf(x, y) : x + y;
    }
    __syncthreads();   // s_red may still be read from the previous reduction
    if ((threadIdx.x & 63) == 0) s_red[threadIdx.x >> 6] = x;
    __syncthreads();
    return is_max ? fmaxf(s_red[0], s_red[1]) : s_red[0] + s_red[1];
}

template <bool WITH_V>
__global__ __launch_bounds__(128) void decode_combine_kernel(const float* __restrict__ glse,
                                                            const float* __restrict__ opart,
                                                            half_t* __restrict__ out,
                                                            float* __restrict__ row_sums,
                                                            int num_split) {
    __shared__ float s_w[kCombineLds];
    __shared__ float s_red[2];
    const int h = blockIdx.x;
    const int b = blockIdx.y;
    const int d = threadIdx.x;
    const size_t base = ((size_t)b * kHeads + h) * num_split;
    float mx = -INFINITY;
    for (int s = d; s < num_split; s += 128) mx = fmaxf(mx, glse[base + s]);
    mx = combine_reduce(mx, true, s_red);
    const float mref = (mx == -INFINITY) ? 0.f : mx;
    float sum = 0.f;
    for (int s = d; s < num_split; s += 128) sum += fast_exp2(glse[base + s] - mref);
    sum = combine_reduce(sum, false, s_red);
    const float lse = (sum > 0.f) ? fast_log2(sum) + mref : -INFINITY;
    if (row_sums && d == 0) row_sums[(size_t)b * kHeads + h] = lse;
    if (WITH_V) {
        const float lref = (lse == -INFINITY) ? 0.f : lse;
        for (int s = d; s < min(num_split, kCombineLds); s += 128) s_w[s] = fast_exp2(glse[base + s] - lref);
        __syncthreads();
        const float* op = opart + base * kDim + d;
        float o = 0.f;
        int s = 0;
        // a split that saw no rows leaves its partial output unwritten: select, never multiply
        for (; s + 8 <= min(num_split, kCombineLds); s += 8) {
            float x[8];
#pragma unroll
            for (int e = 0; e < 8; ++e) x[e] = op[(size_t)(s + e) * kDim];
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const float w = s_w[s + e];
                o += (w > 0.f) ? w * x[e] : 0.f;
            }
        }
        for (; s < num_split; ++s) {
            const float w = (s < kCombineLds) ? s_w[s] : fast_exp2(glse[base + s] - lref);
            const float x = op[(size_t)s * kDim];
            o += (w > 0.f) ? w * x : 0.f;
        }
        out[((size_t)b * kHeads + h) * kDim + d] = (half_t)o;
    }
}

// agg[b,g,j] = fp16( sum_h exp2(s[b,4g+h,j]*scale - lse[b,4g+h]) ), 0 beyond the sequence.
// grid (ceil(stride/2048), G, B), 256 threads x 8 tokens.
// The per-head log-sums come either merged (row_sums_in) or as the splits' partial log-sums
// (glse [B,H,num_split]): then every workgroup merges them itself -- one wavefront per head --
// and the first workgroup of a (sequence, KV head) also writes them to row_sums_out, which saves
// the combine launch of an anchor pass that produces no output.
__global__ __launch_bounds__(256) void decode_aggregate_kernel(const float* __restrict__ scores,
                                                              const float* __restrict__ row_sums_in,
                                                              const float* __restrict__ glse, int num_split,
                                                              float* __restrict__ row_sums_out,
                                                              const int* __restrict__ seqlens,
                                                              half_t* __restrict__ agg,
                                                              int scores_stride, int uniform_len) {
    __shared__ float s_lse[kGroupSize];
    const int g = blockIdx.y;
    const int b = blockIdx.z;
    const int len = seqlens ? seqlens[b] : uniform_len;
    const int j0 = (blockIdx.x * 256 + threadIdx.x) * 8;
    float lse[kGroupSize];
    if (glse != nullptr) {   // uniform over the launch
        const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
        const float* gl = glse + ((size_t)b * kHeads + g * kGroupSize + wave) * num_split;
        float mx = -INFINITY;
        for (int sidx = lane; sidx < num_split; sidx += 64) mx = fmaxf(mx, gl[sidx]);
#pragma unroll
        for (int o = 32; o >= 1; o >>= 1) mx = fmaxf(mx, __shfl_xor(mx, o));
        const float mref = (mx == -INFINITY) ? 0.f : mx;
        float sum = 0.f;
        for (int sidx = lane; sidx < num_split; sidx += 64) sum += fast_exp2(gl[sidx] - mref);
#pragma unroll
        for (int o = 32; o >= 1; o >>= 1) sum += __shfl_xor(sum, o);
        const float v = (sum > 0.f) ? fast_log2(sum) + mref : -INFINITY;
        if (lane == 0) {
            s_lse[wave] = v;
            if (blockIdx.x == 0 && row_sums_out) row_sums_out[(size_t)b * kHeads + g * kGroupSize + wave] = v;
        }
        __syncthreads();
#pragma unroll
        for (int h = 0; h < kGroupSize; ++h) lse[h] = s_lse[h];
    } else {
#pragma unroll
        for (int h = 0; h < kGroupSize; ++h) lse[h] = row_sums_in[(size_t)b * kHeads + g * kGroupSize + h];
    }
    if (j0 >= scores_stride) return;
    float sum[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) sum[e] = 0.f;
    const bool full = (j0 + 8 <= scores_stride) && ((scores_stride & 7) == 0);
    if (j0 < len) {   // codes and references beyond the sequence were never written
#pragma unroll
        for (int h = 0; h < kGroupSize; ++h) {
            const float* row = scores + ((size_t)b * kHeads + g * kGroupSize + h) * scores_stride;
            const uint16_t* sp = reinterpret_cast<const uint16_t*>(row) + j0;
            const float ref = row[scores_stride / 2 + (j0 >> 6)] - lse[h];
            uint32_t q[8];
            if (full) {
                const uint4_t raw = ld_global_16(sp);
#pragma unroll
                for (int e = 0; e < 8; ++e) q[e] = (raw[e >> 1] >> (16 * (e & 1))) & 0xFFFFu;
            } else {
#pragma unroll
                for (int e = 0; e < 8; ++e) q[e] = (j0 + e < len) ? sp[e] : kScoreNone;
            }
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const float pr = fast_exp2(ref - (float)q[e] * (1.f / kScoreSteps));
                sum[e] += (q[e] == kScoreNone) ? 0.f : pr;
            }
        }
    }
    half_t* ap = agg + ((size_t)b * kGroups + g) * scores_stride + j0;
    if (full && ((scores_stride & 7) == 0)) {
        Pack16 o;
#pragma unroll
        for (int e = 0; e < 8; ++e) o.h[e] = (j0 + e < len) ? (half_t)sum[e] : (half_t)0.f;
        *reinterpret_cast<uint4_t*>(ap) = o.u;
    } else {
#pragma unroll
        for (int e = 0; e < 8; ++e)
            if (j0 + e < scores_stride) ap[e] = (j0 + e < len) ? (half_t)sum[e] : (half_t)0.f;
    }
}

}  // namespace

hipError_t launch_decode_split(const DecodeParams& p, bool gather, bool with_v, bool write_scores,
                               hipStream_t stream) {
    dim3 grid(kGroups, p.num_split, p.B), block(write_scores ? kThreads + 64 : kThreads);
    if (gather) {
        hipLaunchKernelGGL((decode_split_kernel<true, true, false>), grid, block, 0, stream, p);
    } else if (write_scores) {
        if (with_v)
            hipLaunchKernelGGL((decode_split_kernel<false, true, true>), grid, block, 0, stream, p);
        else
            hipLaunchKernelGGL((decode_split_kernel<false, false, true>), grid, block, 0, stream, p);
    } else {
        hipLaunchKernelGGL((decode_split_kernel<false, true, false>), grid, block, 0, stream, p);
    }
    return hipGetLastError();
}

hipError_t launch_decode_combine(const float* glse, const float* opart, half_t* out,
                                 float* row_sums, int batch, int num_split, bool with_v,
                                 hipStream_t stream) {
    dim3 grid(kHeads, batch), block(128);
    if (with_v)
        hipLaunchKernelGGL((decode_combine_kernel<true>), grid, block, 0, stream, glse, opart, out,
                           row_sums, num_split);
    else
        hipLaunchKernelGGL((decode_combine_kernel<false>), grid, block, 0, stream, glse, opart, out,
                           row_sums, num_split);
    return hipGetLastError();
}

hipError_t launch_decode_aggregate(const float* scores, const float* row_sums_in, const float* glse,
                                   int num_split, float* row_sums_out, const int* seqlens,
                                   half_t* agg, int batch, int scores_stride, int uniform_len,
                                   hipStream_t stream) {
    dim3 grid((scores_stride + 2047) / 2048, kGroups, batch), block(256);
    hipLaunchKernelGGL(decode_aggregate_kernel, grid, block, 0, stream, scores, row_sums_in, glse,
                       num_split, row_sums_out, seqlens, agg, scores_stride, uniform_len);
    return hipGetLastError();
}

}  // namespace kascade
