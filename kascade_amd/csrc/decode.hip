// Decode-step attention kernels for gfx950: bandwidth-bound split-K streaming of
// K/V rows (gathered through a top-k index list, or dense), log-sum merge, and
// pooled post-softmax scores for anchor layers.
//
// Work decomposition (one launch = all sequences, KV heads and splits):
//   grid  (G, num_split, B), 256 threads = 4 wavefronts.  A wavefront works on
//   tiles of 16 rows:
//   16 lanes fetch one 256-byte row with one 16-byte load each (four rows per
//   instruction), the tile crosses a wavefront-private piece of LDS into the
//   operand layouts of the matrix unit, and both products of the step run there
//   (q.k as 16 keys x 4-of-16 columns, p.v with the tile's keys contracted).
//   The arithmetic is 2 flop/byte, far below the machine balance; the matrix
//   unit is used because it does the dot products without cross-lane reductions,
//   which on the vector unit cost ~110 instructions per row and capped every
//   variant below what HBM delivers.  Every wavefront keeps one online-softmax
//   state per query head; the four states of a workgroup are merged once at the
//   end, the splits by the last workgroup to arrive (or the combine kernel).
#include "decode.h"

#include <type_traits>

namespace kascade {

namespace {

constexpr int kThreads = 256;
// The instruction scheduler otherwise sinks every prefetch load down to its first use (to save
// registers), which serialises load -> wait -> use and removes all memory-level parallelism.
#define KASCADE_SCHED_FENCE() __builtin_amdgcn_sched_barrier(0)
constexpr int kStripRows = 256;               // consecutive tokens a wavefront owns per 1024
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

template <int D, int HS>
struct alignas(16) MergeState {  // one per wavefront after the in-wave merge
    float m[HS];
    float l[HS];
    float acc[HS][D];
};

// PHYS (gather mode over a paged cache): the index lists hold physical cache rows
// (page * page_size + slot, what translate_indices_kernel writes) instead of token positions, so
// the block table is not on the path from a list entry to its K/V row.
// D, T: head dimension (64 or 128) and element type (fp16 or bf16) of Q, K, V and the output; the
// number of KV heads and of query heads per KV head (p.gs) are launch parameters.  The query heads
// of the KV head are columns of the first product, so any number up to 16 rides on the same K/V
// stream; HS (4, 8 or 16 >= p.gs) sizes what is kept per head in LDS.
template <bool GATHER, bool WITH_V, bool WRITE_SCORES, bool PHYS, int D, typename T, int HS>
__global__ __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(2)))
void decode_split_kernel(DecodeParams p) {
    typedef typename Elem<T>::x8 x8_t;
    typedef typename Elem<T>::x4 x4_t;
    typedef typename Elem<T>::x2 x2_t;
    constexpr float kScaleLog2 = ScaleLog2<D>::value;
    const int kvh = p.G;                 // KV heads
    const int gs = p.gs;                 // query heads per KV head (<= HS)
    const int nheads = p.G * gs;         // query heads
    __shared__ int s_row[GATHER ? kSubChunk : 1];
    __shared__ int s_last;
    __shared__ int s_found;   // gather mode: sub-chunk whose index list names the newest token
    // anchor mode: the compact raw scores of kCodePhase * 1024 tokens (see kScoreSteps), written to
    // HBM in one burst per phase; they share their LDS with the merge state, which is only needed
    // after the last burst
    // what fits beside two workgroups' tiles: 40 / 56 KB of codes
    constexpr int kCodePhase = HS == 4 ? (WITH_V ? 5 : 7) : HS == 8 ? (WITH_V ? 2 : 3) : 1;
    constexpr int kPhaseRows = WRITE_SCORES ? kCodePhase * 4 * kStripRows : 64;
    union Shared {
        MergeState<D, HS> merge[4];
        struct {   // head rows 32 bytes apart in the banks: the 4 x 4 lanes of a granule write hit 16 bank pairs
            uint16_t code[HS][kPhaseRows + 16];
            float ref[HS][kPhaseRows / 64];
        } sc;
    };
    __shared__ __attribute__((aligned(16))) Shared s_u;
    MergeState<D, HS>* s_merge = s_u.merge;
    auto& s_code = s_u.sc.code;
    auto& s_ref = s_u.sc.ref;
    // per wavefront one tile of 16 K rows (and V rows) on its way into the matrix layouts
    constexpr int kKtStride = D + 8;    // elements per K row: rows 272 (144) bytes apart, conflict-free both ways
    constexpr int kVtStride = D + 16;   // elements per V row: 288 (160) bytes, conflict-free for the transposing reads
    __shared__ __attribute__((aligned(16))) T s_kt[4][16 * kKtStride];
    __shared__ __attribute__((aligned(16))) T s_vt[WITH_V ? 4 : 1][WITH_V ? 16 * kVtStride : 8];

    const int g = blockIdx.x;       // the 8 KV heads of one token range are adjacent in dispatch order
    const int tid = threadIdx.x;
    const int wave = tid >> 6;
    const int lane = tid & 63;

    // The longest context memory allows a sequence that claims `len` tokens: lengths live in device
    // memory, the host sized every buffer from its own arguments, so each length is cut down to
    // what the block table covers (or the cache holds) and, on an anchor pass, to the row width of
    // the score scratch.  Nothing is read or written beyond those bounds whatever the lengths say.
    auto safe_len = [&](int len) {
        if (p.block_table) len = min(len, p.max_pages << p.page_shift);
        else if (p.kv_stride_tokens > 0) len = min(len, p.kv_stride_tokens);
        if (WRITE_SCORES) len = min(len, p.scores_stride);
        return max(len, 0);
    };
    // rows a (sequence, KV head) pair of (safe) length `len` attends to
    auto rows_for = [&](int len) {
        if (!GATHER) return len;
        int n;
        if (p.topk_percent > 0.f) {
            long long fl = (long long)floor((double)p.topk_percent * (double)len / 100.0);
            n = (int)(((fl + 127) / 128) * 128);
        } else {
            n = p.topk;
        }
        n = min(n, p.topk);
        if (p.seqlens) n = min(n, len);   // never more rows than the sequence holds
        return n;
    };
    // Splits a sequence of `rows` rows occupies: never more than the launch has per sequence.  A
    // sequence longer than the host sized the splits for (its length exceeds the caller's bound)
    // keeps num_split splits and its last split takes every row that is left.
    auto split_count = [&](int rows) {
        return max(1, min(p.num_split, (rows + p.rows_per_split - 1) / p.rows_per_split));
    };
    // Which (sequence, split) this workgroup takes.  With per-sequence lengths the non-empty
    // splits of all sequences are numbered consecutively (sequence-major; at least one split per
    // sequence) and workgroup w of the launch takes number w: the workgroups left over -- a
    // ragged batch has many -- come last in dispatch order and exit at once, instead of being
    // scattered among the working ones, which left some compute units with several streams and
    // others with none (four sequences of 131072..524288 tokens, 512 working workgroups: gather
    // 101 -> 86 us).  One sequence needs none of this; beyond 64 * kMapRounds sequences the
    // workgroups keep their grid position.  Neither do gather launches whose lists all have the
    // same length (no per-sequence budget): every split of the grid has work, and leaving the
    // numbering out takes one dependent trip to memory off the start of every workgroup.
    constexpr int kMapRounds = 4;
    int b, split, nsplit_b, seqlen;
    bool len_cut;
    const bool ragged_rows = !GATHER || p.topk_percent > 0.f;
    if (p.seqlens != nullptr && p.B > 1 && p.B <= 64 * kMapRounds && ragged_rows) {
        // every wavefront works it out for itself: lane l holds sequences l, l + 64, ...; no LDS,
        // no barrier, and the sequence's length comes out of the same loads (all issued first)
        const int w = blockIdx.y + gridDim.y * blockIdx.z;
        int lens[kMapRounds];
        unsigned long long cut[kMapRounds];   // sequences whose length had to be cut down
#pragma unroll
        for (int r = 0; r < kMapRounds; ++r) {
            const int bi = 64 * r + lane;
            const int raw = bi < p.B ? p.seqlens[bi] : 0;
            lens[r] = safe_len(raw);
            cut[r] = __ballot(lens[r] != raw);
        }
        int carry = 0;   // splits of the sequences of earlier rounds (wavefront-uniform)
        b = -1; split = 0; nsplit_b = 1; seqlen = 0; len_cut = false;
#pragma unroll
        for (int r = 0; r < kMapRounds; ++r) {
            if (64 * r < p.B && b < 0) {   // uniform
                const int bi = 64 * r + lane;
                const int cnt = bi < p.B ? split_count(rows_for(lens[r])) : 0;
                int incl = cnt;
#pragma unroll
                for (int o = 1; o < 64; o <<= 1) {
                    const int t = __shfl_up(incl, o);
                    if (lane >= o) incl += t;
                }
                const int excl = carry + incl - cnt;
                const unsigned long long mine = __ballot(bi < p.B && w >= excl && w < excl + cnt);
                if (mine != 0) {
                    const int src = __ffsll((long long)mine) - 1;
                    b = 64 * r + src;
                    split = __builtin_amdgcn_readfirstlane(w - __shfl(excl, src));
                    nsplit_b = __builtin_amdgcn_readfirstlane(__shfl(cnt, src));
                    seqlen = __builtin_amdgcn_readfirstlane(__shfl(lens[r], src));
                    len_cut = (cut[r] >> src) & 1;
                }
                carry += __builtin_amdgcn_readfirstlane(__shfl(incl, 63));
            }
        }
        if (b < 0) return;   // beyond the last working workgroup
    } else {
        b = blockIdx.z;
        split = blockIdx.y;
        nsplit_b = p.num_split;
        const int raw = p.seqlens ? p.seqlens[b] : p.kv_stride_tokens;
        seqlen = safe_len(raw);
        len_cut = seqlen != raw;
    }
    const int n = rows_for(seqlen);  // rows this (b, g) pair attends to
    // contiguous range of this split; every split covers rows_per_split rows, sequences
    // shorter than num_split*rows_per_split leave their last splits empty, and the last split of
    // a sequence runs to the sequence's end
    const long long r0l = (long long)split * p.rows_per_split;
    const int r0 = (int)min((long long)n, r0l);
    const int r1 = (split == nsplit_b - 1) ? n : (int)min((long long)n, r0l + p.rows_per_split);

    // Fused append.  With k_new/v_new the K/V rows of the newest token (position seqlen-1)
    // arrive beside the cache and have to end up in it.  A workgroup that is going to read that
    // row writes it first and waits for its own stores at a barrier; what other workgroups write
    // there is the same bytes.  `write_newest` is uniform over the workgroup.
    // A length that had to be cut down names a slot that does not exist: nothing is appended.
    const int newest = seqlen - 1;
    const bool can_append = p.k_new != nullptr && newest >= 0 && !len_cut;
    int newest_row = -1;   // PHYS: the cache row of the newest token, what a list names it by
    if (PHYS && can_append)
        newest_row = (p.block_table[(size_t)b * p.max_pages + (newest >> p.page_shift)] << p.page_shift) +
                     (newest & ((1 << p.page_shift) - 1));
    auto write_newest = [&]() {
        if (tid < 2 * (D / 8)) {   // one 16-byte chunk of the K row or of the V row per thread
            const int part = tid / (D / 8), c = tid % (D / 8);
            size_t off;
            if (p.block_table) {
                const int pg = p.block_table[(size_t)b * p.max_pages + (newest >> p.page_shift)];
                const int row = (pg << p.page_shift) + (newest & ((1 << p.page_shift) - 1));
                off = (size_t)row * (kvh * D) + (size_t)g * D + c * 8;
            } else {
                off = (size_t)b * p.kv_stride_b + (size_t)g * p.kv_stride_h + (size_t)newest * p.kv_stride_l + c * 8;
            }
            const T* src = (part ? (const T*)p.v_new : (const T*)p.k_new) + ((size_t)b * kvh + g) * D + c * 8;
            T* dst = (part ? (T*)p.v_cache : (T*)p.k_cache) + off;
            *reinterpret_cast<uint4_t*>(dst) = ld_global_16(src);
        }
    };
    if (can_append) {
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

    // ---- tiles of 16 rows on the matrix unit ----
    // Lane roles.  Loading: lane (dq, col) = (lane / 16, lane % 16) takes the 16-byte chunk `col`
    // of rows 4i + dq of a tile, i = 0..3, so 16 lanes fetch one 256-byte row and an instruction
    // four rows.  Computing: the same lane is key `col` / part dq of the A operand of
    // S^T = K Q^T (v_mfma_f32_16x16x32_f16: 16 keys x 16 columns, d contracted 32 at a time; the
    // four query heads are columns 0-3, the rest zero) and ends up with S^T[4dq .. 4dq+3][col]:
    // exactly the B-operand layout of O^T += V^T P^T (v_mfma_f32_16x16x16_f16, the tile's 16 keys
    // contracted), whose A operand V^T is read out of the row-major V tile by the transposing LDS
    // read.  The tiles pass through wavefront-private LDS (no workgroup barrier).  Nothing here is
    // a cross-lane reduction: ~10 vector instructions per row, where dot products on the vector
    // unit needed ~110 and bounded every variant of this kernel.
    const int col = lane & 15, dq = lane >> 4;
    // Loading role: a row is D/8 chunks of 16 bytes, so a wavefront instruction fetches kRowsPerLoad
    // whole rows (4 at D = 128, 8 at D = 64) and a tile of 16 rows takes kLoads of them; lane
    // (lr, lc) takes chunk lc of rows kRowsPerLoad * i + lr.
    constexpr int kChunks = D / 8, kRowsPerLoad = 64 / kChunks, kLoads = 16 / kRowsPerLoad;
    const int lc = lane % kChunks, lr = lane / kChunks;
    x8_t qb[D / 32];   // B operand of the first product: Q[col][32*st + 8*dq, +8)
#pragma unroll
    for (int st = 0; st < D / 32; ++st) {
        PackT<T> t;
        t.u = ld_global_16((const T*)p.Q + ((size_t)b * nheads + g * gs + min(col, gs - 1)) * D + 32 * st + 8 * dq);
        if (col >= gs) t.u = uint4_t{0, 0, 0, 0};
        qb[st] = t.v8;
    }
    // Online softmax state of this lane's column.  With V one running maximum per column (the
    // second product needs a common reference: two cross-lane exchanges per tile); without V
    // every lane keeps the maximum and sum of its own keys and the four parts meet at the end.
    float mcol = -INFINITY, lcol = 0.f;
    constexpr int kOBlocks = D / 16;
    float4_t oacc[WITH_V ? kOBlocks : 1];   // O^T[16*blk + 4*dq + r][col]
#pragma unroll
    for (int blk = 0; blk < (WITH_V ? kOBlocks : 1); ++blk) oacc[blk] = float4_t{0.f, 0.f, 0.f, 0.f};

    const int* idx_row = nullptr;
    // a map built for another KV-head count must not leave the index tensor
    if (GATHER) idx_row = p.idx + ((size_t)b * kvh + max(0, min(p.head_map[g], kvh - 1))) * p.topk;
    const int page_mask = (1 << p.page_shift) - 1;
    const unsigned stride_l = p.kv_stride_l;
    T* kt = &s_kt[wave][0];
    T* vt = &s_vt[wave][0];
    const T* Kc = (const T*)p.K;
    const T* Vc = (const T*)p.V;

    struct Tile {
        uint4_t k[kLoads];
        uint4_t v[WITH_V ? kLoads : 1];
    };
    // `row`: physical row (page * page_size + slot) behind a block table; otherwise the token
    // number of sequence b behind the caller's (batch, token, head) strides, so that a head-major
    // cache is read in place.  Every K/V row is read once per launch: non-temporal loads keep
    // the stream from displacing what the launch does want cached (index lists, block table,
    // the raw scores of an anchor pass).
    auto load_row = [&](auto paged_tag, int row, Tile& tb, int i) {
        constexpr bool PAGED = decltype(paged_tag)::value;
        const size_t off = PAGED ? ((size_t)row * kvh + g) * D + 8 * lc
                                 : (size_t)b * p.kv_stride_b + (size_t)g * p.kv_stride_h +
                                       (size_t)(unsigned)row * stride_l + 8 * lc;
        tb.k[i] = __builtin_nontemporal_load(reinterpret_cast<const uint4_t*>(Kc + off));
        if (WITH_V) tb.v[i] = __builtin_nontemporal_load(reinterpret_cast<const uint4_t*>(Vc + off));
    };
    // One tile: `key0` is the position of this lane's first key within the range, `cn` the number
    // of rows of the range (keys at or beyond it are masked).  Returns this lane's four raw scores.
    // Straight-line on purpose (no early exit): a branch between issuing a tile's loads and
    // consuming them makes the compiler wait for every load in flight.
    auto compute_tile = [&](const Tile& tb, int key0, int cn) -> float4_t {
#pragma unroll
        for (int i = 0; i < kLoads; ++i) {
            *reinterpret_cast<uint4_t*>(&kt[(kRowsPerLoad * i + lr) * kKtStride + 8 * lc]) = tb.k[i];
            if (WITH_V) *reinterpret_cast<uint4_t*>(&vt[(kRowsPerLoad * i + lr) * kVtStride + 8 * lc]) = tb.v[i];
        }
        __builtin_amdgcn_wave_barrier();   // the reads below are other lanes' writes (same wavefront: in order)
        float4_t sc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int st = 0; st < D / 32; ++st) {
            const x8_t a = *reinterpret_cast<const x8_t*>(&kt[col * kKtStride + 32 * st + 8 * dq]);
            sc = Elem<T>::mma_16x16x32(a, qb[st], sc);
        }
#pragma unroll
        for (int e = 0; e < 4; ++e)
            if (key0 + e >= cn) sc[e] = -INFINITY;
        float mx = fmaxf(fmaxf(sc[0], sc[1]), fmaxf(sc[2], sc[3]));
        if (WITH_V) {
            mx = fmaxf(mx, __shfl_xor(mx, 16));
            mx = fmaxf(mx, __shfl_xor(mx, 32));
        }
        mx = fmaxf(mx, mcol);
        const float mref = (mx == -INFINITY) ? 0.f : mx * kScaleLog2;
        const float corr = fast_exp2(mcol * kScaleLog2 - mref);   // mcol = -inf -> 0
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
            if (__any(corr != 1.f)) {   // wavefront-uniform: skip when no maximum moved
#pragma unroll
                for (int blk = 0; blk < kOBlocks; ++blk) oacc[blk] *= corr;
            }
            const x4_t pb = {(T)pe[0], (T)pe[1], (T)pe[2], (T)pe[3]};
            // ds_read_b64_tr_b16: lane (dq, col) points at V[row 4dq + col/4][16blk + 4(col%4), +4)
            // and receives V[rows 4dq .. 4dq+3][16blk + col]
            const T* vp = &vt[(4 * dq + (col >> 2)) * kVtStride + 4 * (col & 3)];
#pragma unroll
            for (int blk = 0; blk < kOBlocks; ++blk) {
                const short4_t raw = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                    (__attribute__((address_space(3))) short4_t*)(vp + 16 * blk));
                oacc[blk] = Elem<T>::mma_16x16x16(raw, pb, oacc[blk]);
            }
        }
        __builtin_amdgcn_wave_barrier();
        return sc;
    };

    // Anchor passes: a granule's raw scores (four consecutive tiles of this wavefront, 64 tokens at
    // position `prow` of the phase buffer) become 16-bit codes below the granule's maximum.
    auto encode_granule = [&](const float4_t (&sc)[4], int prow) {
        float mx = -INFINITY;
#pragma unroll
        for (int j = 0; j < 4; ++j) mx = fmaxf(mx, fmaxf(fmaxf(sc[j][0], sc[j][1]), fmaxf(sc[j][2], sc[j][3])));
        mx = fmaxf(mx, __shfl_xor(mx, 16));
        mx = fmaxf(mx, __shfl_xor(mx, 32));
        const float base = (mx == -INFINITY) ? 0.f : mx;
        if (col < gs) {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                uint32_t q[4];
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const float d = (base - sc[j][e]) * (kScaleLog2 * kScoreSteps);      // >= 0, +inf if masked
                    q[e] = (sc[j][e] == -INFINITY) ? kScoreNone : (uint32_t)fminf(rintf(d), (float)(kScoreNone - 1));
                }
                *reinterpret_cast<uint2*>(&s_code[col][prow + 16 * j + 4 * dq]) =
                    make_uint2(q[0] | (q[1] << 16), q[2] | (q[3] << 16));
            }
            if (dq == 0) s_ref[col][prow >> 6] = base * kScaleLog2;
        }
    };
    // The codes of phase `ph` (tokens [ph * kPhaseRows, +kPhaseRows) of the range) leave in one
    // burst from all threads.  Score stores trickling out while K streams cost the stream far
    // more than their bytes (HBM turning between reads and writes); workgroups of one launch run
    // in step, so their bursts coincide and the device alternates between long read and short
    // write phases.  The streaming wavefronts issue these stores themselves -- loads and stores
    // retire in order on one counter, so the next tiles wait for them -- once per phase.
    auto flush_phase = [&](int ph) {
        const int cn = r1 - r0;
        const int lo = ph * kPhaseRows;
        const int nrows = min(kPhaseRows, cn - lo);
        __syncthreads();
        if (nrows > 0) {
            for (int h = 0; h < gs; ++h) {
                float* row = p.scores + ((size_t)b * nheads + g * gs + h) * p.scores_stride;
                uint16_t* dst = reinterpret_cast<uint16_t*>(row) + r0 + lo;
                for (int i = tid * 8; i < nrows; i += kThreads * 8) {
                    if (i + 8 <= nrows) {
                        __builtin_nontemporal_store(*reinterpret_cast<const uint4_t*>(&s_code[h][i]),
                                                    reinterpret_cast<uint4_t*>(dst + i));
                    } else {
                        for (int e = 0; i + e < nrows; ++e) dst[i + e] = s_code[h][i + e];
                    }
                }
                for (int i = tid; i < (nrows + 63) / 64; i += kThreads)
                    row[p.scores_stride / 2 + ((r0 + lo) >> 6) + i] = s_ref[h][i];
            }
        }
        __syncthreads();
    };

    if constexpr (GATHER) {
        // Index list -> block table -> physical row, staged in LDS one sub-chunk at a time; the
        // wavefronts take the sub-chunk's tiles in turn, two tiles (16 KB) in flight each.
        auto run = [&](auto paged_tag) {
        constexpr bool PAGED = decltype(paged_tag)::value;
        for (int c0 = r0; c0 < r1; c0 += kSubChunk) {
            const int cn = min(kSubChunk, r1 - c0);
            Tile ta, tb;
            // Physical rows, first sub-chunk: every wavefront fetches the rows of its first two
            // tiles straight from the list and has their K/V loads in flight while the sub-chunk
            // is being staged -- one trip to memory less before the first product.  Not when the
            // launch appends the newest token: a tile that names it must be loaded after the write.
            // Loads retire in order, so the order of issue is: these eight list entries, the
            // staging's list loads, the K/V loads of the two tiles (which wait for the eight
            // entries only), and then the staging consumes its entries with the K/V loads still
            // in flight behind them.
            // Only for long lists: with a few tiles per wavefront the staged route is the faster one
            // (batch 1 x 16384 tokens, 128 rows per workgroup: 7.9 us per call against 8.3; 4 x 32768,
            // 416 rows: 17.2 against 18.4; from about 1700 rows on list-direct wins by half a percent).
            const bool early = PHYS && c0 == r0 && !can_append && cn >= 1024;   // uniform over the workgroup
            int er[2][kLoads];
            if (early) {
#pragma unroll
                for (int u = 0; u < 2; ++u)
#pragma unroll
                    for (int i = 0; i < kLoads; ++i)
                        er[u][i] = idx_row[c0 + min(16 * (wave + 4 * u) + kRowsPerLoad * i + lr, cn - 1)];
            }
            auto early_tiles = [&]() {
                if (early) {
                    KASCADE_SCHED_FENCE();
#pragma unroll
                    for (int u = 0; u < 2; ++u)
#pragma unroll
                        for (int i = 0; i < kLoads; ++i)
                            load_row(paged_tag, max(0, min(er[u][i], p.max_row)), u ? tb : ta, i);
                    KASCADE_SCHED_FENCE();
                }
            };
            __syncthreads();
            // all of a thread's index loads first, then all of its block-table loads: two trips to
            // memory per sub-chunk instead of two per entry (the count per thread is a compile-time
            // constant per case, so that short lists do not pay for eight loads)
            auto stage = [&](auto per_tag) {
                constexpr int kPer = decltype(per_tag)::value;
                int toks[kPer], rows[kPer];
#pragma unroll
                for (int j = 0; j < kPer; ++j) toks[j] = idx_row[c0 + min(tid + j * kThreads, cn - 1)];
                early_tiles();
#pragma unroll
                for (int j = 0; j < kPer; ++j) {
                    // a corrupt entry must not leave the sequence (the cache, for physical rows)
                    toks[j] = max(0, min(toks[j], PHYS ? p.max_row : seqlen - 1));
                    rows[j] = (PAGED && !PHYS) ? p.block_table[(size_t)b * p.max_pages + (toks[j] >> p.page_shift)] : toks[j];
                }
#pragma unroll
                for (int j = 0; j < kPer; ++j) {
                    const int i = tid + j * kThreads;
                    if (i < cn) {
                        if (toks[j] == (PHYS ? newest_row : newest)) s_found = c0;
                        s_row[i] = (PAGED && !PHYS) ? (rows[j] << p.page_shift) + (toks[j] & page_mask) : rows[j];
                    }
                }
            };
            if (cn <= kThreads) stage(std::integral_constant<int, 1>{});
            else if (cn <= 2 * kThreads) stage(std::integral_constant<int, 2>{});
            else if (cn <= 4 * kThreads) stage(std::integral_constant<int, 4>{});
            else stage(std::integral_constant<int, kSubChunk / kThreads>{});
            __syncthreads();
            if (can_append && s_found == c0) {   // c0 differs per sub-chunk: no reset needed
                write_newest();
                __syncthreads();
            }
            auto issue = [&](int t, Tile& tb) {   // tile t: rows [16t, 16t+16) of the sub-chunk
#pragma unroll
                for (int i = 0; i < kLoads; ++i)      // past the end: clamped, masked later
                    load_row(paged_tag, s_row[min(16 * t + kRowsPerLoad * i + lr, cn - 1)], tb, i);
            };
            const int ntiles = (cn + 15) / 16;
            int t_first = wave;
            if (early) {   // tiles wave and wave + 4 are in flight already
                compute_tile(ta, 16 * wave + 4 * dq, cn);
                KASCADE_SCHED_FENCE();
                issue(wave + 8, ta);
                KASCADE_SCHED_FENCE();
                compute_tile(tb, 16 * (wave + 4) + 4 * dq, cn);
                KASCADE_SCHED_FENCE();
                t_first = wave + 8;
            } else {
                issue(wave, ta);
            }
            for (int t = t_first; t < ntiles; t += 8) {
                issue(t + 4, tb);
                KASCADE_SCHED_FENCE();   // the scheduler otherwise sinks the loads down to their first use
                compute_tile(ta, 16 * t + 4 * dq, cn);
                KASCADE_SCHED_FENCE();
                issue(t + 8, ta);
                KASCADE_SCHED_FENCE();
                compute_tile(tb, 16 * (t + 4) + 4 * dq, cn);
                KASCADE_SCHED_FENCE();
            }
        }
        };
        if (p.block_table) run(std::true_type{}); else run(std::false_type{});
    } else {
        // Token range [r0, r1) (dense baseline, anchor passes): no staging.  A wavefront owns 256
        // consecutive tokens of every 1024 and walks them in tiles of 16, four consecutive tiles
        // (one 64-token granule of the score codes) per loop iteration: 16 KB in flight per
        // wavefront (two tiles of K and V, or four of K alone), block table entries one round
        // further ahead so that no row address waits for its page number.
        const int cn = r1 - r0;
        const int* bt_row = p.block_table ? p.block_table + (size_t)b * p.max_pages : nullptr;
        constexpr int kDepth = WITH_V ? 2 : 4;
        constexpr int kTilesPerStrip = kStripRows / 16;
        auto run = [&](auto paged_tag) {
        constexpr bool PAGED = decltype(paged_tag)::value;
        // tile k of this wavefront: 16 keys from row (k / 16) * 1024 + wave * 256 + (k % 16) * 16
        auto tile_row = [&](int k) { return (k / kTilesPerStrip) * (4 * kStripRows) + wave * kStripRows + (k % kTilesPerStrip) * 16; };
        auto tok_of = [&](int k, int i) { return min(r0 + tile_row(k) + kRowsPerLoad * i + lr, r1 - 1); };   // past the end: clamped, masked later
        auto fetch_pages = [&](int k, int (&pg)[kLoads]) {
#pragma unroll
            for (int i = 0; i < kLoads; ++i) pg[i] = PAGED ? bt_row[tok_of(k, i) >> p.page_shift] : 0;
        };
        auto issue = [&](int k, const int (&pg)[kLoads], Tile& tb) {
#pragma unroll
            for (int i = 0; i < kLoads; ++i) {
                const int tok = tok_of(k, i);
                load_row(paged_tag, PAGED ? (pg[i] << p.page_shift) + (tok & page_mask) : tok, tb, i);
            }
        };
        if (cn > 0) {
            const int nsup = (cn + 4 * kStripRows - 1) / (4 * kStripRows);
            const int ntile = nsup * kTilesPerStrip;   // the same for every wavefront
            Tile buf[kDepth];
            int pgn[kDepth][kLoads];
#pragma unroll
            for (int j = 0; j < kDepth; ++j) {
                fetch_pages(j, pgn[j]);
                issue(j, pgn[j], buf[j]);
            }
#pragma unroll
            for (int j = 0; j < kDepth; ++j) fetch_pages(kDepth + j, pgn[j]);
            for (int k = 0; k < ntile; k += 4) {   // four consecutive tiles: one granule of 64 tokens
                float4_t sc[4];
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const int jb = j % kDepth;
                    sc[j] = compute_tile(buf[jb], tile_row(k + j) + 4 * dq, cn);
                    KASCADE_SCHED_FENCE();
                    issue(k + kDepth + j, pgn[jb], buf[jb]);      // past the last tile: clamped rows, never used
                    fetch_pages(k + 2 * kDepth + j, pgn[jb]);
                    KASCADE_SCHED_FENCE();
                }
                if (WRITE_SCORES) {
                    const int sup = k / kTilesPerStrip;
                    encode_granule(sc, (sup % kCodePhase) * (4 * kStripRows) + wave * kStripRows + (k % kTilesPerStrip) * 16);
                    if ((k + 4) % (kTilesPerStrip * kCodePhase) == 0) flush_phase(sup / kCodePhase);
                }
            }
            if (WRITE_SCORES && nsup % kCodePhase != 0) flush_phase(nsup / kCodePhase);
        }
        };
        if (bt_row) run(std::true_type{}); else run(std::false_type{});
    }

    // ---- the wavefront's state: columns 0-3, the four parts of a column in lanes col + 16*dq ----
    if (WITH_V) {   // one reference per column: the partial sums just add
        lcol += __shfl_xor(lcol, 16);
        lcol += __shfl_xor(lcol, 32);
    } else {
#pragma unroll
        for (int sh = 16; sh <= 32; sh <<= 1) {
            const float mo = __shfl_xor(mcol, sh), lo = __shfl_xor(lcol, sh);
            const float mx = fmaxf(mcol, mo);
            const float mref = (mx == -INFINITY) ? 0.f : mx * kScaleLog2;
            lcol = lcol * fast_exp2(mcol * kScaleLog2 - mref) + lo * fast_exp2(mo * kScaleLog2 - mref);
            mcol = mx;
        }
    }
    if (col < gs) {
        if (dq == 0) {
            s_merge[wave].m[col] = mcol;
            s_merge[wave].l[col] = lcol;
        }
        if (WITH_V) {
#pragma unroll
            for (int blk = 0; blk < kOBlocks; ++blk)
                *reinterpret_cast<float4_t*>(&s_merge[wave].acc[col][16 * blk + 4 * dq]) = oacc[blk];
        }
    }
    __syncthreads();
    // ---- merge the four wavefronts; thread -> (head, two d's), four heads at a time ----
#pragma unroll
    for (int h = tid >> 6; h < HS; h += 4) {
        if (h >= gs) break;                              // uniform over the wavefront
        const bool has_d = (tid & 63) * 2 < D;           // at D = 64 half of the lanes have no output element
        const int d0 = has_d ? (tid & 63) * 2 : 0;
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
        const size_t ph = ((size_t)b * nheads + g * gs + h) * p.num_split + split;
        const float lse_part = (L > 0.f) ? (fast_log2(L) + mref) : -INFINITY;
        const float inv = (L > 0.f) ? 1.f / L : 0.f;
        if (p.counters == nullptr) {
            if ((tid & 63) == 0) p.glse[ph] = lse_part;
            if (WITH_V && has_d) *reinterpret_cast<float2*>(p.opart + ph * D + d0) = make_float2(o0 * inv, o1 * inv);
        } else {
            // read by another workgroup of this launch: device-coherent stores
            if ((tid & 63) == 0) store_device(p.glse + ph, lse_part);
            if (WITH_V && has_d) store_device2(p.opart + ph * D + d0, o0 * inv, o1 * inv);
        }
    }
    // splits that no workgroup takes (sequences shorter than the longest) count as empty for
    // the kernels that merge all num_split partial log-sums
    if (split == 0) {
        const int missing = p.num_split - nsplit_b;
        for (int i = tid; i < gs * missing; i += kThreads)
            p.glse[((size_t)b * nheads + g * gs + i / missing) * p.num_split + nsplit_b + i % missing] = -INFINITY;
    }
    // ---- fused combine: the last workgroup of (b, g) to arrive merges the splits ----
    // The partial results above are written through to device-coherent memory and the barrier
    // waits for those stores before thread 0 counts this workgroup in; the merging workgroup
    // reads them back with device-coherent loads.  No device-wide fence is involved: one per
    // workgroup would write back and invalidate the L2 that the K/V stream lives in.
    if (p.counters == nullptr) return;
    // Every wavefront waits until its own stores above have been acknowledged (they are
    // write-through at device scope, so an acknowledged store is in device-coherent memory) and
    // only then joins the barrier.  The barrier by itself does not do this: at workgroup scope
    // the compiler may leave the wait for outstanding stores out of the barrier's fences.
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    if (tid == 0) {
        const int arrived = __hip_atomic_fetch_add(&p.counters[b * kvh + g], 1, __ATOMIC_RELAXED,
                                                   __HIP_MEMORY_SCOPE_AGENT);
        s_last = (arrived == nsplit_b - 1);
    }
    __syncthreads();
    if (!s_last) return;
    if (tid == 0)   // ready for the next launch
        __hip_atomic_store(&p.counters[b * kvh + g], 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
#pragma unroll
    for (int hh = wave; hh < HS; hh += 4) {
        if (hh >= gs) break;   // uniform over the wavefront
        // wavefront -> head (four at a time); lanes over the splits for the reductions, then two
        // d's per lane
        const int head = g * gs + hh;
        const int ns = nsplit_b;   // the splits of this sequence that exist
        const size_t base = ((size_t)b * nheads + head) * p.num_split;
        const float* gl = p.glse + base;
        const bool has_d = lane * 2 < D;
        const float* op = p.opart + base * D + (has_d ? lane * 2 : 0);
        // the first partial outputs are requested together with the log-sums, so that short
        // split lists cost one trip to memory, not two
        constexpr int kEarly = 16;
        float2 xe[kEarly];
        if (WITH_V) {
#pragma unroll
            for (int j = 0; j < kEarly; ++j) xe[j] = load_device2(op + (size_t)min(j, ns - 1) * D);
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
        if (p.row_sums && lane == 0) p.row_sums[(size_t)b * nheads + head] = lse;
        if (WITH_V) {
            const float lref = (lse == -INFINITY) ? 0.f : lse;
            float o0 = 0.f, o1 = 0.f;
            float wl = fast_exp2(g0 - lref);   // 0 in lanes beyond the split count
            // batches of kEarly partial outputs, every load of a batch in flight before the first
            // is used (the first batch has been since before the log-sums were read)
            for (int s0 = 0; s0 < ns; s0 += kEarly) {
                if (s0 > 0) {
                    if ((s0 & 63) == 0) wl = (s0 + lane < ns) ? fast_exp2(load_device(gl + s0 + lane) - lref) : 0.f;
#pragma unroll
                    for (int j = 0; j < kEarly; ++j) xe[j] = load_device2(op + (size_t)min(s0 + j, ns - 1) * D);
                }
#pragma unroll
                for (int j = 0; j < kEarly; ++j) {
                    const float w = __shfl(wl, (s0 & 63) + j);   // 0 for splits that do not exist
                    o0 += w * xe[j].x;
                    o1 += w * xe[j].y;
                }
            }
            x2_t o = {(T)o0, (T)o1};
            if (has_d) *reinterpret_cast<x2_t*>((T*)p.out + ((size_t)b * nheads + head) * D + lane * 2) = o;
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

template <bool WITH_V, int D, typename T>
__global__ __launch_bounds__(128) void decode_combine_kernel(const float* __restrict__ glse,
                                                            const float* __restrict__ opart,
                                                            T* __restrict__ out,
                                                            float* __restrict__ row_sums,
                                                            int num_split) {
    __shared__ float s_w[kCombineLds];
    __shared__ float s_red[2];
    const int h = blockIdx.x;
    const int b = blockIdx.y;
    const int nheads = gridDim.x;
    const int d = threadIdx.x;            // threads beyond D only take part in the reductions
    const size_t base = ((size_t)b * nheads + h) * num_split;
    float mx = -INFINITY;
    for (int s = d; s < num_split; s += 128) mx = fmaxf(mx, glse[base + s]);
    mx = combine_reduce(mx, true, s_red);
    const float mref = (mx == -INFINITY) ? 0.f : mx;
    float sum = 0.f;
    for (int s = d; s < num_split; s += 128) sum += fast_exp2(glse[base + s] - mref);
    sum = combine_reduce(sum, false, s_red);
    const float lse = (sum > 0.f) ? fast_log2(sum) + mref : -INFINITY;
    if (row_sums && d == 0) row_sums[(size_t)b * nheads + h] = lse;
    if (WITH_V) {
        const float lref = (lse == -INFINITY) ? 0.f : lse;
        for (int s = d; s < min(num_split, kCombineLds); s += 128) s_w[s] = fast_exp2(glse[base + s] - lref);
        __syncthreads();
        if (d >= D) return;
        const float* op = opart + base * D + d;
        float o = 0.f;
        int s = 0;
        // a split that saw no rows leaves its partial output unwritten: select, never multiply
        for (; s + 8 <= min(num_split, kCombineLds); s += 8) {
            float x[8];
#pragma unroll
            for (int e = 0; e < 8; ++e) x[e] = op[(size_t)(s + e) * D];
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const float w = s_w[s + e];
                o += (w > 0.f) ? w * x[e] : 0.f;
            }
        }
        for (; s < num_split; ++s) {
            const float w = (s < kCombineLds) ? s_w[s] : fast_exp2(glse[base + s] - lref);
            const float x = op[(size_t)s * D];
            o += (w > 0.f) ? w * x : 0.f;
        }
        out[((size_t)b * nheads + h) * D + d] = (T)o;
    }
}

// agg[b,g,j] = fp16( sum_h exp2(s[b,gs g+h,j]*scale - lse[b,gs g+h]) ), 0 beyond the sequence; the sum
// runs over the gs query heads of KV head g.
// grid (ceil(stride/2048), G, B), 256 threads x 8 tokens.
// The per-head log-sums come either merged (row_sums_in) or as the splits' partial log-sums
// (glse [B,H,num_split]): then every workgroup merges them itself -- a wavefront per head, four
// heads at a time -- and the first workgroup of a (sequence, KV head) also writes them to
// row_sums_out, which saves the combine launch of an anchor pass that produces no output.
__global__ __launch_bounds__(256) void decode_aggregate_kernel(const float* __restrict__ scores,
                                                              const float* __restrict__ row_sums_in,
                                                              const float* __restrict__ glse, int num_split,
                                                              float* __restrict__ row_sums_out,
                                                              const int* __restrict__ seqlens,
                                                              half_t* __restrict__ agg, int gs,
                                                              int scores_stride, int uniform_len,
                                                              int len_cap) {
    constexpr int kMaxGroup = 16;
    __shared__ float s_lse[kMaxGroup];
    const int g = blockIdx.y;
    const int b = blockIdx.z;
    const int kvh = gridDim.y, nheads = gridDim.y * gs;
    // the same bound the streaming launch applied to the length: codes beyond it were never written
    const int len = max(0, min(seqlens ? seqlens[b] : uniform_len, len_cap));
    const int j0 = (blockIdx.x * 256 + threadIdx.x) * 8;
    if (glse != nullptr) {   // uniform over the launch
        const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
        for (int h = wave; h < gs; h += 4) {
            const float* gl = glse + ((size_t)b * nheads + g * gs + h) * num_split;
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
                s_lse[h] = v;
                if (blockIdx.x == 0 && row_sums_out) row_sums_out[(size_t)b * nheads + g * gs + h] = v;
            }
        }
    } else if (threadIdx.x < gs) {
        s_lse[threadIdx.x] = row_sums_in[(size_t)b * nheads + g * gs + threadIdx.x];
    }
    __syncthreads();
    if (j0 >= scores_stride) return;
    float sum[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) sum[e] = 0.f;
    const bool full = (j0 + 8 <= scores_stride) && ((scores_stride & 7) == 0);
    if (j0 < len) {   // codes and references beyond the sequence were never written
        for (int h = 0; h < gs; ++h) {
            const float* row = scores + ((size_t)b * nheads + g * gs + h) * scores_stride;
            const uint16_t* sp = reinterpret_cast<const uint16_t*>(row) + j0;
            const float ref = row[scores_stride / 2 + (j0 >> 6)] - s_lse[h];
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
    half_t* ap = agg + ((size_t)b * kvh + g) * scores_stride + j0;
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

namespace {

template <int D, typename T, int HS>
hipError_t launch_split_hs(const DecodeParams& p, bool gather, bool with_v, bool write_scores, hipStream_t stream) {
    dim3 grid(p.G, p.num_split, p.B), block(kThreads);
    if (gather && p.idx_physical) {
        hipLaunchKernelGGL((decode_split_kernel<true, true, false, true, D, T, HS>), grid, block, 0, stream, p);
    } else if (gather) {
        hipLaunchKernelGGL((decode_split_kernel<true, true, false, false, D, T, HS>), grid, block, 0, stream, p);
    } else if (write_scores) {
        if (with_v)
            hipLaunchKernelGGL((decode_split_kernel<false, true, true, false, D, T, HS>), grid, block, 0, stream, p);
        else
            hipLaunchKernelGGL((decode_split_kernel<false, false, true, false, D, T, HS>), grid, block, 0, stream, p);
    } else {
        hipLaunchKernelGGL((decode_split_kernel<false, true, false, false, D, T, HS>), grid, block, 0, stream, p);
    }
    return hipGetLastError();
}

template <int D, typename T>
hipError_t launch_split_t(const DecodeParams& p, bool gather, bool with_v, bool write_scores, hipStream_t stream) {
    if (p.gs <= 4) return launch_split_hs<D, T, 4>(p, gather, with_v, write_scores, stream);
    if (p.gs <= 8) return launch_split_hs<D, T, 8>(p, gather, with_v, write_scores, stream);
    return launch_split_hs<D, T, 16>(p, gather, with_v, write_scores, stream);
}

template <int D, typename T>
hipError_t launch_combine_t(const float* glse, const float* opart, void* out, float* row_sums, int batch, int heads,
                            int num_split, bool with_v, hipStream_t stream) {
    dim3 grid(heads, batch), block(128);
    if (with_v)
        hipLaunchKernelGGL((decode_combine_kernel<true, D, T>), grid, block, 0, stream, glse, opart,
                           static_cast<T*>(out), row_sums, num_split);
    else
        hipLaunchKernelGGL((decode_combine_kernel<false, D, T>), grid, block, 0, stream, glse, opart,
                           static_cast<T*>(out), row_sums, num_split);
    return hipGetLastError();
}

}  // namespace

// head_dim in {64, 128}, elem in {kElemF16, kElemBF16}: checked by the callers
hipError_t launch_decode_split(const DecodeParams& p, bool gather, bool with_v, bool write_scores,
                               hipStream_t stream) {
    if (p.head_dim == 128)
        return p.elem == kElemBF16 ? launch_split_t<128, bf16_t>(p, gather, with_v, write_scores, stream)
                                   : launch_split_t<128, half_t>(p, gather, with_v, write_scores, stream);
    return p.elem == kElemBF16 ? launch_split_t<64, bf16_t>(p, gather, with_v, write_scores, stream)
                               : launch_split_t<64, half_t>(p, gather, with_v, write_scores, stream);
}

hipError_t launch_decode_combine(const float* glse, const float* opart, void* out, float* row_sums,
                                 int batch, int heads, int num_split, bool with_v, int head_dim, int elem,
                                 hipStream_t stream) {
    if (head_dim == 128)
        return elem == kElemBF16
                   ? launch_combine_t<128, bf16_t>(glse, opart, out, row_sums, batch, heads, num_split, with_v, stream)
                   : launch_combine_t<128, half_t>(glse, opart, out, row_sums, batch, heads, num_split, with_v, stream);
    return elem == kElemBF16
               ? launch_combine_t<64, bf16_t>(glse, opart, out, row_sums, batch, heads, num_split, with_v, stream)
               : launch_combine_t<64, half_t>(glse, opart, out, row_sums, batch, heads, num_split, with_v, stream);
}

hipError_t launch_decode_aggregate(const float* scores, const float* row_sums_in, const float* glse,
                                   int num_split, float* row_sums_out, const int* seqlens,
                                   half_t* agg, int batch, int groups, int group_size, int scores_stride,
                                   int uniform_len, int len_cap, hipStream_t stream) {
    dim3 grid((scores_stride + 2047) / 2048, groups, batch), block(256);
    hipLaunchKernelGGL(decode_aggregate_kernel, grid, block, 0, stream, scores, row_sums_in, glse,
                       num_split, row_sums_out, seqlens, agg, group_size, scores_stride, uniform_len, len_cap);
    return hipGetLastError();
}

}  // namespace kascade
