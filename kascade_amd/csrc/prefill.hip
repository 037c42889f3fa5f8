// Prefill attention kernels for gfx950 (fp16/bf16 MFMA 32x32x16, fp32 softmax).
//
// prefill_attn_kernel -- flash attention over one (query block, KV head, batch)
//   per workgroup; 4 wavefronts, wavefront w owns q-head 4g+w and 32*NQB queries,
//   so the four heads of a KV head share every K/V tile staged in LDS.
//   Three key regimes (REUSE): dense causal, gathered top-k rows through the
//   tile's index list, and the within-tile causal diagonal.
//
//   K/V tiles go from global memory straight into LDS (global_load_lds_dwordx4: no staging
//   registers, no LDS store instructions) into one of two buffers, so a tile costs one
//   barrier: wait for the own loads, barrier, start the next tile's loads into the other
//   buffer, compute.  Rows lie in LDS as they lie in memory; the 16-byte chunk c of row R
//   sits at chunk c ^ swz(R), chosen by the lane that fetches it (each lane picks the global
//   chunk that belongs at its LDS position), which makes both read patterns below free of
//   bank conflicts without padding.
//
//   The kernel works on S^T = K Q^T so that each lane owns one query column:
//   row max / row sum are in-lane reductions plus one cross-half exchange, and
//   the exponentiated scores are already in the B-operand layout of the second
//   product O^T = V^T P^T -- P never leaves registers.  The A operand of that product,
//   V^T, comes out of the row-major V tile through the transposing LDS read
//   ds_read_b64_tr_b16 (two per operand: four keys each).
//
// prefill_aggregate_kernel -- pooled tile scores: S = Q_tile K^T with the 128
//   (query, head) rows of a tile held as A operands in registers by every
//   wavefront; each wavefront takes 32 keys of a 128-key tile, so pooling over
//   rows is an in-lane sum over accumulator registers.
#include "prefill.h"
#include "prefill_tile.h"

#include <algorithm>
#include <type_traits>

// Wave priority around the phases of a tile.  Two wavefronts share a SIMD; which of them the
// scheduler serves first when both have an instruction ready decides how well one's softmax hides
// under the other's matrix instructions.  Modes: 0 none; 1 the wavefront in its softmax goes first;
// 2 the one in its products; 4 the one in its second product only; 5 the one in its first product
// only.  Measured at 32K tokens against mode 0 (same box, two rounds): kernels with a second
// product mode 2 -1.1 % (reuse) / -1.4 % (dense), mode 1 +1.2 %, mode 4 +1 %, mode 5 -0.5 %; the
// K-only log-sum pass mode 1 -2.6 %, mode 2 -0.8 %, mode 5 -0.5 %; the pooling kernel mode 2 -1.9 %,
// mode 1 -1.7 %.
#ifndef KASCADE_PRIO_V
#define KASCADE_PRIO_V 2
#endif
#ifndef KASCADE_PRIO_K
#define KASCADE_PRIO_K 1
#endif
#ifndef KASCADE_PRIO_AGG
#define KASCADE_PRIO_AGG 2
#endif

namespace kascade {

namespace {

constexpr int kThreads = 256;
constexpr int kAggKT = 128;        // keys per tile (aggregate kernel)

// phase: 0 = first product begins, 1 = softmax begins, 2 = second product begins (or the tile ends)
template <int MODE> __device__ __forceinline__ void tile_phase(int phase) {
    if (MODE == 1) { if (phase == 1) __builtin_amdgcn_s_setprio(1); else if (phase == 2) __builtin_amdgcn_s_setprio(0); }
    if (MODE == 2) { if (phase == 1) __builtin_amdgcn_s_setprio(0); else if (phase == 2) __builtin_amdgcn_s_setprio(1); }
    if (MODE == 4) { if (phase == 0) __builtin_amdgcn_s_setprio(0); else if (phase == 2) __builtin_amdgcn_s_setprio(1); }
    if (MODE == 5) { if (phase == 0) __builtin_amdgcn_s_setprio(1); else if (phase == 1) __builtin_amdgcn_s_setprio(0); }
}

// Queries are rows [0, Lq) of Q at global positions q_start + row (q_start a multiple of 32);
// keys are positions [0, L) with L = q_start + Lq.  PAGED: K/V are pages [P, page, G, D]
// addressed through the block table, and gathered index rows hold physical row numbers.
// EXACT_SUM: the softmax denominators are summed in fp32 from the unrounded exponentials (the
// passes whose log-sum is an output); otherwise reuse units sum them as they enter the second product.
template <int NQB, bool REUSE, bool WITH_V, bool PAGED, int D, typename T, bool EXACT_SUM = false>
__device__ __forceinline__ void prefill_attn_body(const PrefillParams& p, T* sK, T* sV) {
    typedef typename Elem<T>::x8 x8_t;
    typedef typename Elem<T>::x4 x4_t;
    typedef typename Elem<T>::x2 x2_t;
    typedef AttnTile<D> G_;
    constexpr int kKT = G_::kKT, kKS = G_::kKS, kDB = G_::kDB, kKB = G_::kKB, kChunks = G_::kChunks;
    constexpr int kRPL = G_::kRowsPerLoad, kTileElems = G_::kTileElems;
    constexpr float kScaleLog2 = ScaleLog2<D>::value;
    const HeadSlots hs = head_slots(p.gs);
    const int kvh = p.G, nheads = p.G * hs.gs;
    const T* Qp = (const T*)p.Q;
    const T* Kp = (const T*)p.K;
    const T* Vp = (const T*)p.V;

    constexpr int QT = 32 * NQB;
    const int Lq = p.Lq;            // rows of Q and of the outputs per sequence
    const int nqt = (Lq + QT - 1) / QT;
    int blk, g, b;
    unit_of_workgroup(p.B, p.G * hs.subs, nqt, blk, g, b);   // g: KV head and sub-group
    int q_start, Lqv;               // this sequence's first position and how many of the rows are its own
    chunk_of_sequence(p, b, q_start, Lqv);
    const int L = q_start + Lqv;    // keys of this sequence
    int sub = 0;
    if (hs.subs > 1) {
        sub = g % hs.subs;
        g /= hs.subs;               // the KV head
    }
    const int tq = nqt - 1 - blk;   // long (late) query blocks first
    const int tid = threadIdx.x;
    const int wave = tid >> 6;
    const int lane = tid & 63;
    const int li = lane & 31;
    const int lg = lane >> 5;
    const int q0l = tq * QT;            // first query row of this block
    if (q0l >= Lqv) return;             // a block past this sequence's rows (uniform over the workgroup)
    const int q0 = q_start + q0l;       // its global position
    const int head = g * hs.gs + min(4 * sub + wave, hs.gs - 1);
    const bool real_head = 4 * sub + wave < hs.gs;   // a slot beyond the last head computes along and stores nothing

    // ---- key regime of this block ----
    bool sparse = false;
    int n = 0, ng = 0;
    const int* idx_row = nullptr;
    if (REUSE) {
        // a sequence of a mixed batch keeps the budget it has on its own (the rows are as wide as
        // the longest sequence needs)
        const int width = p.q_start_rows ? min(p.max_topk, topk_width_of(p.topk_percent, L)) : p.max_topk;
        n = (p.rolling && L > 128) ? rolling_budget(p.topk_percent, q0) : width;
        n = min(n, width);
        if (q0 > n) {
            sparse = true;
            ng = (n + kKT - 1) / kKT;
            const int src = max(0, min(p.head_map[g], kvh - 1));   // a map built for another head count must not leave the tensor
            idx_row = p.idx + (((long long)b * kvh + src) * p.T + tq) * p.max_topk;
        }
    }
    const int ntiles = sparse ? ng + 1 : (min(q0 + QT, L) + kKT - 1) / kKT;
    const bool idx_vec = REUSE && (p.max_topk & 3) == 0 && (reinterpret_cast<uintptr_t>(p.idx) & 15) == 0;

    // ---- tile staging: wavefront w fills rows [4w R, 4(w+1) R) of a tile with four loads of R rows
    // each (R = 4 at D = 128, 8 at D = 64); lane = (row within the load, chunk position) ----
    const int wave_u = __builtin_amdgcn_readfirstlane(wave);
    const int lrow = lane / kChunks;
    const int lchunk = lane % kChunks;
    // This lane's four rows sit at LDS rows slot0 + j R (j = load) and hold the four consecutive
    // tile positions pos0 + j: one 16-byte load brings their four indices, one block-table entry
    // covers their page, and the rows of a tile in LDS are a permutation of its keys -- which only
    // the masks need to know (both products contract over the same order).
    const int slot0 = wave * 4 * kRPL + lrow;
    const int pos0 = 4 * (wave * kRPL + lrow);
    int coff[4];                                 // element offset of the chunk this lane fetches for row j
#pragma unroll
    for (int j = 0; j < 4; ++j) coff[j] = (lchunk ^ swz<D>(slot0 + j * kRPL)) * 8;
    // tile position of LDS row `slot`
    auto pos_of_slot = [](int slot) { return 4 * ((slot / (4 * kRPL)) * kRPL + slot % kRPL) + (slot / kRPL) % 4; };
    const T* kbase = PAGED ? Kp + (long long)g * D : Kp + (long long)b * p.k_sb + (long long)g * p.k_sh;
    const T* vbase = PAGED ? Vp + (long long)g * D : Vp + (long long)b * p.k_sb + (long long)g * p.k_sh;
    const int* bt_row = PAGED ? p.block_table + (long long)b * p.max_pages : nullptr;
    const int page_mask = (1 << p.page_shift) - 1;
    const int max_row = PAGED ? (p.num_pages << p.page_shift) - 1 : 0;
    const uint32_t lds_k = lds_address(sK) + wave_u * 4096;   // this wavefront's 4 KB of a K buffer
    const uint32_t lds_v = WITH_V ? lds_address(sV) + wave_u * 4096 : 0;

    // key position `pos` of tile `ti` -> key id (contiguous and diagonal tiles)
    auto tile_key = [&](int ti, int pos) {
        return min((sparse ? q0 : ti * kKT) + pos, L - 1);
    };
    // ids[j]: what the loads of row j of the next tile need, fetched a tile ahead so that the
    // loads never wait on it.  Gathered tiles: the key id (physical row when PAGED).
    // Consecutive keys, PAGED: the block-table entry of the key's page.  Consecutive keys,
    // strided: nothing (addresses follow from the tile index).
    int ids[4];
    int pend_ti = 0;        // tile the ids belong to
    const unsigned row_stride = PAGED ? (unsigned)(kvh * D) : (unsigned)p.k_sl;   // host checks < 2^31
    auto fetch_ids = [&](int ti) {
        pend_ti = ti;
        if (sparse && ti < ng) {   // values are bounded at use
            if (idx_vec) {   // list length and n are multiples of four: a group lies inside the list or outside
                const int4_t v = *reinterpret_cast<const int4_t*>(idx_row + min(ti * kKT + pos0, n - 4));
#pragma unroll
                for (int j = 0; j < 4; ++j) ids[j] = v[j];
            } else {
#pragma unroll
                for (int j = 0; j < 4; ++j) ids[j] = idx_row[min(ti * kKT + pos0 + j, n - 1)];
            }
        } else if (PAGED) {   // four consecutive keys from a multiple of four on: one page
            ids[0] = bt_row[tile_key(ti, pos0) >> p.page_shift];
        }
    };
    // Row addresses of the tile whose ids are held (element offsets from kbase / vbase).  The
    // loads themselves are issued one at a time between the matrix instructions of the first
    // product: a wavefront that issued all eight at once would sit in front of the memory
    // pipeline, which takes 16 cycles per 1 KB load, with nothing running behind it.
    long long off[4];
    auto next_offsets = [&]() {
        if (sparse && pend_ti < ng) {
#pragma unroll
            for (int j = 0; j < 4; ++j) {   // a corrupt index must not leave the tensor
                const int row = max(0, min(ids[j], PAGED ? max_row : L - 1));
                off[j] = (long long)((unsigned long long)(unsigned)row * row_stride) + coff[j];
            }
        } else {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int key = tile_key(pend_ti, pos0 + j);
                const int row = PAGED ? (ids[0] << p.page_shift) + (key & page_mask) : key;
                off[j] = (long long)((unsigned long long)(unsigned)row * row_stride) + coff[j];
            }
        }
    };
    constexpr int kNumLoads = WITH_V ? 8 : 4;
    auto issue_load = [&](int i, int buf) {   // i < 4: K row group i; else V row group i - 4
        if (i < 4) load_to_lds_16(kbase + off[i], lds_k + buf * (kTileElems * 2) + i * 1024);
        else load_to_lds_16(vbase + off[i - 4], lds_v + buf * (kTileElems * 2) + (i - 4) * 1024);
    };
    // LDS read positions (elements, within a tile buffer).  A operand of S^T: row 32 kb + li,
    // chunk 2 ks + lg.  A operand of O^T (two transposing reads h = 0, 1 of four keys each):
    // the 16 lanes of a group address rows 16 s + 8 h + 4 lg + (0..3) of a key block, 16 columns
    // of V from column 32 db + 16 (group & 1) on, and receive one column of the four rows each.
    const int kx = lg ^ swz<D>(li);
    const int krd = li * D;
    const int vcol = lane & 15;
    const int vrow = 4 * lg + (vcol >> 2);                          // + 32 kb + 16 s + 8 h
    const int vchunk = 2 * ((lane >> 4) & 1) + ((vcol >> 1) & 1);    // + 4 db
    const int vrd = vrow * D + 4 * (vcol & 1);

    // Softmax state.  m[] is the reference the exponentials are taken against, in log2 units of
    // the scaled scores.  It follows the running maximum lazily: a tile moves it only when one of
    // its scores lies more than kRefSlack above it, so an exponential never exceeds 2^kRefSlack
    // (representable in fp16 and bf16, sums and products are kept in fp32) and the rescaling of the
    // accumulators -- 64 products per lane -- runs on the first tiles of a unit and then almost
    // never.  The quotient is the same: numerator and denominator carry the same factor.
    constexpr int kPrio = WITH_V ? KASCADE_PRIO_V : KASCADE_PRIO_K;
    constexpr float kRefSlack = 8.f;
    // Reuse units sum the exponentials as they enter the second product (rounded to the element
    // type, two per instruction); the passes whose log-sum feeds the selection sum them in fp32.
    constexpr bool kPairSum = REUSE && WITH_V && !EXACT_SUM;
    float m[NQB], l[NQB];
    float16_t oT[NQB][kDB];
#pragma unroll
    for (int qb = 0; qb < NQB; ++qb) {
        m[qb] = -INFINITY;
        l[qb] = 0.f;
#pragma unroll
        for (int db = 0; db < kDB; ++db)
#pragma unroll
            for (int v = 0; v < 16; ++v) oT[qb][db][v] = 0.f;
    }

    // Order of the tiles.  A sparse unit takes its diagonal tile first: the keys q0 .. q0+31 need
    // no index list, so their loads leave at once and the first products run while the list of
    // the first gathered tile and then its rows are still on their way -- one dependent trip to
    // memory less before the first product of every unit, and units are short (28 tiles on
    // average under rolling budgets).  Softmax is accumulated online, so the order is free.
    auto tile_at = [&](int s) { return (REUSE && sparse) ? (s == 0 ? ng : s - 1) : s; };
    fetch_ids(tile_at(0));
    next_offsets();
#pragma unroll
    for (int i = 0; i < kNumLoads; ++i) issue_load(i, 0);
    if (ntiles > 1) fetch_ids(tile_at(1));

    // ---- Q fragments (B operand of S^T): query li (+32 qb), d chunk 16*ks + 8*lg; requested after
    // the first tile's rows, which the first barrier waits for ----
    x8_t qf[NQB][kKS];
#pragma unroll
    for (int qb = 0; qb < NQB; ++qb) {
        const int ql = q0l + 32 * qb + li;
        const bool ok = ql < Lqv;
        const T* qp = Qp + (long long)b * p.q_sb + (long long)min(ql, Lqv - 1) * p.q_sl +
                      (long long)head * p.q_sh + lg * 8;
#pragma unroll
        for (int ks = 0; ks < kKS; ++ks) {
            PackT<T> t;
            t.u = ld_global_16(qp + ks * 16);
            if (!ok) t.u = uint4_t{0, 0, 0, 0};
            qf[qb][ks] = t.v8;
        }
    }

    // One tile: registers -> LDS, next tile's loads, both products, softmax.  Three copies of
    // the code, each straight-line: tiles that need no mask (all but one or two of a unit), tiles
    // that do (the causal edge, the end of the sequence, a selection that ends inside a tile), and
    // the diagonal tile of a sparse unit (32 keys: half the products).
    constexpr int kFull = 0, kMasked = 1, kDiag = 2;
    auto run_tile = [&](int sq, auto mode_c) {
        constexpr int MODE = decltype(mode_c)::value;
        constexpr int nkb = (MODE == kDiag && QT == 32) ? 1 : kKB;
        const int ti = tile_at(sq);
        const T* bK = sK + (sq & 1) * kTileElems;
        const T* bV = sV + (sq & 1) * kTileElems;
        // own loads of this tile landed; after the barrier everybody's have, and everybody is done
        // reading the other buffer (the tile before), which the next tile's loads may now fill
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
        // The next tile's loads go out between the products below, unconditionally: after the last
        // tile they fetch its rows once more into the idle buffer (1/28 of the traffic on average,
        // from the cache) rather than put a branch between the matrix instructions.
        if (sq + 1 < ntiles) next_offsets();
        const int nbuf = (sq + 1) & 1;

        tile_phase<kPrio>(0);
        // ---- S^T = K_tile Q^T.  Step c = (key block c / kKS, contraction step c % kKS); operands are
        // read from LDS two windows (four steps) ahead of the products that use them, in program
        // order, because LDS reads do not move across the load statements ----
        constexpr int kSteps = nkb * kKS;
        float16_t sT[NQB][nkb];
        float16_t zero16;
#pragma unroll
        for (int v = 0; v < 16; ++v) zero16[v] = 0.f;
        auto read_a = [&](int c) {
            return *reinterpret_cast<const x8_t*>(&bK[32 * (c / kKS) * D + krd + ((2 * (c % kKS)) ^ kx) * 8]);
        };
        constexpr int kAhead = (kKB <= 2) ? 2 : 1;   // windows read ahead (registers are scarcer at D = 64)
        x8_t aw[kAhead + 1][2];
#pragma unroll
        for (int c = 0; c < 2 * kAhead && c < kSteps; ++c) aw[c >> 1][c & 1] = read_a(c);
#pragma unroll
        for (int w = 0; w < kSteps / 2; ++w) {
            if (2 * (w + kAhead) < kSteps) {
                aw[(w + kAhead) % (kAhead + 1)][0] = read_a(2 * (w + kAhead));
                aw[(w + kAhead) % (kAhead + 1)][1] = read_a(2 * (w + kAhead) + 1);
            }
            __builtin_amdgcn_sched_barrier(0);   // the scheduler would sink the reads to their use
#pragma unroll
            for (int i = 0; i < 2; ++i) {
                const int kb = (2 * w + i) / kKS, ks = (2 * w + i) % kKS;
#pragma unroll
                for (int qb = 0; qb < NQB; ++qb)   // the first product starts from a constant zero
                    sT[qb][kb] = Elem<T>::mma_32x32x16(aw[w % (kAhead + 1)][i], qf[qb][ks], ks == 0 ? zero16 : sT[qb][kb]);
            }
            if (w < kNumLoads) issue_load(w, nbuf);
        }
#pragma unroll
        for (int i = kSteps / 2; i < kNumLoads; ++i) issue_load(i, nbuf);
        if (sq + 2 < ntiles) fetch_ids(tile_at(sq + 2));
        // ---- masks: accumulator v of key block kb is LDS row 32kb + 8(v/4) + 4lg + v%4 of the tile ----
        if (MODE != kFull) {
            const bool diag_here = MODE == kDiag || (sparse && ti == ng);
            if (sparse && !diag_here) {   // a selection that ends inside this tile
#pragma unroll
                for (int qb = 0; qb < NQB; ++qb)
#pragma unroll
                    for (int kb = 0; kb < nkb; ++kb)
#pragma unroll
                        for (int v = 0; v < 16; ++v) {
                            const int pos = ti * kKT + pos_of_slot(32 * kb + 8 * (v >> 2) + 4 * lg + (v & 3));
                            if (pos >= n) sT[qb][kb][v] = -INFINITY;
                        }
            } else {                           // the causal edge and the end of the sequence
                const int kstart = diag_here ? q0 : ti * kKT;
#pragma unroll
                for (int qb = 0; qb < NQB; ++qb) {
                    const int q = q0 + 32 * qb + li;   // global position
#pragma unroll
                    for (int kb = 0; kb < nkb; ++kb)
#pragma unroll
                        for (int v = 0; v < 16; ++v) {
                            const int key = kstart + pos_of_slot(32 * kb + 8 * (v >> 2) + 4 * lg + (v & 3));
                            if (key > q || key >= L) sT[qb][kb][v] = -INFINITY;
                        }
                }
            }
        }
        // ---- online softmax (one query column per lane pair: lanes li and li + 32) ----
        tile_phase<kPrio>(1);
        x8_t pf[NQB][2 * nkb];
#pragma unroll
        for (int qb = 0; qb < NQB; ++qb) {
            float mx = -INFINITY;
#pragma unroll
            for (int kb = 0; kb < nkb; ++kb)
#pragma unroll
                for (int v = 0; v < 16; ++v) mx = fmaxf(mx, sT[qb][kb][v]);
            const float ms = mx * kScaleLog2;
            if (__any(ms > m[qb] + kRefSlack)) {   // wavefront-uniform
                const float mnew = fmaxf(m[qb], max_with_other_half(ms));   // the same in both lanes of a column
                const float corr = (mnew == -INFINITY) ? 1.f : fast_exp2(m[qb] - mnew);
                m[qb] = mnew;
                l[qb] *= corr;
                if (WITH_V) {
#pragma unroll
                    for (int db = 0; db < kDB; ++db)
#pragma unroll
                        for (int v = 0; v < 16; ++v) oT[qb][db][v] *= corr;
                }
            }
            const float mu = (m[qb] == -INFINITY) ? 0.f : m[qb];
#pragma unroll
            for (int kb = 0; kb < nkb; ++kb)
#pragma unroll
                for (int v = 0; v < 16; ++v)
                    sT[qb][kb][v] = fast_exp2(__builtin_fmaf(sT[qb][kb][v], kScaleLog2, -mu));
            float sum = 0.f;
            if (WITH_V) {
#pragma unroll
                for (int s = 0; s < 2 * nkb; ++s) {
                    x8_t t;
#pragma unroll
                    for (int e = 0; e < 8; ++e) t[e] = (T)sT[qb][s >> 1][8 * (s & 1) + e];
                    pf[qb][s] = t;
                }
            }
            if (kPairSum) {
#pragma unroll
                for (int s = 0; s < 2 * nkb; ++s)
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const x2_t pr = {pf[qb][s][2 * e], pf[qb][s][2 * e + 1]};
                        sum = Elem<T>::add_pair(pr, sum);
                    }
            } else {
#pragma unroll
                for (int kb = 0; kb < nkb; ++kb)
#pragma unroll
                    for (int v = 0; v < 16; ++v) sum += sT[qb][kb][v];
            }
            l[qb] += sum;   // per-lane partial sum (own key positions)
        }
        tile_phase<kPrio>(2);
        // ---- O^T += V^T P^T: step s covers the keys of accumulators 8(s&1) .. 8(s&1)+7 of key block
        // s/2, i.e. rows 16 s + 8 h + 4 lg + (0..3), h = 0, 1, of the tile.  The operands of a block
        // of 32 output rows are read while the block before it is multiplied ----
        if (WITH_V) {
            constexpr int kPS = 2 * nkb;
            auto read_v = [&](int db, int s, int h) {
                const int row = 16 * s + 8 * h;   // + vrow; only its low four bits enter swz
                const T* vp = bV + row * D + vrd + ((4 * db + vchunk) ^ swz<D>(row + vrow)) * 8;
                return __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) short4_t*)vp);
            };
            // steps in groups of kGrp (a group = 2 kGrp transposing reads, kGrp products per query block)
            constexpr int kGrp = (kKB <= 2) ? 4 : 2;
            constexpr int kGroupsPV = kDB * kPS / kGrp;
            short4_t av[2][kGrp][2];
#pragma unroll
            for (int i = 0; i < kGrp; ++i)
#pragma unroll
                for (int h = 0; h < 2; ++h) av[0][i][h] = read_v(i / kPS, i % kPS, h);
#pragma unroll
            for (int gq = 0; gq < kGroupsPV; ++gq) {
                if (gq + 1 < kGroupsPV) {
#pragma unroll
                    for (int i = 0; i < kGrp; ++i)
#pragma unroll
                        for (int h = 0; h < 2; ++h)
                            av[(gq + 1) & 1][i][h] = read_v((kGrp * (gq + 1) + i) / kPS, (kGrp * (gq + 1) + i) % kPS, h);
                }
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int i = 0; i < kGrp; ++i) {
                    const int db = (kGrp * gq + i) / kPS, s = (kGrp * gq + i) % kPS;
                    const short8_t both = __builtin_shufflevector(av[gq & 1][i][0], av[gq & 1][i][1], 0, 1, 2, 3, 4, 5, 6, 7);
                    const x8_t a = __builtin_bit_cast(x8_t, both);
#pragma unroll
                    for (int qb = 0; qb < NQB; ++qb)
                        oT[qb][db] = Elem<T>::mma_32x32x16(a, pf[qb][s], oT[qb][db]);
                }
            }
        }
    };

    {
        int sq = 0;
        if (REUSE && sparse) {   // a copy of its own where it halves the tile's products (64-key tiles)
            if (kKB <= 2) run_tile(0, std::integral_constant<int, kDiag>{});
            else run_tile(0, std::integral_constant<int, kMasked>{});
            sq = 1;
        }
        // tiles wholly below the unit's first query and inside the sequence / wholly inside the selection
        const int full_end = (REUSE && sparse) ? 1 + n / kKT : min((q0 + 1) / kKT, L / kKT);
        for (; sq < full_end; ++sq) run_tile(sq, std::integral_constant<int, kFull>{});
        for (; sq < ntiles; ++sq) run_tile(sq, std::integral_constant<int, kMasked>{});
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // no load may land in LDS after the workgroup has left

    // ---- epilogue (rows are local to this call).  A lane holds one query's output spread over its
    // registers; the rows go through the wavefront's share of the (now idle) K buffers so that they
    // leave as whole rows: 16-byte stores, four rows per instruction ----
    static_assert(!WITH_V || NQB == 1, "the output pass is written for 32 queries per wavefront");
    if (WITH_V) __syncthreads();   // everybody is done with the tile buffers
#pragma unroll
    for (int qb = 0; qb < NQB; ++qb) {
        const int ql = q0l + 32 * qb + li;
        const float lt = sum_with_other_half(l[qb]);
        if (p.log_sum && lg == 0 && ql < Lqv && real_head)
            p.log_sum[((long long)b * Lq + ql) * nheads + head] = fast_log2(lt) + m[qb];
        if (WITH_V) {
            T* so = sK + wave * (32 * D);
            const float inv = 1.f / lt;
#pragma unroll
            for (int db = 0; db < kDB; ++db)
#pragma unroll
                for (int v4 = 0; v4 < 4; ++v4) {   // d = 32 db + 8 v4 + 4 lg .. +3: chunk 4 db + v4 of row li
                    x4_t o = {(T)(oT[qb][db][4 * v4 + 0] * inv), (T)(oT[qb][db][4 * v4 + 1] * inv),
                              (T)(oT[qb][db][4 * v4 + 2] * inv), (T)(oT[qb][db][4 * v4 + 3] * inv)};
                    *reinterpret_cast<x4_t*>(&so[li * D + (((4 * db + v4) ^ (li & (kChunks - 1))) * 8) + 4 * lg]) = o;
                }
            __builtin_amdgcn_wave_barrier();   // the reads below are other lanes' writes (same wavefront: in order)
#pragma unroll
            for (int j = 0; j < 32 / kRPL; ++j) {
                const int r = j * kRPL + lrow;
                const uint4_t row = *reinterpret_cast<const uint4_t*>(&so[r * D + lchunk * 8]);
                const int qr = q0l + r;
                if (qr < Lqv && real_head)   // the output is not read again by these kernels: keep it out of the caches
                    __builtin_nontemporal_store(row, reinterpret_cast<uint4_t*>(
                        (T*)p.O + (((long long)b * Lq + qr) * nheads + head) * D + ((lchunk ^ (r & (kChunks - 1))) * 8)));
            }
        }
    }
}


// 32 queries per wavefront: register budget capped so that two workgroups share a
// compute unit (64 KB of LDS each: two K and two V tile buffers).
template <bool REUSE, bool WITH_V, bool PAGED, int D, typename T, bool EXACT_SUM = false>
__global__ __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(2)))
void prefill_attn_kernel_q32(PrefillParams p) {
    __shared__ __attribute__((aligned(1024))) T sK[2 * AttnTile<D>::kTileElems];
    __shared__ __attribute__((aligned(1024))) T sV[WITH_V ? 2 * AttnTile<D>::kTileElems : 8];
    prefill_attn_body<1, REUSE, WITH_V, PAGED, D, T, EXACT_SUM>(p, sK, sV);
}

// 64 queries per wavefront for the K-only log-sum pass, whose state fits 256 registers: two
// workgroups per compute unit, and the MFMA results stay in ordinary registers (with the full
// 512-register budget the compiler parks them in accumulation registers and copies each one out
// before the softmax).
template <int D, typename T>
__global__ __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(2)))
void prefill_attn_kernel_q64(PrefillParams p) {
    __shared__ __attribute__((aligned(1024))) T sK[2 * AttnTile<D>::kTileElems];
    prefill_attn_body<2, false, false, false, D, T>(p, sK, static_cast<T*>(nullptr));
}

// Pooled tile scores: out[b,g,t,key] = sum over the 32 queries of tile t and the 4 q-heads of g
// of exp2(s*scale - log_sum), for keys before the tile's first (global) position.
// Two workgroups per compute unit (register budget 256): one wavefront's exponentials run
// under the other's matrix instructions.
//
// A wavefront takes 32 keys of every 128-key tile and nobody else reads them.  Their rows go
// from global memory straight into the wavefront's own LDS area (whole rows per load: read as
// B operands directly, a 16-byte piece of 32 different rows per instruction, the same bytes kept
// the data-return path of the memory pipeline busy 96 % of the kernel) and come back as B
// operands (lane = key, 8 elements at d = 16 ks + 8 lg) from the chunk-permuted rows.  Two buffers
// per wavefront, no barrier in the tile loop: the loads of the next tile are issued one per
// contraction step and waited for at the top of that tile.
template <bool PAGED, int D, typename T>
__global__ __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(2)))
void prefill_aggregate_kernel(PrefillParams p) {
    typedef typename Elem<T>::x8 x8_t;
    constexpr int kKS = D / 16;
    constexpr int kChunks = D / 8;
    constexpr int kRPL = 64 / kChunks;          // rows per load instruction
    constexpr int kLoads = 32 / kRPL;           // load instructions per wavefront and tile
    constexpr int kWaveElems = 32 * D;          // a wavefront's 32 rows
    constexpr float kScaleLog2 = ScaleLog2<D>::value;
    const HeadSlots hs = head_slots(p.gs);
    const int kvh = p.G, nheads = p.G * hs.gs;
    const T* Qp = (const T*)p.Q;
    const T* Kp = (const T*)p.K;
    __shared__ __attribute__((aligned(1024))) T sK[2 * 4 * kWaveElems];
    __shared__ __attribute__((aligned(16))) float s_lse[128];

    const int Ls = p.L;                  // width of a row of pooled scores
    const int Lq = p.Lq;
    int blk, g, b;
    unit_of_workgroup(p.B, p.G, p.T, blk, g, b);
    int q_start, Lqv;                    // this sequence's first position and how many of the rows are its own
    chunk_of_sequence(p, b, q_start, Lqv);
    const int L = q_start + Lqv;         // keys of this sequence
    const int t = p.T - 1 - blk;
    const int tid = threadIdx.x;
    const int wave = tid >> 6;
    const int lane = tid & 63;
    const int li = lane & 31;
    const int lg = lane >> 5;
    const int tl = t * kTile;            // first query row of the tile
    const int ts = q_start + tl;         // its global position
    half_t* out = p.agg + (((long long)b * kvh + g) * p.T + t) * Ls;
    const half_t neg_inf = (half_t)(-INFINITY);

    const int ntiles = tl < Lqv ? (ts + kAggKT - 1) / kAggKT : 0;   // a tile past the sequence's rows pools nothing
    if (ntiles > 0) {
        // A operands: row block rb = head slot rb of this launch's sub-group, row li = query tl+li
        const int head0 = g * hs.gs + 4 * p.vsub;
        x8_t qa[kGroupSize][kKS];
#pragma unroll
        for (int rb = 0; rb < kGroupSize; ++rb) {
            const int q = tl + li;
            const bool ok = q < Lqv;
            const T* qp = Qp + (long long)b * p.q_sb + (long long)min(q, Lqv - 1) * p.q_sl +
                          (long long)min(head0 + rb, g * hs.gs + hs.gs - 1) * p.q_sh + lg * 8;
#pragma unroll
            for (int ks = 0; ks < kKS; ++ks) {
                PackT<T> x;
                x.u = ld_global_16(qp + ks * 16);
                if (!ok) x.u = uint4_t{0, 0, 0, 0};
                qa[rb][ks] = x.v8;
            }
        }
        if (tid < 128) {
            const int q = tl + (tid & 31);
            // a query row past the chunk, or a slot past the KV head's last query head, adds exp2(-inf) = 0
            const bool counts = q < Lqv && 4 * p.vsub + (tid >> 5) < hs.gs;
            s_lse[tid] = counts ? p.log_sum_in[((long long)b * Lq + q) * nheads + head0 + (tid >> 5)] : INFINITY;
        }

        // ---- staging: load j of a tile covers rows j kRPL + lrow of the wavefront's 32 ----
        const int wave_u = __builtin_amdgcn_readfirstlane(wave);
        const int lrow = lane / kChunks;
        const int lchunk = lane % kChunks;
        const T* kbase = PAGED ? Kp + (long long)g * D : Kp + (long long)b * p.k_sb + (long long)g * p.k_sh;
        const unsigned row_stride = PAGED ? (unsigned)(kvh * D) : (unsigned)p.k_sl;
        const int* bt_row = PAGED ? p.block_table + (long long)b * p.max_pages : nullptr;
        const int page_mask = (1 << p.page_shift) - 1;
        const uint32_t lds_w = lds_address(sK) + wave_u * (kWaveElems * 2);   // + buf * 4 * kWaveElems * 2
        const T* my_k = sK + wave * kWaveElems;
        // block-table entry of the key this lane stands for (row lane & 31 of the wavefront's 32),
        // fetched a tile ahead; the lanes of a load pick theirs up with a lane permutation
        int pg_next = 0;
        auto fetch_page = [&](int ti) {
            if (PAGED) pg_next = bt_row[min(ti * kAggKT + 32 * wave + li, L - 1) >> p.page_shift];
        };
        int pg_cur = 0;   // entries of the tile whose loads are being issued
        auto issue_load = [&](int ti, int j, int buf) {
            const int row = j * kRPL + lrow;
            const int key = min(ti * kAggKT + 32 * wave + row, L - 1);
            int src = key;
            if (PAGED) {
                const int pgv = __builtin_amdgcn_ds_bpermute(row << 2, pg_cur);
                src = (pgv << p.page_shift) + (key & page_mask);
            }
            const T* gp = kbase + (long long)((unsigned long long)(unsigned)src * row_stride) +
                          (lchunk ^ swz<D>(row)) * 8;
            load_to_lds_16(gp, lds_w + buf * (4 * kWaveElems * 2) + j * 1024);
        };
        fetch_page(0);
        pg_cur = pg_next;
#pragma unroll
        for (int j = 0; j < kLoads; ++j) issue_load(0, j, 0);
        if (ntiles > 1) fetch_page(1);
        const int kx = lg ^ swz<D>(li);
        __syncthreads();   // s_lse

        for (int ti = 0; ti < ntiles; ++ti) {
            // this tile's rows have landed (and the next tile's block-table entries arrived)
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            const T* bK = my_k + (ti & 1) * (4 * kWaveElems);
            const int tn = min(ti + 1, ntiles - 1);   // after the last tile: its rows once more, unused
            const int nbuf = (ti + 1) & 1;
            pg_cur = pg_next;
            if (ti + 2 < ntiles) fetch_page(ti + 2);

            float16_t acc[kGroupSize];
            float16_t zero16;   // the first product of a tile starts from a constant zero
#pragma unroll
            for (int v = 0; v < 16; ++v) zero16[v] = 0.f;
            auto read_b = [&](int ks) {
                return *reinterpret_cast<const x8_t*>(&bK[li * D + ((2 * ks) ^ kx) * 8]);
            };
            x8_t kb[3];
            kb[0] = read_b(0);
            if (kKS > 1) kb[1] = read_b(1);
#pragma unroll
            for (int ks = 0; ks < kKS; ++ks) {
                if (ks + 2 < kKS) kb[(ks + 2) % 3] = read_b(ks + 2);
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int rb = 0; rb < kGroupSize; ++rb)
                    acc[rb] = Elem<T>::mma_32x32x16(qa[rb][ks], kb[ks % 3], ks == 0 ? zero16 : acc[rb]);
                if (ks < kLoads) issue_load(tn, ks, nbuf);
            }
#pragma unroll
            for (int j = kKS; j < kLoads; ++j) issue_load(tn, j, nbuf);
            // accumulator v of row block rb is query row 8(v/4) + 4lg + v%4, column = key li
            tile_phase<KASCADE_PRIO_AGG>(1);
            float sum = 0.f;
#pragma unroll
            for (int rb = 0; rb < kGroupSize; ++rb)
#pragma unroll
                for (int v4 = 0; v4 < 4; ++v4) {
                    const float4_t ls = *reinterpret_cast<const float4_t*>(&s_lse[rb * 32 + 8 * v4 + 4 * lg]);
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        sum += fast_exp2(acc[rb][4 * v4 + e] * kScaleLog2 - ls[e]);
                }
            sum = sum_with_other_half(sum);
            tile_phase<KASCADE_PRIO_AGG>(2);
            const int key = ti * kAggKT + 32 * wave + li;
            if (lg == 0 && key < Ls) {
                if (key < ts)   // a later sub-group of the KV head adds to what the earlier ones left
                    out[key] = (half_t)(p.accumulate ? sum + (float)out[key] : sum);
                else if (p.fill_invalid)
                    out[key] = neg_inf;
            }
        }
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // no load may land in LDS after the workgroup has left
    }
    if (p.fill_invalid) {
        for (int key = ntiles * kAggKT + tid; key < Ls; key += kThreads) out[key] = neg_inf;
    }
}

}  // namespace

namespace {

template <int D, typename T>
hipError_t launch_attn_t(const PrefillParams& p, bool reuse, bool with_v, int nqb, hipStream_t stream) {
    const int qt = 32 * nqb;
    const bool paged = p.block_table != nullptr;
    const int nqt = (p.Lq + qt - 1) / qt;
    const int gv = p.G * head_slots(p.gs).subs;   // (KV head, sub-group of four query heads) pairs
    dim3 grid(nqt, gv, p.B), block(kThreads);
    if (pairs_fill_xcds(p.B, gv)) {
        const long long total = (long long)nqt * gv * p.B;
        if (total > 0x7fffffffLL) return hipErrorInvalidConfiguration;
        grid = dim3((unsigned)total);
    }
    if (reuse && p.log_sum) {   // a reuse pass that also reports its log-sums: fp32 sums
        if (paged)
            hipLaunchKernelGGL((prefill_attn_kernel_q32<true, true, true, D, T, true>), grid, block, 0, stream, p);
        else
            hipLaunchKernelGGL((prefill_attn_kernel_q32<true, true, false, D, T, true>), grid, block, 0, stream, p);
    } else if (paged) {
        if (reuse)
            hipLaunchKernelGGL((prefill_attn_kernel_q32<true, true, true, D, T>), grid, block, 0, stream, p);
        else if (with_v)
            hipLaunchKernelGGL((prefill_attn_kernel_q32<false, true, true, D, T>), grid, block, 0, stream, p);
        else
            hipLaunchKernelGGL((prefill_attn_kernel_q32<false, false, true, D, T>), grid, block, 0, stream, p);
    } else if (reuse) {
        hipLaunchKernelGGL((prefill_attn_kernel_q32<true, true, false, D, T>), grid, block, 0, stream, p);
    } else if (nqb == 2) {   // K-only log-sum pass
        hipLaunchKernelGGL((prefill_attn_kernel_q64<D, T>), grid, block, 0, stream, p);
    } else {
        if (with_v)
            hipLaunchKernelGGL((prefill_attn_kernel_q32<false, true, false, D, T>), grid, block, 0, stream, p);
        else
            hipLaunchKernelGGL((prefill_attn_kernel_q32<false, false, false, D, T>), grid, block, 0, stream, p);
    }
    return hipGetLastError();
}

template <int D, typename T>
hipError_t launch_aggregate_t(const PrefillParams& p, hipStream_t stream) {
    dim3 grid(p.T, p.G, p.B), block(kThreads);
    if (pairs_fill_xcds(p.B, p.G)) {
        const long long total = (long long)p.T * p.G * p.B;
        if (total > 0x7fffffffLL) return hipErrorInvalidConfiguration;
        grid = dim3((unsigned)total);
    }
    if (p.block_table)
        hipLaunchKernelGGL((prefill_aggregate_kernel<true, D, T>), grid, block, 0, stream, p);
    else
        hipLaunchKernelGGL((prefill_aggregate_kernel<false, D, T>), grid, block, 0, stream, p);
    return hipGetLastError();
}

}  // namespace

// p.head_dim in {64, 128}, p.elem in {kElemF16, kElemBF16}: checked by the callers
hipError_t launch_prefill_attn(const PrefillParams& p, bool reuse, bool with_v, int nqb,
                               hipStream_t stream) {
    if (p.head_dim == 128)
        return p.elem == kElemBF16 ? launch_attn_t<128, bf16_t>(p, reuse, with_v, nqb, stream)
                                   : launch_attn_t<128, half_t>(p, reuse, with_v, nqb, stream);
    return p.elem == kElemBF16 ? launch_attn_t<64, bf16_t>(p, reuse, with_v, nqb, stream)
                               : launch_attn_t<64, half_t>(p, reuse, with_v, nqb, stream);
}

hipError_t launch_prefill_aggregate(const PrefillParams& p0, hipStream_t stream) {
    // one launch per sub-group of four query heads; the launches after the first add to the
    // pooled scores (launches on a stream run in order)
    PrefillParams p = p0;
    const int subs = head_slots(p.gs).subs;
    for (int v = 0; v < subs; ++v) {
        p.vsub = v;
        p.accumulate = v > 0;
        hipError_t e;
        if (p.head_dim == 128)
            e = p.elem == kElemBF16 ? launch_aggregate_t<128, bf16_t>(p, stream) : launch_aggregate_t<128, half_t>(p, stream);
        else
            e = p.elem == kElemBF16 ? launch_aggregate_t<64, bf16_t>(p, stream) : launch_aggregate_t<64, half_t>(p, stream);
        if (e != hipSuccess) return e;
    }
    return hipSuccess;
}

// idx[i] (token position) -> physical row of the paged cache, in place or to another buffer.
__global__ void translate_indices_kernel(const int* __restrict__ idx, int* __restrict__ out,
                                         const int* __restrict__ block_table, long long per_seq,
                                         int max_pages, int page_shift, int L) {
    const int b = blockIdx.y;
    const int* bt = block_table + (long long)b * max_pages;
    const int mask = (1 << page_shift) - 1;
    for (long long i = blockIdx.x * (long long)blockDim.x + threadIdx.x; i < per_seq;
         i += (long long)gridDim.x * blockDim.x) {
        const int tok = max(0, min(idx[b * per_seq + i], L - 1));
        out[b * per_seq + i] = (bt[tok >> page_shift] << page_shift) + (tok & mask);
    }
}

hipError_t launch_translate_indices(const int* idx, int* out, const int* block_table, int B,
                                    long long per_seq, int max_pages, int page_shift, int L,
                                    hipStream_t stream) {
    if (per_seq <= 0 || B <= 0) return hipSuccess;
    const int blocks = (int)std::min<long long>((per_seq + 255) / 256, 4096);
    hipLaunchKernelGGL(translate_indices_kernel, dim3(blocks, B), dim3(256), 0, stream, idx, out,
                       block_table, per_seq, max_pages, page_shift, L);
    return hipGetLastError();
}

}  // namespace kascade
