// Pieces of the prefill attention kernels (prefill.hip): tile geometry, the
// LDS chunk permutation, direct-to-LDS loads, the workgroup -> unit mapping and the budgets.
#pragma once
#include "prefill.h"

namespace kascade {
namespace {

// Tile geometry of the attention kernel per head dimension.  A tile is 16 KB of K (and of V)
// whatever D: 64 keys at D = 128, 128 keys at D = 64, so a wavefront always stages a tile with
// four 1 KB loads per tensor, both products issue 16 matrix instructions per tile and wavefront,
// and the score registers a narrower head frees hold the extra keys.
template <int D> struct AttnTile {
    static constexpr int kKT = 64 * 128 / D;     // keys per tile
    static constexpr int kKS = D / 16;           // contraction steps of S^T = K Q^T
    static constexpr int kDB = D / 32;           // 32-row blocks of O^T
    static constexpr int kKB = kKT / 32;         // 32-key blocks of a tile
    static constexpr int kChunks = D / 8;        // 16-byte chunks of a row
    static constexpr int kRowsPerLoad = 64 / kChunks;   // rows one wavefront-wide 16-byte load covers
    static constexpr int kTileElems = kKT * D;   // 16 KB of K (and of V) whatever D
};

// Chunk permutation of a tile row in LDS (see the head of the file).  What it must give:
// 16 lanes reading the same chunk of 16 consecutive rows (A operand of S^T), and 32 lanes
// reading 4 consecutive rows x 4 consecutive chunks in 8-byte halves (transposing read of V),
// each touch all 64 banks once.  Rows are 256 bytes (D = 128: the row does not move the bank)
// or 128 bytes (D = 64: the row parity picks the bank half, three more row bits permute).
template <int D> __device__ __forceinline__ int swz(int row);
template <> __device__ __forceinline__ int swz<128>(int row) { return ((row & 3) << 2) | ((row >> 2) & 3); }
template <> __device__ __forceinline__ int swz<64>(int row) { return (((row >> 1) & 1) << 2) | ((row >> 2) & 3); }

// One wavefront-wide load of 16 bytes per lane from global memory into LDS: lane i's bytes
// land at lds_base + 16 i (lds_base wavefront-uniform).  Counted by vmcnt like any load; the
// compiler does not know that it writes LDS, so whoever reads the bytes waits for vmcnt and
// passes a barrier first (the tile loop does both once per tile).
__device__ __forceinline__ void load_to_lds_16(const void* gptr, uint32_t lds_base) {
    asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off"
                 :: "v"(gptr), "s"(lds_base) : "m0");
}
template <typename P> __device__ __forceinline__ uint32_t lds_address(P* ptr) {
    return (uint32_t)(size_t)(__attribute__((address_space(3))) void*)ptr;
}

// Workgroup -> (query block, KV head, sequence).  Workgroups go to the eight XCDs round-robin in
// launch order and each XCD has an L2 of its own.  When the number of (sequence, KV head) pairs
// is a multiple of eight the launch is one-dimensional and consecutive workgroups take eight
// different pairs: all units of a pair, which read the same K/V rows, run on one XCD.
__host__ __device__ inline bool pairs_fill_xcds(int B, int G) { return (B * G) % 8 == 0; }
__device__ __forceinline__ void unit_of_workgroup(int B, int G, int nblocks, int& blk, int& g, int& b) {
    if (pairs_fill_xcds(B, G)) {
        const int i = blockIdx.x;
        const int r = i >> 3;
        const int pair = (r / nblocks) * 8 + (i & 7);
        blk = r % nblocks;
        g = pair % G;
        b = pair / G;
    } else {
        blk = blockIdx.x;
        g = blockIdx.y;
        b = blockIdx.z;
    }
}

__device__ __forceinline__ int rolling_budget(float pct, int tile_start) {
    long long fl = (long long)floor((double)pct * (double)tile_start / 100.0);
    if (fl < 128) fl = 128;
    return (int)(((fl + 127) / 128) * 128);
}

// Index-row width the host gives a prompt of L keys: min(128 ceil(min(max(128, floor(pct L / 100)), L) / 128), L).
__device__ __forceinline__ int topk_width_of(float pct, int L) {
    long long k = (long long)floor((double)pct * (double)L / 100.0);
    if (k < 128) k = 128;
    if (k > L) k = L;
    k = ((k + 127) / 128) * 128;
    return (int)(k > L ? L : k);
}

// Where sequence b's rows of a chunked call stand: first global position and number of rows.
__device__ __forceinline__ void chunk_of_sequence(const PrefillParams& p, int b, int& q_start, int& rows) {
    q_start = p.q_start;
    rows = p.Lq;
    if (p.q_start_rows) {
        q_start = max(0, min(p.q_start_rows[b], p.q_start)) & ~(kTile - 1);
        if (p.q_len_rows) rows = max(0, min(p.q_len_rows[b], p.Lq));
    }
}

}  // namespace
}  // namespace kascade
