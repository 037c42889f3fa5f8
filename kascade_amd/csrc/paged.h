// Host-visible launchers of the cache bookkeeping kernels (paged.hip).
#pragma once
#include "common.h"

namespace kascade {

hipError_t launch_paged_kv_append(half_t* Kp, half_t* Vp, const half_t* k_new, const half_t* v_new,
                                  const int* start_pos, const int* block_table, int batch,
                                  int n_new, int max_pages, int page_shift, long long sb,
                                  long long sl, long long sh, int groups, int head_dim,
                                  hipStream_t stream);

hipError_t launch_decode_budgets(int* seqlens, int advance, float percent, int batch, int* valid_rows,
                                 int* n_sel_rows, hipStream_t stream);

struct RopeAppendParams {
    const half_t* q_in;       // [B,n,H,D] through (q_sb, q_sl, q_sh)
    const half_t* k_in;       // [B,n,G,D] through (kv_sb, kv_sl, kv_sh); v_in shares the strides
    const half_t* v_in;
    const float* cos_sin;     // [max_pos, D]: cos of the 64 pair angles, then their sin
    const half_t* q_weight;   // [D] or null: RMS normalisation of every query head
    const half_t* k_weight;   // [D] or null
    const int* start_pos;     // [B]; token t of sequence b sits at start_pos[b] + pos_offset + t
    half_t* q_out;            // [B,n,H,D] contiguous
    half_t* Kp;               // [num_pages, page, G, D]
    half_t* Vp;
    const int* block_table;   // [B,max_pages]
    long long q_sb, q_sl, q_sh, kv_sb, kv_sl, kv_sh;
    float eps;
    int pos_offset, batch, n_new, max_pages, page_shift, max_pos;
};

hipError_t launch_rope_append(const RopeAppendParams& p, hipStream_t stream);

}  // namespace kascade
