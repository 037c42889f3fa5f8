// Host-visible launchers of the cache bookkeeping kernels (paged.hip).
#pragma once
#include "common.h"

namespace kascade {

hipError_t launch_paged_kv_append(half_t* Kp, half_t* Vp, const half_t* k_new, const half_t* v_new,
                                  const int* start_pos, const int* block_table, int batch,
                                  int n_new, const int* n_new_rows, int max_pages, int page_shift, long long sb,
                                  long long sl, long long sh, int groups, int head_dim,
                                  hipStream_t stream);

hipError_t launch_decode_budgets(int* seqlens, int advance, float percent, int batch, int groups,
                                 int* valid_rows, int* n_sel_rows, hipStream_t stream);

struct RopeAppendParams {   // element tensors are fp16 or bf16 (elem), H = gs G query heads
    const void* q_in;         // [B,n,H,D] through (q_sb, q_sl, q_sh)
    const void* k_in;         // [B,n,G,D] through (kv_sb, kv_sl, kv_sh); v_in shares the strides
    const void* v_in;
    const float* cos_sin;     // [max_pos, D]: cos of the D/2 pair angles, then their sin
    const void* q_weight;     // [D] or null: RMS normalisation of every query head
    const void* k_weight;     // [D] or null
    const int* start_pos;     // [B]; token t of sequence b sits at start_pos[b] + pos_offset + t
    void* q_out;              // [B,n,H,D] contiguous
    void* Kp;                 // [num_pages, page, G, D]
    void* Vp;
    const int* block_table;   // [B,max_pages]
    long long q_sb, q_sl, q_sh, kv_sb, kv_sl, kv_sh;
    float eps;
    int pos_offset, batch, n_new, max_pages, page_shift, max_pos;
    int G, head_dim, elem, gs;
};

hipError_t launch_rope_append(const RopeAppendParams& p, hipStream_t stream);

}  // namespace kascade
