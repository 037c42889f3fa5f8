// Host-visible launchers of the cache bookkeeping kernels (paged.hip).
#pragma once
#include "common.h"

namespace kascade {

hipError_t launch_paged_kv_append(half_t* Kp, half_t* Vp, const half_t* k_new, const half_t* v_new,
                                  const int* start_pos, const int* block_table, int batch,
                                  int n_new, int max_pages, int page_shift, long long sb,
                                  long long sl, long long sh, hipStream_t stream);

hipError_t launch_decode_budgets(int* seqlens, int advance, float percent, int batch, int* valid_rows,
                                 int* n_sel_rows, hipStream_t stream);

}  // namespace kascade
