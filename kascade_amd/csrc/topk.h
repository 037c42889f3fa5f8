// Host-visible launcher of the top-k selection kernel (topk.hip).
#pragma once
#include "common.h"

namespace kascade {

hipError_t launch_topk(const half_t* scores, int* out_idx, int rows, long long row_stride,
                       int uniform_len, const int* valid_len, const int* n_sel, int period, int k,
                       int fill, hipStream_t stream);

}  // namespace kascade
