// Host-visible launcher of the top-k selection kernel (topk.hip).
#pragma once
#include "common.h"

namespace kascade {

hipError_t launch_topk(const half_t* scores, int* out_idx, int rows, long long row_stride,
                       int uniform_len, const int* valid_len, const int* n_sel, int period, int k,
                       int fill, hipStream_t stream);

// Multi-workgroup variant for long rows.  Returns 0 bytes when the single-workgroup kernel
// is the right choice (short rows, or too many rows for the 8 KB/row workspace).
long long topk_split_workspace_bytes(int rows, long long row_len);
hipError_t launch_topk_split(const half_t* scores, int* out_idx, int rows, long long row_stride,
                             int max_len, int uniform_len, const int* valid_len, const int* n_sel,
                             int period, int k, int fill, void* workspace, hipStream_t stream);

}  // namespace kascade
