// Host-visible launchers of the diagnostic read kernels (diag.hip).
#pragma once
#include "common.h"

namespace kascade {

hipError_t launch_diag_stream_read(const void* src, long long bytes, void* sink, int blocks, hipStream_t stream);
hipError_t launch_diag_gather_rows(const void* a0, const void* a1, const int* rows, long long n_rows,
                                   int rows_per_block, long long row_stride_bytes, void* sink,
                                   hipStream_t stream);

}  // namespace kascade
