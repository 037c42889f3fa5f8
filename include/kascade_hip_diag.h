/*
 * kascade_hip_diag.h -- measurement helpers exported by libkascade_hip.so.
 *
 * Not part of the attention path and not something a replacement of the reference's kernel
 * objects binds: the benchmark uses these two read-only kernels to put the decode kernels'
 * bandwidth next to what the device gives a kernel that does no arithmetic.  Same calling
 * convention as kascade_hip.h (0 / -1, kascade_get_last_error()).
 */
#ifndef KASCADE_HIP_DIAG_H
#define KASCADE_HIP_DIAG_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Read-only kernels with no arithmetic, for measuring what the device delivers to the two access
 * patterns of the decode path (no counterpart in the reference; used by the benchmark only).
 * Nothing is written except, never in practice, 16 bytes at `sink`.
 *   stream_read: reads `bytes` bytes of src, 16 bytes per lane, four loads in flight per lane.
 *   gather_rows: for each of the n_rows entries of row_ids reads the 256 bytes at
 *                rows_a + row_ids[i]*row_stride_bytes (and the same row of rows_b when non-NULL),
 *                16 lanes per row; every id must address a row inside the arrays. */
int kascade_diag_stream_read_call(const void* src, int64_t bytes, void* sink, void* stream);
int kascade_diag_gather_rows_call(const void* rows_a, const void* rows_b, const int32_t* row_ids,
                                  int64_t n_rows, int64_t row_stride_bytes, void* sink, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* KASCADE_HIP_DIAG_H */
