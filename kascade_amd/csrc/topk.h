// Host-visible launcher of the top-k selection kernel (topk.hip).
#pragma once
#include "common.h"

namespace kascade {

// Optional second output of a selection: the selected positions as rows of a paged cache.
struct TopkRows {
    int* out_rows;            // [rows, k], or null: no second output
    const int* block_table;   // [sequences, max_pages]
    int max_pages;
    int page_shift;
    int rows_per_seq;         // consecutive score rows that belong to one sequence
};

hipError_t launch_topk(const half_t* scores, int* out_idx, int rows, long long row_stride,
                       int uniform_len, const int* valid_len, const int* n_sel, int period, int k,
                       int fill, const TopkRows* tr, hipStream_t stream);

// Multi-workgroup variant for long rows.  Returns 0 bytes when the single-workgroup kernel
// is the right choice (short rows, or too many rows for the 8 KB/row workspace).
long long topk_split_workspace_bytes(int rows, long long row_len);
// longest row (entries) the one-workgroup selection keeps in registers (the tensor must start 16-byte
// aligned; rows that start off a boundary count 7 slots more)
int topk_max_register_row();
hipError_t launch_topk_split(const half_t* scores, int* out_idx, int rows, long long row_stride,
                             int max_len, int uniform_len, const int* valid_len, const int* n_sel,
                             int period, int k, int fill, void* workspace, const TopkRows* tr,
                             hipStream_t stream);

// Reorders the first min(k, valid length) entries of every row of idx [rows, k] by descending score
// (equal scores: ascending position); workspace: topk_sort_workspace_bytes(rows, k) bytes (0 for
// short lists, which are sorted in LDS).
long long topk_sort_workspace_bytes(int rows, int k);
hipError_t launch_topk_sort_rows(const half_t* scores, int* idx, void* workspace, int rows,
                                 long long row_stride, int uniform_len, const int* valid_len,
                                 int period, int k, hipStream_t stream);

}  // namespace kascade
