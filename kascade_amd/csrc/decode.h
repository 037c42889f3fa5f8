// Host-visible launchers of the decode kernels (decode.hip).
#pragma once
#include "common.h"

namespace kascade {

struct DecodeParams {
    // Q, K, V, the new rows and the output hold elements of kind `elem` (fp16 or bf16); G KV heads,
    // H = gs G query heads, head dimension head_dim (64 or 128).
    const void* Q;          // [B,H,D]
    const void* K;          // pages [P,page,G,D], or a strided [B,tokens,G,D] view
    const void* V;
    const int* seqlens;     // [B] or null
    const int* idx;         // [B,G,topk] logical token ids (gather mode); physical cache rows with idx_physical
    const int* head_map;    // [G] (gather mode)
    const int* block_table; // [B,max_pages] or null
    float* glse;            // [B,H,num_split]
    float* opart;           // [B,H,num_split,D]
    float* scores;          // [B,H,scores_stride] floats of scratch: compact raw scores (anchor mode)
    // Fused combine: with counters != null ([B*G] ints, zero before the first launch and zero
    // again after every launch) the last split workgroup of each (b, g) merges the splits into
    // out [B,H,D] and row_sums [B,H] (either may be null), and no combine launch is needed.
    // Fused append: with k_new != null the rows k_new/v_new [B,G,D] of each sequence's newest
    // token (position seqlen-1) are written into k_cache / v_cache by the launch itself.
    const void* k_new;
    const void* v_new;
    void* k_cache;
    void* v_cache;
    int* counters;
    void* out;
    float* row_sums;
    int idx_physical;       // gather mode over pages: idx holds cache rows (page * page_size + slot)
    int max_row;            // ... each clamped to [0, max_row]
    int max_pages;
    int page_shift;
    int kv_stride_tokens;   // without seqlens: tokens per sequence; with: an upper bound
    // Without a block table, element (b, token, g, 0) of K and V sits at
    // b*kv_stride_b + token*kv_stride_l + g*kv_stride_h (multiples of 8 elements).
    long long kv_stride_b;
    long long kv_stride_h;
    unsigned kv_stride_l;
    int topk;
    float topk_percent;
    int scores_stride;
    int num_split;
    int rows_per_split;     // multiple of 64; num_split*rows_per_split >= longest row list
    int B;
    int G;                  // KV heads
    int head_dim;           // 64 or 128
    int elem;               // kElemF16 or kElemBF16
    int gs;                 // query heads per KV head: 1 to 16
};

hipError_t launch_decode_split(const DecodeParams& p, bool gather, bool with_v, bool write_scores,
                               hipStream_t stream);
hipError_t launch_decode_combine(const float* glse, const float* opart, void* out, float* row_sums,
                                 int batch, int heads, int num_split, bool with_v, int head_dim, int elem,
                                 hipStream_t stream);
// Log-sums per head: merged (row_sums_in), or glse [B,H,num_split] to be merged by the kernel,
// which then also writes them to row_sums_out.  len_cap: the bound the streaming launch put on
// every sequence length (block-table coverage or cache length, and the score row width).
hipError_t launch_decode_aggregate(const float* scores, const float* row_sums_in, const float* glse,
                                   int num_split, float* row_sums_out, const int* seqlens,
                                   half_t* agg, int batch, int groups, int group_size, int scores_stride,
                                   int uniform_len, int len_cap, hipStream_t stream);

}  // namespace kascade
