// Host-visible launchers of the prefill kernels (prefill.hip).
#pragma once
#include "common.h"

namespace kascade {

struct PrefillParams {
    // Queries are rows [0, Lq) of Q at global positions q_start + row; keys are positions
    // [0, L), L = q_start + Lq.  A whole-prompt call has q_start = 0 and Lq = L.
    // Q, K, V and O hold elements of kind `elem` (fp16 or bf16); G KV heads, H = gs G query heads,
    // head dimension head_dim (64 or 128).  A workgroup always works on four head slots of one
    // KV head: the KV head's gs query heads are taken four at a time, ceil(gs/4) "sub-groups" --
    // the attention kernels launch one workgroup per (KV head, sub-group), the pooling kernel is
    // launched once per sub-group (vsub) and adds to the pooled scores of the earlier ones.  A
    // slot beyond the KV head's last query head computes along on that head's data and leaves
    // nothing behind: no output, no log-sum, nothing in the pooled sums.
    const void* Q;            // [B,Lq,H,D] through (q_sb, q_sl, q_sh)
    const void* K;            // [B,L,G,D] through (k_sb, k_sl, k_sh); V shares the strides.
    const void* V;            //   Paged: [num_pages, page, G, D] contiguous, strides unused
    const int* idx;           // [B,G,T,max_topk] (reuse); physical rows when paged
    const int* head_map;      // [G] (reuse)
    const float* log_sum_in;  // [B,Lq,H] (aggregate)
    float* log_sum;           // [B,Lq,H] or null (attention kernel output)
    void* O;                  // [B,Lq,H,D] contiguous
    half_t* agg;              // [B,G,T,L] (aggregate)
    const int* block_table;   // [B,max_pages] or null (strided K/V)
    // Chunked prefill of a batch whose sequences stand at different positions (both null: every
    // sequence starts at q_start and has Lq rows).  q_start_rows[b]: first global position of
    // sequence b's rows (a multiple of 32, at most q_start); q_len_rows[b]: how many of the Lq rows
    // of Q belong to it (null: all).  Rows beyond are left alone: no output, no log-sum, no scores.
    const int* q_start_rows;
    const int* q_len_rows;
    long long q_sb, q_sl, q_sh;
    long long k_sb, k_sl, k_sh;
    int B, L, T;              // T = ceil(Lq / 32) query tiles of this call
    int Lq, q_start;
    int max_pages, page_shift, num_pages;
    int max_topk;
    int rolling;
    float topk_percent;
    int fill_invalid;
    int G;                    // KV heads
    int head_dim;             // 64 or 128
    int elem;                 // kElemF16 or kElemBF16
    int gs;                   // query heads per KV head: 1 to 16 (0 = 4)
    int vsub, accumulate;     // pooling kernel: sub-group of this launch; add to what agg holds
};

// Query heads per KV head and the sub-groups of four head slots they take.
struct HeadSlots {
    int gs, subs;
};
__host__ __device__ inline HeadSlots head_slots(int gs) {
    if (gs <= 0) gs = 4;
    return HeadSlots{gs, (gs + 3) / 4};
}

hipError_t launch_prefill_attn(const PrefillParams& p, bool reuse, bool with_v, int nqb,
                               hipStream_t stream);
hipError_t launch_prefill_aggregate(const PrefillParams& p, hipStream_t stream);
// out[b,i] = physical cache row of token idx[b,i] (clamped to [0, L)); out may alias idx.
hipError_t launch_translate_indices(const int* idx, int* out, const int* block_table, int B,
                                    long long per_seq, int max_pages, int page_shift, int L,
                                    hipStream_t stream);

}  // namespace kascade
