// Host-visible launchers of the prefill kernels (prefill.hip).
#pragma once
#include "common.h"

namespace kascade {

struct PrefillParams {
    const half_t* Q;          // [B,L,H,D] through (q_sb, q_sl, q_sh)
    const half_t* K;          // [B,L,G,D] through (k_sb, k_sl, k_sh); V shares the strides
    const half_t* V;
    const int* idx;           // [B,G,T,max_topk] (reuse)
    const int* head_map;      // [G] (reuse)
    const float* log_sum_in;  // [B,L,H] (aggregate)
    float* log_sum;           // [B,L,H] or null (attention kernel output)
    half_t* O;                // [B,L,H,D] contiguous
    half_t* agg;              // [B,G,T,L] (aggregate)
    long long q_sb, q_sl, q_sh;
    long long k_sb, k_sl, k_sh;
    int B, L, T;
    int max_topk;
    int rolling;
    float topk_percent;
    int fill_invalid;
};

hipError_t launch_prefill_attn(const PrefillParams& p, bool reuse, bool with_v, int nqb,
                               hipStream_t stream);
hipError_t launch_prefill_aggregate(const PrefillParams& p, hipStream_t stream);

}  // namespace kascade
