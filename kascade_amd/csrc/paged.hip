// Paged KV-cache append: scatter the new tokens' K/V rows into their page slots.
// One 16-byte chunk per thread; grid covers B * n_new * G * (D/8) chunks for K and V.  Elements are
// 16 bits wide (fp16 or bf16: the kernel only moves them).
#include "paged.h"

namespace kascade {

namespace {

__global__ __launch_bounds__(256) void paged_kv_append_kernel(
    half_t* __restrict__ Kp, half_t* __restrict__ Vp, const half_t* __restrict__ k_new,
    const half_t* __restrict__ v_new, const int* __restrict__ start_pos,
    const int* __restrict__ block_table, int batch, int n_new, int max_pages, int page_shift,
    long long sb, long long sl, long long sh, int groups, int head_dim) {
    const int chunks = head_dim / 8;
    const long long total = (long long)batch * n_new * groups * chunks;
    const long long c = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (c >= total) return;
    const int col = (int)(c % chunks);
    const int g = (int)((c / chunks) % groups);
    const long long bt = c / (chunks * groups);
    const int t = (int)(bt % n_new);
    const int b = (int)(bt / n_new);
    const int tok = start_pos[b] + t;
    // a position before the sequence or beyond what the block table covers has no slot: skipped,
    // like rope_append_kernel does (reading the table there would land in another sequence's row)
    if (tok < 0 || (tok >> page_shift) >= max_pages) return;
    const int pg = block_table[(long long)b * max_pages + (tok >> page_shift)];
    const long long row = ((long long)pg << page_shift) + (tok & ((1 << page_shift) - 1));
    const long long dst = (row * groups + g) * head_dim + col * 8;
    const long long src = b * sb + t * sl + g * sh + col * 8;
    *reinterpret_cast<uint4_t*>(Kp + dst) = ld_global_16(k_new + src);
    *reinterpret_cast<uint4_t*>(Vp + dst) = ld_global_16(v_new + src);
}

// Per (sequence, KV head) row of a ragged decode step: how many pooled scores are valid and how
// many of them the selection keeps, n(b) = 128*ceil(floor(percent*len_b/100)/128), optionally
// after adding `advance` to every length in place (the step's new token).
__global__ __launch_bounds__(256) void decode_budgets_kernel(int* __restrict__ seqlens, int advance,
                                                             float percent, int batch,
                                                             int* __restrict__ valid_rows,
                                                             int* __restrict__ n_sel_rows) {
    // a single workgroup: the barrier puts the in-place update after every read of a length
    for (int i = threadIdx.x; i < batch * kGroups; i += blockDim.x) {
        const int len = seqlens[i / kGroups] + advance;
        const long long fl = (long long)floor((double)percent * (double)len / 100.0);
        if (valid_rows) valid_rows[i] = len;
        if (n_sel_rows) n_sel_rows[i] = (int)(((fl + 127) / 128) * 128);
    }
    __syncthreads();
    if (advance != 0)
        for (int b = threadIdx.x; b < batch; b += blockDim.x) seqlens[b] += advance;
}


// One workgroup per token, one 16-lane row per head: 32 query heads, 8 key heads, 8 value heads
// = 48 rows, three per 16-lane group (two query heads; a key head or a value head).  Query and
// key heads are (optionally) RMS-normalised over the head dimension, then rotated by the token's
// position in the "rotate half" pairing (i, i + 64): the partner element sits 8 lanes away in the
// row.  Queries go to a dense [B,n,H,D] tensor; keys and values go straight to their page slots.
// The position, the page and the angles are the same for the whole workgroup.
__global__ __launch_bounds__(256) void rope_append_kernel(RopeAppendParams p) {
    const int lane = threadIdx.x & 15;
    const int grp = threadIdx.x >> 4;                       // 0..15
    const int t = blockIdx.x % p.n_new;
    const int b = blockIdx.x / p.n_new;
    const int pos = p.start_pos[b] + p.pos_offset + t;
    if (pos < 0) return;
    const bool cache_ok = (pos >> p.page_shift) < p.max_pages;
    const bool is_v = grp >= kGroups;                       // third row of this group: key or value head
    const int g_kv = grp & (kGroups - 1);

    // all loads first
    Pack16 x[3], wq, wk;
    const half_t* qrow = p.q_in + b * p.q_sb + t * p.q_sl;
    x[0].u = ld_global_16(qrow + grp * p.q_sh + lane * 8);
    x[1].u = ld_global_16(qrow + (grp + 16) * p.q_sh + lane * 8);
    x[2].u = ld_global_16((is_v ? p.v_in : p.k_in) + b * p.kv_sb + t * p.kv_sl + g_kv * p.kv_sh + lane * 8);
    if (p.q_weight) wq.u = ld_global_16(p.q_weight + lane * 8);
    if (p.k_weight) wk.u = ld_global_16(p.k_weight + lane * 8);
    const int pc = pos < p.max_pos ? pos : p.max_pos - 1;
    const float* cs = p.cos_sin + (long long)pc * kDim + (lane & 7) * 8;
    float c[8], sn[8];
    *reinterpret_cast<float4_t*>(c) = *reinterpret_cast<const float4_t*>(cs);
    *reinterpret_cast<float4_t*>(c + 4) = *reinterpret_cast<const float4_t*>(cs + 4);
    *reinterpret_cast<float4_t*>(sn) = *reinterpret_cast<const float4_t*>(cs + kDim / 2);
    *reinterpret_cast<float4_t*>(sn + 4) = *reinterpret_cast<const float4_t*>(cs + kDim / 2 + 4);
    long long cache_row = 0;
    if (cache_ok) {
        const int pg = p.block_table[(long long)b * p.max_pages + (pos >> p.page_shift)];
        cache_row = ((long long)pg << p.page_shift) + (pos & ((1 << p.page_shift) - 1));
    }
    const float sign = lane < 8 ? -1.f : 1.f;

    auto rotate = [&](Pack16 v, const half_t* w, const Pack16& wv) {
        if (w) {
            float ss = 0.f;
#pragma unroll
            for (int e = 0; e < 8; ++e) ss += (float)v.h[e] * (float)v.h[e];
            ss = row16_sum(ss);
            const float inv = 1.0f / sqrtf(ss * (1.0f / kDim) + p.eps);
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const half_t n = (half_t)((float)v.h[e] * inv);          // normalised, in storage type
                v.h[e] = (half_t)((float)n * (float)wv.h[e]);            // times the weight, rounded once
            }
        }
        Pack16 y;   // the partner half of the head: lanes 8 apart within the row of 16
#pragma unroll
        for (int d = 0; d < 4; ++d)
            y.u[d] = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v.u[d], 0x128, 0xF, 0xF, false);  // row_ror:8
#pragma unroll
        for (int e = 0; e < 8; ++e) v.h[e] = (half_t)((float)v.h[e] * c[e] + sign * ((float)y.h[e] * sn[e]));
        return v;
    };

    half_t* qdst = p.q_out + (long long)blockIdx.x * kHeads * kDim + lane * 8;
    *reinterpret_cast<uint4_t*>(qdst + grp * kDim) = rotate(x[0], p.q_weight, wq).u;
    *reinterpret_cast<uint4_t*>(qdst + (grp + 16) * kDim) = rotate(x[1], p.q_weight, wq).u;
    if (cache_ok) {
        const long long off = (cache_row * kGroups + g_kv) * kDim + lane * 8;
        if (is_v)      // uniform over the 16 lanes of a row, so the row-wide exchanges above stay whole
            *reinterpret_cast<uint4_t*>(p.Vp + off) = x[2].u;
        else
            *reinterpret_cast<uint4_t*>(p.Kp + off) = rotate(x[2], p.k_weight, wk).u;
    }
}

}  // namespace

hipError_t launch_decode_budgets(int* seqlens, int advance, float percent, int batch, int* valid_rows,
                                 int* n_sel_rows, hipStream_t stream) {
    hipLaunchKernelGGL(decode_budgets_kernel, dim3(1), dim3(256), 0, stream, seqlens, advance, percent,
                       batch, valid_rows, n_sel_rows);
    return hipGetLastError();
}

hipError_t launch_paged_kv_append(half_t* Kp, half_t* Vp, const half_t* k_new, const half_t* v_new,
                                  const int* start_pos, const int* block_table, int batch,
                                  int n_new, int max_pages, int page_shift, long long sb,
                                  long long sl, long long sh, int groups, int head_dim,
                                  hipStream_t stream) {
    const long long total = (long long)batch * n_new * groups * (head_dim / 8);
    if (total == 0) return hipSuccess;
    dim3 grid((unsigned)((total + 255) / 256)), block(256);
    hipLaunchKernelGGL(paged_kv_append_kernel, grid, block, 0, stream, Kp, Vp, k_new, v_new,
                       start_pos, block_table, batch, n_new, max_pages, page_shift, sb, sl, sh, groups, head_dim);
    return hipGetLastError();
}

hipError_t launch_rope_append(const RopeAppendParams& p, hipStream_t stream) {
    const long long rows = (long long)p.batch * p.n_new * (kHeads + 2 * kGroups);
    if (rows == 0) return hipSuccess;
    hipLaunchKernelGGL(rope_append_kernel, dim3((unsigned)(p.batch * p.n_new)), dim3(256), 0, stream, p);
    return hipGetLastError();
}

}  // namespace kascade
