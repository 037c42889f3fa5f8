// Paged KV-cache append: scatter the new tokens' K/V rows into their page slots.
// One 16-byte chunk per thread; grid covers B * n_new * G * (D/8) chunks for K and V.  Elements are
// 16 bits wide (fp16 or bf16: the kernel only moves them).
#include "paged.h"

namespace kascade {

namespace {

__global__ __launch_bounds__(256) void paged_kv_append_kernel(
    half_t* __restrict__ Kp, half_t* __restrict__ Vp, const half_t* __restrict__ k_new,
    const half_t* __restrict__ v_new, const int* __restrict__ start_pos,
    const int* __restrict__ block_table, int batch, int n_new, const int* __restrict__ n_new_rows,
    int max_pages, int page_shift, long long sb, long long sl, long long sh, int groups, int head_dim) {
    const int chunks = head_dim / 8;
    const long long total = (long long)batch * n_new * groups * chunks;
    const long long c = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (c >= total) return;
    const int col = (int)(c % chunks);
    const int g = (int)((c / chunks) % groups);
    const long long bt = c / (chunks * groups);
    const int t = (int)(bt % n_new);
    const int b = (int)(bt / n_new);
    if (n_new_rows && t >= n_new_rows[b]) return;   // this sequence brings fewer rows than the batch's widest
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
                                                             float percent, int batch, int groups,
                                                             int* __restrict__ valid_rows,
                                                             int* __restrict__ n_sel_rows) {
    // a single workgroup: the barrier puts the in-place update after every read of a length
    for (int i = threadIdx.x; i < batch * groups; i += blockDim.x) {
        const int cur = seqlens[i / groups];
        const int len = cur > 0 ? cur + advance : cur;   // length 0: an empty slot of the batch, left alone
        const long long fl = (long long)floor((double)percent * (double)len / 100.0);
        if (valid_rows) valid_rows[i] = len;
        if (n_sel_rows) n_sel_rows[i] = (int)(((fl + 127) / 128) * 128);
    }
    __syncthreads();
    if (advance != 0)
        for (int b = threadIdx.x; b < batch; b += blockDim.x)
            if (seqlens[b] > 0) seqlens[b] += advance;
}


// One workgroup per token, one row of D/8 lanes per head: H query heads, G key heads, G value
// heads = H + 2G rows, taken 256/(D/8) at a time, three at once (the reference's shape is one trip:
// two query heads and a key or value head per row of lanes).  Query and key heads are
// (optionally) RMS-normalised over the head dimension, then rotated by the token's position in
// the "rotate half" pairing (i, i + D/2): the partner element sits D/16 lanes away in the row.
// Queries go to a dense [B,n,H,D] tensor; keys and values go straight to their page slots.
// The position, the page and the angles are the same for the whole workgroup.
template <int D, typename T>
__global__ __launch_bounds__(256) void rope_append_kernel(RopeAppendParams p) {
    constexpr int kRowLanes = D / 8;                        // 16 or 8
    constexpr int kRowsPerTrip = 256 / kRowLanes;           // 16 or 32
    const int lane = threadIdx.x % kRowLanes;
    const int grp = threadIdx.x / kRowLanes;
    const int t = blockIdx.x % p.n_new;
    const int b = blockIdx.x / p.n_new;
    const int pos = p.start_pos[b] + p.pos_offset + t;
    if (pos < 0) return;
    const bool cache_ok = (pos >> p.page_shift) < p.max_pages;
    const int G = p.G, Hq = p.gs * G, nrows = Hq + 2 * G;
    const T* q_in = static_cast<const T*>(p.q_in);
    const T* k_in = static_cast<const T*>(p.k_in);
    const T* v_in = static_cast<const T*>(p.v_in);

    PackT<T> wq, wk;
    if (p.q_weight) wq.u = ld_global_16(static_cast<const T*>(p.q_weight) + lane * 8);
    if (p.k_weight) wk.u = ld_global_16(static_cast<const T*>(p.k_weight) + lane * 8);
    const int pc = pos < p.max_pos ? pos : p.max_pos - 1;
    const float* cs = p.cos_sin + (long long)pc * D + (lane % (kRowLanes / 2)) * 8;
    float c[8], sn[8];
    *reinterpret_cast<float4_t*>(c) = *reinterpret_cast<const float4_t*>(cs);
    *reinterpret_cast<float4_t*>(c + 4) = *reinterpret_cast<const float4_t*>(cs + 4);
    *reinterpret_cast<float4_t*>(sn) = *reinterpret_cast<const float4_t*>(cs + D / 2);
    *reinterpret_cast<float4_t*>(sn + 4) = *reinterpret_cast<const float4_t*>(cs + D / 2 + 4);
    long long cache_row = 0;
    if (cache_ok) {
        const int pg = p.block_table[(long long)b * p.max_pages + (pos >> p.page_shift)];
        cache_row = ((long long)pg << p.page_shift) + (pos & ((1 << p.page_shift) - 1));
    }
    const float sign = lane < kRowLanes / 2 ? -1.f : 1.f;

    // Called per row of lanes (16 or 8): the exchanges stay inside the row, so rows of different
    // kinds may take different branches.
    auto rotate = [&](PackT<T> v, bool norm, const PackT<T>& wv) {
        if (norm) {
            float ss = 0.f;
#pragma unroll
            for (int e = 0; e < 8; ++e) ss += (float)v.e[e] * (float)v.e[e];
            if constexpr (kRowLanes == 16) {
                ss = row16_sum(ss);
            } else {   // rows of 8 lanes: three exchanges within the half row
                ss += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, ss), 0xB1, 0xF, 0xF, false));
                ss += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, ss), 0x4E, 0xF, 0xF, false));
                ss += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, ss), 0x141, 0xF, 0xF, false));
            }
            const float inv = 1.0f / sqrtf(ss * (1.0f / D) + p.eps);
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const T n = (T)((float)v.e[e] * inv);                  // normalised, in storage type
                v.e[e] = (T)((float)n * (float)wv.e[e]);               // times the weight, rounded once
            }
        }
        PackT<T> y;   // the partner half of the head: D/16 lanes away within the row
#pragma unroll
        for (int d = 0; d < 4; ++d) {
            if constexpr (kRowLanes == 16)
                y.u[d] = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v.u[d], 0x128, 0xF, 0xF, false);  // row_ror:8
            else
                y.u[d] = (uint32_t)__builtin_amdgcn_ds_swizzle((int)v.u[d], 0x101F);                      // lane ^ 4
        }
#pragma unroll
        for (int e = 0; e < 8; ++e) v.e[e] = (T)((float)v.e[e] * c[e] + sign * ((float)y.e[e] * sn[e]));
        return v;
    };

    const T* qrow = q_in + b * p.q_sb + t * p.q_sl;
    const long long kvoff = b * p.kv_sb + t * p.kv_sl;
    for (int row0 = 0; row0 < nrows; row0 += 3 * kRowsPerTrip) {   // uniform over the workgroup
        // all loads first, none behind a branch (a row past the last one reads row 0 again)
        PackT<T> x[3];
#pragma unroll
        for (int j = 0; j < 3; ++j) {
            int r = row0 + grp + j * kRowsPerTrip;
            r = r < nrows ? r : 0;
            const T* src = r < Hq ? qrow + r * p.q_sh
                         : r < Hq + G ? k_in + kvoff + (r - Hq) * p.kv_sh
                                      : v_in + kvoff + (r - Hq - G) * p.kv_sh;
            x[j].u = ld_global_16(src + lane * 8);
        }
#pragma unroll
        for (int j = 0; j < 3; ++j) {
            const int r = row0 + grp + j * kRowsPerTrip;   // the same for all lanes of a row
            if (r < Hq) {
                *reinterpret_cast<uint4_t*>(static_cast<T*>(p.q_out) + ((long long)blockIdx.x * Hq + r) * D + lane * 8) =
                    rotate(x[j], p.q_weight != nullptr, wq).u;
            } else if (r < nrows && cache_ok) {
                const bool is_k = r < Hq + G;
                const long long off = (cache_row * G + (is_k ? r - Hq : r - Hq - G)) * D + lane * 8;
                if (is_k)
                    *reinterpret_cast<uint4_t*>(static_cast<T*>(p.Kp) + off) = rotate(x[j], p.k_weight != nullptr, wk).u;
                else
                    *reinterpret_cast<uint4_t*>(static_cast<T*>(p.Vp) + off) = x[j].u;
            }
        }
    }
}

}  // namespace

hipError_t launch_decode_budgets(int* seqlens, int advance, float percent, int batch, int groups,
                                 int* valid_rows, int* n_sel_rows, hipStream_t stream) {
    hipLaunchKernelGGL(decode_budgets_kernel, dim3(1), dim3(256), 0, stream, seqlens, advance, percent,
                       batch, groups, valid_rows, n_sel_rows);
    return hipGetLastError();
}

hipError_t launch_paged_kv_append(half_t* Kp, half_t* Vp, const half_t* k_new, const half_t* v_new,
                                  const int* start_pos, const int* block_table, int batch,
                                  int n_new, const int* n_new_rows, int max_pages, int page_shift, long long sb,
                                  long long sl, long long sh, int groups, int head_dim,
                                  hipStream_t stream) {
    const long long total = (long long)batch * n_new * groups * (head_dim / 8);
    if (total == 0) return hipSuccess;
    dim3 grid((unsigned)((total + 255) / 256)), block(256);
    hipLaunchKernelGGL(paged_kv_append_kernel, grid, block, 0, stream, Kp, Vp, k_new, v_new,
                       start_pos, block_table, batch, n_new, n_new_rows, max_pages, page_shift, sb, sl, sh, groups, head_dim);
    return hipGetLastError();
}

hipError_t launch_rope_append(const RopeAppendParams& p, hipStream_t stream) {
    if ((long long)p.batch * p.n_new == 0) return hipSuccess;
    const dim3 grid((unsigned)(p.batch * p.n_new)), block(256);
    if (p.head_dim == 128 && p.elem == kElemF16)
        hipLaunchKernelGGL((rope_append_kernel<128, half_t>), grid, block, 0, stream, p);
    else if (p.head_dim == 128 && p.elem == kElemBF16)
        hipLaunchKernelGGL((rope_append_kernel<128, bf16_t>), grid, block, 0, stream, p);
    else if (p.head_dim == 64 && p.elem == kElemF16)
        hipLaunchKernelGGL((rope_append_kernel<64, half_t>), grid, block, 0, stream, p);
    else if (p.head_dim == 64 && p.elem == kElemBF16)
        hipLaunchKernelGGL((rope_append_kernel<64, bf16_t>), grid, block, 0, stream, p);
    else
        return hipErrorInvalidValue;
    return hipGetLastError();
}

}  // namespace kascade
