// Shared device/host helpers for the gfx950 kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace kascade {

constexpr int kHeads = 32;     // query heads
constexpr int kGroups = 8;     // KV heads
constexpr int kGroupSize = 4;  // query heads per KV head
constexpr int kDim = 128;      // head dimension
constexpr int kTile = 32;      // prefill query tile
// D^-0.5 * log2(e): softmax is evaluated as exp2(s*kScaleLog2 - m*kScaleLog2)
constexpr float kScaleLog2 = 0.12751743082459868f;

typedef _Float16 half_t;
typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef float float4_t __attribute__((ext_vector_type(4)));
typedef float float16_t __attribute__((ext_vector_type(16)));
typedef uint32_t uint4_t __attribute__((ext_vector_type(4)));
typedef int int4_t __attribute__((ext_vector_type(4)));

typedef __bf16 bf16_t;
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x4_t __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef short short4_t __attribute__((ext_vector_type(4)));
typedef short short8_t __attribute__((ext_vector_type(8)));

// Element types of Q, K, V and the attention output (pooled scores are fp16 for both).
enum ElemKind { kElemF16 = 0, kElemBF16 = 1 };

// D^-0.5 * log2(e) for the head dimensions the kernels are built for
template <int D> struct ScaleLog2;
template <> struct ScaleLog2<128> { static constexpr float value = 0.12751743082459868f; };
template <> struct ScaleLog2<64> { static constexpr float value = 0.18033688011112042f; };

// Vector types and matrix instructions per element type.  Both types have the same operand
// layouts, so the kernels are written once over Elem<T>.
template <typename T> struct Elem;
template <> struct Elem<half_t> {
    typedef half2_t x2; typedef half4_t x4; typedef half8_t x8;
    static __device__ __forceinline__ float4_t mma_16x16x32(x8 a, x8 b, float4_t c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
    }
    static __device__ __forceinline__ float4_t mma_16x16x16(short4_t a, x4 b, float4_t c) {
        return __builtin_amdgcn_mfma_f32_16x16x16f16(__builtin_bit_cast(x4, a), b, c, 0, 0, 0);
    }
    static __device__ __forceinline__ float16_t mma_32x32x16(x8 a, x8 b, float16_t c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
    }
    // acc + p.x + p.y in fp32 (one instruction for two elements)
    static __device__ __forceinline__ float add_pair(x2 p, float acc) {
        const x2 ones = {(half_t)1.f, (half_t)1.f};
        return __builtin_amdgcn_fdot2(p, ones, acc, false);
    }
};
template <> struct Elem<bf16_t> {
    typedef bf16x2_t x2; typedef bf16x4_t x4; typedef bf16x8_t x8;
    static __device__ __forceinline__ float4_t mma_16x16x32(x8 a, x8 b, float4_t c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
    }
    static __device__ __forceinline__ float4_t mma_16x16x16(short4_t a, x4 b, float4_t c) {
        return __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(a, __builtin_bit_cast(short4_t, b), c, 0, 0, 0);
    }
    static __device__ __forceinline__ float16_t mma_32x32x16(x8 a, x8 b, float16_t c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
    }
    static __device__ __forceinline__ float add_pair(x2 p, float acc) {
        const x2 ones = {(bf16_t)1.f, (bf16_t)1.f};
        return __builtin_amdgcn_fdot2_f32_bf16(p, ones, acc, false);
    }
};

template <typename T> union PackT {  // one 16-byte transaction seen as 8 elements of type T
    uint4_t u;
    typename Elem<T>::x8 v8;
    T e[8];
};

union Pack16 {  // one 16-byte global/LDS transaction seen as 8 halves
    uint4_t u;
    half8_t h8;
    half2_t h2[4];
    half_t h[8];
};

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }
__device__ __forceinline__ float fast_log2(float x) { return __builtin_amdgcn_logf(x); }

// Sum over the 16 lanes of a DPP row; every lane of the row receives the total.
__device__ __forceinline__ float row16_sum(float x) {
    x += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0xB1, 0xF, 0xF, false));   // quad_perm [1,0,3,2]
    x += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0x4E, 0xF, 0xF, false));   // quad_perm [2,3,0,1]
    x += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0x141, 0xF, 0xF, false));  // row_half_mirror
    x += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0x140, 0xF, 0xF, false));  // row_mirror
    return x;
}

// max(x in this lane, x in lane ^ 32) without a trip through LDS (gfx950 lane-half swap)
__device__ __forceinline__ float max_with_other_half(float x) {
    const uint32_t u = __builtin_bit_cast(uint32_t, x);
    const auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);   // {low half twice, high half twice}
    return fmaxf(__builtin_bit_cast(float, (uint32_t)r[0]), __builtin_bit_cast(float, (uint32_t)r[1]));
}
__device__ __forceinline__ float sum_with_other_half(float x) {
    const uint32_t u = __builtin_bit_cast(uint32_t, x);
    const auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
    return __builtin_bit_cast(float, (uint32_t)r[0]) + __builtin_bit_cast(float, (uint32_t)r[1]);
}

__device__ __forceinline__ uint4_t ld_global_16(const void* p) {
    return *reinterpret_cast<const uint4_t*>(p);
}

inline int ilog2_exact(int x) {  // host: log2 of a power of two, -1 otherwise
    if (x <= 0 || (x & (x - 1))) return -1;
    int s = 0;
    while ((1 << s) < x) ++s;
    return s;
}

}  // namespace kascade
