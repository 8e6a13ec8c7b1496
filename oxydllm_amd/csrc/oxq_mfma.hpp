// Matrix-core operand helpers shared by the tile kernels: the bit-exact
// T((q - z) * s) dequantisation of a pair of weights and the
// v_mfma_f32_16x16x32_{f16,bf16} wrappers.
#pragma once

#include "oxq_device.hpp"

namespace oxq {

template <typename TT> struct MfmaOps;

template <> struct MfmaOps<F16Traits> {
    // exact (bias+q) - (bias+z), then one correctly rounded multiply
    __device__ static __forceinline__ uint32_t dequant_pair(uint32_t p, uint32_t negzb, uint32_t s) {
        const half2_t d = __builtin_bit_cast(half2_t, p) + __builtin_bit_cast(half2_t, negzb);
        return __builtin_bit_cast(uint32_t, d * __builtin_bit_cast(half2_t, s));
    }
    __device__ static __forceinline__ uint32_t splat(float v) {
        const uint16_t h = F16Traits::from_f32(v);
        return (uint32_t)h | ((uint32_t)h << 16);
    }
    __device__ static __forceinline__ float4_t mfma(const uint32_t a[4], const uint32_t b[4], float4_t c) {
        u32x4_t av = {a[0], a[1], a[2], a[3]}, bv = {b[0], b[1], b[2], b[3]};
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8_t, av),
                                                      __builtin_bit_cast(half8_t, bv), c, 0, 0, 0);
    }
};

template <> struct MfmaOps<BF16Traits> {
    __device__ static __forceinline__ uint32_t dequant_pair(uint32_t p, uint32_t negzb, uint32_t s) {
        // widen (exact), subtract (exact), multiply (exact in f32), round once to bf16
        const float lo = (__builtin_bit_cast(float, p << 16) + __builtin_bit_cast(float, negzb << 16)) *
                         __builtin_bit_cast(float, s << 16);
        const float hi = (__builtin_bit_cast(float, p & 0xFFFF0000u) +
                          __builtin_bit_cast(float, negzb & 0xFFFF0000u)) *
                         __builtin_bit_cast(float, s & 0xFFFF0000u);
        return (uint32_t)BF16Traits::from_f32(lo) | ((uint32_t)BF16Traits::from_f32(hi) << 16);
    }
    __device__ static __forceinline__ uint32_t splat(float v) {
        const uint16_t h = BF16Traits::from_f32(v);
        return (uint32_t)h | ((uint32_t)h << 16);
    }
    __device__ static __forceinline__ float4_t mfma(const uint32_t a[4], const uint32_t b[4], float4_t c) {
        u32x4_t av = {a[0], a[1], a[2], a[3]}, bv = {b[0], b[1], b[2], b[3]};
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, av),
                                                       __builtin_bit_cast(bf16x8_t, bv), c, 0, 0, 0);
    }
};

}  // namespace oxq
