// Device-side helpers shared by the gfx950 kernels: 16-bit type traits,
// packed-nibble unpack into dot2/MFMA operand pairs, wave reductions and the
// deterministic split-K arrival protocol.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdint>
#include <type_traits>

namespace oxq {

typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float float4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));

constexpr int WAVE = 64;

__device__ __forceinline__ uint32_t perm_b32(uint32_t hi, uint32_t lo, uint32_t sel) {
    return __builtin_amdgcn_perm(hi, lo, sel);
}
// (lo16(a), lo16(b)) and (hi16(a), hi16(b)) as {low half, high half}
__device__ __forceinline__ uint32_t pack_lo16(uint32_t a, uint32_t b) {
    return perm_b32(b, a, 0x05040100u);
}
__device__ __forceinline__ uint32_t pack_hi16(uint32_t a, uint32_t b) {
    return perm_b32(b, a, 0x07060302u);
}

// AWQ 4-bit slot -> column offset inside the 8 columns of a word.
__device__ __forceinline__ constexpr int awq_slot_col(int slot) {
    return ((slot & 3) << 1) | (slot >> 2);
}

// The AND masks live in VGPRs: v_and_or_b32 may read only one scalar/literal
// operand, and with both the mask and the exponent pattern as literals the
// compiler splits every unpack into v_and + v_or.
struct NibbleMasks {
    uint32_t m0, m1;
};
__device__ __forceinline__ uint32_t vgpr_const(uint32_t c) {
    uint32_t r;
    asm volatile("v_mov_b32 %0, %1" : "=v"(r) : "s"(c));
    return r;
}
__device__ __forceinline__ NibbleMasks nibble_masks() {
    return NibbleMasks{vgpr_const(0x000F000Fu), vgpr_const(0x00F000F0u)};
}

// Raw buffer resources: base + 32-bit lane offset + scalar offset addressing, so
// row addresses cost scalar ALU only; out-of-range reads return zero.
constexpr int BUFFER_RSRC_FLAGS = 0x00020000;
__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void *p, uint32_t bytes) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(p), 0, (int)bytes, BUFFER_RSRC_FLAGS);
}

// ---------------------------------------------------------------------------
// Element-type traits.  `pair` registers hold two 16-bit floats.
//
// unpack4(t, p): t holds two 16-bit halves of 4 nibbles each; p[i] receives
// the pair {nibble i of the low half, nibble i of the high half} as two
// floats equal to BIAS(i) + nibble.  The OR-with-exponent trick makes the
// conversion exact: an f16 with exponent 2^10 (2^6) has ulp 1 at mantissa bit
// 0 (bit 4); a bf16 with exponent 2^7 has ulp 1 at mantissa bit 0.
// ---------------------------------------------------------------------------
struct F16Traits {
    using elem_t = _Float16;
    static constexpr int DTYPE = 1;
    static constexpr uint32_t ONES = 0x3C003C00u;
    __device__ static __forceinline__ float bias(int i) { return (i & 1) ? 64.0f : 1024.0f; }
    __device__ static __forceinline__ void unpack4(uint32_t t, uint32_t p[4], const NibbleMasks &k) {
        p[0] = (t & k.m0) | 0x64006400u;
        p[1] = (t & k.m1) | 0x54005400u;
        const uint32_t t8 = t >> 8;
        p[2] = (t8 & k.m0) | 0x64006400u;
        p[3] = (t8 & k.m1) | 0x54005400u;
    }
    // one nibble position (0..3 of each 16-bit half) -> pair of bias(i) + nibble
    __device__ static __forceinline__ uint32_t unpack1(uint32_t t, int i, const NibbleMasks &k) {
        const uint32_t u = (i & 2) ? (t >> 8) : t;
        return (i & 1) ? ((u & k.m1) | 0x54005400u) : ((u & k.m0) | 0x64006400u);
    }
    // two bytes (low byte of each half) -> pair of 1024 + byte
    __device__ static __forceinline__ uint32_t unpack_bytes(uint32_t t) {
        return (t & 0x00FF00FFu) | 0x64006400u;
    }
    static constexpr float BYTE_BIAS = 1024.0f;
    __device__ static __forceinline__ float dot2(uint32_t a, uint32_t b, float c) {
        return __builtin_amdgcn_fdot2(__builtin_bit_cast(half2_t, a),
                                      __builtin_bit_cast(half2_t, b), c, false);
    }
    __device__ static __forceinline__ float to_f32(uint16_t v) {
        return (float)__builtin_bit_cast(_Float16, v);
    }
    __device__ static __forceinline__ uint16_t from_f32(float f) {
        return __builtin_bit_cast(uint16_t, (_Float16)f);
    }
};

struct BF16Traits {
    using elem_t = __bf16;
    static constexpr int DTYPE = 2;
    static constexpr uint32_t ONES = 0x3F803F80u;
    __device__ static __forceinline__ float bias(int) { return 128.0f; }
    __device__ static __forceinline__ void unpack4(uint32_t t, uint32_t p[4], const NibbleMasks &k) {
        p[0] = (t & k.m0) | 0x43004300u;
        p[1] = ((t >> 4) & k.m0) | 0x43004300u;
        p[2] = ((t >> 8) & k.m0) | 0x43004300u;
        p[3] = ((t >> 12) & k.m0) | 0x43004300u;
    }
    __device__ static __forceinline__ uint32_t unpack1(uint32_t t, int i, const NibbleMasks &k) {
        const uint32_t u = i ? (t >> (4 * i)) : t;
        return (u & k.m0) | 0x43004300u;
    }
    // bytes need 8 significant bits: go through f32 (exact), keep the high halves
    __device__ static __forceinline__ uint32_t unpack_bytes(uint32_t t) {
        const float lo = (float)(t & 0xFFu);
        const float hi = (float)((t >> 16) & 0xFFu);
        return (__builtin_bit_cast(uint32_t, lo) >> 16) |
               (__builtin_bit_cast(uint32_t, hi) & 0xFFFF0000u);
    }
    static constexpr float BYTE_BIAS = 0.0f;
    __device__ static __forceinline__ float dot2(uint32_t a, uint32_t b, float c) {
        return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, a),
                                               __builtin_bit_cast(bf16x2_t, b), c, false);
    }
    __device__ static __forceinline__ float to_f32(uint16_t v) {
        return __builtin_bit_cast(float, ((uint32_t)v) << 16);
    }
    __device__ static __forceinline__ uint16_t from_f32(float f) {  // round to nearest even
        uint32_t u = __builtin_bit_cast(uint32_t, f);
        if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x0040u);
        u += 0x7fffu + ((u >> 16) & 1u);
        return (uint16_t)(u >> 16);
    }
};

// E8M0 -> f32 power of two; 0xFF is NaN (mxfp4.rs:25-31), 0 is the subnormal 2^-127.
// Gate functions of the gated activations (ffn_kernels.metal:5-17), f32 in and out; shared by the
// stand-alone activation kernel and the fused gate|up epilogue so that both give the same bits.
// a * b rounded to f32 by one v_mul_f32, kept out of the compiler's sight: otherwise a narrowing
// conversion that follows may be merged with the multiply into a mixed-precision fma, which rounds
// once and turns a -0 product into +0, and two kernels finishing the same activation would differ
// in those bits.  With this the last step is the same everywhere: f32 product, then one narrowing.
__device__ __forceinline__ float mul_f32_rn(float a, float b) {
    float r;
    asm("v_mul_f32 %0, %1, %2" : "=v"(r) : "v"(a), "v"(b));
    return r;
}
// The logistic function through the hardware's exp2 and reciprocal (v_exp_f32, v_rcp_f32: an ulp each), five
// instructions where expf and an IEEE division take about forty - in a matmul epilogue that nothing overlaps
// (one workgroup a CU at prefill sizes) the difference is a tenth of the kernel.  The results are rounded to a
// 16-bit type afterwards; every kernel here takes these same functions, so they agree among themselves bit for
// bit.  e^-x = inf for very negative x gives 1 / inf = 0: the limit.
__device__ __forceinline__ float logistic_f32(float x) {
    return __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(x * -1.4426950408889634f));
}
__device__ __forceinline__ float silu_f32(float x) { return x * logistic_f32(x); }
// GPT-OSS clamped SwiGLU of one (gate, up) pair, alpha = 1.702 (moe.rs:152-173)
__device__ __forceinline__ float gpt_oss_swiglu_f32(float gate, float up, float limit) {
    gate = fminf(gate, limit);
    up = fminf(fmaxf(up, -limit), limit);
    const float sig = logistic_f32(gate * 1.702f);
    return mul_f32_rn(up + 1.0f, gate * sig);
}
__device__ __forceinline__ float gelu_tanh_f32(float x) {
    // 0.5 x (1 + tanh t) = x / (1 + e^(-2t)): no cancellation in the negative tail, where 1 + tanh t is tiny
    const float k0 = 0.7978845608028654f, k1 = 0.044715f;
    return x * logistic_f32(2.0f * (k0 * (x + k1 * x * x * x)));
}

__device__ __forceinline__ float e8m0_to_f32(uint32_t s) {
    const uint32_t bits = (s == 0xFFu) ? 0x7FC00000u : (s == 0u ? 0x00400000u : (s << 23));
    return __builtin_bit_cast(float, bits);
}

// ---------------------------------------------------------------------------
// Reductions
// ---------------------------------------------------------------------------
// Whole-wave reductions that leave the result in every lane, on the DPP lane permutes (pairs, quads,
// halves of 8 and rows of 16) and four lane reads for the rows: about twenty instructions, where the
// same butterfly through ds_bpermute is six trips through the LDS crossbar.  All 64 lanes must be active.
template <typename V, typename F>
__device__ __forceinline__ V wave_all_reduce(V v, F op) {
    static_assert(sizeof(V) == 4, "32-bit values");
    auto dpp = [](V x, auto ctrl) {
        return __builtin_bit_cast(V, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), decltype(ctrl)::value,
                                                                0xF, 0xF, false));
    };
    v = op(v, dpp(v, std::integral_constant<int, 0xB1>{}));   // quad_perm [1,0,3,2]: lane ^ 1
    v = op(v, dpp(v, std::integral_constant<int, 0x4E>{}));   // quad_perm [2,3,0,1]: lane ^ 2
    v = op(v, dpp(v, std::integral_constant<int, 0x141>{}));  // row_half_mirror: the other quad of 8
    v = op(v, dpp(v, std::integral_constant<int, 0x140>{}));  // row_mirror: the other half of 16
    const int b = __builtin_bit_cast(int, v);
    const V r0 = __builtin_bit_cast(V, __builtin_amdgcn_readlane(b, 0)), r1 = __builtin_bit_cast(V, __builtin_amdgcn_readlane(b, 16));
    const V r2 = __builtin_bit_cast(V, __builtin_amdgcn_readlane(b, 32)), r3 = __builtin_bit_cast(V, __builtin_amdgcn_readlane(b, 48));
    return op(op(r0, r1), op(r2, r3));
}

// v[l] + v[l ^ 16] and v[l] + v[l ^ 32] in every lane: v_permlane16_swap / v_permlane32_swap exchange
// the odd rows (upper half) of one register with the even rows (lower half) of the other, so with the
// value in both, the two results hold the two partners of every lane.  Vector ALU, no LDS crossbar.
__device__ __forceinline__ float add_lane_xor16(float v) {
    const uint32_t b = __builtin_bit_cast(uint32_t, v);
    const auto r = __builtin_amdgcn_permlane16_swap(b, b, false, false);
    const uint32_t r0 = r[0], r1 = r[1];
    return __builtin_bit_cast(float, r0) + __builtin_bit_cast(float, r1);
}
__device__ __forceinline__ float add_lane_xor32(float v) {
    const uint32_t b = __builtin_bit_cast(uint32_t, v);
    const auto r = __builtin_amdgcn_permlane32_swap(b, b, false, false);
    const uint32_t r0 = r[0], r1 = r[1];
    return __builtin_bit_cast(float, r0) + __builtin_bit_cast(float, r1);
}

template <int WIDTH>
__device__ __forceinline__ float wave_sum_xor(float v) {  // butterfly over WIDTH lanes
    if constexpr (WIDTH == 64) {
        return wave_all_reduce(v, [](float a, float b) { return a + b; });
    } else {
#pragma unroll
        for (int off = WIDTH / 2; off > 0; off >>= 1) v += __shfl_xor(v, off, WAVE);
        return v;
    }
}

// ---------------------------------------------------------------------------
// Deterministic split-K.
//
// Each of `splits` workgroups that share an output tile stores its f32 partial
// tile to the workspace; the partials are summed in slice order 0..splits-1,
// so the result does not depend on which workgroup finishes first.  Two ways
// to run that sum:
//
//  * a second kernel (splitk_reduce_kernel): plain stores, the kernel boundary
//    publishes them, every CU takes part in the reduction;
//  * fused: the last workgroup to arrive at the tile's counter does the sum.
//    Partials are written and read with device-scope relaxed atomics
//    (write-through / cache-bypassing accesses on gfx950), the arrival is a
//    device-scope atomic add issued after the workgroup's stores have
//    completed (s_waitcnt + barrier).  No cache write-back or invalidate is
//    needed, which on this part costs more than the whole GEMV.  The counter is
//    left at zero for the next launch.
// ---------------------------------------------------------------------------
__device__ __forceinline__ void st_agent(float *p, float v) {
    __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ float ld_agent(const float *p) {
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

__device__ __forceinline__ bool splitk_arrive(unsigned *counters, unsigned tile, unsigned splits) {
    __shared__ unsigned s_last;
    __atomic_signal_fence(__ATOMIC_SEQ_CST);
    __builtin_amdgcn_s_waitcnt(0);  // this wave's partial stores have completed
    __syncthreads();
    if (threadIdx.x == 0 && threadIdx.y == 0 && threadIdx.z == 0) {
        const unsigned old = __hip_atomic_fetch_add(&counters[tile], 1u, __ATOMIC_RELAXED,
                                                    __HIP_MEMORY_SCOPE_AGENT);
        const unsigned last = (old + 1u == splits) ? 1u : 0u;
        if (last)
            __hip_atomic_store(&counters[tile], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        s_last = last;
    }
    __syncthreads();
    __atomic_signal_fence(__ATOMIC_SEQ_CST);
    return s_last != 0u;
}

}  // namespace oxq
