// Dense dequantization of AWQ / GPTQ packed weights to [K, N] in the scales'
// dtype.  Reference semantics: quant_kernels.metal:188-215 (awq_dequantize_impl)
// and 508-545 (gptq_dequantize_impl): T((float(q) - float(z)) * float(s)).
// The integer difference is exact and the f32 product of a small integer with
// a 16-bit float is exact, so the only rounding is the final conversion to T:
// the result is bit-identical to the CPU dequant (awq.rs:612-633, 561-590)
// converted with round-to-nearest-even.
//
// HBM-bound: reads 0.5 (or 1) byte and writes 2 bytes per element.

#include "oxq_device.hpp"
#include "oxq_internal.hpp"

namespace oxq {

template <typename TT, int BITS>
__global__ __launch_bounds__(256) void awq_dequant_kernel(const uint32_t *__restrict__ qw,
                                                          const uint32_t *__restrict__ qz,
                                                          const uint16_t *__restrict__ sc,
                                                          uint16_t *__restrict__ out, int K, int N,
                                                          int packed_out, int gshift) {
    constexpr int PF = 32 / BITS;
    constexpr uint32_t MASK = (1u << BITS) - 1u;
    const int j = blockIdx.x * blockDim.x + threadIdx.x;  // packed word column
    const int k = blockIdx.y;
    if (j >= packed_out || k >= K) return;
    const int g = k >> gshift;
    const uint32_t ww = qw[(size_t)k * packed_out + j];
    const uint32_t zw = qz[(size_t)g * packed_out + j];
    const uint16_t *srow = sc + (size_t)g * N + (size_t)j * PF;
    uint16_t vals[PF];
#pragma unroll
    for (int s = 0; s < PF; ++s) {
        const int col = (BITS == 4) ? awq_slot_col(s) : s;
        const int q = (int)((ww >> (BITS * s)) & MASK);
        const int z = (int)((zw >> (BITS * s)) & MASK);
        const float v = (float)(q - z) * TT::to_f32(srow[col]);
        vals[col] = TT::from_f32(v);
    }
    uint16_t *o = out + (size_t)k * N + (size_t)j * PF;
#pragma unroll
    for (int c = 0; c < PF; ++c) o[c] = vals[c];
}

template <typename TT, int BITS>
__global__ __launch_bounds__(256) void gptq_dequant_kernel(const uint32_t *__restrict__ qw,
                                                           const uint32_t *__restrict__ qz,
                                                           const uint16_t *__restrict__ sc,
                                                           uint16_t *__restrict__ out, int K, int N,
                                                           int gshift) {
    constexpr int PF = 32 / BITS;
    constexpr uint32_t MASK = (1u << BITS) - 1u;
    const int n = blockIdx.x * blockDim.x + threadIdx.x;
    const int iw = blockIdx.y;
    if (n >= N || iw * PF >= K) return;
    const uint32_t ww = qw[(size_t)iw * N + n];
    const int packed_out = N / PF;
#pragma unroll
    for (int s = 0; s < PF; ++s) {
        const int k = iw * PF + s;
        const int g = k >> gshift;
        const uint32_t zw = qz[(size_t)g * packed_out + n / PF];
        const int zp1 = (int)((zw >> (BITS * (n % PF))) & MASK) + 1;
        const int q = (int)((ww >> (BITS * s)) & MASK);
        const float v = (float)(q - zp1) * TT::to_f32(sc[(size_t)g * N + n]);
        out[(size_t)k * N + n] = TT::from_f32(v);
    }
}

int launch_wna16_dequant(oxq_ctx *ctx, hipStream_t s, const Wna16Problem &p, void *out_kn) {
    const int K = (int)p.K, N = (int)p.N;
    const int pf = 32 / p.bits;
    dim3 block(256);
    const uint16_t *sc = (const uint16_t *)p.scales;
    uint16_t *out = (uint16_t *)out_kn;
    if (p.pack_dim == OXQ_PACK_OUT) {
        const int packed_out = N / pf;
        dim3 grid((unsigned)ceil_div(packed_out, 256), (unsigned)K);
        set_plan(ctx, p.bits == 4 ? "awq_dequant_w4" : "awq_dequant_w8", grid, block, 1, 1, 0);
        if (ctx->plan_only) return OXQ_OK;
#define OXQ_LAUNCH(TT, BITS)                                                              \
    hipLaunchKernelGGL((awq_dequant_kernel<TT, BITS>), grid, block, 0, s, p.qweight, p.qzeros, sc, \
                       out, K, N, packed_out, p.group_shift)
        if (p.dtype == OXQ_F16) {
            if (p.bits == 4) OXQ_LAUNCH(F16Traits, 4); else OXQ_LAUNCH(F16Traits, 8);
        } else {
            if (p.bits == 4) OXQ_LAUNCH(BF16Traits, 4); else OXQ_LAUNCH(BF16Traits, 8);
        }
#undef OXQ_LAUNCH
    } else {
        dim3 grid((unsigned)ceil_div(N, 256), (unsigned)(K / pf));
        set_plan(ctx, p.bits == 4 ? "gptq_dequant_w4" : "gptq_dequant_w8", grid, block, 1, 1, 0);
        if (ctx->plan_only) return OXQ_OK;
#define OXQ_LAUNCH(TT, BITS)                                                               \
    hipLaunchKernelGGL((gptq_dequant_kernel<TT, BITS>), grid, block, 0, s, p.qweight, p.qzeros, sc, \
                       out, K, N, p.group_shift)
        if (p.dtype == OXQ_F16) {
            if (p.bits == 4) OXQ_LAUNCH(F16Traits, 4); else OXQ_LAUNCH(F16Traits, 8);
        } else {
            if (p.bits == 4) OXQ_LAUNCH(BF16Traits, 4); else OXQ_LAUNCH(BF16Traits, 8);
        }
#undef OXQ_LAUNCH
    }
    OXQ_HIP_CHECK(hipGetLastError());
    return OXQ_OK;
}

}  // namespace oxq
