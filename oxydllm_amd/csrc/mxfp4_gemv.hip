// MXFP4 (E2M1 values, one E8M0 scale per 32) expert GEMV and dense dequant.
//
// Reference semantics: mxfp4.rs:13-64 (code table, low nibble first,
// scale 2^(s-127), 0xFF -> NaN) and quant_kernels.metal:3104-3173
// (mxfp4_gemv_batch_bf16: bf16 x/y, f32 accumulation).  The grouped form runs
// every active expert of one MoE projection in a single launch; it replaces
// the per-expert loop of moe.rs:593-605.
//
// One wave per output row; a lane owns whole 32-element blocks (one aligned
// 128-bit load each) and strides over the row.  HBM-bound.

#include "oxq_device.hpp"
#include "oxq_internal.hpp"

namespace oxq {

// E2M1 code -> f32: sign | exponent e (2 bits) | mantissa m (1 bit);
// e == 0 is the subnormal {0, 0.5}; else (1 + m/2) * 2^(e-1).
__device__ __forceinline__ float fp4_to_f32(uint32_t c) {
    const uint32_t e = (c >> 1) & 3u, m = c & 1u;
    uint32_t bits = e ? (((126u + e) << 23) | (m << 22)) : (m ? 0x3F000000u : 0u);
    bits |= (c & 8u) << 28;
    return __builtin_bit_cast(float, bits);
}

// E8M0 -> f32 power of two; 0xFF is NaN (mxfp4.rs:25-31), 0 is the subnormal 2^-127.
__device__ __forceinline__ float e8m0_to_f32(uint32_t s) {
    const uint32_t bits = (s == 0xFFu) ? 0x7FC00000u : (s == 0u ? 0x00400000u : (s << 23));
    return __builtin_bit_cast(float, bits);
}

__device__ __forceinline__ void decode_block(const u32x4_t q, float scale, float w[32]) {
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int b = 0; b < 4; ++b) {
            const uint32_t byte = (q[i] >> (8 * b)) & 0xFFu;
            w[8 * i + 2 * b] = fp4_to_f32(byte & 0xFu) * scale;
            w[8 * i + 2 * b + 1] = fp4_to_f32(byte >> 4) * scale;
        }
}

// Block dot product on the gfx950 conversion path: v_cvt_scalef32_pk_bf16_fp4
// turns one byte (two E2M1 codes, low nibble first) into a bf16 pair - every
// E2M1 value is exact in bf16 - and v_dot2_f32_bf16 multiplies it with the
// matching activation pair into an f32 accumulator.  One conversion and one
// dot per two weights; the E8M0 scale multiplies the block sum once.
// The activation pair is taken as a by-value uint32_t: bit-casting an element
// of a vector lvalue directly made the compiler read element 0 every time.
__device__ __forceinline__ float dot2_fp4(float acc, uint32_t xpair, bf16x2_t wpair) {
    return __builtin_amdgcn_fdot2_f32_bf16(wpair, __builtin_bit_cast(bf16x2_t, xpair), acc, false);
}

__device__ __forceinline__ float block_dot_bf16(const u32x4_t q, const uint16_t *__restrict__ xr) {
    const u32x4_t *xp = (const u32x4_t *)xr;
    float acc = 0.0f;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const u32x4_t xv = xp[i];
        const uint32_t w = q[i], x0 = xv[0], x1 = xv[1], x2 = xv[2], x3 = xv[3];
        acc = dot2_fp4(acc, x0, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(w, 1.0f, 0));
        acc = dot2_fp4(acc, x1, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(w, 1.0f, 1));
        acc = dot2_fp4(acc, x2, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(w, 1.0f, 2));
        acc = dot2_fp4(acc, x3, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(w, 1.0f, 3));
    }
    return acc;
}

// grid.x = row quads, grid.y = expert (1 for the plain form).
// offsets == nullptr: plain form, rows 0..M-1 of x / y.
template <int MB>
__global__ __launch_bounds__(256) void mxfp4_gemv_kernel(
    const uint16_t *__restrict__ x, const uint8_t *__restrict__ blocks,
    const uint8_t *__restrict__ scales, const uint16_t *__restrict__ bias,
    uint16_t *__restrict__ y, const int32_t *__restrict__ offsets,
    const int32_t *__restrict__ token_ids, int M, int K, int N) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int n = blockIdx.x * 4 + wave;
    if (n >= N) return;
    const int e = blockIdx.y;
    int p0 = 0, p1 = M;
    if (offsets) {
        p0 = offsets[e];
        p1 = offsets[e + 1];
        if (p1 <= p0) return;
    }
    const int nb = K >> 5;
    const size_t row = (size_t)e * N + n;
    const u32x4_t *brow = (const u32x4_t *)blocks + row * nb;
    const uint8_t *srow = scales + row * nb;
    const float bv = bias ? BF16Traits::to_f32(bias[row]) : 0.0f;

    for (int pbase = p0; pbase < p1; pbase += MB) {
        const int rows = min(MB, p1 - pbase);
        const uint16_t *xrow[MB];
#pragma unroll
        for (int m = 0; m < MB; ++m) {
            const int p = pbase + (m < rows ? m : 0);
            const int src = token_ids ? token_ids[p] : p;
            xrow[m] = x + (size_t)src * K;
        }
        float acc[MB];
#pragma unroll
        for (int m = 0; m < MB; ++m) acc[m] = 0.0f;
        for (int b = lane; b < nb; b += 64) {
            const u32x4_t q = brow[b];
            const float scale = e8m0_to_f32(srow[b]);
#pragma unroll
            for (int m = 0; m < MB; ++m)
                if (m < rows) acc[m] = fmaf(scale, block_dot_bf16(q, xrow[m] + (size_t)b * 32), acc[m]);
        }
#pragma unroll
        for (int m = 0; m < MB; ++m) {
            if (m < rows) {
                const float tot = wave_sum_xor<64>(acc[m]);
                if (lane == 0) y[(size_t)(pbase + m) * N + n] = BF16Traits::from_f32(tot + bv);
            }
        }
    }
}

__global__ __launch_bounds__(256) void mxfp4_dequant_kernel(const uint8_t *__restrict__ blocks,
                                                            const uint8_t *__restrict__ scales,
                                                            float *__restrict__ out, size_t nblocks) {
    const size_t b = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (b >= nblocks) return;
    float w[32];
    decode_block(((const u32x4_t *)blocks)[b], e8m0_to_f32(scales[b]), w);
    float *o = out + b * 32;
#pragma unroll
    for (int i = 0; i < 32; ++i) o[i] = w[i];
}

int launch_mxfp4_gemv(oxq_ctx *ctx, hipStream_t s, const Mxfp4Problem &p) {
    const bool grouped = p.n_experts > 0;
    dim3 grid((unsigned)ceil_div(p.N, 4), grouped ? (unsigned)p.n_experts : 1u), block(256);
    set_plan(ctx, grouped ? "mxfp4_moe_gemv_bf16" : "mxfp4_gemv_bf16", grid, block, 1, 1, 0);
    if (ctx->plan_only) return OXQ_OK;
    if (((uintptr_t)p.blocks & 15) || ((uintptr_t)p.x & 15) || (p.K % 8))
        return fail(OXQ_ERR_UNSUPPORTED, "mxfp4 gemv: blocks and x must be 16-byte aligned");
    const int M = (int)p.M, K = (int)p.K, N = (int)p.N;
    const int64_t rows_hint = grouped ? 8 : p.M;
#define OXQ_GO(MBv)                                                                                   \
    hipLaunchKernelGGL((mxfp4_gemv_kernel<MBv>), grid, block, 0, s, (const uint16_t *)p.x, p.blocks,  \
                       p.scales, (const uint16_t *)p.bias, (uint16_t *)p.y, p.expert_offsets,        \
                       p.token_ids, M, K, N)
    if (rows_hint <= 1) OXQ_GO(1);
    else if (rows_hint <= 2) OXQ_GO(2);
    else if (rows_hint <= 4) OXQ_GO(4);
    else OXQ_GO(8);
#undef OXQ_GO
    OXQ_HIP_CHECK(hipGetLastError());
    return OXQ_OK;
}

int launch_mxfp4_dequant(oxq_ctx *ctx, hipStream_t s, const Mxfp4Problem &p, float *out_nk) {
    const size_t nblocks = (size_t)p.N * (p.K >> 5);
    dim3 grid((unsigned)ceil_div((int64_t)nblocks, 256)), block(256);
    set_plan(ctx, "mxfp4_dequant", grid, block, 1, 1, 0);
    if (ctx->plan_only) return OXQ_OK;
    if ((uintptr_t)p.blocks & 15)
        return fail(OXQ_ERR_UNSUPPORTED, "mxfp4 dequant: blocks must be 16-byte aligned");
    hipLaunchKernelGGL(mxfp4_dequant_kernel, grid, block, 0, s, p.blocks, p.scales, out_nk, nblocks);
    OXQ_HIP_CHECK(hipGetLastError());
    return OXQ_OK;
}

}  // namespace oxq
