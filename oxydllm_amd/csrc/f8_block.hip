// Block-scaled F8E4M3 (fn variant) weights: widening cast, dense BF16 dequant and GEMV.
//
// Reference semantics (quant_kernels.metal:3738-3934, host side metal_ops.rs:5500-5811): a
// weight value is bf16( f32(bf16(f8)) * scale ), scale = the F32 entry of the block grid
// that tiles the [out, in] weight (the loader's cast chain, replayed bit for bit; the inner
// bf16 rounding is exact because E4M3 has 3 mantissa bits); the GEMV accumulates
// f32(x) * f32(w) in f32 and writes BF16, 1 <= m <= 8, one writer per output and a fixed
// summation order.  The hardware conversion (v_cvt_pk_f32_fp8, OCP E4M3 on this target:
// bias 7, S.1111.111 = NaN, no infinity) decodes two bytes per instruction.
//
// GEMV: one wave per output row; lanes stride over 16-byte chunks of the row (16 weights,
// one scale when the block width is a multiple of 16), each weight decoded once and used
// for all m rows of x; the wave's partial sums meet in a fixed-order butterfly.

#include "oxq_device.hpp"
#include "oxq_internal.hpp"

namespace oxq {

typedef float f8_f2_t __attribute__((ext_vector_type(2)));

__device__ __forceinline__ uint32_t f8_pack_bf16(float lo, float hi) {
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(f8_f2_t{lo, hi}, bf16x2_t));
}

// four bytes of `w` -> f32
__device__ __forceinline__ void f8x4_to_f32(uint32_t w, float o[4]) {
    const f8_f2_t lo = __builtin_amdgcn_cvt_pk_f32_fp8((int)w, false);
    const f8_f2_t hi = __builtin_amdgcn_cvt_pk_f32_fp8((int)w, true);
    o[0] = lo[0], o[1] = lo[1], o[2] = hi[0], o[3] = hi[1];
}

__global__ __launch_bounds__(256) void cast_f8e4m3_f32_kernel(const uint8_t *__restrict__ in,
                                                              float *__restrict__ out, size_t n) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n) return;
    const uint32_t b = in[i];
    out[i] = __builtin_amdgcn_cvt_pk_f32_fp8((int)b, false)[0];
}

__global__ __launch_bounds__(256) void f8_block_dequant_bf16_kernel(const uint8_t *__restrict__ in,
                                                                    const float *__restrict__ scales,
                                                                    uint16_t *__restrict__ out, int cols,
                                                                    size_t n, int block_r, int block_c,
                                                                    int s_cols) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n) return;
    const int r = (int)(i / cols), c = (int)(i % cols);
    const float w = __builtin_amdgcn_cvt_pk_f32_fp8((int)(uint32_t)in[i], false)[0];  // exact in bf16
    const float sc = scales[(size_t)(r / block_r) * s_cols + c / block_c];
    out[i] = (uint16_t)f8_pack_bf16(w * sc, 0.0f);
}

// CHUNKED: 16 weights share one scale and rows are 16-byte aligned (block_c % 16 == 0,
// K % 16 == 0); otherwise one weight per lane and step.
template <int MB, bool CHUNKED>
__global__ __launch_bounds__(256) void f8_gemv_kernel(const uint16_t *__restrict__ x,
                                                      const uint8_t *__restrict__ w,
                                                      const float *__restrict__ scales,
                                                      uint16_t *__restrict__ y, int M, int K, int N,
                                                      int block_r, int block_c, int s_cols) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int n = blockIdx.x * 4 + wave;
    if (n >= N) return;
    const uint8_t *wrow = w + (size_t)n * K;
    const float *srow = scales + (size_t)(n / block_r) * s_cols;
    float acc[MB];
#pragma unroll
    for (int m = 0; m < MB; ++m) acc[m] = 0.0f;
    if (CHUNKED) {
        for (int c = lane; c < (K >> 4); c += 64) {
            const u32x4_t q = __builtin_nontemporal_load((const u32x4_t *)(wrow + (size_t)c * 16));  // read once
            const float sc = srow[(c * 16) / block_c];
            const uint32_t q0 = q[0], q1 = q[1], q2 = q[2], q3 = q[3];
            const uint32_t qw[4] = {q0, q1, q2, q3};
            float wf[16];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                float t[4];
                f8x4_to_f32(qw[i], t);
                const uint32_t p0 = f8_pack_bf16(t[0] * sc, t[1] * sc), p1 = f8_pack_bf16(t[2] * sc, t[3] * sc);
                wf[4 * i] = __builtin_bit_cast(float, p0 << 16);
                wf[4 * i + 1] = __builtin_bit_cast(float, p0 & 0xFFFF0000u);
                wf[4 * i + 2] = __builtin_bit_cast(float, p1 << 16);
                wf[4 * i + 3] = __builtin_bit_cast(float, p1 & 0xFFFF0000u);
            }
#pragma unroll
            for (int m = 0; m < MB; ++m) {
                if (m < M) {
                    const u32x4_t *xp = (const u32x4_t *)(x + (size_t)m * K + (size_t)c * 16);
#pragma unroll
                    for (int h = 0; h < 2; ++h) {
                        const u32x4_t xv = xp[h];
                        const uint32_t x0 = xv[0], x1 = xv[1], x2 = xv[2], x3 = xv[3];
                        const uint32_t xs[4] = {x0, x1, x2, x3};
#pragma unroll
                        for (int i = 0; i < 4; ++i) {
                            acc[m] = fmaf(__builtin_bit_cast(float, xs[i] << 16), wf[8 * h + 2 * i], acc[m]);
                            acc[m] = fmaf(__builtin_bit_cast(float, xs[i] & 0xFFFF0000u), wf[8 * h + 2 * i + 1], acc[m]);
                        }
                    }
                }
            }
        }
    } else {
        for (int k = lane; k < K; k += 64) {
            const float t = __builtin_amdgcn_cvt_pk_f32_fp8((int)(uint32_t)wrow[k], false)[0];
            const float wv = __builtin_bit_cast(float, f8_pack_bf16(t * srow[k / block_c], 0.0f) << 16);
#pragma unroll
            for (int m = 0; m < MB; ++m)
                if (m < M) acc[m] = fmaf(BF16Traits::to_f32(x[(size_t)m * K + k]), wv, acc[m]);
        }
    }
#pragma unroll
    for (int m = 0; m < MB; ++m) {
        if (m < M) {
            const float tot = wave_sum_xor<64>(acc[m]);
            if (lane == 0) y[(size_t)m * N + n] = (uint16_t)f8_pack_bf16(tot, 0.0f);
        }
    }
}

int launch_cast_f8e4m3_f32(oxq_ctx *ctx, hipStream_t s, const uint8_t *in, float *out, size_t n) {
    dim3 grid((unsigned)ceil_div((int64_t)n, 256)), block(256);
    set_plan(ctx, "cast_f8e4m3_f32", grid, block, 1, 1, 0);
    if (ctx->plan_only || n == 0) return OXQ_OK;
    hipLaunchKernelGGL(cast_f8e4m3_f32_kernel, grid, block, 0, s, in, out, n);
    OXQ_HIP_CHECK(hipGetLastError());
    return OXQ_OK;
}

int launch_f8_block_dequant(oxq_ctx *ctx, hipStream_t s, const F8Problem &p, uint16_t *out) {
    const size_t n = (size_t)p.N * p.K;
    dim3 grid((unsigned)ceil_div((int64_t)n, 256)), block(256);
    set_plan(ctx, "f8_block_dequant_bf16", grid, block, 1, 1, 0);
    if (ctx->plan_only || n == 0) return OXQ_OK;
    hipLaunchKernelGGL(f8_block_dequant_bf16_kernel, grid, block, 0, s, p.w, p.scales, out, (int)p.K, n,
                       (int)p.block_r, (int)p.block_c, (int)p.s_cols);
    OXQ_HIP_CHECK(hipGetLastError());
    return OXQ_OK;
}

template <bool CHUNKED>
static void f8_gemv_go(hipStream_t s, dim3 grid, const F8Problem &p, const uint16_t *x, uint16_t *y, int rows) {
    dim3 block(256);
#define OXQ_F8(MBv)                                                                                       \
    hipLaunchKernelGGL((f8_gemv_kernel<MBv, CHUNKED>), grid, block, 0, s, x, p.w, p.scales, y, rows, (int)p.K, \
                       (int)p.N, (int)p.block_r, (int)p.block_c, (int)p.s_cols)
    if (rows <= 1) OXQ_F8(1);
    else if (rows <= 2) OXQ_F8(2);
    else if (rows <= 4) OXQ_F8(4);
    else OXQ_F8(8);
#undef OXQ_F8
}

// any m: rows of x are taken 8 at a time (the tile matmul handles large m where it applies)
int launch_f8_gemv(oxq_ctx *ctx, hipStream_t s, const F8Problem &p) {
    const bool chunked = p.K % 16 == 0 && p.block_c % 16 == 0 && ((uintptr_t)p.w & 15) == 0 &&
                         ((uintptr_t)p.x & 15) == 0;
    dim3 grid((unsigned)ceil_div(p.N, 4)), block(256);
    set_plan(ctx, chunked ? "f8_gemv_bf16" : "f8_gemv_bf16_bytes", grid, block, 1, (uint32_t)ceil_div(p.M, 8), 0);
    if (ctx->plan_only) return OXQ_OK;
    for (int64_t m0 = 0; m0 < p.M; m0 += 8) {
        const int rows = (int)std::min<int64_t>(8, p.M - m0);
        const uint16_t *x = (const uint16_t *)p.x + (size_t)m0 * p.K;
        uint16_t *y = (uint16_t *)p.y + (size_t)m0 * p.N;
        if (chunked) f8_gemv_go<true>(s, grid, p, x, y, rows);
        else f8_gemv_go<false>(s, grid, p, x, y, rows);
    }
    OXQ_HIP_CHECK(hipGetLastError());
    return OXQ_OK;
}

}  // namespace oxq
