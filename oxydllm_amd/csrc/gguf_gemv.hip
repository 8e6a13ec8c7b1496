// GGUF block-quant GEMV (Q4_0, Q8_0, Q4_K, Q6_K) over the raw ggml block bytes,
// and the matching dense dequant.
//
// Reference semantics: the weight is row n = K/QK consecutive blocks
// (linear.rs:225-240); element values follow the ggml formats as the reference
// restates them in quant_kernels.metal:2342-2384 (Q8_0/Q4_0), 2438-2482 (Q4_K)
// and 2518-2554 (Q6_K); y = x . W^T with f32 accumulation
// (quant_kernels.metal:792-870, 1097-1221, 1223-1436, 1681-1838).
//
// Work unit = 32 consecutive elements of one row (a whole Q4_0/Q8_0 block, one
// of the 8 sub-blocks of a K-quant super-block).  One wave per output row,
// lanes stride over the row's units, so 64 lanes read 64 consecutive units.
// All block offsets are even, so the bytes are fetched as 16-bit words.
// HBM-bound: every weight byte is read once per 8 activation rows.

#include "oxq_device.hpp"
#include "oxq_internal.hpp"

namespace oxq {

__device__ __forceinline__ uint32_t ld16(const uint8_t *p) { return *(const uint16_t *)p; }
__device__ __forceinline__ float ld_f16(const uint8_t *p) {
    return (float)__builtin_bit_cast(_Float16, *(const uint16_t *)p);
}

template <int FMT> struct GgufFmt;
template <> struct GgufFmt<OXQ_GGUF_Q4_0> { static constexpr int BE = 32, BB = 18; };
template <> struct GgufFmt<OXQ_GGUF_Q8_0> { static constexpr int BE = 32, BB = 34; };
template <> struct GgufFmt<OXQ_GGUF_Q4_K> { static constexpr int BE = 256, BB = 144; };
template <> struct GgufFmt<OXQ_GGUF_Q6_K> { static constexpr int BE = 256, BB = 210; };

// Decode unit `u` (32 elements) of the row starting at `row` into w[0..31].
template <int FMT>
__device__ __forceinline__ void decode_unit(const uint8_t *__restrict__ row, int u, float w[32]) {
    if constexpr (FMT == OXQ_GGUF_Q4_0) {
        const uint8_t *p = row + (size_t)u * 18;
        const float d = ld_f16(p);
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const uint32_t q = ld16(p + 2 + 2 * i);  // bytes 2i, 2i+1
            w[2 * i] = (float)((int)(q & 0xF) - 8) * d;
            w[2 * i + 16] = (float)((int)((q >> 4) & 0xF) - 8) * d;
            w[2 * i + 1] = (float)((int)((q >> 8) & 0xF) - 8) * d;
            w[2 * i + 17] = (float)((int)((q >> 12) & 0xF) - 8) * d;
        }
    } else if constexpr (FMT == OXQ_GGUF_Q8_0) {
        const uint8_t *p = row + (size_t)u * 34;
        const float d = ld_f16(p);
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const uint32_t q = ld16(p + 2 + 2 * i);
            w[2 * i] = (float)(int)(int8_t)(q & 0xFF) * d;
            w[2 * i + 1] = (float)(int)(int8_t)(q >> 8) * d;
        }
    } else if constexpr (FMT == OXQ_GGUF_Q4_K) {
        const int b = u >> 3, sb = u & 7;
        const uint8_t *p = row + (size_t)b * 144;
        const float d = ld_f16(p), dmin = ld_f16(p + 2);
        const uint8_t *sc = p + 4;
        uint32_t scv, mnv;
        if (sb < 4) {  // get_scale_min_k4
            scv = sc[sb] & 63u;
            mnv = sc[sb + 4] & 63u;
        } else {
            scv = (sc[sb + 4] & 0x0Fu) | ((uint32_t)(sc[sb - 4] >> 6) << 4);
            mnv = ((uint32_t)sc[sb + 4] >> 4) | ((uint32_t)(sc[sb] >> 6) << 4);
        }
        const float sc_v = d * (float)scv;
        const float m_v = dmin * (float)mnv;
        const uint8_t *qs = p + 16 + (sb >> 1) * 32;
        const int sh = (sb & 1) * 4;
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const uint32_t q = ld16(qs + 2 * i);
            w[2 * i] = sc_v * (float)((q >> sh) & 0xF) - m_v;
            w[2 * i + 1] = sc_v * (float)((q >> (8 + sh)) & 0xF) - m_v;
        }
    } else {  // Q6_K
        const int b = u >> 3, sub = u & 7;
        const int h = sub >> 2, quad = sub & 3;
        const uint8_t *p = row + (size_t)b * 210;
        const uint8_t *ql = p + 64 * h + (quad & 1) * 32;
        const uint8_t *qh = p + 128 + 32 * h;
        const int8_t *scales = (const int8_t *)(p + 192);
        const float d = ld_f16(p + 208);
        const float s0 = d * (float)scales[8 * h + 2 * quad];
        const float s1 = d * (float)scales[8 * h + 2 * quad + 1];
        const int shl = (quad < 2) ? 0 : 4;
        const int shh = 2 * quad;
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const uint32_t l16 = ld16(ql + 2 * i);
            const uint32_t h16 = ld16(qh + 2 * i);
            const int q0 = (int)(((l16 >> shl) & 0xF) | (((h16 >> shh) & 3) << 4)) - 32;
            const int q1 = (int)(((l16 >> (8 + shl)) & 0xF) | (((h16 >> (8 + shh)) & 3) << 4)) - 32;
            const float sv = (i < 8) ? s0 : s1;  // elements 0..15 / 16..31
            w[2 * i] = sv * (float)q0;
            w[2 * i + 1] = sv * (float)q1;
        }
    }
}

template <bool BF16X>
__device__ __forceinline__ float dot32(const void *__restrict__ xv, const float w[32]) {
    float acc = 0.0f;
    if constexpr (BF16X) {
        const u32x4_t *xp = (const u32x4_t *)xv;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const u32x4_t v = xp[i];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                acc = fmaf(__builtin_bit_cast(float, v[j] << 16), w[8 * i + 2 * j], acc);
                acc = fmaf(__builtin_bit_cast(float, v[j] & 0xFFFF0000u), w[8 * i + 2 * j + 1], acc);
            }
        }
    } else {
        const float4_t *xp = (const float4_t *)xv;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const float4_t v = xp[i];
#pragma unroll
            for (int j = 0; j < 4; ++j) acc = fmaf(v[j], w[4 * i + j], acc);
        }
    }
    return acc;
}

template <int FMT, bool BF16X, int MB>
__global__ __launch_bounds__(256) void gguf_gemv_kernel(const void *__restrict__ x,
                                                        const uint8_t *__restrict__ w,
                                                        const void *__restrict__ bias,
                                                        void *__restrict__ y, int M, int K, int N) {
    constexpr int XB = BF16X ? 2 : 4;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int n = blockIdx.x * 4 + wave;
    if (n >= N) return;
    const int units = K >> 5;
    const size_t row_bytes = (size_t)(K / GgufFmt<FMT>::BE) * GgufFmt<FMT>::BB;
    const uint8_t *row = w + (size_t)n * row_bytes;
    float acc[MB];
#pragma unroll
    for (int m = 0; m < MB; ++m) acc[m] = 0.0f;
    for (int u = lane; u < units; u += 64) {
        float wf[32];
        decode_unit<FMT>(row, u, wf);
#pragma unroll
        for (int m = 0; m < MB; ++m) {
            if (m < M) {
                const uint8_t *xr = (const uint8_t *)x + ((size_t)m * K + (size_t)u * 32) * XB;
                acc[m] += dot32<BF16X>(xr, wf);
            }
        }
    }
#pragma unroll
    for (int m = 0; m < MB; ++m) {
        if (m < M) {
            float tot = wave_sum_xor<64>(acc[m]);
            if (lane == 0) {
                if constexpr (BF16X) {
                    if (bias) tot += BF16Traits::to_f32(((const uint16_t *)bias)[n]);
                    ((uint16_t *)y)[(size_t)m * N + n] = BF16Traits::from_f32(tot);
                } else {
                    if (bias) tot += ((const float *)bias)[n];
                    ((float *)y)[(size_t)m * N + n] = tot;
                }
            }
        }
    }
}

template <int FMT>
__global__ __launch_bounds__(256) void gguf_dequant_kernel(const uint8_t *__restrict__ w,
                                                           float *__restrict__ out, int K, int N) {
    const int units = K >> 5;
    const size_t row_bytes = (size_t)(K / GgufFmt<FMT>::BE) * GgufFmt<FMT>::BB;
    const size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= (size_t)N * units) return;
    const int n = (int)(idx / units), u = (int)(idx % units);
    float wf[32];
    decode_unit<FMT>(w + (size_t)n * row_bytes, u, wf);
    float *o = out + (size_t)n * K + (size_t)u * 32;
#pragma unroll
    for (int i = 0; i < 32; ++i) o[i] = wf[i];
}

template <int FMT, bool BF16X>
static void launch_rows(hipStream_t s, dim3 grid, const GgufProblem &p, const uint8_t *x,
                        uint8_t *y, int rows) {
    const int K = (int)p.K, N = (int)p.N;
    dim3 block(256);
    if (rows <= 1)
        hipLaunchKernelGGL((gguf_gemv_kernel<FMT, BF16X, 1>), grid, block, 0, s, x, p.w, p.bias, y, rows, K, N);
    else if (rows <= 2)
        hipLaunchKernelGGL((gguf_gemv_kernel<FMT, BF16X, 2>), grid, block, 0, s, x, p.w, p.bias, y, rows, K, N);
    else if (rows <= 4)
        hipLaunchKernelGGL((gguf_gemv_kernel<FMT, BF16X, 4>), grid, block, 0, s, x, p.w, p.bias, y, rows, K, N);
    else
        hipLaunchKernelGGL((gguf_gemv_kernel<FMT, BF16X, 8>), grid, block, 0, s, x, p.w, p.bias, y, rows, K, N);
}

static const char *fmt_name(int q) {
    switch (q) {
    case OXQ_GGUF_Q4_0: return "q4_0";
    case OXQ_GGUF_Q8_0: return "q8_0";
    case OXQ_GGUF_Q4_K: return "q4k";
    default: return "q6k";
    }
}

int launch_gguf_gemv(oxq_ctx *ctx, hipStream_t s, const GgufProblem &p) {
    dim3 grid((unsigned)ceil_div(p.N, 4)), block(256);
    const bool bf = p.act_dtype == OXQ_BF16;
    const uint32_t chunks = (uint32_t)ceil_div(p.M, 8);
    char name[64];
    snprintf(name, sizeof name, "gguf_%s_gemv_%s", fmt_name(p.quant), bf ? "bf16" : "f32");
    set_plan(ctx, name, grid, block, 1, chunks, 0);
    if (ctx->plan_only) return OXQ_OK;
    const size_t xb = bf ? 2 : 4;
    // m > 8: activation rows are processed 8 at a time (the weight is re-read
    // per chunk; a tiled kernel for large m is future work).
    for (int64_t m0 = 0; m0 < p.M; m0 += 8) {
        const int rows = (int)((p.M - m0) < 8 ? (p.M - m0) : 8);
        const uint8_t *x = (const uint8_t *)p.x + (size_t)m0 * p.K * xb;
        uint8_t *y = (uint8_t *)p.y + (size_t)m0 * p.N * xb;
#define OXQ_FMT(F)                                              \
    if (bf) launch_rows<F, true>(s, grid, p, x, y, rows);       \
    else launch_rows<F, false>(s, grid, p, x, y, rows)
        switch (p.quant) {
        case OXQ_GGUF_Q4_0: OXQ_FMT(OXQ_GGUF_Q4_0); break;
        case OXQ_GGUF_Q8_0: OXQ_FMT(OXQ_GGUF_Q8_0); break;
        case OXQ_GGUF_Q4_K: OXQ_FMT(OXQ_GGUF_Q4_K); break;
        default: OXQ_FMT(OXQ_GGUF_Q6_K); break;
        }
#undef OXQ_FMT
    }
    OXQ_HIP_CHECK(hipGetLastError());
    return OXQ_OK;
}

int launch_gguf_dequant(oxq_ctx *ctx, hipStream_t s, const GgufProblem &p, float *out_nk) {
    const int K = (int)p.K, N = (int)p.N;
    const size_t units = (size_t)N * (K >> 5);
    dim3 grid((unsigned)ceil_div((int64_t)units, 256)), block(256);
    char name[64];
    snprintf(name, sizeof name, "gguf_%s_dequant", fmt_name(p.quant));
    set_plan(ctx, name, grid, block, 1, 1, 0);
    if (ctx->plan_only) return OXQ_OK;
    switch (p.quant) {
    case OXQ_GGUF_Q4_0: hipLaunchKernelGGL((gguf_dequant_kernel<OXQ_GGUF_Q4_0>), grid, block, 0, s, p.w, out_nk, K, N); break;
    case OXQ_GGUF_Q8_0: hipLaunchKernelGGL((gguf_dequant_kernel<OXQ_GGUF_Q8_0>), grid, block, 0, s, p.w, out_nk, K, N); break;
    case OXQ_GGUF_Q4_K: hipLaunchKernelGGL((gguf_dequant_kernel<OXQ_GGUF_Q4_K>), grid, block, 0, s, p.w, out_nk, K, N); break;
    default: hipLaunchKernelGGL((gguf_dequant_kernel<OXQ_GGUF_Q6_K>), grid, block, 0, s, p.w, out_nk, K, N); break;
    }
    OXQ_HIP_CHECK(hipGetLastError());
    return OXQ_OK;
}

}  // namespace oxq
