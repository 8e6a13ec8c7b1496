// GGUF block-quant GEMV (Q4_0, Q4_1, Q5_0, Q5_1, Q8_0, Q2_K, Q3_K, Q4_K, Q5_K, Q6_K)
// over the raw ggml block bytes, and the matching dense dequant.
//
// Reference semantics: the weight is row n = K/QK consecutive blocks
// (linear.rs:225-240); element values follow the ggml formats as the reference
// restates them in quant_kernels.metal:2315-2640 (one dequant strip per format);
// y = x . W^T with f32 accumulation (quant_kernels.metal:709-2300, one gemv per format).
//
// Work unit = 32 consecutive elements of one row (a whole Q4_0/Q8_0 block, one
// of the 8 sub-blocks of a K-quant super-block).  One wave per output row,
// lanes stride over the row's units, so 64 lanes read 64 consecutive units.
// All block offsets are even, so the bytes are fetched as 16-bit words.
// HBM-bound: every weight byte is read once per 8 activation rows.

#include "gguf_decode.hpp"

#include <cstdlib>

namespace oxq {

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

// ---------------------------------------------------------------------------
// GEMV with rows and activations staged in LDS.
//
// With one wave per row reading global memory directly, every wave re-reads the
// activations from L2 and fetches its blocks with two-byte loads, and the decode
// spends about five vector instructions per weight (extract, convert, subtract the
// offset, scale, multiply-add).  Here a workgroup copies its `rpwg` consecutive rows -
// one contiguous byte range - and the activations into LDS with 16-byte loads, and the
// per-unit arithmetic is factored the way the reference's kernels factor it
// (quant_kernels.metal:1097-1221, 1681-1838): the raw integers are converted once,
//     y_unit = scale * (sum q_i x_i) - offset * (sum x_i),
// and the sums of x over 16 elements are computed once per workgroup, not per row.
// ---------------------------------------------------------------------------
// Activations sit in LDS unit by unit: the CPU 16-byte chunks of unit u at u * (CPU + 1) * 16, one
// pad chunk after each unit.  Consecutive lanes (units) then read at a pitch of 144 (f32) or 80 (bf16)
// bytes, which puts every 8 neighbouring lanes on the 8 different 16-byte bank groups, and a chunk's
// offset inside its unit is an immediate of the load (one address register a unit).  Behind the
// activations: the sums of x over every 16 elements (two floats a unit), computed once per workgroup.
// 8 consecutive activations (index 8*o .. 8*o+7 of the unit at `xu`) as f32:
template <bool BF16X>
__device__ __forceinline__ void ld_x8(const unsigned char *xu, int o, float out[8]) {
    if constexpr (BF16X) {
        const u32x4_t v = *(const u32x4_t *)(xu + o * 16);
        const uint32_t v0 = v[0], v1 = v[1], v2 = v[2], v3 = v[3];
        const uint32_t vv[4] = {v0, v1, v2, v3};
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            out[2 * j] = __builtin_bit_cast(float, vv[j] << 16);
            out[2 * j + 1] = __builtin_bit_cast(float, vv[j] & 0xFFFF0000u);
        }
    } else {
        const float4_t a = *(const float4_t *)(xu + (2 * o) * 16);
        const float4_t b = *(const float4_t *)(xu + (2 * o + 1) * 16);
        out[0] = a[0], out[1] = a[1], out[2] = a[2], out[3] = a[3];
        out[4] = b[0], out[5] = b[1], out[6] = b[2], out[7] = b[3];
    }
}

// PW (one activation row, one weight row per wave, the launcher checks the sizes): every wave
// fetches its own weight row and only the activations meet at the barrier.  Staged jointly the
// kernel is the sum of its parts (4096 x 4096 Q4_K, M = 1: 6.9 us = 2.65 us launch and activations
// + 1.85 us weights + 2.5 us decode and dot, each measured with the others cut out): nobody
// computes until the last row of the workgroup has arrived.
template <int FMT, bool BF16X, int MB, bool PW>
__global__ __launch_bounds__(PW ? 1024 : 512) void gguf_gemv_lds_kernel(const void *__restrict__ x,
                                                            const uint8_t *__restrict__ w,
                                                            const void *__restrict__ bias,
                                                            void *__restrict__ y, int M, int K, int N,
                                                            int rpwg, size_t total_bytes) {
    constexpr int XB = BF16X ? 2 : 4;
    extern __shared__ __attribute__((aligned(16))) unsigned char gg_lds[];
    constexpr int CPU = 32 * XB / 16;                                 // 16-byte chunks per unit
    constexpr int XP = (CPU + 1) * 16;                                // bytes of one unit's activations + pad
    const size_t xrow_bytes = ((size_t)(K >> 5) * (XP + 8) + 15) & ~(size_t)15;  // units, then 2 sums a unit
    unsigned char *lds_x = gg_lds;                                   // [MB] chunked activations
    unsigned char *lds_w = gg_lds + (size_t)MB * xrow_bytes;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int n0 = blockIdx.x * rpwg;
    const int nrows = min(rpwg, N - n0);
    const int units = K >> 5;
    const size_t row_bytes = (size_t)(K / GgufFmt<FMT>::BE) * GgufFmt<FMT>::BB;
    const size_t start = (size_t)n0 * row_bytes, a0 = start & ~(size_t)15;
    const int head = (int)(start - a0);
    const int wchunks = (int)((head + (size_t)nrows * row_bytes + 15) >> 4);
    const int cpr = K * XB / 16;  // chunks per activation row
    const int nthr = blockDim.x, nwaves = blockDim.x >> 6;
    constexpr int CB = 4;
    constexpr int WCH = 6;  // 16-byte chunks per lane that hold one weight row (PW)
    // chunks that lie wholly inside the tensor; only the tensor's very last chunk can be partial
    const int full = (int)min((size_t)wchunks, (total_bytes - a0) >> 4);
    const u32x4_t *wsrc = (const u32x4_t *)(w + a0);
    // sums of x over every 16 elements, once per workgroup (every row's decode needs them: the offset
    // terms of the formats multiply them).  Association: the elements of a 16-byte chunk in order, then
    // the chunks of the half unit pairwise - what the wave-per-row form gets from lane exchanges.
    auto chunk_sum = [](const u32x4_t v) {
        float sx = 0.0f;
        if constexpr (BF16X) {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const uint32_t e = v[j];
                sx += __builtin_bit_cast(float, e << 16) + __builtin_bit_cast(float, e & 0xFFFF0000u);
            }
        } else {
#pragma unroll
            for (int j = 0; j < 4; ++j) sx += __builtin_bit_cast(float, (uint32_t)v[j]);
        }
        return sx;
    };
    auto stage_sums = [&]() {
        constexpr int HC = CPU / 2;
        for (int t = threadIdx.x; t < MB * 2 * units; t += nthr) {
            const int m = MB == 1 ? 0 : t / (2 * units), hu = t - m * 2 * units;
            if (m < M) {
                unsigned char *xr = lds_x + m * xrow_bytes;
                const u32x4_t *c = (const u32x4_t *)(xr + (hu >> 1) * XP + (hu & 1) * HC * 16);
                float sx = chunk_sum(c[0]) + chunk_sum(c[1]);
                if constexpr (HC == 4) sx += chunk_sum(c[2]) + chunk_sum(c[3]);
                ((float *)(xr + (size_t)units * XP))[hu] = sx;
            }
        }
    };
    if constexpr (PW) {
        // one straight-line batch of activation loads, then the wave's own row: the compiler can count
        // the younger loads, so storing the activations leaves the weights in flight
        // (buffer loads: out-of-range lanes need no branch, which would make the count unknowable)
        constexpr int OOB = 0x7FFFFF00;
        const __amdgpu_buffer_rsrc_t rs_x = make_rsrc(x, (uint32_t)cpr * 16u);
        const __amdgpu_buffer_rsrc_t rs_w = make_rsrc(w + a0, (uint32_t)full * 16u);
        u32x4_t xv[CB], wv[WCH];
#pragma unroll
        for (int b = 0; b < CB; ++b)
            xv[b] = __builtin_amdgcn_raw_buffer_load_b128(rs_x, ((int)threadIdx.x + b * nthr) * 16, 0, 0);
        const size_t rb = head + (size_t)wave * row_bytes;  // the row's bytes inside the workgroup's span
        const int wc0 = (int)(rb >> 4);
        const int wc1 = wave < nrows ? min((int)((rb + row_bytes + 15) >> 4), full) : wc0;
#pragma unroll
        for (int q = 0; q < WCH; ++q) {
            const int c = wc0 + lane + 64 * q;
            wv[q] = __builtin_amdgcn_raw_buffer_load_b128(rs_w, c < wc1 ? c * 16 : OOB, 0, 2);  // nontemporal
        }
        // stores without a branch as well (a load whose only use is conditional gets moved into the
        // branch): lanes past the row write the unused padding chunk of the layout, unit index `units`
#pragma unroll
        for (int b = 0; b < CB; ++b) {
            const int g = (int)threadIdx.x + b * nthr;
            const int u = g / CPU, cc = g - u * CPU;
            *(u32x4_t *)(lds_x + (g < cpr ? u * XP + cc * 16 : CPU * 16)) = xv[b];  // else: unit 0's pad
            // the sums of x over 16 elements, from the registers that carry x: a chunk's own elements,
            // then the HC chunks of a half unit, which neighbouring lanes hold (lane ^ 1, lane ^ 2)
            constexpr int HC = CPU / 2;
            float sx = chunk_sum(xv[b]);
            sx += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, sx), 0xB1, 0xF, 0xF, false));
            if constexpr (HC == 4)
                sx += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, sx), 0x4E, 0xF, 0xF, false));
            if (g < cpr && (cc & (HC - 1)) == 0) ((float *)(lds_x + (size_t)units * XP))[2 * u + cc / HC] = sx;
        }
        __syncthreads();  // the one barrier comes before the wait for the wave's own weight row
#pragma unroll
        for (int q = 0; q < WCH; ++q) {
            const int c = wc0 + lane + 64 * q;
            if (c < wc1) ((u32x4_t *)lds_w)[c] = wv[q];
        }
        if (full < wchunks && wave == nrows - 1 && lane == 0) {  // the tensor's last, partial chunk: byte by byte
            const size_t off = a0 + (size_t)full * 16;
            uint32_t t[4] = {0u, 0u, 0u, 0u};
            for (int i = 0; i < 16; ++i)
                if (off + i < total_bytes) t[i >> 2] |= (uint32_t)w[off + i] << (8 * (i & 3));
            ((u32x4_t *)lds_w)[full] = u32x4_t{t[0], t[1], t[2], t[3]};
        }
    } else {
    // Staging copies in batches of 4 loads per thread: with one load per loop trip every
    // trip pays a full memory round trip before its LDS store.
    for (int base = threadIdx.x; base < full; base += nthr * CB) {
        u32x4_t v[CB];
#pragma unroll
        for (int b = 0; b < CB; ++b) {
            const int c = base + b * nthr;
            v[b] = c < full ? __builtin_nontemporal_load(wsrc + c) : u32x4_t{0u, 0u, 0u, 0u};  // read once
        }
#pragma unroll
        for (int b = 0; b < CB; ++b) {
            const int c = base + b * nthr;
            if (c < full) ((u32x4_t *)lds_w)[c] = v[b];
        }
    }
    if (full < wchunks && threadIdx.x == 0) {  // the tensor's last, partial chunk: byte by byte
        const size_t off = a0 + (size_t)full * 16;
        uint32_t t[4] = {0u, 0u, 0u, 0u};
        for (int i = 0; i < 16; ++i)
            if (off + i < total_bytes) t[i >> 2] |= (uint32_t)w[off + i] << (8 * (i & 3));
        ((u32x4_t *)lds_w)[full] = u32x4_t{t[0], t[1], t[2], t[3]};
    }
    // activations, row by row (no division per chunk): chunk g of a row holds elements 16 / XB * g ...
#pragma unroll
    for (int m = 0; m < MB; ++m) {
        if (m < M) {
            const u32x4_t *xsrc = (const u32x4_t *)x + (size_t)m * cpr;
            unsigned char *xdst = lds_x + m * xrow_bytes;
            for (int base = threadIdx.x; base < cpr; base += nthr * CB) {
                u32x4_t v[CB];
#pragma unroll
                for (int b = 0; b < CB; ++b) {
                    const int g = base + b * nthr;
                    v[b] = g < cpr ? xsrc[g] : u32x4_t{0u, 0u, 0u, 0u};
                }
#pragma unroll
                for (int b = 0; b < CB; ++b) {
                    const int g = base + b * nthr;
                    if (g < cpr) {
                        const int u = g / CPU, cc = g - u * CPU;  // CPU is a power of two
                        *(u32x4_t *)(xdst + (size_t)u * XP + cc * 16) = v[b];
                    }
                }
            }
        }
    }
    __syncthreads();
    stage_sums();
    __syncthreads();
    }
    for (int r = wave; r < nrows; r += nwaves) {
        const uint8_t *row = lds_w + head + (size_t)r * row_bytes;
        const int n = n0 + r;
        float acc[MB];
#pragma unroll
        for (int m = 0; m < MB; ++m) acc[m] = 0.0f;
        // unit `u` of the row against every activation row
        auto add_unit = [&](int u) {
            float q[32], c0, c1, d0, d1;
            unit_ints<FMT>(row, u, q, c0, c1, d0, d1);
#pragma unroll
            for (int m = 0; m < MB; ++m) {
                if (m < M) {
                    const unsigned char *xr = lds_x + m * xrow_bytes;
                    const unsigned char *xu = xr + u * XP;
                    const float2 sx = *(const float2 *)(xr + (size_t)units * XP + u * 8);
                    float dot0 = 0.0f, dot1 = 0.0f;
#pragma unroll
                    for (int o = 0; o < 4; ++o) {
                        float xv[8];
                        ld_x8<BF16X>(xu, o, xv);
#pragma unroll
                        for (int i = 0; i < 8; ++i) {
                            if (o < 2) dot0 = fmaf(q[8 * o + i], xv[i], dot0);
                            else dot1 = fmaf(q[8 * o + i], xv[i], dot1);
                        }
                    }
                    acc[m] += (c0 * dot0 + c1 * dot1) - (d0 * sx.x + d1 * sx.y);
                }
            }
        };
        for (int u = lane; u < units; u += 64) add_unit(u);
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

static const char *fmt_name(int q) {
    switch (q) {
    case OXQ_GGUF_Q4_0: return "q4_0";
    case OXQ_GGUF_Q8_0: return "q8_0";
    case OXQ_GGUF_Q4_K: return "q4k";
    case OXQ_GGUF_Q4_1: return "q4_1";
    case OXQ_GGUF_Q5_0: return "q5_0";
    case OXQ_GGUF_Q5_1: return "q5_1";
    case OXQ_GGUF_Q2_K: return "q2k";
    case OXQ_GGUF_Q3_K: return "q3k";
    case OXQ_GGUF_Q5_K: return "q5k";
    default: return "q6k";
    }
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

template <int FMT, bool BF16X, int MB, bool PW = false>
static int launch_rows_lds_mb(hipStream_t s, const GgufProblem &p, const uint8_t *x, uint8_t *y, int rows,
                              int rpwg, size_t lds) {
    static LdsGrant lds_grant;  // one per instantiation
    OXQ_HIP_CHECK(lds_grant.ensure((const void *)gguf_gemv_lds_kernel<FMT, BF16X, MB, PW>, lds));
    const int K = (int)p.K, N = (int)p.N;
    const size_t total = (size_t)N * (size_t)(K / GgufFmt<FMT>::BE) * GgufFmt<FMT>::BB;
    // one wave per row at a time: 8 waves for 8 rows (x is staged once per 8 rows), else 4; the
    // wave-per-row form also runs 16 rows on 16 waves
    dim3 grid((unsigned)ceil_div(N, rpwg)), block(PW && rpwg >= 16 ? 1024 : rpwg >= 8 ? 512 : 256);
    hipLaunchKernelGGL((gguf_gemv_lds_kernel<FMT, BF16X, MB, PW>), grid, block, lds, s, x, p.w, p.bias, y, rows, K,
                       N, rpwg, total);
    return OXQ_OK;
}

template <int FMT, bool BF16X>
static int launch_rows_lds(const oxq_ctx *ctx, hipStream_t s, const GgufProblem &p, const uint8_t *x, uint8_t *y,
                           int rows, int rpwg, size_t lds) {
    if (rows <= 1) {
        // a wave per weight row needs: 8 waves for the 8 rows, the row in 6 chunks a lane, x in one batch
        const size_t row_bytes = (size_t)(p.K / GgufFmt<FMT>::BE) * GgufFmt<FMT>::BB;
        if ((rpwg == 8 || rpwg == 16) && row_bytes + 30 <= 6 * 64 * 16 &&
            p.K * (BF16X ? 2 : 4) / 16 <= 4 * 64 * rpwg && tune(ctx, OXQ_TUNE_GGUF_PW, 1) != 0)
            return launch_rows_lds_mb<FMT, BF16X, 1, true>(s, p, x, y, rows, rpwg, lds);
        return launch_rows_lds_mb<FMT, BF16X, 1>(s, p, x, y, rows, rpwg, lds);
    }
    if (rows <= 2) return launch_rows_lds_mb<FMT, BF16X, 2>(s, p, x, y, rows, rpwg, lds);
    if (rows <= 4) return launch_rows_lds_mb<FMT, BF16X, 4>(s, p, x, y, rows, rpwg, lds);
    return launch_rows_lds_mb<FMT, BF16X, 8>(s, p, x, y, rows, rpwg, lds);
}

static size_t gguf_row_bytes(int quant, int64_t K) {
    int64_t be = 0, bb = 0;
    oxq_gguf_block_layout(quant, &be, &bb);
    return (size_t)(K / be) * (size_t)bb;
}

int launch_gguf_gemv(oxq_ctx *ctx, hipStream_t s, const GgufProblem &p) {
    const bool bf = p.act_dtype == OXQ_BF16;
    const size_t xb = bf ? 2 : 4;
    const size_t row_bytes = gguf_row_bytes(p.quant, p.K);
    const bool aligned = ((uintptr_t)p.x & 15) == 0 && ((uintptr_t)p.w & 15) == 0 && (p.K * xb) % 16 == 0 &&
                         !tune(ctx, OXQ_TUNE_FORCE_GENERIC, 0);
    // The staged kernel for `mb` activation rows a pass: x (per row K/32 units of 32 elements + one 16-byte
    // pad each, then two sums a unit) and `rpwg` weight rows in LDS.  8 rows on 8 waves; for one activation
    // row OXQ_GGUF_RPWG=16 runs 16 rows on 16 waves, which halves the activation traffic (every workgroup
    // stages all of x): measured slower on 4096 x 4096 (Q4_0 5.5 against 5.1 us, Q6_K 6.8 against 6.0 us); 16
    // rows on 8 waves of two rows each: 6.0 and 7.5 us.  64 KB of LDS a workgroup (two or more per CU) while
    // at least 4 weight rows fit beside x; otherwise up to 150 KB, one workgroup per CU, if 8 rows fit then
    // (a down projection: K = 14336 is 68 KB of f32 x alone; Q4_1 14336 x 4096 at one row 31 -> 17 us; with
    // 4 rows a workgroup the staged kernel is no faster than a wave per row from global memory).
    struct Staged {
        bool ok;
        int rpwg;
        size_t lds;
    };
    auto staged = [&](int mb) -> Staged {
        const size_t x_lds = (size_t)mb * ((((size_t)(p.K >> 5) * ((32 * xb / 16 + 1) * 16 + 8)) + 15) & ~(size_t)15);
        const bool wave_per_row = mb == 1 && row_bytes + 30 <= 6 * 64 * 16 && tune(ctx, OXQ_TUNE_GGUF_PW, 1) != 0;
        int rpwg = tune(ctx, OXQ_TUNE_GGUF_RPWG, 8);
        if (rpwg < 1) rpwg = 1;
        if (rpwg > 8 && !(wave_per_row && rpwg == 16 && p.K * (int64_t)xb / 16 <= 4 * 64 * 16)) rpwg = 8;
        const int rp0 = rpwg;
        auto lds_cap_of = [](int r) { return (size_t)(r == 16 ? 128 : 64) * 1024; };
        while (rpwg > 1 && x_lds + (size_t)rpwg * row_bytes + 32 > lds_cap_of(rpwg)) rpwg >>= 1;
        size_t cap = lds_cap_of(rpwg);
        if ((rpwg < 4 || x_lds + (size_t)rpwg * row_bytes + 32 > cap) && rp0 >= 8 && tune(ctx, OXQ_TUNE_GGUF_BIG_LDS, 1) != 0 &&
            x_lds + (size_t)8 * row_bytes + 32 <= (size_t)150 * 1024)
            rpwg = 8, cap = (size_t)150 * 1024;
        const size_t lds = x_lds + (size_t)rpwg * row_bytes + 32;
        return Staged{aligned && lds <= cap, rpwg, lds};
    };
    // rows of x a pass: as many of the 8 the kernels take as still leave a staged kernel (the weight is re-read
    // per pass, which costs less than the unstaged kernel: 4096 x 4096 f32 at 8 rows 59 -> 26 us in two passes)
    const int64_t mrows = p.M < 8 ? p.M : 8;
    int mb = mrows <= 1 ? 1 : mrows <= 2 ? 2 : mrows <= 4 ? 4 : 8;
    Staged st = staged(mb);
    while (!st.ok && mb > 1) {
        mb >>= 1;
        st = staged(mb);
    }
    const bool use_lds = st.ok;
    const int rpwg = st.rpwg;
    const size_t lds = st.lds;
    const int pass = use_lds ? mb : 8;  // rows of x a launch
    const uint32_t chunks = (uint32_t)ceil_div(p.M, pass);
    char name[64];
    snprintf(name, sizeof name, "gguf_%s_gemv_%s%s", fmt_name(p.quant), bf ? "bf16" : "f32", use_lds ? "_lds" : "");
    dim3 grid((unsigned)(use_lds ? ceil_div(p.N, rpwg) : ceil_div(p.N, 4))), block(use_lds && rpwg >= 16 ? 1024 : use_lds && rpwg >= 8 ? 512 : 256);
    set_plan(ctx, name, grid, block, 1, chunks, 0);
    if (ctx->plan_only) return OXQ_OK;
    // more rows than a pass takes: the weight is re-read per pass (beyond 8 rows the tile matmul serves)
    for (int64_t m0 = 0; m0 < p.M; m0 += pass) {
        const int rows = (int)((p.M - m0) < pass ? (p.M - m0) : pass);
        const uint8_t *x = (const uint8_t *)p.x + (size_t)m0 * p.K * xb;
        uint8_t *y = (uint8_t *)p.y + (size_t)m0 * p.N * xb;
#define OXQ_FMT(F)                                                                  \
    if (use_lds) {                                                                  \
        int rc = bf ? launch_rows_lds<F, true>(ctx, s, p, x, y, rows, rpwg, lds)         \
                    : launch_rows_lds<F, false>(ctx, s, p, x, y, rows, rpwg, lds);       \
        if (rc != OXQ_OK) return rc;                                                \
    } else if (bf) launch_rows<F, true>(s, grid, p, x, y, rows);                    \
    else launch_rows<F, false>(s, grid, p, x, y, rows)
        switch (p.quant) {
        case OXQ_GGUF_Q4_0: OXQ_FMT(OXQ_GGUF_Q4_0); break;
        case OXQ_GGUF_Q8_0: OXQ_FMT(OXQ_GGUF_Q8_0); break;
        case OXQ_GGUF_Q4_K: OXQ_FMT(OXQ_GGUF_Q4_K); break;
        case OXQ_GGUF_Q4_1: OXQ_FMT(OXQ_GGUF_Q4_1); break;
        case OXQ_GGUF_Q5_0: OXQ_FMT(OXQ_GGUF_Q5_0); break;
        case OXQ_GGUF_Q5_1: OXQ_FMT(OXQ_GGUF_Q5_1); break;
        case OXQ_GGUF_Q2_K: OXQ_FMT(OXQ_GGUF_Q2_K); break;
        case OXQ_GGUF_Q3_K: OXQ_FMT(OXQ_GGUF_Q3_K); break;
        case OXQ_GGUF_Q5_K: OXQ_FMT(OXQ_GGUF_Q5_K); break;
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
#define OXQ_DQ(F) \
    case F: hipLaunchKernelGGL((gguf_dequant_kernel<F>), grid, block, 0, s, p.w, out_nk, K, N); break
    switch (p.quant) {
        OXQ_DQ(OXQ_GGUF_Q4_0);
        OXQ_DQ(OXQ_GGUF_Q8_0);
        OXQ_DQ(OXQ_GGUF_Q4_K);
        OXQ_DQ(OXQ_GGUF_Q4_1);
        OXQ_DQ(OXQ_GGUF_Q5_0);
        OXQ_DQ(OXQ_GGUF_Q5_1);
        OXQ_DQ(OXQ_GGUF_Q2_K);
        OXQ_DQ(OXQ_GGUF_Q3_K);
        OXQ_DQ(OXQ_GGUF_Q5_K);
    default: hipLaunchKernelGGL((gguf_dequant_kernel<OXQ_GGUF_Q6_K>), grid, block, 0, s, p.w, out_nk, K, N); break;
    }
#undef OXQ_DQ
    OXQ_HIP_CHECK(hipGetLastError());
    return OXQ_OK;
}

}  // namespace oxq
