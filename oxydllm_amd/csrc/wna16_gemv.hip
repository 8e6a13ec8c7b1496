// Fused dequant + GEMV for AWQ / GPTQ packed weights, 1 <= M <= 8 rows.
//
//   y[m, n] = sum_k x[m, k] * (q[k, n] - z[k/g, n]) * s[k/g, n]      (AWQ)
//   y[m, n] = sum_k x[m, k] * (q[k, n] - (z[k/g, n] + 1)) * s[k/g, n] (GPTQ)
//
// Reference semantics: quant_kernels.metal:3349-3499 (awq_gemv[_batch]_det_impl)
// and 3501-3648 (gptq_gemv[_batch]_det_impl): f32 accumulation, deterministic
// fixed-order reduction of the K slices, result cast to the activation dtype.
//
// Two kernel families:
//   *_generic  one packed word per lane per row, f32 math exactly as the
//              reference writes it; accepts every shape the reference accepts.
//   awq_gemv_fast / gptq_gemv_fast  the bandwidth path, 4- and 8-bit: 128/64/32-bit
//              coalesced loads, nibbles or bytes turned into exact 16-bit floats
//              with one AND-OR, rows paired so v_dot2_f32_{f16,bf16} does two MACs
//              per lane, zero-point and scale applied once per group.
//
// Both split K across workgroups and combine the slices with the
// last-arriver protocol of oxq_device.hpp (bitwise run-to-run deterministic).
// HBM-bound: the packed weights are read exactly once.

#include "oxq_device.hpp"
#include "oxq_internal.hpp"

#include <cstdlib>

namespace oxq {

// ---------------------------------------------------------------------------
// Shared epilogue: the last workgroup of a column tile sums the slices.
// ---------------------------------------------------------------------------
template <typename TT>
__device__ __forceinline__ void splitk_finish(const float *__restrict__ ws,
                                              const uint16_t *__restrict__ bias,
                                              uint16_t *__restrict__ y, int M, int N, int S,
                                              int n0, int tile_cols, int nthreads, int tid) {
    constexpr int CPT = 4;  // outputs per thread whose slice loads are in flight together
    const int total = M * tile_cols;
    for (int base = tid; base < total; base += nthreads * CPT) {
        float tot[CPT];
#pragma unroll
        for (int c = 0; c < CPT; ++c) tot[c] = 0.0f;
        for (int s0 = 0; s0 < S; s0 += 8) {
            float v[CPT][8];
#pragma unroll
            for (int c = 0; c < CPT; ++c) {
                const int idx = base + c * nthreads;
                const int m = idx / tile_cols;
                const int n = n0 + idx % tile_cols;
                const bool ok = idx < total && n < N;
#pragma unroll
                for (int u = 0; u < 8; ++u)
                    v[c][u] = (ok && s0 + u < S) ? ld_agent(ws + ((size_t)(s0 + u) * M + m) * N + n) : 0.0f;
            }
#pragma unroll
            for (int c = 0; c < CPT; ++c)
#pragma unroll
                for (int u = 0; u < 8; ++u) tot[c] += v[c][u];  // slice order
        }
#pragma unroll
        for (int c = 0; c < CPT; ++c) {
            const int idx = base + c * nthreads;
            const int m = idx / tile_cols;
            const int n = n0 + idx % tile_cols;
            if (idx < total && n < N) {
                float t = tot[c];
                if (bias) t += TT::to_f32(bias[n]);
                y[(size_t)m * N + n] = TT::from_f32(t);
            }
        }
    }
}

// Stand-alone reduction of the K slices (second launch): every thread owns 4
// consecutive outputs and issues the loads of 8 slices at a time.
template <typename TT>
__global__ __launch_bounds__(256) void splitk_reduce_kernel(const float *__restrict__ ws,
                                                            const uint16_t *__restrict__ bias,
                                                            uint16_t *__restrict__ y, size_t total,
                                                            int N, int S) {
    const size_t i4 = ((size_t)blockIdx.x * 256 + threadIdx.x) * 4;
    if (i4 >= total) return;
    float4_t tot = {0.f, 0.f, 0.f, 0.f};
    for (int s0 = 0; s0 < S; s0 += 8) {
        float4_t v[8];
#pragma unroll
        for (int u = 0; u < 8; ++u)
            v[u] = (s0 + u < S) ? *(const float4_t *)(ws + (size_t)(s0 + u) * total + i4)
                                : float4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int u = 0; u < 8; ++u) tot += v[u];
    }
    uint16_t o[4];
#pragma unroll
    for (int c = 0; c < 4; ++c) {
        float t = tot[c];
        if (bias) t += TT::to_f32(bias[(i4 + c) % N]);
        o[c] = TT::from_f32(t);
    }
    *(uint2 *)(y + i4) = uint2{(uint32_t)o[0] | ((uint32_t)o[1] << 16),
                               (uint32_t)o[2] | ((uint32_t)o[3] << 16)};
}

int launch_splitk_reduce(oxq_ctx *ctx, hipStream_t s, const float *ws, const void *bias, void *y,
                         int64_t M, int64_t N, int S, int dtype) {
    const size_t total = (size_t)M * N;  // N % 4 == 0 for every caller
    dim3 grid((unsigned)ceil_div((int64_t)(total / 4), 256)), block(256);
    add_launch(ctx);
    if (ctx->plan_only) return OXQ_OK;
    if (dtype == OXQ_F16)
        hipLaunchKernelGGL((splitk_reduce_kernel<F16Traits>), grid, block, 0, s, ws,
                           (const uint16_t *)bias, (uint16_t *)y, total, (int)N, S);
    else
        hipLaunchKernelGGL((splitk_reduce_kernel<BF16Traits>), grid, block, 0, s, ws,
                           (const uint16_t *)bias, (uint16_t *)y, total, (int)N, S);
    OXQ_HIP_CHECK(hipGetLastError());
    return OXQ_OK;
}

// ---------------------------------------------------------------------------
// Generic AWQ-layout kernel (4- and 8-bit).  256 threads = 64 word columns x 4
// interleaved row phases.
// ---------------------------------------------------------------------------
template <typename TT, int BITS, int MB>
__global__ __launch_bounds__(256) void awq_gemv_generic(
    const uint16_t *__restrict__ x, const uint32_t *__restrict__ qw,
    const uint32_t *__restrict__ qz, const uint16_t *__restrict__ sc,
    const uint16_t *__restrict__ bias, uint16_t *__restrict__ y, float *__restrict__ ws,
    unsigned *__restrict__ counters, int M, int K, int N, int packed_out, int gshift, int kchunk,
    int S, int fused) {
    constexpr int PF = 32 / BITS;
    constexpr uint32_t MASK = (1u << BITS) - 1u;
    __shared__ float red[4][64][PF];
    const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
    const int j = blockIdx.x * 64 + tx;
    const int slice = blockIdx.y;
    const int k0 = slice * kchunk;
    const int k1 = min(K, k0 + kchunk);

    float acc[MB][PF];
#pragma unroll
    for (int m = 0; m < MB; ++m)
#pragma unroll
        for (int s = 0; s < PF; ++s) acc[m][s] = 0.0f;

    if (j < packed_out) {
        int last_g = -1;
        float zf[PF], sf[PF];
        constexpr int UL = 8;  // packed words in flight per lane
        for (int ib = k0 + ty; ib < k1; ib += 4 * UL) {
          uint32_t wwb[UL];
#pragma unroll
          for (int u = 0; u < UL; ++u) {
              const int i = ib + 4 * u;
              wwb[u] = i < k1 ? qw[(size_t)i * packed_out + j] : 0u;
          }
#pragma unroll
          for (int u = 0; u < UL; ++u) {
            const int i = ib + 4 * u;
            if (i >= k1) break;
            const int g = i >> gshift;
            if (g != last_g) {
                const uint32_t zw = qz[(size_t)g * packed_out + j];
#pragma unroll
                for (int s = 0; s < PF; ++s) {
                    const int col = (BITS == 4) ? awq_slot_col(s) : s;
                    zf[s] = (float)((zw >> (BITS * s)) & MASK);
                    sf[s] = TT::to_f32(sc[(size_t)g * N + (size_t)j * PF + col]);
                }
                last_g = g;
            }
            const uint32_t ww = wwb[u];
            float w[PF];
#pragma unroll
            for (int s = 0; s < PF; ++s) w[s] = ((float)((ww >> (BITS * s)) & MASK) - zf[s]) * sf[s];
#pragma unroll
            for (int m = 0; m < MB; ++m) {
                if (m < M) {
                    const float xv = TT::to_f32(x[(size_t)m * K + i]);
#pragma unroll
                    for (int s = 0; s < PF; ++s) acc[m][s] = fmaf(xv, w[s], acc[m][s]);
                }
            }
          }
        }
    }

    const int tile_cols = 64 * PF;
    const int n0 = blockIdx.x * tile_cols;
#pragma unroll
    for (int m = 0; m < MB; ++m) {
        if (m < M) {
#pragma unroll
            for (int s = 0; s < PF; ++s) red[ty][tx][s] = acc[m][s];
            __syncthreads();
            if (ty == 0 && j < packed_out) {
#pragma unroll
                for (int s = 0; s < PF; ++s) {
                    const int col = (BITS == 4) ? awq_slot_col(s) : s;
                    const float tot = red[0][tx][s] + red[1][tx][s] + red[2][tx][s] + red[3][tx][s];
                    const int n = j * PF + col;
                    if (S == 1) {
                        const float b = bias ? TT::to_f32(bias[n]) : 0.0f;
                        y[(size_t)m * N + n] = TT::from_f32(tot + b);
                    } else if (fused) {
                        st_agent(ws + ((size_t)slice * M + m) * N + n, tot);
                    } else {
                        ws[((size_t)slice * M + m) * N + n] = tot;
                    }
                }
            }
            __syncthreads();
        }
    }
    if (S > 1 && fused && splitk_arrive(counters, blockIdx.x, S))
        splitk_finish<TT>(ws, bias, y, M, N, S, n0, tile_cols, 256, threadIdx.x);
}

// ---------------------------------------------------------------------------
// Generic GPTQ-layout kernel (4- and 8-bit).  One output column per lane; a
// word holds PF consecutive k for that column.  256 threads = 64 columns x 4
// interleaved word-row phases.
// ---------------------------------------------------------------------------
template <typename TT, int BITS, int MB>
__global__ __launch_bounds__(256) void gptq_gemv_generic(
    const uint16_t *__restrict__ x, const uint32_t *__restrict__ qw,
    const uint32_t *__restrict__ qz, const uint16_t *__restrict__ sc,
    const uint16_t *__restrict__ bias, uint16_t *__restrict__ y, float *__restrict__ ws,
    unsigned *__restrict__ counters, int M, int K, int N, int gshift, int wchunk, int S, int fused) {
    constexpr int PF = 32 / BITS;
    constexpr uint32_t MASK = (1u << BITS) - 1u;
    __shared__ float red[4][64];
    const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
    const int n = blockIdx.x * 64 + tx;
    const int slice = blockIdx.y;
    const int packed_in = K / PF;
    const int w0 = slice * wchunk;
    const int w1 = min(packed_in, w0 + wchunk);
    const int packed_out = N / PF;

    float acc[MB];
#pragma unroll
    for (int m = 0; m < MB; ++m) acc[m] = 0.0f;

    if (n < N) {
        int last_g = -1;
        float zp1 = 0.0f, sv = 0.0f;
        const uint32_t zshift = BITS * (n % PF);
        constexpr int UL = 8;  // packed words in flight per lane
        for (int ib = w0 + ty; ib < w1; ib += 4 * UL) {
          uint32_t wwb[UL];
#pragma unroll
          for (int u = 0; u < UL; ++u) {
              const int iw = ib + 4 * u;
              wwb[u] = iw < w1 ? qw[(size_t)iw * N + n] : 0u;
          }
#pragma unroll
          for (int u = 0; u < UL; ++u) {
            const int iw = ib + 4 * u;
            if (iw >= w1) break;
            const int g = (iw * PF) >> gshift;
            if (g != last_g) {
                const uint32_t zw = qz[(size_t)g * packed_out + n / PF];
                zp1 = (float)((zw >> zshift) & MASK) + 1.0f;
                sv = TT::to_f32(sc[(size_t)g * N + n]);
                last_g = g;
            }
            const uint32_t ww = wwb[u];
            float w[PF];
#pragma unroll
            for (int s = 0; s < PF; ++s) w[s] = sv * ((float)((ww >> (BITS * s)) & MASK) - zp1);
#pragma unroll
            for (int m = 0; m < MB; ++m) {
                if (m < M) {
                    const uint16_t *xr = x + (size_t)m * K + (size_t)iw * PF;
#pragma unroll
                    for (int s = 0; s < PF; ++s) acc[m] = fmaf(TT::to_f32(xr[s]), w[s], acc[m]);
                }
            }
          }
        }
    }
    const int n0 = blockIdx.x * 64;
#pragma unroll
    for (int m = 0; m < MB; ++m) {
        if (m < M) {
            red[ty][tx] = acc[m];
            __syncthreads();
            if (ty == 0 && n < N) {
                const float tot = red[0][tx] + red[1][tx] + red[2][tx] + red[3][tx];
                if (S == 1) {
                    const float b = bias ? TT::to_f32(bias[n]) : 0.0f;
                    y[(size_t)m * N + n] = TT::from_f32(tot + b);
                } else if (fused) {
                    st_agent(ws + ((size_t)slice * M + m) * N + n, tot);
                } else {
                    ws[((size_t)slice * M + m) * N + n] = tot;
                }
            }
            __syncthreads();
        }
    }
    if (S > 1 && fused && splitk_arrive(counters, blockIdx.x, S))
        splitk_finish<TT>(ws, bias, y, M, N, S, n0, 64, 256, threadIdx.x);
}

// ---------------------------------------------------------------------------
// Fast 4-bit AWQ kernel.
//
// Geometry: a workgroup of WAVES waves owns a slab of LPR*WPL packed words
// (LPR*WPL*8 output columns) and `gpw` consecutive quantization groups of K.
// A lane owns WPL consecutive words of a row (one 32*WPL-bit load) and walks
// row pairs (k, k+1): the low/high 16-bit halves of the two rows' words are
// interleaved with one v_perm, after which a single AND-OR per slot yields the
// pair {bias+q[k], bias+q[k+1]} as 16-bit floats, consumed by one dot2 against
// {x[k], x[k+1]}.  Per group and column the lane then applies
//     y += s * (acc - (bias + z) * sum_k x[k])
// which removes both the conversion bias and the zero-point in f32.
//
// 8-bit layers run the same kernel with 4 columns per word in identity order: after the
// same row-pair interleave, bytes 0/2 of a register are one column's pair and bytes 1/3 the next
// column's (f16: 1024 + q by AND-OR; bf16: through f32).
// ---------------------------------------------------------------------------
template <int WPL> struct WordVec;
template <> struct WordVec<4> {
    typedef uint32_t type __attribute__((ext_vector_type(4)));
    __device__ static __forceinline__ type load(__amdgpu_buffer_rsrc_t r, int voff, int soff) {
        return __builtin_amdgcn_raw_buffer_load_b128(r, voff, soff, 2);  // weights are read once: nontemporal
    }
};
template <> struct WordVec<2> {
    typedef uint32_t type __attribute__((ext_vector_type(2)));
    __device__ static __forceinline__ type load(__amdgpu_buffer_rsrc_t r, int voff, int soff) {
        return __builtin_amdgcn_raw_buffer_load_b64(r, voff, soff, 2);
    }
};
template <> struct WordVec<1> {
    typedef uint32_t type __attribute__((ext_vector_type(1)));
    __device__ static __forceinline__ type load(__amdgpu_buffer_rsrc_t r, int voff, int soff) {
        type v;
        v[0] = __builtin_amdgcn_raw_buffer_load_b32(r, voff, soff, 2);
        return v;
    }
};

template <typename TT, int BITS, int MB, int WPL, int WPG, int GPB, int RPW, int PS>
__global__ __launch_bounds__(WPG * GPB * 64) void awq_gemv_fast(
    const uint16_t *__restrict__ x, const uint32_t *__restrict__ qw,
    const uint32_t *__restrict__ qz, const uint16_t *__restrict__ sc,
    const uint16_t *__restrict__ bias, uint16_t *__restrict__ y, float *__restrict__ ws,
    unsigned *__restrict__ counters, int M, int K, int N, int gshift, int gpw, int S, int fused) {
    // WPG waves share one quantization group (they take interleaved row pairs),
    // GPB groups are processed side by side by one workgroup.
    typedef WordVec<WPL> WV;
    typedef typename WV::type wvec_t;
    constexpr int WAVES = WPG * GPB;
    constexpr int LPR = 64 / RPW;          // lanes per row
    constexpr int CPW = 32 / BITS;         // columns per word
    constexpr int NC = WPL * CPW;          // columns per lane
    constexpr int SLAB_COLS = LPR * NC;
    constexpr int ROWS_PER_CHUNK = 2 * WPG * RPW * PS;
    __shared__ float red[WAVES][SLAB_COLS];

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int wg = wave / WPG, wr = wave % WPG;  // group slot, row phase (wave-uniform)
    const int cl = lane % LPR, sub = lane / LPR;
    const int PW = N / CPW;                // words per row
    const int rowbytes = PW * 4;
    const int jw = (blockIdx.x * LPR + cl) * WPL;
    const bool valid = jw < PW;
    const int G = K >> gshift;
    const int slice = blockIdx.y;
    const int g0 = slice * gpw;
    const int g1 = min(G, g0 + gpw);
    const int chunks = (1 << gshift) / ROWS_PER_CHUNK;

    const __amdgpu_buffer_rsrc_t rs_w = make_rsrc(qw, (uint32_t)K * (uint32_t)rowbytes);
    const __amdgpu_buffer_rsrc_t rs_x = make_rsrc(x, (uint32_t)M * (uint32_t)K * 2u);
    const int voff_w = (2 * sub * PW + jw) * 4;  // this lane's row pair and word column
    const int voff_x = 2 * sub * 2;
    const NibbleMasks nm = nibble_masks();

    float yacc[MB][NC];
#pragma unroll
    for (int m = 0; m < MB; ++m)
#pragma unroll
        for (int c = 0; c < NC; ++c) yacc[m][c] = 0.0f;

    if (valid) {
        for (int g = g0 + wg; g < g1; g += GPB) {
            const wvec_t zw = *(const wvec_t *)(qz + (size_t)g * PW + jw);
            const uint16_t *srow = sc + (size_t)g * N + (size_t)jw * CPW;
            uint32_t sv[WPL][CPW / 2];  // the word's CPW scales, two per register
#pragma unroll
            for (int c = 0; c < WPL; ++c) {
                if constexpr (BITS == 4) {
                    const u32x4_t v = *(const u32x4_t *)(srow + c * 8);
#pragma unroll
                    for (int q = 0; q < 4; ++q) sv[c][q] = v[q];
                } else {
                    const uint2 v = *(const uint2 *)(srow + c * 4);
                    sv[c][0] = v.x;
                    sv[c][1] = v.y;
                }
            }
            float acc[MB][NC];
            float xs[MB];
#pragma unroll
            for (int m = 0; m < MB; ++m) {
                xs[m] = 0.0f;
#pragma unroll
                for (int c = 0; c < NC; ++c) acc[m][c] = 0.0f;
            }
            for (int ch = 0; ch < chunks; ++ch) {
                const int kb = (g << gshift) + ch * ROWS_PER_CHUNK;
                wvec_t wa[PS], wb[PS];
                uint32_t xp[MB][PS];
#pragma unroll
                for (int t = 0; t < PS; ++t) {
                    const int ru = kb + 2 * (wr * RPW + t * (WPG * RPW));  // wave-uniform row
                    wa[t] = WV::load(rs_w, voff_w, ru * rowbytes);
                    wb[t] = WV::load(rs_w, voff_w, (ru + 1) * rowbytes);
#pragma unroll
                    for (int m = 0; m < MB; ++m) {
                        const int mm = m < M ? m : M - 1;
                        xp[m][t] = __builtin_amdgcn_raw_buffer_load_b32(rs_x, voff_x, (mm * K + ru) * 2, 0);
                    }
                }
#pragma unroll
                for (int t = 0; t < PS; ++t) {
#pragma unroll
                    for (int c = 0; c < WPL; ++c) {
                        uint32_t p[CPW];
                        const uint32_t lo = pack_lo16(wa[t][c], wb[t][c]), hi = pack_hi16(wa[t][c], wb[t][c]);
                        if constexpr (BITS == 4) {
                            TT::unpack4(lo, p, nm);
                            TT::unpack4(hi, p + 4, nm);
                        } else {
                            p[0] = TT::unpack_bytes(lo);
                            p[1] = TT::unpack_bytes(lo >> 8);
                            p[2] = TT::unpack_bytes(hi);
                            p[3] = TT::unpack_bytes(hi >> 8);
                        }
#pragma unroll
                        for (int m = 0; m < MB; ++m)
#pragma unroll
                            for (int s = 0; s < CPW; ++s)
                                acc[m][c * CPW + s] = TT::dot2(p[s], xp[m][t], acc[m][c * CPW + s]);
                    }
#pragma unroll
                    for (int m = 0; m < MB; ++m) xs[m] = TT::dot2(TT::ONES, xp[m][t], xs[m]);
                }
            }
            // group epilogue: remove bias and zero-point, apply the scale
#pragma unroll
            for (int c = 0; c < WPL; ++c) {
                const uint32_t zword = zw[c];
#pragma unroll
                for (int s = 0; s < CPW; ++s) {
                    const int col = BITS == 4 ? awq_slot_col(s) : s;
                    const uint32_t spair = sv[c][col >> 1];
                    const uint16_t sbits = (col & 1) ? (uint16_t)(spair >> 16) : (uint16_t)(spair & 0xFFFFu);
                    const float scale = TT::to_f32(sbits);
                    const float zb = (float)((zword >> (BITS * s)) & ((1u << BITS) - 1u)) +
                                     (BITS == 4 ? TT::bias(s) : TT::BYTE_BIAS);
#pragma unroll
                    for (int m = 0; m < MB; ++m) {
                        const float v = fmaf(-zb, xs[m], acc[m][c * CPW + s]);
                        yacc[m][c * CPW + s] = fmaf(scale, v, yacc[m][c * CPW + s]);
                    }
                }
            }
        }
    }

    // combine the RPW row phases inside the wave, then the waves through LDS
    const int n0 = blockIdx.x * SLAB_COLS;
#pragma unroll
    for (int m = 0; m < MB; ++m) {
        if (m < M) {
#pragma unroll
            for (int c = 0; c < NC; ++c) {
                float v = yacc[m][c];
                if constexpr (LPR == 16) {  // lanes l, l ^ 16, l ^ 32, l ^ 48 on the gfx950 lane-swap instructions
                    v = add_lane_xor16(v);
                    v = add_lane_xor32(v);
                } else {
#pragma unroll
                    for (int off = LPR; off < 64; off <<= 1) v += __shfl_xor(v, off, WAVE);
                }
                yacc[m][c] = v;
            }
            if (sub == 0) {
#pragma unroll
                for (int c = 0; c < WPL; ++c)
#pragma unroll
                    for (int s = 0; s < CPW; ++s)
                        red[wave][cl * NC + c * CPW + (BITS == 4 ? awq_slot_col(s) : s)] = yacc[m][c * CPW + s];
            }
            __syncthreads();
            for (int col = threadIdx.x; col < SLAB_COLS; col += WAVES * 64) {
                const int n = n0 + col;
                if (n < N) {
                    float tot = 0.0f;
#pragma unroll
                    for (int w = 0; w < WAVES; ++w) tot += red[w][col];
                    if (S == 1) {
                        const float b = bias ? TT::to_f32(bias[n]) : 0.0f;
                        y[(size_t)m * N + n] = TT::from_f32(tot + b);
                    } else if (fused) {
                        st_agent(ws + ((size_t)slice * M + m) * N + n, tot);
                    } else {
                        ws[((size_t)slice * M + m) * N + n] = tot;
                    }
                }
            }
            __syncthreads();
        }
    }
    if (S > 1 && fused && splitk_arrive(counters, blockIdx.x, S))
        splitk_finish<TT>(ws, bias, y, M, N, S, n0, SLAB_COLS, WAVES * 64, threadIdx.x);
}

// ---------------------------------------------------------------------------
// Fast 4-bit GPTQ kernel.
//
// A GPTQ word holds 8 consecutive k of ONE column, so a lane that loads 4 words
// (one 128-bit load = 4 adjacent columns of a word row) owns 4 output columns
// outright: no cross-lane reduction.  Masks 0x000F000F / 0x00F000F0 on the word
// and on word >> 8 give the k pairs (0,4) (1,5) (2,6) (3,7) as exact 16-bit
// floats (bias 1024 / 64 for f16, 128 for bf16); the matching activation pairs
// {x[k], x[k+4]} are wave-uniform, built once per workgroup in LDS and read
// with one 128-bit LDS load per word row.  Per group:
//     y += s * (acc - bias_even*Xe - bias_odd*Xo - (z+1)*(Xe+Xo)),
// Xe / Xo = sums of x over even / odd nibble positions of the lane's word rows.
// One wave owns a whole quantization group (16 word rows at g=128), 8 waves =
// 8 groups per workgroup, 256 columns per workgroup; K slices go to the workspace.
// ---------------------------------------------------------------------------
//
// 8-bit layers run the same kernel: a word holds 4 consecutive k, bytes 0/2 and 1/3 become the k
// pairs (0,2) (1,3) as exact floats (f16: 1024 + q by AND-OR; bf16: through f32), a chunk of 16
// word rows is 64 k, and the lane's four zeros are one qzeros word.
template <typename TT, int BITS, int MB>
__global__ __launch_bounds__(512) void gptq_gemv_fast(
    const uint16_t *__restrict__ x, const uint32_t *__restrict__ qw,
    const uint32_t *__restrict__ qz, const uint16_t *__restrict__ sc,
    const uint16_t *__restrict__ bias, uint16_t *__restrict__ y, float *__restrict__ ws,
    unsigned *__restrict__ counters, int M, int K, int N, int gshift, int gpw, int S, int fused) {
    constexpr int WAVES = 8;
    constexpr int PF = 32 / BITS;          // k per word
    constexpr int XW = PF / 2;             // x pairs (words) per word row
    constexpr int WR = 16;                 // word rows per chunk (128 k at 4 bits, 64 k at 8)
    constexpr int CK = WR * PF;            // k per chunk
    constexpr int RK = 1024;               // k staged per round
    __shared__ __attribute__((aligned(16))) uint32_t xl[MB][RK / PF][XW];  // permuted x pairs
    __shared__ float red[WAVES][256];

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int n4 = blockIdx.x * 64 + lane;             // 4-column unit of this lane
    const int n0 = n4 * 4;
    const bool valid = n0 < N;
    const int slice = blockIdx.y;
    const int G = K >> gshift;
    const int g0 = slice * gpw, g1 = min(G, g0 + gpw);
    const int rowbytes = N * 4;
    const __amdgpu_buffer_rsrc_t rs_w = make_rsrc(qw, (uint32_t)(K / PF) * (uint32_t)rowbytes);
    const int voff_w = n0 * 4;
    const NibbleMasks nm = nibble_masks();

    float yacc[MB][4];
#pragma unroll
    for (int m = 0; m < MB; ++m)
#pragma unroll
        for (int c = 0; c < 4; ++c) yacc[m][c] = 0.0f;

    // rounds of up to RK k: stage permuted x, then each wave walks its share
    const int k_lo = g0 << gshift, k_hi = g1 << gshift;
    for (int kr = k_lo; kr < k_hi; kr += RK) {
        const int kr_end = min(k_hi, kr + RK);
        const int nwr = (kr_end - kr) / PF;            // word rows in this round
        __syncthreads();
        for (int idx = threadIdx.x; idx < MB * nwr; idx += WAVES * 64) {
            const int m = idx / nwr, r = idx % nwr;
            const int mm = m < M ? m : M - 1;
            if constexpr (BITS == 4) {
                const u32x4_t d = *(const u32x4_t *)(x + (size_t)mm * K + kr + r * 8);
                u32x4_t o;
                o[0] = pack_lo16(d[0], d[2]);  // (x0, x4)
                o[1] = pack_hi16(d[0], d[2]);  // (x1, x5)
                o[2] = pack_lo16(d[1], d[3]);  // (x2, x6)
                o[3] = pack_hi16(d[1], d[3]);  // (x3, x7)
                *(u32x4_t *)(&xl[m][r][0]) = o;
            } else {
                const uint2 d = *(const uint2 *)(x + (size_t)mm * K + kr + r * 4);
                *(uint2 *)(&xl[m][r][0]) = uint2{pack_lo16(d.x, d.y), pack_hi16(d.x, d.y)};  // (x0, x2) (x1, x3)
            }
        }
        __syncthreads();
        // chunks of 16 word rows are dealt round-robin to the waves
        const int nchunks = nwr / WR;
        for (int ch = wave; ch < nchunks; ch += WAVES) {
            const int kc = kr + ch * CK;
            const int g = kc >> gshift;
            u32x4_t w[WR];
#pragma unroll
            for (int t = 0; t < WR; ++t)
                w[t] = __builtin_amdgcn_raw_buffer_load_b128(rs_w, voff_w, (kc / PF + t) * rowbytes, 2);  // nontemporal
            const uint32_t zw = valid ? qz[(size_t)g * (N / PF) + n0 / PF] : 0u;
            uint2 sv = valid ? *(const uint2 *)(sc + (size_t)g * N + n0) : uint2{0u, 0u};
            float acc[MB][4], xe[MB], xo[MB];
#pragma unroll
            for (int m = 0; m < MB; ++m) {
                xe[m] = 0.0f;
                xo[m] = 0.0f;
#pragma unroll
                for (int c = 0; c < 4; ++c) acc[m][c] = 0.0f;
            }
#pragma unroll
            for (int t = 0; t < WR; ++t) {
                uint32_t xp[MB][XW];
#pragma unroll
                for (int m = 0; m < MB; ++m) {
                    if constexpr (BITS == 4) {
                        const u32x4_t v = *(const u32x4_t *)(&xl[m][ch * WR + t][0]);
#pragma unroll
                        for (int q = 0; q < XW; ++q) xp[m][q] = v[q];
                    } else {
                        const uint2 v = *(const uint2 *)(&xl[m][ch * WR + t][0]);
                        xp[m][0] = v.x;
                        xp[m][1] = v.y;
                    }
                }
#pragma unroll
                for (int c = 0; c < 4; ++c) {
                    uint32_t p[XW];
                    if constexpr (BITS == 4) {
                        TT::unpack4(w[t][c], p, nm);  // pairs (0,4) (1,5) (2,6) (3,7)
                    } else {
                        p[0] = TT::unpack_bytes(w[t][c]);       // (0,2)
                        p[1] = TT::unpack_bytes(w[t][c] >> 8);  // (1,3)
                    }
#pragma unroll
                    for (int m = 0; m < MB; ++m)
#pragma unroll
                        for (int q = 0; q < XW; ++q) acc[m][c] = TT::dot2(p[q], xp[m][q], acc[m][c]);
                }
#pragma unroll
                for (int m = 0; m < MB; ++m) {
                    if constexpr (BITS == 4) {
                        xe[m] = TT::dot2(TT::ONES, xp[m][0], xe[m]);
                        xe[m] = TT::dot2(TT::ONES, xp[m][XW - 2], xe[m]);
                        xo[m] = TT::dot2(TT::ONES, xp[m][1], xo[m]);
                        xo[m] = TT::dot2(TT::ONES, xp[m][XW - 1], xo[m]);
                    } else {  // one conversion bias for every byte: a single sum
                        xe[m] = TT::dot2(TT::ONES, xp[m][0], xe[m]);
                        xe[m] = TT::dot2(TT::ONES, xp[m][1], xe[m]);
                    }
                }
            }
            // a chunk lies inside one group (group size >= 128): apply scale / zero
            const int zsh = (n0 % PF) * BITS;
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                const uint32_t spair = c < 2 ? sv.x : sv.y;
                const float scale = TT::to_f32((c & 1) ? (uint16_t)(spair >> 16) : (uint16_t)(spair & 0xFFFFu));
                const float zp1 = (float)((zw >> (zsh + BITS * c)) & ((1u << BITS) - 1u)) + 1.0f;
#pragma unroll
                for (int m = 0; m < MB; ++m) {
                    float v;
                    if constexpr (BITS == 4) {
                        v = acc[m][c] - TT::bias(0) * xe[m] - TT::bias(1) * xo[m];
                        v = fmaf(-zp1, xe[m] + xo[m], v);
                    } else {
                        v = fmaf(-(zp1 + TT::BYTE_BIAS), xe[m], acc[m][c]);
                    }
                    yacc[m][c] = fmaf(scale, v, yacc[m][c]);
                }
            }
        }
    }

    const int nbase = blockIdx.x * 256;
#pragma unroll
    for (int m = 0; m < MB; ++m) {
        if (m < M) {
            __syncthreads();
            *(float4_t *)(&red[wave][lane * 4]) = float4_t{yacc[m][0], yacc[m][1], yacc[m][2], yacc[m][3]};
            __syncthreads();
            for (int col = threadIdx.x; col < 256; col += WAVES * 64) {
                const int n = nbase + col;
                if (n < N) {
                    float tot = 0.0f;
#pragma unroll
                    for (int w8 = 0; w8 < WAVES; ++w8) tot += red[w8][col];
                    if (S == 1) {
                        const float b = bias ? TT::to_f32(bias[n]) : 0.0f;
                        y[(size_t)m * N + n] = TT::from_f32(tot + b);
                    } else if (fused) {
                        st_agent(ws + ((size_t)slice * M + m) * N + n, tot);
                    } else {
                        ws[((size_t)slice * M + m) * N + n] = tot;
                    }
                }
            }
        }
    }
    if (S > 1 && fused && splitk_arrive(counters, blockIdx.x, S))
        splitk_finish<TT>(ws, bias, y, M, N, S, nbase, 256, WAVES * 64, threadIdx.x);
}

// ---------------------------------------------------------------------------
// Host dispatch
// ---------------------------------------------------------------------------
// 1: the last workgroup of a tile sums the slices; 0: a second launch does.
// The fused form saves a launch but its sum runs on one workgroup per tile, so
// it only pays for few slices.
static int splitk_fused(const oxq_ctx *ctx, int S) {
    if (S <= 1) return 0;
    if (ctx->splitk_mode == 1) return 1;
    if (ctx->splitk_mode == 2) return 0;
    return S <= 4 ? 1 : 0;
}

static int pick_mb(int64_t M) { return M <= 1 ? 1 : (M <= 2 ? 2 : (M <= 4 ? 4 : 8)); }

template <typename TT, int BITS, int MB, int WPL, int WPG, int GPB, int RPW, int PS>
static int launch_awq_fast_t(oxq_ctx *ctx, hipStream_t s, const Wna16Problem &p, int gpw) {
    constexpr int LPR = 64 / RPW;
    const int PW = (int)(p.N * BITS / 32);
    const int G = (int)(p.K >> p.group_shift);
    const int S = (int)ceil_div(G, gpw);
    dim3 grid((unsigned)ceil_div(PW, LPR * WPL), (unsigned)S);
    dim3 block(WPG * GPB * 64);
    const uint64_t ws_bytes = S > 1 ? (uint64_t)S * p.M * p.N * 4 : 0;
    char name[64];
    snprintf(name, sizeof name, "awq%d_gemv_fast_%s_m%d_w%d_g%dx%d_r%d_p%d", BITS,
             TT::DTYPE == 1 ? "f16" : "bf16", MB, WPL, WPG, GPB, RPW, PS);
    set_plan(ctx, name, grid, block, S, 1, ws_bytes);
    if (ctx->plan_only) {
        if (S > 1 && !splitk_fused(ctx, S)) add_launch(ctx);
        return OXQ_OK;
    }
    if (ws_bytes > ctx->workspace_bytes || grid.x > ctx->n_counters)
        return fail(OXQ_ERR_WORKSPACE, "w4a16 gemv: needs %llu workspace bytes, ctx holds %zu",
                    (unsigned long long)ws_bytes, ctx->workspace_bytes);
    const int fused = splitk_fused(ctx, S);
    hipLaunchKernelGGL((awq_gemv_fast<TT, BITS, MB, WPL, WPG, GPB, RPW, PS>), grid, block, 0, s,
                       (const uint16_t *)p.x, p.qweight, p.qzeros, (const uint16_t *)p.scales,
                       (const uint16_t *)p.bias, (uint16_t *)p.y, (float *)ctx->workspace,
                       ctx->counters, (int)p.M, (int)p.K, (int)p.N, p.group_shift, gpw, S, fused);
    OXQ_HIP_CHECK(hipGetLastError());
    if (S > 1 && !fused)
        return launch_splitk_reduce(ctx, s, (const float *)ctx->workspace, p.bias, p.y, p.M, p.N, S,
                                    p.dtype);
    return OXQ_OK;
}

// Geometry table.  rows per chunk = 2 * WPG * RPW * PS must divide the group size.
template <typename TT, int BITS>
static int launch_awq_fast(oxq_ctx *ctx, hipStream_t s, const Wna16Problem &p) {
    constexpr int CPW = 32 / BITS;
    const int mb = pick_mb(p.M);
    const int G = (int)(p.K >> p.group_shift);
    const int gs = (int)p.group_size;
    int cfg = tune(ctx, OXQ_TUNE_GEMV_CFG, -1);
    int gpw_env = tune(ctx, OXQ_TUNE_GEMV_GPW, 0);
    auto gpw_for = [&](int slab_cols, int gpb) {
        if (gpw_env > 0) return gpw_env;
        const int slabs = (int)ceil_div(p.N, slab_cols);
        int S = (int)ceil_div(ctx->num_cus, slabs);  // about one workgroup per CU
        if (S > G) S = G;
        if (S < 1) S = 1;
        int gpw = (int)ceil_div(G, S);
        gpw = (int)ceil_div(gpw, gpb) * gpb;       // whole rounds of GPB groups
        return gpw;
    };
    if (mb == 1) {
        if (cfg < 0) cfg = gs >= 128 ? 4 : 0;  // measured best on MI355X at K=4096, N=14336
        if (gs >= 128) {
            switch (cfg) {
            case 1: return launch_awq_fast_t<TT, BITS, 1, 4, 4, 2, 2, 8>(ctx, s, p, gpw_for(1024 * CPW / 8, 2));
            case 2: return launch_awq_fast_t<TT, BITS, 1, 4, 4, 4, 4, 4>(ctx, s, p, gpw_for(512 * CPW / 8, 4));
            case 4: return launch_awq_fast_t<TT, BITS, 1, 4, 2, 4, 4, 8>(ctx, s, p, gpw_for(512 * CPW / 8, 4));
            case 5: return launch_awq_fast_t<TT, BITS, 1, 4, 1, 8, 8, 8>(ctx, s, p, gpw_for(256 * CPW / 8, 8));
            case 6: return launch_awq_fast_t<TT, BITS, 1, 4, 1, 4, 8, 8>(ctx, s, p, gpw_for(256 * CPW / 8, 4));
            default: return launch_awq_fast_t<TT, BITS, 1, 4, 4, 1, 2, 8>(ctx, s, p, gpw_for(1024 * CPW / 8, 1));
            }
        }
        return launch_awq_fast_t<TT, BITS, 1, 4, 4, 1, 2, 4>(ctx, s, p, gpw_for(1024 * CPW / 8, 1));
    }
    const bool ps8 = gs >= 128;
    if (mb == 2)
        return ps8 ? launch_awq_fast_t<TT, BITS, 2, 4, 4, 1, 2, 8>(ctx, s, p, gpw_for(1024 * CPW / 8, 1))
                   : launch_awq_fast_t<TT, BITS, 2, 4, 4, 1, 2, 4>(ctx, s, p, gpw_for(1024 * CPW / 8, 1));
    if (mb == 4)
        return ps8 ? launch_awq_fast_t<TT, BITS, 4, 2, 4, 1, 2, 8>(ctx, s, p, gpw_for(512 * CPW / 8, 1))
                   : launch_awq_fast_t<TT, BITS, 4, 2, 4, 1, 2, 4>(ctx, s, p, gpw_for(512 * CPW / 8, 1));
    return ps8 ? launch_awq_fast_t<TT, BITS, 8, 1, 4, 1, 2, 8>(ctx, s, p, gpw_for(256 * CPW / 8, 1))
               : launch_awq_fast_t<TT, BITS, 8, 1, 4, 1, 2, 4>(ctx, s, p, gpw_for(256 * CPW / 8, 1));
}

static bool awq_fast_ok(const Wna16Problem &p) {
    if ((p.bits != 4 && p.bits != 8) || p.pack_dim != OXQ_PACK_OUT) return false;
    if (p.N % 32 != 0 || p.K % 2 != 0) return false;
    if (p.group_size < 64) return false;  // 2 * WPG * RPW * PS rows per chunk
    if ((uint64_t)p.K * (uint64_t)(p.N * p.bits / 8) >= (1ull << 31)) return false;  // 32-bit buffer offsets
    if ((uint64_t)p.M * (uint64_t)p.K * 2 >= (1ull << 31)) return false;
    if (((uintptr_t)p.qweight | (uintptr_t)p.qzeros | (uintptr_t)p.scales) & 15) return false;
    if ((uintptr_t)p.x & 3) return false;
    return true;
}

template <typename TT, int BITS>
static int launch_generic_t(oxq_ctx *ctx, hipStream_t s, const Wna16Problem &p) {
    constexpr int PF = 32 / BITS;
    const int mb = pick_mb(p.M);
    const bool awq = p.pack_dim == OXQ_PACK_OUT;
    const int tiles = awq ? (int)ceil_div(p.N / PF, 64) : (int)ceil_div(p.N, 64);
    const int64_t units = awq ? p.K : p.K / PF;  // rows (AWQ) or word rows (GPTQ) to split
    int S = (int)ceil_div(2 * ctx->num_cus, tiles);
    // keep whole groups per slice so each slice reloads scales rarely
    const int64_t unit_group = awq ? p.group_size : (p.group_size / PF > 0 ? p.group_size / PF : 1);
    int64_t chunk = ceil_div(units, S);
    chunk = ceil_div(chunk, unit_group) * unit_group;
    if (chunk < 4) chunk = 4;
    S = (int)ceil_div(units, chunk);
    dim3 grid((unsigned)tiles, (unsigned)S), block(256);
    const uint64_t ws_bytes = S > 1 ? (uint64_t)S * p.M * p.N * 4 : 0;
    char name[64];
    snprintf(name, sizeof name, "%s_gemv_generic_w%d_%s_m%d", awq ? "awq" : "gptq", BITS,
             TT::DTYPE == 1 ? "f16" : "bf16", mb);
    set_plan(ctx, name, grid, block, S, 1, ws_bytes);
    // the stand-alone reduce handles 4 outputs per thread
    const int fused = (p.N % 4 != 0 && S > 1) ? 1 : splitk_fused(ctx, S);
    if (ctx->plan_only) {
        if (S > 1 && !fused) add_launch(ctx);
        return OXQ_OK;
    }
    if (ws_bytes > ctx->workspace_bytes || grid.x > ctx->n_counters)
        return fail(OXQ_ERR_WORKSPACE, "wna16 gemv: needs %llu workspace bytes, ctx holds %zu",
                    (unsigned long long)ws_bytes, ctx->workspace_bytes);
#define OXQ_GO(MBv)                                                                              \
    if (awq)                                                                                     \
        hipLaunchKernelGGL((awq_gemv_generic<TT, BITS, MBv>), grid, block, 0, s,                 \
                           (const uint16_t *)p.x, p.qweight, p.qzeros, (const uint16_t *)p.scales, \
                           (const uint16_t *)p.bias, (uint16_t *)p.y, (float *)ctx->workspace,   \
                           ctx->counters, (int)p.M, (int)p.K, (int)p.N, (int)(p.N / PF),         \
                           p.group_shift, (int)chunk, S, fused);                                 \
    else                                                                                         \
        hipLaunchKernelGGL((gptq_gemv_generic<TT, BITS, MBv>), grid, block, 0, s,                \
                           (const uint16_t *)p.x, p.qweight, p.qzeros, (const uint16_t *)p.scales, \
                           (const uint16_t *)p.bias, (uint16_t *)p.y, (float *)ctx->workspace,   \
                           ctx->counters, (int)p.M, (int)p.K, (int)p.N, p.group_shift, (int)chunk, S, fused)
    switch (mb) {
    case 1: OXQ_GO(1); break;
    case 2: OXQ_GO(2); break;
    case 4: OXQ_GO(4); break;
    default: OXQ_GO(8); break;
    }
#undef OXQ_GO
    OXQ_HIP_CHECK(hipGetLastError());
    if (S > 1 && !fused)
        return launch_splitk_reduce(ctx, s, (const float *)ctx->workspace, p.bias, p.y, p.M, p.N, S,
                                    p.dtype);
    return OXQ_OK;
}

static bool gptq_fast_ok(const Wna16Problem &p) {
    if ((p.bits != 4 && p.bits != 8) || p.pack_dim != OXQ_PACK_IN) return false;
    if (p.N % 8 != 0 || p.K % 128 != 0 || p.group_size < 128) return false;
    if (((uintptr_t)p.qweight | (uintptr_t)p.x) & 15) return false;
    if (((uintptr_t)p.scales) & 7) return false;
    if ((uint64_t)(p.K * p.bits / 32) * (uint64_t)p.N * 4 >= (1ull << 31)) return false;
    return true;
}

template <typename TT, int BITS>
static int launch_gptq_fast(oxq_ctx *ctx, hipStream_t s, const Wna16Problem &p) {
    const int mb = pick_mb(p.M);
    const int G = (int)(p.K >> p.group_shift);
    const int slabs = (int)ceil_div(p.N, 256);
    int S = (int)ceil_div(ctx->num_cus, slabs);
    if (S > G) S = G;
    if (S < 1) S = 1;
    int gpw = tune(ctx, OXQ_TUNE_GEMV_GPW, (int)ceil_div(G, S));
    S = (int)ceil_div(G, gpw);
    dim3 grid((unsigned)slabs, (unsigned)S), block(512);
    const uint64_t ws_bytes = S > 1 ? (uint64_t)S * p.M * p.N * 4 : 0;
    char name[64];
    snprintf(name, sizeof name, "gptq%d_gemv_fast_%s_m%d", BITS, TT::DTYPE == 1 ? "f16" : "bf16", mb);
    set_plan(ctx, name, grid, block, S, 1, ws_bytes);
    const int fused = splitk_fused(ctx, S);
    if (ctx->plan_only) {
        if (S > 1 && !fused) add_launch(ctx);
        return OXQ_OK;
    }
    if (ws_bytes > ctx->workspace_bytes || grid.x > ctx->n_counters)
        return fail(OXQ_ERR_WORKSPACE, "gptq gemv: needs %llu workspace bytes, ctx holds %zu",
                    (unsigned long long)ws_bytes, ctx->workspace_bytes);
#define OXQ_GO(MBv)                                                                               \
    hipLaunchKernelGGL((gptq_gemv_fast<TT, BITS, MBv>), grid, block, 0, s, (const uint16_t *)p.x, \
                       p.qweight, p.qzeros, (const uint16_t *)p.scales, (const uint16_t *)p.bias, \
                       (uint16_t *)p.y, (float *)ctx->workspace, ctx->counters, (int)p.M, (int)p.K, \
                       (int)p.N, p.group_shift, gpw, S, fused)
    switch (mb) {
    case 1: OXQ_GO(1); break;
    case 2: OXQ_GO(2); break;
    case 4: OXQ_GO(4); break;
    default: OXQ_GO(8); break;
    }
#undef OXQ_GO
    OXQ_HIP_CHECK(hipGetLastError());
    if (S > 1 && !fused)
        return launch_splitk_reduce(ctx, s, (const float *)ctx->workspace, p.bias, p.y, p.M, p.N, S,
                                    p.dtype);
    return OXQ_OK;
}

int launch_wna16_gemv(oxq_ctx *ctx, hipStream_t s, const Wna16Problem &p) {
    const bool f16 = p.dtype == OXQ_F16;
    // 2..8 rows of f16 on 4-bit AWQ: the matrix-core tile kernel reads the weights once for all
    // rows (13 - 14 us against 17 - 33 us for the dot2 kernel at 4096 x 14336).  Its B operand is
    // the dequantized weight rounded to f16, 2^-12 relative: far inside the tolerance; bf16, whose
    // rounding is 2^-9, keeps the kernel that never rounds the weight.
    if (p.M >= 2 && f16 && awq4_mfma_ok(p) && tune(ctx, OXQ_TUNE_GEMV_TILE, 1) && !tune(ctx, OXQ_TUNE_FORCE_GENERIC, 0))
        return launch_wna16_mfma(ctx, s, p);
    // GPTQ words feed the matrix cores as they are stored (gptq_tile.hip): 64-column strips, K inside the
    // workgroup (layers of few strips: K slices and the slice-ordered sum), the same time for 1 - 16 rows where
    // the dot-product kernel's arithmetic grows with the rows.  Like that kernel it never rounds a dequantized
    // weight at these row counts.  A single row of a layer of few strips stays with the dot-product kernel
    // (4096 x 4096: 7.1 against 7.3 us; 8-bit also two rows: 8.4 against 9.0); from there on the tile kernel
    // is ahead (14336 x 4096 at 2 / 8 rows: 10.5 / 10.7 against 11.2 / 21.0 us).
    if (gptq_tile_ok(p) && !tune(ctx, OXQ_TUNE_FORCE_GENERIC, 0)) {
        const int v = tune(ctx, OXQ_TUNE_GPTQ_TILE, 1);
        const bool wide = p.N >= 96 * 64;
        if (v == 2 || (v == 1 && (wide || p.M >= (p.bits == 4 ? 2 : 4)))) return launch_gptq_tile(ctx, s, p);
    }
    if (gptq_fast_ok(p) && !tune(ctx, OXQ_TUNE_FORCE_GENERIC, 0)) {
        if (p.bits == 4)
            return f16 ? launch_gptq_fast<F16Traits, 4>(ctx, s, p) : launch_gptq_fast<BF16Traits, 4>(ctx, s, p);
        return f16 ? launch_gptq_fast<F16Traits, 8>(ctx, s, p) : launch_gptq_fast<BF16Traits, 8>(ctx, s, p);
    }
    if (awq_fast_ok(p) && !tune(ctx, OXQ_TUNE_FORCE_GENERIC, 0)) {
        if (p.bits == 4)
            return f16 ? launch_awq_fast<F16Traits, 4>(ctx, s, p) : launch_awq_fast<BF16Traits, 4>(ctx, s, p);
        return f16 ? launch_awq_fast<F16Traits, 8>(ctx, s, p) : launch_awq_fast<BF16Traits, 8>(ctx, s, p);
    }
    if (p.bits == 4)
        return f16 ? launch_generic_t<F16Traits, 4>(ctx, s, p) : launch_generic_t<BF16Traits, 4>(ctx, s, p);
    return f16 ? launch_generic_t<F16Traits, 8>(ctx, s, p) : launch_generic_t<BF16Traits, 8>(ctx, s, p);
}

}  // namespace oxq
