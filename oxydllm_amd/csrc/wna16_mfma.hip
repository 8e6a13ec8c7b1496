// Batched W4A16 tile GEMM on the matrix cores (M >= 9 rows).
//
//   y[M, N] = x[M, K] . dequant(W)[K, N],  f32 accumulation, result in x's dtype.
//
// Reference semantics: mpp_gemm.metal:84-266 (staged quant GEMM: the B tile is
// dequantized to the 16-bit activation type, T((q - z) * s), before the matrix
// unit; f32 accumulate).  The B operand built here is bit-identical to the
// dense dequant op's output for the same elements.
//
// AWQ 4-bit mapping onto v_mfma_f32_16x16x32_{f16,bf16}: lane (c = lane % 16,
// kb = lane / 16) reads the packed word of column group c for the 8 rows
// k0 + 8*kb .. +7.  Those 8 words hold, per nibble slot s, the 8 consecutive-k
// values of output column 8*j + order(s): exactly one B fragment per slot, so
// 8 MFMAs per K-step of 32 cover 128 output columns with no cross-lane
// movement; the AWQ interleave is absorbed by the column index of each
// MFMA's result.  Rows are paired with v_perm so one AND-OR produces two
// exact 16-bit integers, then (q - z) * s is a packed add + packed multiply.
//
// A workgroup of 4 waves covers 16*MT rows x 512 columns; K is split across
// workgroups and combined with the deterministic last-arriver protocol.

#include "oxq_device.hpp"
#include "oxq_internal.hpp"

#include <cstdlib>

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

template <typename TT, int MT>
__global__ __launch_bounds__(256) void awq4_mfma_kernel(
    const uint16_t *__restrict__ x, const uint32_t *__restrict__ qw,
    const uint32_t *__restrict__ qz, const uint16_t *__restrict__ sc,
    const uint16_t *__restrict__ bias, uint16_t *__restrict__ y, float *__restrict__ ws,
    unsigned *__restrict__ counters, int M, int K, int N, int gshift, int kslice, int S) {
    typedef MfmaOps<TT> Ops;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int c = lane & 15, kb = lane >> 4;
    const int PW = N >> 3;
    const int jw = blockIdx.x * 64 + wave * 16 + c;  // packed word column of this lane
    const bool col_ok = jw < PW;
    const int jws = col_ok ? jw : PW - 1;            // clamp loads, discard results
    const int slice = blockIdx.y;
    const int m0 = blockIdx.z * (16 * MT);
    const int k_begin = slice * kslice;
    const int k_end = min(K, k_begin + kslice);

    float4_t acc[MT][8];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int s = 0; s < 8; ++s) acc[mt][s] = float4_t{0.f, 0.f, 0.f, 0.f};

    // activation rows of this lane's A fragments (clamped; extra rows are discarded)
    const uint16_t *xrow[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
        int r = m0 + mt * 16 + c;
        r = r < M ? r : M - 1;
        xrow[mt] = x + (size_t)r * K;
    }

    uint32_t negzb[8], sp[8];
    int cur_g = -1;
    for (int k0 = k_begin; k0 < k_end; k0 += 32) {
        const int g = k0 >> gshift;
        if (g != cur_g) {  // wave-uniform
            const uint32_t zw = qz[(size_t)g * PW + jws];
            const u32x4_t sv = *(const u32x4_t *)(sc + (size_t)g * N + (size_t)jws * 8);
#pragma unroll
            for (int s = 0; s < 8; ++s) {
                const int col = awq_slot_col(s);
                const uint32_t pr = sv[col >> 1];
                const uint32_t sb = (col & 1) ? (pr >> 16) : (pr & 0xFFFFu);
                sp[s] = sb | (sb << 16);
                negzb[s] = Ops::splat(-((float)((zw >> (4 * s)) & 0xFu) + TT::bias(s)));
            }
            cur_g = g;
        }
        uint32_t w[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) w[i] = qw[(size_t)(k0 + kb * 8 + i) * PW + jws];
        uint32_t a[MT][4];
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            const u32x4_t av = *(const u32x4_t *)(xrow[mt] + k0 + kb * 8);
            a[mt][0] = av[0]; a[mt][1] = av[1]; a[mt][2] = av[2]; a[mt][3] = av[3];
        }
        uint32_t b[8][4];
#pragma unroll
        for (int pp = 0; pp < 4; ++pp) {
            uint32_t p[8];
            TT::unpack4(pack_lo16(w[2 * pp], w[2 * pp + 1]), p);
            TT::unpack4(pack_hi16(w[2 * pp], w[2 * pp + 1]), p + 4);
#pragma unroll
            for (int s = 0; s < 8; ++s) b[s][pp] = Ops::dequant_pair(p[s], negzb[s], sp[s]);
        }
#pragma unroll
        for (int s = 0; s < 8; ++s)
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) acc[mt][s] = Ops::mfma(a[mt], b[s], acc[mt][s]);
    }

    // D layout: lane (c, rb = lane / 16) holds rows 4*rb + i, column c of each tile.
    const int rb = kb;
    const int nbase = jw * 8;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int m = m0 + mt * 16 + rb * 4 + i;
            if (m < M && col_ok) {
                float v[8];
#pragma unroll
                for (int s = 0; s < 8; ++s) v[awq_slot_col(s)] = acc[mt][s][i];
                if (S == 1) {
                    uint32_t o[4];
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        float lo = v[2 * q], hi = v[2 * q + 1];
                        if (bias) {
                            lo += TT::to_f32(bias[nbase + 2 * q]);
                            hi += TT::to_f32(bias[nbase + 2 * q + 1]);
                        }
                        o[q] = (uint32_t)TT::from_f32(lo) | ((uint32_t)TT::from_f32(hi) << 16);
                    }
                    *(u32x4_t *)(y + (size_t)m * N + nbase) = u32x4_t{o[0], o[1], o[2], o[3]};
                } else {
                    float *dst = ws + ((size_t)slice * M + m) * N + nbase;
                    *(float4_t *)dst = float4_t{v[0], v[1], v[2], v[3]};
                    *(float4_t *)(dst + 4) = float4_t{v[4], v[5], v[6], v[7]};
                }
            }
        }
    }
    if (S > 1 && splitk_arrive(counters, blockIdx.z * gridDim.x + blockIdx.x, S)) {
        const int tile_cols = 512;
        const int n0 = blockIdx.x * tile_cols;
        const int rows = min(16 * MT, M - m0);
        for (int idx = threadIdx.x; idx < rows * tile_cols; idx += 256) {
            const int m = m0 + idx / tile_cols;
            const int n = n0 + idx % tile_cols;
            if (n >= N) continue;
            float tot = 0.0f;
            for (int s = 0; s < S; ++s) tot += ws[((size_t)s * M + m) * N + n];
            if (bias) tot += TT::to_f32(bias[n]);
            y[(size_t)m * N + n] = TT::from_f32(tot);
        }
    }
}

static int env_int(const char *name, int dflt) {
    const char *v = getenv(name);
    return (v && *v) ? atoi(v) : dflt;
}

template <typename TT>
static int launch_awq4_mfma(oxq_ctx *ctx, hipStream_t s, const Wna16Problem &p) {
    const int M = (int)p.M, K = (int)p.K, N = (int)p.N;
    const int mt = M <= 16 ? 1 : (M <= 32 ? 2 : (M <= 48 ? 3 : 4));
    const int mtiles = (int)ceil_div(M, 16 * mt);
    const int ctiles = (int)ceil_div(N, 512);
    // K slices: whole groups (and whole 32-row MFMA steps), about one workgroup per CU
    const int step = (int)(p.group_size > 32 ? p.group_size : 32);
    const int units = K / step;
    int S = env_int("OXQ_MFMA_SPLITK", ctx->num_cus / (mtiles * ctiles));
    if (S < 1) S = 1;
    if (S > units) S = units;
    const int kslice = (int)ceil_div(units, S) * step;
    S = (int)ceil_div(K, kslice);
    // keep the partials inside the workspace
    while (S > 1 && (uint64_t)S * M * N * 4 > ctx->workspace_bytes) --S;
    const int kslice2 = (int)ceil_div(units, S) * step;
    S = (int)ceil_div(K, kslice2);
    dim3 grid((unsigned)ctiles, (unsigned)S, (unsigned)mtiles), block(256);
    const uint64_t ws_bytes = S > 1 ? (uint64_t)S * M * N * 4 : 0;
    char name[64];
    snprintf(name, sizeof name, "awq4_mfma_%s_mt%d", TT::DTYPE == 1 ? "f16" : "bf16", mt);
    set_plan(ctx, name, grid, block, S, 1, ws_bytes);
    if (ctx->plan_only) return OXQ_OK;
    if (ws_bytes > ctx->workspace_bytes || (size_t)ctiles * mtiles > ctx->n_counters)
        return fail(OXQ_ERR_WORKSPACE, "w4a16 tile gemm: needs %llu workspace bytes, ctx holds %zu",
                    (unsigned long long)ws_bytes, ctx->workspace_bytes);
#define OXQ_GO(MTv)                                                                              \
    hipLaunchKernelGGL((awq4_mfma_kernel<TT, MTv>), grid, block, 0, s, (const uint16_t *)p.x,    \
                       p.qweight, p.qzeros, (const uint16_t *)p.scales, (const uint16_t *)p.bias, \
                       (uint16_t *)p.y, (float *)ctx->workspace, ctx->counters, M, K, N,         \
                       p.group_shift, kslice2, S)
    switch (mt) {
    case 1: OXQ_GO(1); break;
    case 2: OXQ_GO(2); break;
    case 3: OXQ_GO(3); break;
    default: OXQ_GO(4); break;
    }
#undef OXQ_GO
    OXQ_HIP_CHECK(hipGetLastError());
    return OXQ_OK;
}

static bool awq4_mfma_ok(const Wna16Problem &p) {
    if (p.bits != 4 || p.pack_dim != OXQ_PACK_OUT) return false;
    if (p.K % 32 != 0 || p.N % 8 != 0) return false;
    if (p.group_size % 32 != 0) return false;  // a 32-row MFMA step stays inside one group
    if (((uintptr_t)p.x | (uintptr_t)p.scales | (uintptr_t)p.y) & 15) return false;
    return true;
}

int launch_wna16_mfma(oxq_ctx *ctx, hipStream_t s, const Wna16Problem &p) {
    if (awq4_mfma_ok(p) && !env_int("OXQ_FORCE_GENERIC", 0))
        return p.dtype == OXQ_F16 ? launch_awq4_mfma<F16Traits>(ctx, s, p)
                                  : launch_awq4_mfma<BF16Traits>(ctx, s, p);
    // Layouts without a tile kernel (GPTQ, 8-bit, unaligned shapes): run the
    // GEMV kernel over chunks of 8 rows, as the reference does below its
    // tile-GEMM threshold (linear.rs:457-480).
    uint32_t launches = 0;
    const size_t eb = 2;
    for (int64_t m0 = 0; m0 < p.M; m0 += 8) {
        Wna16Problem c = p;
        c.M = (p.M - m0) < 8 ? (p.M - m0) : 8;
        c.x = (const uint8_t *)p.x + (size_t)m0 * p.K * eb;
        c.y = (uint8_t *)p.y + (size_t)m0 * p.N * eb;
        int rc = launch_wna16_gemv(ctx, s, c);
        if (rc != OXQ_OK) return rc;
        ++launches;
    }
    ctx->plan.launches = launches;
    return OXQ_OK;
}

}  // namespace oxq
