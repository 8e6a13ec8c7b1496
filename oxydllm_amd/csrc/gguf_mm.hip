// GGUF block-quant tile matmul for m > 8 (prefill) on the matrix cores, bf16 activations.
//
// Reference semantics (quant_kernels.metal:2303-3102, gguf_*_mul_mm_bf16; host side
// metal_ops.rs:5856-5989): a strip of weight rows is dequantized block by block, each value
// rounded to bf16, and multiplied with the bf16 activations, f32 accumulation, bf16 output:
//     y[m][n] = bf16( sum_k f32(x[m][k]) * f32(bf16(w[n][k])) ) (+ bias).
//
// Tile: 64 weight rows x (16 * MT) tokens x 256 elements of K per stage, 256 threads; wave w
// owns weight rows 16w..16w+15 against all MT token tiles.
//   1. the stage's raw bytes - 256 elements of each row, one super-block or eight small
//      blocks, contiguous - and the token tile go to LDS with 16-byte loads (each row's
//      segment from the 16-byte boundary below its first byte: block rows are only
//      2-byte aligned);
//   2. lane (r = l % 16, kb = l / 16) decodes units kb and kb + 4 of row r (32 weights
//      each) from LDS and rounds them to bf16.  Those registers are the A operands of eight
//      v_mfma_f32_16x16x32_bf16 steps as they are: inside a step the k index only has to
//      agree between A and B, so step (unit u, quarter j) multiplies elements
//      32 u + 8 j .. + 7 of row r with the same elements of the tokens, which lane
//      (token l % 16, kb) reads from the token tile.  The weights never go back to LDS,
//      and a weight is decoded once per 16 * MT tokens;
//   3. lane (l % 16, l / 16) ends up with 4 consecutive output columns of token l % 16.
// The next stage's global loads are issued before step 2 and land in LDS after the MFMAs.
// The token tile is padded to a pitch of 528 bytes: the 16 rows a quarter wave reads or
// writes then start 4 banks apart.
// Shapes with few tiles also split K over grid.z: every slice stores its f32 partial tile
// to the workspace with plain stores, and a second kernel adds the slices in slice order
// (the kernel boundary publishes the partials; the result does not depend on timing).

#include "gguf_decode.hpp"

#include <algorithm>
#include <cstdlib>

namespace oxq {

constexpr int MM_BN = 64;     // weight rows per workgroup
constexpr int MM_BK = 256;    // elements of K per stage
constexpr int MM_TP = 528;    // token tile row pitch in bytes (512 + 16)

template <int FMT> struct GgufSeg {
    static constexpr int SEG = MM_BK / GgufFmt<FMT>::BE * GgufFmt<FMT>::BB;  // bytes per row per stage
    static constexpr int RAWC = ((SEG + 14 + 15) / 16) | 1;                  // 16-byte chunks per row, odd
    static constexpr int RAWP = RAWC * 16;
    static constexpr int NRAW = (MM_BN * RAWC + 255) / 256;                   // chunks per thread
};

__device__ __forceinline__ uint32_t pack_bf16(float lo, float hi) {
    typedef float f2_t __attribute__((ext_vector_type(2)));
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(f2_t{lo, hi}, bf16x2_t));
}

template <int FMT, int MT>
__global__ __launch_bounds__(256) void gguf_mm_kernel(const uint16_t *__restrict__ x,
                                                      const uint8_t *__restrict__ w,
                                                      const uint16_t *__restrict__ bias,
                                                      uint16_t *__restrict__ y, float *__restrict__ ws,
                                                      int M, int K, int N, size_t total_bytes,
                                                      int stages_per_slice) {
    using S = GgufSeg<FMT>;
    extern __shared__ __attribute__((aligned(16))) unsigned char mm_lds[];
    unsigned char *raw = mm_lds;                          // [64][RAWP]
    unsigned char *xt = raw + MM_BN * S::RAWP;            // [16 MT][528] bf16 tokens
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int ni = lane & 15, kb = lane >> 4;
    const int n0 = blockIdx.x * MM_BN, m0 = blockIdx.y * (16 * MT);
    const int units = K >> 5;
    const int s_begin = blockIdx.z * stages_per_slice;
    const int s_end = min((units + 7) >> 3, s_begin + stages_per_slice);  // > s_begin for every slice
    const size_t row_bytes = (size_t)(K / GgufFmt<FMT>::BE) * GgufFmt<FMT>::BB;

    u32x4_t rreg[S::NRAW], xreg[2 * MT];
    auto load_stage = [&](int s) {
#pragma unroll
        for (int i = 0; i < S::NRAW; ++i) {
            const int c = tid + 256 * i;
            const int r = c / S::RAWC, cc = c - r * S::RAWC;
            u32x4_t v = {0u, 0u, 0u, 0u};
            if (r < MM_BN) {
                const int n = min(n0 + r, N - 1);
                const size_t start = (size_t)n * row_bytes + (size_t)s * S::SEG;
                const size_t off = (start & ~(size_t)15) + (size_t)cc * 16;
                if (off + 16 <= total_bytes) {
                    v = *(const u32x4_t *)(w + off);
                } else if (off < total_bytes) {  // the tensor's last, partial chunk
                    uint32_t t[4] = {0u, 0u, 0u, 0u};
                    for (int b = 0; b < 16; ++b)
                        if (off + b < total_bytes) t[b >> 2] |= (uint32_t)w[off + b] << (8 * (b & 3));
                    v = u32x4_t{t[0], t[1], t[2], t[3]};
                }
            }
            rreg[i] = v;
        }
#pragma unroll
        for (int i = 0; i < 2 * MT; ++i) {
            const int c = tid + 256 * i;
            const int r = c >> 5, cc = c & 31;
            const int m = min(m0 + r, M - 1);
            const int k = s * MM_BK + cc * 8;
            const bool valid = k < K;
            const u32x4_t v = *(const u32x4_t *)(x + (size_t)m * K + (valid ? k : 0));
            xreg[i] = valid ? v : u32x4_t{0u, 0u, 0u, 0u};
        }
    };
    auto commit_stage = [&]() {
#pragma unroll
        for (int i = 0; i < S::NRAW; ++i) {
            const int c = tid + 256 * i;
            if (c < MM_BN * S::RAWC) *(u32x4_t *)(raw + (size_t)c * 16) = rreg[i];
        }
#pragma unroll
        for (int i = 0; i < 2 * MT; ++i) {
            const int c = tid + 256 * i;
            *(u32x4_t *)(xt + (c >> 5) * MM_TP + (c & 31) * 16) = xreg[i];
        }
    };

    float4_t acc[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) acc[mt] = float4_t{0.f, 0.f, 0.f, 0.f};

    const int dr = 16 * wave + ni;  // the weight row this lane decodes and multiplies
    const int dn = min(n0 + dr, N - 1);
    load_stage(s_begin);
    for (int s = s_begin; s < s_end; ++s) {
        commit_stage();
        __syncthreads();
        load_stage(min(s + 1, s_end - 1));
        const int head = (int)(((size_t)dn * row_bytes + (size_t)s * S::SEG) & 15);
        const uint8_t *seg = raw + dr * S::RAWP + head;
        u32x4_t a[2][4];
#pragma unroll
        for (int pass = 0; pass < 2; ++pass) {
            const int u = kb + 4 * pass;
            uint32_t o[16];
            if (s * 8 + u < units) {
                float wf[32];
                decode_unit<FMT>(seg, u, wf);
#pragma unroll
                for (int i = 0; i < 16; ++i) o[i] = pack_bf16(wf[2 * i], wf[2 * i + 1]);
            } else {  // past the end of K (the token tile holds zeros there as well)
#pragma unroll
                for (int i = 0; i < 16; ++i) o[i] = 0u;
            }
#pragma unroll
            for (int j = 0; j < 4; ++j) a[pass][j] = u32x4_t{o[4 * j], o[4 * j + 1], o[4 * j + 2], o[4 * j + 3]};
        }
#pragma unroll
        for (int pass = 0; pass < 2; ++pass)
#pragma unroll
            for (int j = 0; j < 4; ++j)
#pragma unroll
                for (int mt = 0; mt < MT; ++mt) {
                    const u32x4_t bv =
                        *(const u32x4_t *)(xt + (16 * mt + ni) * MM_TP + (kb + 4 * pass) * 64 + j * 16);
                    acc[mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, a[pass][j]),
                                                                      __builtin_bit_cast(bf16x8_t, bv), acc[mt], 0, 0, 0);
                }
        __syncthreads();
    }

    // D[i][j]: lane (j = ni, i = 4 kb + r) holds weight rows n0 + 16 wave + 4 kb + r of token ni
    const int nb0 = n0 + 16 * wave + 4 * kb;
    if (gridDim.z > 1) {  // f32 partial tile of this K slice (the launcher guarantees N % 4 == 0)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            const int m = m0 + 16 * mt + ni;
            if (m < M && nb0 < N) *(float4_t *)(ws + ((size_t)blockIdx.z * M + m) * N + nb0) = acc[mt];
        }
        return;
    }
    float bvals[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) bvals[r] = (bias && nb0 + r < N) ? BF16Traits::to_f32(bias[nb0 + r]) : 0.0f;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
        const int m = m0 + 16 * mt + ni;
        if (m >= M) continue;
        uint16_t *yr = y + (size_t)m * N + nb0;
        if ((N & 3) == 0 && nb0 + 3 < N) {
            const uint32_t lo = pack_bf16(acc[mt][0] + bvals[0], acc[mt][1] + bvals[1]);
            const uint32_t hi = pack_bf16(acc[mt][2] + bvals[2], acc[mt][3] + bvals[3]);
            typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));
            *(u32x2_t *)yr = u32x2_t{lo, hi};
        } else {
#pragma unroll
            for (int r = 0; r < 4; ++r)
                if (nb0 + r < N) yr[r] = BF16Traits::from_f32(acc[mt][r] + bvals[r]);
        }
    }
}

struct MmPlan {
    int mt, ks, stages_per_slice;
};

template <int FMT, int MT>
static int launch_mm_go(oxq_ctx *ctx, hipStream_t s, const GgufProblem &p, dim3 grid, size_t lds, size_t total,
                        int sps) {
    static bool attr_set = false;
    if (!attr_set) {
        OXQ_HIP_CHECK(hipFuncSetAttribute((const void *)gguf_mm_kernel<FMT, MT>,
                                          hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
        attr_set = true;
    }
    hipLaunchKernelGGL((gguf_mm_kernel<FMT, MT>), grid, dim3(256), lds, s, (const uint16_t *)p.x, p.w,
                       (const uint16_t *)p.bias, (uint16_t *)p.y, (float *)ctx->workspace, (int)p.M, (int)p.K,
                       (int)p.N, total, sps);
    OXQ_HIP_CHECK(hipGetLastError());
    return OXQ_OK;
}

// Tile choice: 64 rows x up to 64 tokens (128-token tiles were measured: +10 % at m = 2048
// for the 4-bit formats, slower for the others, whose kernels then need > 256 registers).  When that grid cannot fill the 256 CUs, K is
// split over up to 8 slices of at least two stages.
static MmPlan plan_mm(const oxq_ctx *ctx, const GgufProblem &p) {
    MmPlan pl;
    pl.mt = p.M > 32 ? 4 : p.M > 16 ? 2 : 1;
    if (const char *e = getenv("OXQ_GGUF_MM_MT")) pl.mt = atoi(e) == 1 ? 1 : atoi(e) == 2 ? 2 : 4;
    const int stages = (int)ceil_div(p.K, MM_BK);
    const int64_t tiles = ceil_div(p.N, MM_BN) * ceil_div(p.M, 16 * pl.mt);
    pl.ks = 1;
    if (tiles < 192) pl.ks = (int)std::min<int64_t>({ceil_div(256, tiles), 8, std::max(1, stages / 2)});
    if (const char *e = getenv("OXQ_GGUF_MM_KS")) pl.ks = std::max(1, std::min(atoi(e), stages));
    // the reduction kernel works on groups of 4 columns; the workspace bounds the split
    if (p.N % 4 != 0) pl.ks = 1;
    while (pl.ks > 1 && (size_t)pl.ks * p.M * p.N * 4 > ctx->workspace_bytes) --pl.ks;
    pl.stages_per_slice = (int)ceil_div(stages, pl.ks);
    pl.ks = (int)ceil_div(stages, pl.stages_per_slice);  // no empty slice
    return pl;
}

template <int FMT>
static int launch_mm_fmt(oxq_ctx *ctx, hipStream_t s, const GgufProblem &p, const char *fname) {
    using S = GgufSeg<FMT>;
    const MmPlan pl = plan_mm(ctx, p);
    const int mt = pl.mt;
    const size_t lds = (size_t)MM_BN * S::RAWP + (size_t)16 * mt * MM_TP;
    const size_t total = (size_t)p.N * (size_t)(p.K / GgufFmt<FMT>::BE) * GgufFmt<FMT>::BB;
    dim3 grid((unsigned)ceil_div(p.N, MM_BN), (unsigned)ceil_div(p.M, 16 * mt), (unsigned)pl.ks);
    char name[64];
    snprintf(name, sizeof name, "gguf_%s_mul_mm_bf16_mt%d", fname, mt);
    set_plan(ctx, name, grid, dim3(256), pl.ks, 1, pl.ks > 1 ? (size_t)pl.ks * p.M * p.N * 4 : 0);
    if (ctx->plan_only) {
        if (pl.ks > 1) add_launch(ctx);
        return OXQ_OK;
    }
    int rc;
    switch (mt) {
    case 1: rc = launch_mm_go<FMT, 1>(ctx, s, p, grid, lds, total, pl.stages_per_slice); break;
    case 2: rc = launch_mm_go<FMT, 2>(ctx, s, p, grid, lds, total, pl.stages_per_slice); break;
    default: rc = launch_mm_go<FMT, 4>(ctx, s, p, grid, lds, total, pl.stages_per_slice); break;
    }
    if (rc != OXQ_OK || pl.ks == 1) return rc;
    return launch_splitk_reduce(ctx, s, (const float *)ctx->workspace, p.bias, p.y, p.M, p.N, pl.ks, OXQ_BF16);
}

bool gguf_mm_eligible(const GgufProblem &p) {
    return p.act_dtype == OXQ_BF16 && p.M > 8 && ((uintptr_t)p.x & 15) == 0 && ((uintptr_t)p.w & 15) == 0 &&
           (p.K % 8) == 0;
}

int launch_gguf_mm(oxq_ctx *ctx, hipStream_t s, const GgufProblem &p) {
    switch (p.quant) {
    case OXQ_GGUF_Q4_0: return launch_mm_fmt<OXQ_GGUF_Q4_0>(ctx, s, p, "q4_0");
    case OXQ_GGUF_Q8_0: return launch_mm_fmt<OXQ_GGUF_Q8_0>(ctx, s, p, "q8_0");
    case OXQ_GGUF_Q4_K: return launch_mm_fmt<OXQ_GGUF_Q4_K>(ctx, s, p, "q4k");
    case OXQ_GGUF_Q6_K: return launch_mm_fmt<OXQ_GGUF_Q6_K>(ctx, s, p, "q6k");
    case OXQ_GGUF_Q4_1: return launch_mm_fmt<OXQ_GGUF_Q4_1>(ctx, s, p, "q4_1");
    case OXQ_GGUF_Q5_0: return launch_mm_fmt<OXQ_GGUF_Q5_0>(ctx, s, p, "q5_0");
    case OXQ_GGUF_Q5_1: return launch_mm_fmt<OXQ_GGUF_Q5_1>(ctx, s, p, "q5_1");
    case OXQ_GGUF_Q2_K: return launch_mm_fmt<OXQ_GGUF_Q2_K>(ctx, s, p, "q2k");
    case OXQ_GGUF_Q3_K: return launch_mm_fmt<OXQ_GGUF_Q3_K>(ctx, s, p, "q3k");
    case OXQ_GGUF_Q5_K: return launch_mm_fmt<OXQ_GGUF_Q5_K>(ctx, s, p, "q5k");
    default: return OXQ_ERR_ARG;
    }
}

}  // namespace oxq
