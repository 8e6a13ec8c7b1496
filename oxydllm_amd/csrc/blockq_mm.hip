// Block-quant tile matmul for m > 8 (prefill) on the matrix cores, bf16 activations: the ten
// GGUF formats, MXFP4 (plain and grouped by expert) and block-scaled F8E4M3.
//
// Reference semantics (quant_kernels.metal:2303-3102, gguf_*_mul_mm_bf16; host side
// metal_ops.rs:5856-5989): a strip of weight rows is dequantized block by block, each value
// rounded to bf16, and multiplied with the bf16 activations, f32 accumulation, bf16 output:
//     y[m][n] = bf16( sum_k f32(x[m][k]) * f32(bf16(w[n][k])) ) (+ bias).
// MXFP4 (quant_kernels.metal:3175-3240 mxfp4_mul_mm_bf16, metal_ops.rs:6112-6195) is the same
// with E2M1 code x E8M0 scale, which bf16 holds exactly.
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
// MXFP4 blocks are 16 bytes and aligned: each lane loads its two blocks and their scale bytes
// straight into registers (one stage ahead) and converts them with
// v_cvt_scalef32_pk_bf16_fp4, which applies the block scale as it widens two codes.
// F8E4M3 rows are plain bytes: two 16-byte loads per unit, v_cvt_pk_f32_fp8, the block scale
// in f32 and one rounding to bf16 - the reference's dequantized weight bit for bit
// (quant_kernels.metal:3877-3911), so this kernel is its "dequantize, then matmul" path for
// m > 8 (moe.rs:106-113) without the dense weight in memory.
// Grouped form (mixture of experts): blockIdx.y walks the (expert, token tile) pairs of the
// expert offsets; rows are gathered through the token list and written per routed pair.
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

__device__ __forceinline__ uint32_t pack_bf16(float lo, float hi) {
    typedef float f2_t __attribute__((ext_vector_type(2)));
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(f2_t{lo, hi}, bf16x2_t));
}

struct MmArgs {
    const uint16_t *x;        // [rows, K] bf16
    const uint8_t *w;         // GGUF block bytes / MXFP4 blocks
    const uint8_t *scales;    // MXFP4 E8M0 scales
    const uint16_t *bias;     // [N] ([E, N] grouped) or nullptr
    uint16_t *y;              // [M, N] ([pairs, N] grouped)
    float *ws;                // split-K partial tiles
    const int32_t *offsets;   // grouped: [E + 1] pair offsets per expert, else nullptr
    const int32_t *token_ids; // grouped: x row of each pair, or nullptr = the pair index
    const float *f8_scales;   // F8: F32 block-scale grid
    int f8_block_r, f8_block_c, f8_s_cols;
    int n_experts;
    int M, K, N;
    size_t total_bytes;       // GGUF: size of the weight tensor
    int stages_per_slice;
};

// ---- weight sources: raw bytes of one stage -> the lane's eight A operands -----------------
// load(s): issue the global loads of stage s into registers; commit(): make the loaded stage
// current (GGUF: store it to LDS; the caller's barrier follows); decode(s, pass, a): bf16
// weights 32 u .. 32 u + 31 (u = kb + 4 pass) of the lane's row as four 8-element operands.
template <int FMT> struct GgufSource {
    static constexpr bool HAS_RESIDUE = true;   // a decoded weight is an f32 value
    static constexpr int SEG = MM_BK / GgufFmt<FMT>::BE * GgufFmt<FMT>::BB;  // bytes per row per stage
    static constexpr int RAWC = ((SEG + 14 + 15) / 16) | 1;                  // 16-byte chunks per row, odd
    static constexpr int RAWP = RAWC * 16;
    static constexpr int NRAW = (MM_BN * RAWC + 255) / 256;                   // chunks per thread
    static constexpr int LDS_BYTES = MM_BN * RAWP;
    u32x4_t rreg[NRAW];
    const uint8_t *w;
    unsigned char *raw;
    size_t row_bytes, total_bytes;
    int n0, N, tid, dr, dn, kb, units;

    __device__ __forceinline__ void init(const MmArgs &a, unsigned char *lds, int n0_, int /*expert*/, int dr_,
                                         int kb_) {
        w = a.w, raw = lds, total_bytes = a.total_bytes;
        row_bytes = (size_t)(a.K / GgufFmt<FMT>::BE) * GgufFmt<FMT>::BB;
        n0 = n0_, N = a.N, tid = threadIdx.x, dr = dr_, kb = kb_, units = a.K >> 5;
        dn = min(n0 + dr, N - 1);
    }
    __device__ __forceinline__ void load(int s) {
#pragma unroll
        for (int i = 0; i < NRAW; ++i) {
            const int c = tid + 256 * i;
            const int r = c / RAWC, cc = c - r * RAWC;
            u32x4_t v = {0u, 0u, 0u, 0u};
            if (r < MM_BN) {
                const int n = min(n0 + r, N - 1);
                const size_t start = (size_t)n * row_bytes + (size_t)s * SEG;
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
    }
    __device__ __forceinline__ void commit() {
#pragma unroll
        for (int i = 0; i < NRAW; ++i) {
            const int c = tid + 256 * i;
            if (c < MM_BN * RAWC) *(u32x4_t *)(raw + (size_t)c * 16) = rreg[i];
        }
    }
    // HILO: also the rounding residue w - bf16(w), itself rounded to bf16 (relative error of
    // the pair 2^-17): the decode range keeps the f32 weights of the reference's GEMV kernels
    template <bool HILO>
    __device__ __forceinline__ void decode(int s, int pass, u32x4_t a[4], u32x4_t lo[4]) const {
        const int u = kb + 4 * pass;
        const int head = (int)(((size_t)dn * row_bytes + (size_t)s * SEG) & 15);
        uint32_t o[16], ol[16];
        if (s * 8 + u < units) {
            // stored integers converted once, then one fma a weight: scale * q - offset, the value
            // of the format's dequant (both products exact in f32 or rounded the same single time)
            float wf[32], c0, c1, d0, d1;
            unit_ints<FMT>(raw + dr * RAWP + head, u, wf, c0, c1, d0, d1);
#pragma unroll
            for (int i = 0; i < 32; ++i) wf[i] = fmaf(i < 16 ? c0 : c1, wf[i], -(i < 16 ? d0 : d1));
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                o[i] = pack_bf16(wf[2 * i], wf[2 * i + 1]);
                if (HILO)
                    ol[i] = pack_bf16(wf[2 * i] - __builtin_bit_cast(float, o[i] << 16),
                                      wf[2 * i + 1] - __builtin_bit_cast(float, o[i] & 0xFFFF0000u));
            }
        } else {  // past the end of K (the token tile holds zeros there as well)
#pragma unroll
            for (int i = 0; i < 16; ++i) o[i] = 0u, ol[i] = 0u;
        }
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            a[j] = u32x4_t{o[4 * j], o[4 * j + 1], o[4 * j + 2], o[4 * j + 3]};
            if (HILO) lo[j] = u32x4_t{ol[4 * j], ol[4 * j + 1], ol[4 * j + 2], ol[4 * j + 3]};
        }
    }
};

struct Mxfp4Source {
    static constexpr bool HAS_RESIDUE = false;
    static constexpr int LDS_BYTES = 0;
    const u32x4_t *brow;   // the lane's row of 16-byte blocks
    const uint8_t *srow;   // and of scale bytes
    u32x4_t nq[2], q[2];
    uint32_t ne[2], e[2];
    int nb, kb;

    __device__ __forceinline__ void init(const MmArgs &a, unsigned char *, int n0, int expert, int dr, int kb_) {
        nb = a.K >> 5, kb = kb_;
        const size_t row = (size_t)expert * a.N + min(n0 + dr, a.N - 1);
        brow = (const u32x4_t *)a.w + row * nb;
        srow = a.scales + row * nb;
    }
    __device__ __forceinline__ void load(int s) {
#pragma unroll
        for (int pass = 0; pass < 2; ++pass) {
            const int b = min(s * 8 + kb + 4 * pass, nb - 1);
            nq[pass] = brow[b];
            ne[pass] = srow[b];
        }
    }
    __device__ __forceinline__ void commit() {
        q[0] = nq[0], q[1] = nq[1], e[0] = ne[0], e[1] = ne[1];
    }
    template <bool HILO>  // E2M1 x E8M0 is exact in bf16: no residue
    __device__ __forceinline__ void decode(int s, int pass, u32x4_t a[4], u32x4_t *) const {
        const bool valid = s * 8 + kb + 4 * pass < nb;  // blocks past the row contribute zero
        const float sc = e8m0_to_f32(e[pass]);
        const u32x4_t t = q[pass];
        const uint32_t t0 = t[0], t1 = t[1], t2 = t[2], t3 = t[3];
        const uint32_t wj[4] = {valid ? t0 : 0u, valid ? t1 : 0u, valid ? t2 : 0u, valid ? t3 : 0u};
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const uint32_t c = wj[j];  // 8 codes, low nibble first
            a[j] = u32x4_t{__builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(c, sc, 0)),
                           __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(c, sc, 1)),
                           __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(c, sc, 2)),
                           __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(c, sc, 3))};
        }
    }
};

struct F8Source {
    static constexpr bool HAS_RESIDUE = false;
    static constexpr int LDS_BYTES = 0;
    const u32x4_t *wrow;   // the lane's row, 16-byte chunks
    const float *srow;     // its row of the scale grid
    u32x4_t nq[2][2], q[2][2];
    float nsc[2], sc[2];
    int units, kb, block_c;

    __device__ __forceinline__ void init(const MmArgs &a, unsigned char *, int n0, int, int dr, int kb_) {
        units = a.K >> 5, kb = kb_, block_c = a.f8_block_c;
        const int n = min(n0 + dr, a.N - 1);
        wrow = (const u32x4_t *)(a.w + (size_t)n * a.K);
        srow = a.f8_scales + (size_t)(n / a.f8_block_r) * a.f8_s_cols;
    }
    __device__ __forceinline__ void load(int s) {
#pragma unroll
        for (int pass = 0; pass < 2; ++pass) {
            const int u = min(s * 8 + kb + 4 * pass, units - 1);
            nq[pass][0] = wrow[2 * u];
            nq[pass][1] = wrow[2 * u + 1];
            nsc[pass] = srow[(u * 32) / block_c];  // block_c % 32 == 0: one scale per unit
        }
    }
    __device__ __forceinline__ void commit() {
#pragma unroll
        for (int pass = 0; pass < 2; ++pass) q[pass][0] = nq[pass][0], q[pass][1] = nq[pass][1], sc[pass] = nsc[pass];
    }
    template <bool HILO>  // the weight is a bf16 value by definition: no residue
    __device__ __forceinline__ void decode(int s, int pass, u32x4_t a[4], u32x4_t *) const {
        typedef float f2_t __attribute__((ext_vector_type(2)));
        const bool valid = s * 8 + kb + 4 * pass < units;
        const float scl = sc[pass];
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const u32x4_t t = q[pass][h];
            const uint32_t t0 = t[0], t1 = t[1], t2 = t[2], t3 = t[3];
            const uint32_t wj[4] = {valid ? t0 : 0u, valid ? t1 : 0u, valid ? t2 : 0u, valid ? t3 : 0u};
            uint32_t o[8];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const f2_t lo = __builtin_amdgcn_cvt_pk_f32_fp8((int)wj[i], false);
                const f2_t hi = __builtin_amdgcn_cvt_pk_f32_fp8((int)wj[i], true);
                o[2 * i] = pack_bf16(lo[0] * scl, lo[1] * scl);
                o[2 * i + 1] = pack_bf16(hi[0] * scl, hi[1] * scl);
            }
            a[2 * h] = u32x4_t{o[0], o[1], o[2], o[3]};
            a[2 * h + 1] = u32x4_t{o[4], o[5], o[6], o[7]};
        }
    }
};

template <class SRC, int MT, bool HILO>
__global__ __launch_bounds__(256) void blockq_mm_kernel(const MmArgs a) {
    extern __shared__ __attribute__((aligned(16))) unsigned char mm_lds[];
    unsigned char *xt = mm_lds + SRC::LDS_BYTES;          // [16 MT][528] bf16 tokens
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int ni = lane & 15, kb = lane >> 4;
    const int K = a.K, N = a.N;
    const int n0 = blockIdx.x * MM_BN;
    // the rows [m0, m_end) of x / y this workgroup covers, and its expert
    int m0 = blockIdx.y * (16 * MT), m_end = a.M, expert = 0;
    if (a.offsets) {  // grouped: blockIdx.y -> (expert, token tile); all values block-uniform
        int rem = blockIdx.y, e = 0;
        for (; e < a.n_experts; ++e) {
            const int tiles = (a.offsets[e + 1] - a.offsets[e] + 16 * MT - 1) / (16 * MT);
            if (rem < tiles) break;
            rem -= tiles;
        }
        if (e == a.n_experts) return;
        expert = e;
        m0 = a.offsets[e] + rem * (16 * MT);
        m_end = a.offsets[e + 1];
    }
    const int units = K >> 5;
    const int s_begin = blockIdx.z * a.stages_per_slice;
    const int s_end = min((units + 7) >> 3, s_begin + a.stages_per_slice);  // > s_begin for every slice

    SRC src;
    src.init(a, mm_lds, n0, expert, 16 * wave + ni, kb);

    // token rows this thread copies: chunk c = tid + 256 i -> row c / 32, 16-byte chunk c % 32
    const uint16_t *xrow[2 * MT];
#pragma unroll
    for (int i = 0; i < 2 * MT; ++i) {
        const int m = min(m0 + ((tid + 256 * i) >> 5), m_end - 1);
        xrow[i] = a.x + (size_t)(a.token_ids ? a.token_ids[m] : m) * K;
    }
    u32x4_t xreg[2 * MT];
    auto load_x = [&](int s) {
#pragma unroll
        for (int i = 0; i < 2 * MT; ++i) {
            const int k = s * MM_BK + (tid & 31) * 8;
            const bool valid = k < K;
            const u32x4_t v = *(const u32x4_t *)(xrow[i] + (valid ? k : 0));
            xreg[i] = valid ? v : u32x4_t{0u, 0u, 0u, 0u};
        }
    };

    float4_t acc[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) acc[mt] = float4_t{0.f, 0.f, 0.f, 0.f};

    src.load(s_begin);
    load_x(s_begin);
    for (int s = s_begin; s < s_end; ++s) {
        src.commit();
#pragma unroll
        for (int i = 0; i < 2 * MT; ++i) {
            const int c = tid + 256 * i;
            *(u32x4_t *)(xt + (c >> 5) * MM_TP + (c & 31) * 16) = xreg[i];
        }
        __syncthreads();
        const int sn = min(s + 1, s_end - 1);
        src.load(sn);
        load_x(sn);
        u32x4_t av[2][4], al[HILO ? 2 : 1][4];
        src.template decode<HILO>(s, 0, av[0], al[0]);
        src.template decode<HILO>(s, 1, av[1], al[HILO ? 1 : 0]);
#pragma unroll
        for (int pass = 0; pass < 2; ++pass)
#pragma unroll
            for (int j = 0; j < 4; ++j)
#pragma unroll
                for (int mt = 0; mt < MT; ++mt) {
                    const u32x4_t bv =
                        *(const u32x4_t *)(xt + (16 * mt + ni) * MM_TP + (kb + 4 * pass) * 64 + j * 16);
                    acc[mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, av[pass][j]),
                                                                      __builtin_bit_cast(bf16x8_t, bv), acc[mt], 0, 0, 0);
                    if (HILO)
                        acc[mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
                            __builtin_bit_cast(bf16x8_t, al[HILO ? pass : 0][j]), __builtin_bit_cast(bf16x8_t, bv),
                            acc[mt], 0, 0, 0);
                }
        __syncthreads();
    }

    // D[i][j]: lane (j = ni, i = 4 kb + r) holds weight rows n0 + 16 wave + 4 kb + r of token ni
    const int nb0 = n0 + 16 * wave + 4 * kb;
    if (gridDim.z > 1) {  // f32 partial tile of this K slice (the launcher guarantees N % 4 == 0)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            const int m = m0 + 16 * mt + ni;
            if (m < m_end && nb0 < N) *(float4_t *)(a.ws + ((size_t)blockIdx.z * a.M + m) * N + nb0) = acc[mt];
        }
        return;
    }
    const uint16_t *bias = a.bias ? a.bias + (size_t)expert * N : nullptr;
    float bvals[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) bvals[r] = (bias && nb0 + r < N) ? BF16Traits::to_f32(bias[nb0 + r]) : 0.0f;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
        const int m = m0 + 16 * mt + ni;
        if (m >= m_end) continue;
        uint16_t *yr = a.y + (size_t)m * N + nb0;
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

template <class SRC, int MT, bool HILO = false>
static int launch_mm_go(hipStream_t s, const MmArgs &a, dim3 grid, size_t lds) {
    static LdsGrant lds_grant;  // one per instantiation
    OXQ_HIP_CHECK(lds_grant.ensure((const void *)blockq_mm_kernel<SRC, MT, HILO>, lds));
    hipLaunchKernelGGL((blockq_mm_kernel<SRC, MT, HILO>), grid, dim3(256), lds, s, a);
    OXQ_HIP_CHECK(hipGetLastError());
    return OXQ_OK;
}

// Tile choice: 64 rows x up to 64 tokens (128-token tiles were measured: +10 % at m = 2048
// for the 4-bit formats, slower for the others, whose kernels then need > 256 registers).
// When that grid cannot fill the 256 CUs, K is split over up to 8 slices of at least two
// stages.  `rows` = tokens (plain) or routed pairs (grouped, never split).
static MmPlan plan_mm(const oxq_ctx *ctx, int64_t rows, int64_t K, int64_t N, bool grouped, oxq_tune_key mt_key,
                      oxq_tune_key ks_key) {
    MmPlan pl;
    pl.mt = rows > 32 ? 4 : rows > 16 ? 2 : 1;
    if (tune_given(ctx, mt_key)) pl.mt = tune(ctx, mt_key, 4) == 1 ? 1 : tune(ctx, mt_key, 4) == 2 ? 2 : 4;
    const int stages = (int)ceil_div(K, MM_BK);
    const int64_t tiles = ceil_div(N, MM_BN) * ceil_div(rows, 16 * pl.mt);
    pl.ks = 1;
    if (tiles < 192) pl.ks = (int)std::min<int64_t>({ceil_div(256, tiles), 8, std::max(1, stages / 2)});
    if (tune_given(ctx, ks_key)) pl.ks = std::max(1, std::min(tune(ctx, ks_key, 1), stages));
    // the reduction kernel works on groups of 4 columns; the workspace bounds the split
    if (N % 4 != 0 || grouped) pl.ks = 1;
    while (pl.ks > 1 && (size_t)pl.ks * rows * N * 4 > ctx->workspace_bytes) --pl.ks;
    pl.stages_per_slice = (int)ceil_div(stages, pl.ks);
    pl.ks = (int)ceil_div(stages, pl.stages_per_slice);  // no empty slice
    return pl;
}

// hilo: (GGUF, m <= 8) keep the rounding residue of every weight, see GgufSource::decode
template <class SRC>
static int launch_mm_src(oxq_ctx *ctx, hipStream_t s, MmArgs &a, const char *name_prefix, oxq_tune_key mt_key, oxq_tune_key ks_key,
                         bool hilo = false) {
    const bool grouped = a.offsets != nullptr;
    const MmPlan pl = plan_mm(ctx, a.M, a.K, a.N, grouped, mt_key, ks_key);
    const int mt = pl.mt;
    a.ws = (float *)ctx->workspace;
    a.stages_per_slice = pl.stages_per_slice;
    const size_t lds = (size_t)SRC::LDS_BYTES + (size_t)16 * mt * MM_TP;
    // grouped: sum over experts of ceil(pairs_e / tile) <= pairs / tile + experts
    const int64_t ytiles = grouped ? a.M / (16 * mt) + a.n_experts : ceil_div(a.M, 16 * mt);
    if (ytiles > 65535)
        return fail(OXQ_ERR_UNSUPPORTED, "%s mul_mm: %lld token tiles exceed the grid limit of 65535", name_prefix,
                    (long long)ytiles);
    dim3 grid((unsigned)ceil_div(a.N, MM_BN), (unsigned)ytiles, (unsigned)pl.ks);
    char name[64];
    hilo = hilo && mt == 1 && SRC::HAS_RESIDUE;
    snprintf(name, sizeof name, "%s_mul_mm_bf16_mt%d%s", name_prefix, mt, hilo ? "_f32w" : "");
    set_plan(ctx, name, grid, dim3(256), pl.ks, 1, pl.ks > 1 ? (size_t)pl.ks * a.M * a.N * 4 : 0);
    if (ctx->plan_only) {
        if (pl.ks > 1) add_launch(ctx);
        return OXQ_OK;
    }
    int rc;
    switch (mt) {
    case 1:
        if constexpr (SRC::HAS_RESIDUE) {
            if (hilo) {
                rc = launch_mm_go<SRC, 1, true>(s, a, grid, lds);
                break;
            }
        }
        rc = launch_mm_go<SRC, 1>(s, a, grid, lds);
        break;
    case 2: rc = launch_mm_go<SRC, 2>(s, a, grid, lds); break;
    default: rc = launch_mm_go<SRC, 4>(s, a, grid, lds); break;
    }
    if (rc != OXQ_OK || pl.ks == 1) return rc;
    return launch_splitk_reduce(ctx, s, (const float *)ctx->workspace, a.bias, a.y, a.M, a.N, pl.ks, OXQ_BF16);
}

bool gguf_mm_eligible(const oxq_ctx *ctx, const GgufProblem &p) {
    const int min_m = tune(ctx, OXQ_TUNE_GGUF_MM_MIN_M, 3);  // measured 4096^2: m = 2 GEMV 9.1 / tile 10.6 us, m = 4 16.0 / 10.5
    return p.act_dtype == OXQ_BF16 && p.M >= min_m && ((uintptr_t)p.x & 15) == 0 && ((uintptr_t)p.w & 15) == 0 &&
           (p.K % 8) == 0;
}

int launch_gguf_mm(oxq_ctx *ctx, hipStream_t s, const GgufProblem &p) {
    int64_t be = 0, bb = 0;
    if (oxq_gguf_block_layout(p.quant, &be, &bb) != OXQ_OK) return OXQ_ERR_ARG;
    MmArgs a = {};
    a.x = (const uint16_t *)p.x, a.w = p.w, a.bias = (const uint16_t *)p.bias, a.y = (uint16_t *)p.y;
    a.M = (int)p.M, a.K = (int)p.K, a.N = (int)p.N;
    a.total_bytes = (size_t)p.N * (size_t)(p.K / be) * (size_t)bb;
    const bool hilo = p.M <= 8;  // the decode range (GgufQuantMatmul): weights are not rounded to bf16
#define OXQ_GG(F, NAME) \
    case F: return launch_mm_src<GgufSource<F>>(ctx, s, a, NAME, OXQ_TUNE_GGUF_MM_MT, OXQ_TUNE_GGUF_MM_KS, hilo)
    switch (p.quant) {
        OXQ_GG(OXQ_GGUF_Q4_0, "gguf_q4_0");
        OXQ_GG(OXQ_GGUF_Q8_0, "gguf_q8_0");
        OXQ_GG(OXQ_GGUF_Q4_K, "gguf_q4k");
        OXQ_GG(OXQ_GGUF_Q6_K, "gguf_q6k");
        OXQ_GG(OXQ_GGUF_Q4_1, "gguf_q4_1");
        OXQ_GG(OXQ_GGUF_Q5_0, "gguf_q5_0");
        OXQ_GG(OXQ_GGUF_Q5_1, "gguf_q5_1");
        OXQ_GG(OXQ_GGUF_Q2_K, "gguf_q2k");
        OXQ_GG(OXQ_GGUF_Q3_K, "gguf_q3k");
        OXQ_GG(OXQ_GGUF_Q5_K, "gguf_q5k");
    default: return OXQ_ERR_ARG;
    }
#undef OXQ_GG
}

// m > 8 (plain) / more routed pairs than the decode kernels are built for (grouped)
int launch_mxfp4_mm(oxq_ctx *ctx, hipStream_t s, const Mxfp4Problem &p) {
    const bool grouped = p.n_experts > 0;
    MmArgs a = {};
    a.x = (const uint16_t *)p.x, a.w = p.blocks, a.scales = p.scales, a.bias = (const uint16_t *)p.bias;
    a.y = (uint16_t *)p.y;
    a.M = (int)(grouped ? p.n_pairs : p.M), a.K = (int)p.K, a.N = (int)p.N;
    if (grouped) {
        a.offsets = p.expert_offsets, a.token_ids = p.token_ids, a.n_experts = (int)p.n_experts;
    }
    if (!ctx->plan_only && (((uintptr_t)p.blocks & 15) || ((uintptr_t)p.x & 15)))
        return fail(OXQ_ERR_UNSUPPORTED, "mxfp4 mul_mm: blocks and x must be 16-byte aligned");
    return launch_mm_src<Mxfp4Source>(ctx, s, a, grouped ? "mxfp4_moe" : "mxfp4", OXQ_TUNE_MXFP4_MM_MT, OXQ_TUNE_MXFP4_MM_KS);
}

bool f8_mm_eligible(const oxq_ctx *ctx, const F8Problem &p) {
    const int min_m = tune(ctx, OXQ_TUNE_F8_MM_MIN_M, 3);  // measured 4096^2 at m = 8: GEMV 19.9 us, tile matmul 11.5 us
    return p.M >= min_m && p.K % 32 == 0 && p.block_c % 32 == 0 && ((uintptr_t)p.x & 15) == 0 &&
           ((uintptr_t)p.w & 15) == 0;
}

int launch_f8_mm(oxq_ctx *ctx, hipStream_t s, const F8Problem &p) {
    MmArgs a = {};
    a.x = (const uint16_t *)p.x, a.w = p.w, a.y = (uint16_t *)p.y;
    a.M = (int)p.M, a.K = (int)p.K, a.N = (int)p.N;
    a.f8_scales = p.scales, a.f8_block_r = (int)p.block_r, a.f8_block_c = (int)p.block_c;
    a.f8_s_cols = (int)p.s_cols;
    return launch_mm_src<F8Source>(ctx, s, a, "f8", OXQ_TUNE_F8_MM_MT, OXQ_TUNE_F8_MM_KS);
}

}  // namespace oxq
