// GPTQ (pack_dim = in) layers on the checkpoint layout, any number of rows of x: the matrix-core
// kernel of the stateless gptq_matmul / mpp_quant_matmul ops (metal_ops.rs:2281-2303, 2748-2797;
// kernels quant_kernels.metal:3349-3499 and mpp_gemm.metal:84-266) without a repacked copy.
//
// The GPTQ word is already what a lane of v_mfma_f32_16x16x32 wants: qweight[K / pf][N] holds pf
// consecutive rows of K of ONE column, and a lane's B operand is 8 consecutive rows of K of one
// column.  A lane (ni = l % 16, kb = l / 16) loads 16 bytes = the words of columns 4 ni .. 4 ni + 3 of
// word row 4 t + kb (4-bit; rows 8 t + 2 kb and + 1 for 8-bit): 16 lanes cover 256 contiguous bytes
// of a word row, a wave load four (eight) such rows - whole 128-byte lines, the same number of loads
// as on the tile-major copy.  Column tile f of the MFMA is the lanes' word f.
//
// unpack4 pairs nibble i with nibble i + 4 (rows i and i + 4 of the word), bytes pair 0 with 2 and
// 1 with 3; a dot product does not care in which order its terms come as long as both operands agree,
// so the x block is put into LDS with the halves of every 16-byte chunk in that order (four
// v_perm_b32 a chunk, once a block) and the weights are never shuffled.
//
// Arithmetic: up to 32 rows (the reach of the reference's fused GEMV, linear.rs:450-480) the folded
// form, which never rounds a dequantized weight; above it B = T((q - (z + 1)) * s), bit-identical to the
// dense dequant (f16: exact packed add, one rounding in the packed multiply; bf16: exact f32 fma, one
// conversion), as the reference's staged GEMM rounds B.  f32 accumulation, the 8 waves' partial tiles
// added in wave order.  One workgroup a 64-column strip and 16 MT rows, the waves split K in contiguous
// runs of 128-row blocks: one launch, no workspace, deterministic.  Layers of few strips are also cut into
// K slices (grid.z), whose f32 partial tiles a second launch adds in slice order.

#include "pk4_common.hpp"

namespace oxq {

template <typename TT, int BITS> struct GptqDeq;
// f16: nibbles sit on 1024 (even positions) or 64 (odd), bytes on 1024; -(bias + z1) is exact
template <int BITS> struct GptqDeq<F16Traits, BITS> {
    uint32_t ce, co, cs;
    __device__ __forceinline__ void prep(uint32_t z1, uint32_t s16) {
        const uint32_t e = 0xE400u | z1, o = BITS == 4 ? (0xD400u | (z1 << 4)) : e;
        ce = e | (e << 16), co = o | (o << 16), cs = s16 | (s16 << 16);
    }
    __device__ __forceinline__ uint32_t deq(uint32_t p, int odd) const {
        return MfmaOps<F16Traits>::dequant_pair(p, odd ? co : ce, cs);
    }
};
// bf16: nibbles sit on 128, bytes on 0; fma(bias + q, s, -(bias + z1) s) in f32 is exact
template <int BITS> struct GptqDeq<BF16Traits, BITS> {
    float sf, c;
    __device__ __forceinline__ void prep(uint32_t z1, uint32_t s16) {
        sf = __builtin_bit_cast(float, s16 << 16);
        c = -((BITS == 4 ? 128.0f : 0.0f) + (float)z1) * sf;
    }
    __device__ __forceinline__ uint32_t deq(uint32_t p, int) const {
        const float lo = __builtin_fmaf(__builtin_bit_cast(float, p << 16), sf, c);
        const float hi = __builtin_fmaf(__builtin_bit_cast(float, p & 0xFFFF0000u), sf, c);
        return __builtin_bit_cast(uint32_t, __builtin_convertvector(float2_t{lo, hi}, bf16x2_t));
    }
};

template <typename TT, int BITS, int MT, int PER, int D, bool FOLD>
__global__ __launch_bounds__(512) void gptq_tile_kernel(const uint16_t *__restrict__ x, const uint32_t *__restrict__ qw,
                                                        const uint32_t *__restrict__ qz,
                                                        const uint16_t *__restrict__ sc,
                                                        const uint16_t *__restrict__ bias, uint16_t *__restrict__ y,
                                                        float *__restrict__ ws, int M, int K, int N, int gshift) {
    typedef MfmaOps<TT> Ops;
    constexpr int PF = 32 / BITS;     // rows of K a word
    constexpr int WL = BITS / 4;      // 16-byte loads a lane and MFMA step
    constexpr int XL = 2 * MT;        // 16-byte loads a lane and half block of x (64 rows of K)
    constexpr int STAGE = 16 * MT * 128;
    // One row tile in straight-line code: the wave's whole share of x is put into LDS before the first block
    // (2 PER stages a wave), requested ahead of the weights.  Otherwise x travels by half blocks through two
    // stages a wave, and every request for it queues behind the weights requested before it.
    constexpr bool XFRONT = MT == 1 && PER > 0;
    constexpr int NSTAGE = XFRONT ? 2 * PER : 2;
    constexpr uint32_t OOB = 0x80000000u;
    constexpr int WAUX = MT <= 2 ? 2 : 0;  // up to 32 rows one workgroup reads a strip's weights, once: nontemporal
    extern __shared__ __attribute__((aligned(16))) unsigned char pk4_lds[];

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int ni = lane & 15, kb = lane >> 4;
    const int j = blockIdx.x, m0 = blockIdx.y * 16 * MT;
    // K slices (grid.z; narrow layers): slice z owns blocks [z * NBS, (z + 1) * NBS) and writes an f32 partial tile
    const int NBT = K >> 7;
    const int NBS = (NBT + (int)gridDim.z - 1) / (int)gridDim.z;
    const int s0 = blockIdx.z * NBS;
    const int NB = s0 + NBS < NBT ? NBS : NBT - s0;   // blocks of this slice
    const int per = PER ? PER : (NB + 7) >> 3;  // PER: K / 128 = 8 PER, one slice (launcher)
    const int b0 = s0 + wave * per;
    const int b1 = b0 + per < s0 + NB ? b0 + per : s0 + NB;
    unsigned char *slot = pk4_lds + wave * NSTAGE * STAGE;

    const int wrow = N * 4;  // bytes a word row
    const __amdgpu_buffer_rsrc_t rs_w = make_rsrc(qw, (uint32_t)(K / PF) * (uint32_t)wrow);
    const __amdgpu_buffer_rsrc_t rs_z = make_rsrc(qz, (uint32_t)(K >> gshift) * (uint32_t)(N / PF) * 4u);
    const __amdgpu_buffer_rsrc_t rs_s = make_rsrc(sc, (uint32_t)(K >> gshift) * (uint32_t)N * 2u);
    // this workgroup's rows only: the descriptor's 32-bit size holds them whatever M is
    const int rows = M - m0 < 16 * MT ? M - m0 : 16 * MT;
    const __amdgpu_buffer_rsrc_t rs_x = make_rsrc(x + (size_t)m0 * K, (uint32_t)rows * (uint32_t)K * 2u);
    const uint32_t voff_w = (uint32_t)(kb * WL) * (uint32_t)wrow + (uint32_t)(64 * j + 4 * ni) * 4u;
    const uint32_t voff_s = (uint32_t)(64 * j + 4 * ni) * 2u;
    // the zero points of the lane's four columns lie in one word
    const uint32_t voff_z = BITS == 4 ? (uint32_t)(8 * j + (ni >> 1)) * 4u : (uint32_t)(16 * j + ni) * 4u;
    const int zsh = BITS == 4 ? 16 * (ni & 1) : 0;
    // x load i of a half block: rows 8 i .. 8 i + 7, 8 lanes a row (128 bytes: whole lines); rows past M lie
    // beyond the descriptor.  In LDS a row of a stage is 128 bytes, its 16-byte chunks xor-ed with bits 1..3 of
    // the row number: the row-wise writes and the fragment reads (16 rows x one chunk) are conflict-free.
    const int xrow = lane >> 3, xch = lane & 7;
    const uint32_t xo0 = (uint32_t)xrow * (uint32_t)K * 2u + (uint32_t)xch * 16u;
    const uint32_t xstep = (uint32_t)K * 16u;  // 8 rows
    const int a_rd = ni * 128;                  // fragment (mt, step u of the half): row 16 mt + ni, chunk 4 u + kb
    const NibbleMasks nm = nibble_masks();

    struct WB {
        u32x4_t q[4][WL];
        uint32_t z;
        uint32_t s[2];
    };
    auto load_w = [&](int b, WB &w) {
        // a block past the wave's share is requested beyond the descriptor: zeros, which add nothing
        const uint32_t live = b < b1 ? 0u : OOB;
        const int g = (b << 7) >> gshift;
#pragma unroll
        for (int t = 0; t < 4; ++t)
#pragma unroll
            for (int u = 0; u < WL; ++u)
                w.q[t][u] = __builtin_amdgcn_raw_buffer_load_b128(rs_w, (int)(voff_w + live + (uint32_t)u * wrow),
                                                                 ((b * 4 + t) * 4 * WL) * wrow, WAUX);
        w.z = __builtin_amdgcn_raw_buffer_load_b32(rs_z, (int)(voff_z + live), g * (N / PF) * 4, 0);
        const auto sv = __builtin_amdgcn_raw_buffer_load_b64(rs_s, (int)(voff_s + live), g * N * 2, 0);
        w.s[0] = sv[0], w.s[1] = sv[1];
    };
    u32x4_t xr[XL];
    auto load_x = [&](int b, int h) {
        const uint32_t live = b < b1 ? 0u : OOB;
#pragma unroll
        for (int i = 0; i < XL; ++i)
            xr[i] = __builtin_amdgcn_raw_buffer_load_b128(rs_x, (int)(xo0 + (uint32_t)i * xstep + live), b * 256 + h * 128, 0);
    };
    auto stage_x = [&](int h) {  // h: LDS stage
#pragma unroll
        for (int i = 0; i < XL; ++i) {
            const u32x4_t n = xr[i];
            u32x4_t o;
            if (BITS == 4) o = u32x4_t{pack_lo16(n[0], n[2]), pack_hi16(n[0], n[2]), pack_lo16(n[1], n[3]), pack_hi16(n[1], n[3])};
            else o = u32x4_t{pack_lo16(n[0], n[1]), pack_hi16(n[0], n[1]), pack_lo16(n[2], n[3]), pack_hi16(n[2], n[3])};
            // row 8 i + xrow: bits 1..3 of it are 4 (i & 1) | (xrow >> 1)
            *(u32x4_t *)(slot + h * STAGE + i * 1024 + xrow * 128 + ((xch ^ ((4 * (i & 1)) | (xrow >> 1))) << 4)) = o;
        }
    };

    float4_t acc[MT][4];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int f = 0; f < 4; ++f) acc[mt][f] = float4_t{0.f, 0.f, 0.f, 0.f};

    // Tile form (more than 32 rows): B = T((q - z1) s), the accumulators run over the whole of K.
    // Folded form (up to 32 rows, the reach of the reference's fused GEMV, which never rounds a dequantized
    // weight): the matrix cores multiply x by the exact integers bias + q, one more MFMA a step against a
    // fragment of ones gives the row sums of x in the accumulator layout (and one against the biases where
    // they differ by nibble position), and per block y += s (acc - (bias + z1) rowsum) in f32.
    constexpr bool TWO_BIASES = FOLD && BITS == 4 && TT::DTYPE == 1;
    constexpr float UBIAS = TWO_BIASES ? 0.0f : BITS == 4 ? 128.0f : TT::BYTE_BIAS;  // the bias every position shares
    GptqDeq<TT, BITS> dq[4];
    float sf[4], cb[4];
    float4_t blk[FOLD ? MT : 1][4], r0[FOLD ? MT : 1], r1[FOLD ? MT : 1];
    auto pairs = [&](const WB &w) {
#pragma unroll
        for (int f = 0; f < 4; ++f) {
            const uint32_t z1 = BITS == 4 ? ((w.z >> (zsh + 4 * f)) & 0xFu) + 1u : ((w.z >> (8 * f)) & 0xFFu) + 1u;
            const uint32_t s16 = (f & 1) ? (w.s[f >> 1] >> 16) : (w.s[f >> 1] & 0xFFFFu);
            if (FOLD) sf[f] = TT::to_f32((uint16_t)s16), cb[f] = (float)z1 + UBIAS;
            else dq[f].prep(z1, s16);
        }
        if (FOLD) {
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) {
                r0[mt] = r1[mt] = float4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int f = 0; f < 4; ++f) blk[mt][f] = float4_t{0.f, 0.f, 0.f, 0.f};
            }
        }
    };
    auto half = [&](const WB &w, int h, int st) {  // half h of the block, in LDS stage st
#pragma unroll
        for (int u = 0; u < 2; ++u) {
            const int t = 2 * h + u;
            uint32_t a[MT][4];
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) {
                const u32x4_t av = *(const u32x4_t *)(slot + st * STAGE + mt * 2048 + a_rd + ((((4 * u + kb) ^ (ni >> 1)) & 7) << 4));
                a[mt][0] = av[0], a[mt][1] = av[1], a[mt][2] = av[2], a[mt][3] = av[3];
            }
            if (FOLD) {
                const uint32_t ones[4] = {TT::ONES, TT::ONES, TT::ONES, TT::ONES};
                const uint32_t biases[4] = {0x64006400u, 0x54005400u, 0x64006400u, 0x54005400u};  // f16 1024, 64 (unpack4)
#pragma unroll
                for (int mt = 0; mt < MT; ++mt) {
                    r0[mt] = Ops::mfma(a[mt], ones, r0[mt]);
                    if (TWO_BIASES) r1[mt] = Ops::mfma(a[mt], biases, r1[mt]);
                }
            }
#pragma unroll
            for (int f = 0; f < 4; ++f) {
                uint32_t bq[4];
                if (BITS == 4) {
                    uint32_t p[4];
                    TT::unpack4(w.q[t][0][f], p, nm);
#pragma unroll
                    for (int i = 0; i < 4; ++i) bq[i] = FOLD ? p[i] : dq[f].deq(p[i], i & 1);
                } else {
#pragma unroll
                    for (int v = 0; v < 2; ++v) {
                        const uint32_t wd = w.q[t][v % WL][f];
                        const uint32_t lo = TT::unpack_bytes(wd), hi = TT::unpack_bytes(wd >> 8);
                        bq[2 * v] = FOLD ? lo : dq[f].deq(lo, 0);
                        bq[2 * v + 1] = FOLD ? hi : dq[f].deq(hi, 0);
                    }
                }
#pragma unroll
                for (int mt = 0; mt < MT; ++mt) {
                    if (FOLD) blk[mt][f] = Ops::mfma(a[mt], bq, blk[mt][f]);
                    else acc[mt][f] = Ops::mfma(a[mt], bq, acc[mt][f]);
                }
            }
        }
    };
    auto fold = [&]() {
        if (!FOLD) return;
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
            for (int f = 0; f < 4; ++f)
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const float corr = TWO_BIASES ? __builtin_fmaf(cb[f], r0[mt][e], r1[mt][e]) : cb[f] * r0[mt][e];
                    acc[mt][f][e] = __builtin_fmaf(sf[f], blk[mt][f][e] - corr, acc[mt][f][e]);
                }
    };
    // one block: its first half of x is in the x registers and its weights in w; block bn (D - 1 further on)
    // is requested into wn, the register set of the block before this one
    auto block = [&](int b, const WB &w, int bn, WB &wn, bool more) {
        stage_x(0);
        load_x(b, 1);
        if (more) load_w(bn, wn);
        __builtin_amdgcn_sched_barrier(0);  // requests stay where they are written (the scheduler sinks them to their use)
        pairs(w);
        half(w, 0, 0);
        stage_x(1);
        load_x(b + 1, 0);
        __builtin_amdgcn_sched_barrier(0);
        half(w, 1, 1);
        fold();
    };
    // the same with x already in LDS: block i of the wave's share sits in stages 2 i and 2 i + 1
    auto block_xfront = [&](int i, const WB &w, int bn, WB &wn, bool more) {
        if (more) load_w(bn, wn);
        __builtin_amdgcn_sched_barrier(0);
        pairs(w);
        half(w, 0, 2 * i);
        half(w, 1, 2 * i + 1);
        fold();
    };

    // D register sets of weights in a ring, D - 1 blocks requested ahead.
    WB w[D];
    if (XFRONT) {
        // x of the whole share first (the vector-memory counter runs in issue order: what is needed first is
        // requested first), then the weights; x is in LDS by the time the first block's weights arrive
        u32x4_t xa[NSTAGE][XL];
#pragma unroll
        for (int st = 0; st < NSTAGE; ++st)
#pragma unroll
            for (int i = 0; i < XL; ++i)
                xa[st][i] = __builtin_amdgcn_raw_buffer_load_b128(rs_x, (int)(xo0 + (uint32_t)i * xstep), (b0 * 2 + st) * 128, 0);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int i = 0; i < D - 1 && i < PER; ++i) load_w(b0 + i, w[i]);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int st = 0; st < NSTAGE; ++st) {
#pragma unroll
            for (int i = 0; i < XL; ++i) xr[i] = xa[st][i];
            stage_x(st);
        }
#pragma unroll
        for (int i = 0; i < PER; ++i) block_xfront(i, w[i % D], b0 + i + D - 1, w[(i + D - 1) % D], i + D - 1 < PER);
    } else if (PER) {
        // K = 8 PER blocks: straight-line code, every wave PER blocks; D = PER requests a wave's whole share
        // before it waits for any of it
        load_x(b0, 0);
#pragma unroll
        for (int i = 0; i < D - 1 && i < PER; ++i) load_w(b0 + i, w[i]);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int i = 0; i < PER; ++i) block(b0 + i, w[i % D], b0 + i + D - 1, w[(i + D - 1) % D], i + D - 1 < PER);
    } else if (b0 < b1) {
        // any K: a loop whose body is D blocks, so that every set keeps its registers (a rotating ring would
        // be copied at the loop's end, and a copy waits for the load behind it); blocks past the share
        // are zeros
        load_x(b0, 0);
#pragma unroll
        for (int i = 0; i < D - 1; ++i) load_w(b0 + i, w[i]);
        for (int b = b0; b < b1; b += D) {
#pragma unroll
            for (int i = 0; i < D; ++i) block(b + i, w[i], b + i + D - 1, w[(i + D - 1) % D], true);
        }
    }
    __syncthreads();  // the partial tiles go where other waves' x stages were
    pk4_epilogue_lanes<TT, MT>(acc, bias, y, M, N, j, m0, wave, lane,
                               gridDim.z > 1 ? ws + (size_t)blockIdx.z * M * N : nullptr);
}

// 128-row blocks inside one quantization group, 64-column strips, 32-bit buffer offsets, 16-byte rows
bool gptq_tile_ok(const Wna16Problem &p) {
    if ((p.bits != 4 && p.bits != 8) || p.pack_dim != OXQ_PACK_IN) return false;
    if (p.K % 128 != 0 || p.N % 64 != 0 || p.group_size % 128 != 0 || !is_pow2(p.group_size)) return false;
    if (((uintptr_t)p.qweight | (uintptr_t)p.x | (uintptr_t)p.y) & 15) return false;
    if (((uintptr_t)p.scales | (uintptr_t)p.bias) & 7) return false;
    if ((uint64_t)(p.K * p.bits / 32) * (uint64_t)p.N * 4 >= (1ull << 31)) return false;
    if ((uint64_t)(p.M < 64 ? p.M : 64) * (uint64_t)p.K * 2 >= (1ull << 31)) return false;
    return true;
}

template <typename TT, int BITS, int MT, int PER, int D>
static int gptq_tile_go(hipStream_t s, dim3 grid, const Wna16Problem &p, float *ws) {
    constexpr bool FOLD = MT <= 2;
    // 8 partial tiles of 16 MT x 64 f32; the x stages are as large, or 2 PER stages of 2 KB a wave when x goes first
    const size_t lds = MT == 1 && PER > 2 ? (size_t)8 * 2 * PER * 2048 : (size_t)8 * MT * 4096;
    static LdsGrant lds_grant;
    OXQ_HIP_CHECK(lds_grant.ensure((const void *)gptq_tile_kernel<TT, BITS, MT, PER, D, FOLD>, lds));
    hipLaunchKernelGGL((gptq_tile_kernel<TT, BITS, MT, PER, D, FOLD>), grid, dim3(512), lds, s, (const uint16_t *)p.x, p.qweight,
                       p.qzeros, (const uint16_t *)p.scales, (const uint16_t *)p.bias, (uint16_t *)p.y, ws, (int)p.M,
                       (int)p.K, (int)p.N, p.group_shift);
    OXQ_HIP_CHECK(hipGetLastError());
    return OXQ_OK;
}

// Weight ring: as deep as the registers beside the accumulators and the x half block allow.  K = 4096 and
// 5120 (4 or 5 blocks a wave) run as straight-line code.
template <typename TT, int BITS, int MT>
static int gptq_tile_per(hipStream_t s, dim3 grid, int per, const Wna16Problem &p, float *ws) {
    constexpr bool f16 = TT::DTYPE == 1;
    constexpr int DMAX = BITS == 4 ? (MT == 1 ? 5 : MT == 2 ? 4 : 2) : (MT == 1 ? (f16 ? 4 : 3) : MT == 2 ? 3 : 2);
    if (per == 4) return gptq_tile_go<TT, BITS, MT, 4, (DMAX < 4 ? DMAX : 4)>(s, grid, p, ws);
    if (per == 5) return gptq_tile_go<TT, BITS, MT, 5, (DMAX < 5 ? DMAX : 5)>(s, grid, p, ws);
    return gptq_tile_go<TT, BITS, MT, 0, 2>(s, grid, p, ws);
}

template <typename TT, int BITS>
static int gptq_tile_mt(hipStream_t s, dim3 grid, int mt, const Wna16Problem &p, float *ws) {
    const int64_t NB = p.K / 128;
    const int per = grid.z == 1 && NB % 8 == 0 ? (int)(NB / 8) : 0;  // straight-line code: one slice of 32 or 40 blocks
    switch (mt) {
    case 1: return gptq_tile_per<TT, BITS, 1>(s, grid, per, p, ws);
    case 2: return gptq_tile_per<TT, BITS, 2>(s, grid, per, p, ws);
    default: return gptq_tile_per<TT, BITS, 4>(s, grid, per, p, ws);
    }
}

// K slices for a layer of few strips: as many as bring the launch to about one workgroup a CU, at least
// 8 blocks (one a wave) each; their f32 partial tiles are added in slice order by a second launch.
int gptq_tile_slices(const oxq_ctx *ctx, const Wna16Problem &p) {
    const int mt = p.M > 32 ? 4 : (int)((p.M + 15) / 16);
    const int64_t tiles = (p.N / 64) * ceil_div(p.M, 16 * mt), NB = p.K / 128;
    int ks = 1;
    if (tiles <= 96 && NB >= 32) ks = (int)std::max<int64_t>(1, std::min<int64_t>(256 / tiles, NB / 8));
    else if (tiles <= 128 && NB >= 64) ks = 2;  // half a round of workgroups and a long K
    ks = tune(ctx, OXQ_TUNE_GPTQ_TILE_KS, ks);
    return (int)std::max<int64_t>(1, std::min<int64_t>(ks, NB));
}

int launch_gptq_tile(oxq_ctx *ctx, hipStream_t s, const Wna16Problem &p) {
    const int mt = p.M > 32 ? 4 : (int)((p.M + 15) / 16);  // three row tiles run as four (their sum divides over 8 waves)
    const int ks = gptq_tile_slices(ctx, p);
    dim3 grid((unsigned)(p.N / 64), (unsigned)ceil_div(p.M, 16 * mt), (unsigned)ks);
    const size_t ws_bytes = ks > 1 ? (size_t)ks * p.M * p.N * 4 : 0;
    char name[64];
    snprintf(name, sizeof name, "gptq%d_tile_%s_mt%d", p.bits, p.dtype == OXQ_F16 ? "f16" : "bf16", mt);
    set_plan(ctx, name, grid, dim3(512), ks, 1, ws_bytes);
    if (ctx->plan_only) {
        if (ks > 1) add_launch(ctx);
        return OXQ_OK;
    }
    if (ws_bytes > ctx->workspace_bytes)
        return fail(OXQ_ERR_WORKSPACE, "gptq tile: %d K slices need %zu workspace bytes, ctx holds %zu", ks, ws_bytes,
                    ctx->workspace_bytes);
    float *ws = (float *)ctx->workspace;
    const bool f16 = p.dtype == OXQ_F16;
    int rc;
    if (p.bits == 4) rc = f16 ? gptq_tile_mt<F16Traits, 4>(s, grid, mt, p, ws) : gptq_tile_mt<BF16Traits, 4>(s, grid, mt, p, ws);
    else rc = f16 ? gptq_tile_mt<F16Traits, 8>(s, grid, mt, p, ws) : gptq_tile_mt<BF16Traits, 8>(s, grid, mt, p, ws);
    if (rc != OXQ_OK || ks == 1) return rc;
    return launch_splitk_reduce(ctx, s, ws, p.bias, p.y, p.M, p.N, ks, p.dtype);
}

}  // namespace oxq
