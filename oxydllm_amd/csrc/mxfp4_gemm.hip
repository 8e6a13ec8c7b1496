// Resident MXFP4 experts at prefill sizes (moe.rs:563-607 runs every expert's tokens through its projections;
// mxfp4.rs:119-154 is the layer): the decomposition of pk4n_gemm_kernel on the tile-major expert copy.
//
// The copy (mxfp4_repack_kernel) stores a tile of 16 weight rows as chunks of 1 KB - 128 elements of K, lane
// (ni, kb) the 16 bytes of block 4 c + kb of row ni, whose four words are the chunk's four MFMA steps - which is
// the shape of a block of the 16-column AWQ layout.  So a workgroup takes 64 rows of one expert's pairs and, a wave,
// four neighbouring tiles (64 weight rows = 64 columns of y): the pairs' rows of x come from global memory straight
// into LDS (gathered through the token list, a chunk of K at a time, two buffers, one barrier a chunk), every wave
// streams its tiles through a ring of two chunks, turns a word into an MFMA B fragment with four
// v_cvt_scalef32_pk_bf16_fp4 (the values are exact in bf16, so this is the tile matmul's B) and keeps the whole K in
// its accumulators.  Row tiles of 16 MT rows: 16 or 32 where an expert has few pairs (the weights are then read once
// per tile and most of a 64-row tile would be empty rows), 64, and 128 at long prefills.  (The K split inside the
// workgroup that serves AWQ layers at mid sizes was slower than this form at every pair count: with 32 experts there
// are always enough workgroups, and the stream of weights is what a short launch waits for.)
#include "oxq_device.hpp"
#include "oxq_internal.hpp"
#include "oxq_mfma.hpp"
#include "pk4_common.hpp"

#include <type_traits>

namespace oxq {

constexpr int MXG_WAVES = 8;

template <int MT>
__global__ __launch_bounds__(512) void mxfp4_gemm_kernel(const uint16_t *__restrict__ x, const unsigned char *__restrict__ pw,
                                                         const unsigned char *__restrict__ ps, const uint16_t *__restrict__ bias,
                                                         uint16_t *__restrict__ y, const int32_t *__restrict__ offsets,
                                                         const int32_t *__restrict__ token_ids, int K, int N, int NC, int NG,
                                                         int E, uint32_t x_bytes, int swiglu, float limit) {
    typedef MfmaOps<BF16Traits> Ops;
    constexpr int ROWS = 16 * MT, XBUF = ROWS * 256;
    constexpr int XV = ROWS >= 32 ? ROWS / 32 : 1;  // loads of x a wave issues per chunk: 4 rows each (16 rows: waves 0..3 only)
    constexpr int OOB = 0x7FFFFF00;
    extern __shared__ __attribute__((aligned(16))) unsigned char mxg_lds[];

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int ni = lane & 15, kb = lane >> 4;
    // blockIdx.y -> (expert, row tile of its pairs); all values workgroup-uniform
    int rem = blockIdx.y, e = 0;
    for (; e < E; ++e) {
        const int tiles = (offsets[e + 1] - offsets[e] + ROWS - 1) / ROWS;
        if (rem < tiles) break;
        rem -= tiles;
    }
    if (e == E) return;  // the whole workgroup, before any barrier
    const int m0 = offsets[e] + rem * ROWS, m_end = offsets[e + 1];
    const int j = (int)blockIdx.x * MXG_WAVES + wave;  // the wave's 64 columns: tiles 4 j .. 4 j + 3
    const int ntiles = N >> 4, nb = K >> 5;
    const int live_tiles = min(4, ntiles - 4 * j);  // wave-uniform; <= 0: a wave past the last tile
    const bool live = live_tiles > 0;

    const size_t et = (size_t)e * ntiles + (live ? 4 * j : 0);
    const __amdgpu_buffer_rsrc_t rs_w = make_rsrc(pw + et * nb * 256, live ? (uint32_t)live_tiles * (uint32_t)nb * 256u : 0u);
    const __amdgpu_buffer_rsrc_t rs_s = make_rsrc(ps + et * NG * 256, live ? (uint32_t)live_tiles * (uint32_t)NG * 256u : 0u);
    const __amdgpu_buffer_rsrc_t rs_x = make_rsrc(x, x_bytes);
    const int voff_w = lane * 16, voff_s = lane * 4;
    // x: load q of a wave brings rows 4 (XV wave + q) .. + 3 of a chunk straight into LDS, lane l the 16 bytes that
    // belong at position l % 16 of row l / 16.  Piece p = 4 kb + st of a row's 128 elements (what lane group kb reads
    // in step st) is kept at position (4 st + kb) ^ (row % 16): the four lane groups of a fragment read then start in
    // different banks (at position p ^ row, groups 0 and 2 would meet 128 bytes apart: four conflict cycles a read).
    // Rows past the expert's pairs, and the elements past K in the last chunk, get an offset beyond the descriptor:
    // LDS receives zeros.
    int xo[XV], xc[XV];
#pragma unroll
    for (int q = 0; q < XV; ++q) {
        const int r = 4 * (wave * XV + q) + (lane >> 4);
        const int m = m0 + r;
        const int pos = (lane & 15) ^ (r & 15);
        xc[q] = ((pos & 3) << 2) | (pos >> 2);  // the piece kept at this position
        int src = 0;
        if (m < m_end) src = token_ids ? token_ids[m] : m;
        xo[q] = m < m_end ? src * K * 2 + (xc[q] << 4) : OOB;
    }
    // fragment of step st, row tile mt (+ 4096 mt): row ni, elements 32 kb + 8 st .. + 7 of the chunk = piece 4 kb + st
    int a_rd[4];
#pragma unroll
    for (int st = 0; st < 4; ++st) a_rd[st] = ni * 256 + (((4 * st + kb) ^ ni) << 4);

    u32x4_t wring[2][4];
    uint32_t sring[4];
    const bool loads_x = 4 * wave * XV < ROWS;  // wave-uniform
    auto dma_x = [&](int c) {
        const int lim = (K - c * 128) >> 3;  // 16-byte pieces of the row left in this chunk (<= 0 past the row)
        if (!loads_x) return;
#pragma unroll
        for (int q = 0; q < XV; ++q)
            pk4g_load_lds16(rs_x, mxg_lds + (c & 1) * XBUF + (wave * XV + q) * 1024, xc[q] < lim ? xo[q] : OOB, c * 256);
    };
    // blocks past the row, and tiles past the layer's last, lie beyond the tile but not beyond what the range check
    // looks at (the lane's offset, not the scalar one): the lane carries an offset that is
    auto load_w = [&](int c, u32x4_t (&w)[4]) {
        const int vo = 4 * c + kb < nb ? voff_w : OOB;
#pragma unroll
        for (int f = 0; f < 4; ++f) w[f] = __builtin_amdgcn_raw_buffer_load_b128(rs_w, f < live_tiles ? vo : OOB, f * nb * 256 + c * 1024, 0);
    };
    auto load_s = [&](int c) {
        const int vo = c < NC ? voff_s : OOB;
#pragma unroll
        for (int f = 0; f < 4; ++f) sring[f] = __builtin_amdgcn_raw_buffer_load_b32(rs_s, f < live_tiles ? vo : OOB, (f * NG + (c >> 2)) * 256, 0);
    };

    dma_x(0);
    __builtin_amdgcn_sched_barrier(0);  // requests keep this order: the wait counts rely on it
    load_s(0);
    load_w(0, wring[0]);
    __builtin_amdgcn_sched_barrier(0);
    float4_t acc[MT][4];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int f = 0; f < 4; ++f) acc[mt][f] = float4_t{0.f, 0.f, 0.f, 0.f};
    pk4g_wait_vmcnt<8>();
    __syncthreads();

    // one chunk, its weights in ring half CUR; eight ring loads are younger than the chunk's loads of x
    auto round = [&](int c, auto cur_c) {
        constexpr int CUR = decltype(cur_c)::value;
        dma_x(c + 1);
        __builtin_amdgcn_sched_barrier(0);
        load_w(c + 1, wring[CUR ^ 1]);
        __builtin_amdgcn_sched_barrier(0);
        const unsigned char *buf = mxg_lds + (c & 1) * XBUF;
        float scale[4];
#pragma unroll
        for (int f = 0; f < 4; ++f) scale[f] = e8m0_to_f32((sring[f] >> (8 * (c & 3))) & 0xFFu);
        load_s(c + 1);
#pragma unroll
        for (int st = 0; st < 4; ++st) {
            // four row tiles at a time: at 128 rows the fragments of all eight beside the accumulators do not fit the
            // registers, and a B fragment is four conversions to make again
            constexpr int MH = MT < 4 ? MT : 4;
#pragma unroll
            for (int h = 0; h < MT; h += MH) {
                uint32_t a[MH][4];
#pragma unroll
                for (int mt = 0; mt < MH; ++mt) {
                    const u32x4_t av = *(const u32x4_t *)(buf + (h + mt) * 4096 + a_rd[st]);
                    a[mt][0] = av[0], a[mt][1] = av[1], a[mt][2] = av[2], a[mt][3] = av[3];
                }
#pragma unroll
                for (int f = 0; f < 4; ++f) {
                    const uint32_t w = wring[CUR][f][st];
                    uint32_t b[4];
                    b[0] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(w, scale[f], 0));
                    b[1] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(w, scale[f], 1));
                    b[2] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(w, scale[f], 2));
                    b[3] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(w, scale[f], 3));
#pragma unroll
                    for (int mt = 0; mt < MH; ++mt) acc[h + mt][f] = Ops::mfma(a[mt], b, acc[h + mt][f]);
                }
            }
        }
        __builtin_amdgcn_sched_barrier(0);
        pk4g_wait_vmcnt<8>();  // this wave's part of the next chunk of x is in LDS
        __syncthreads();
    };
    {
        int c = 0;
        for (; c + 1 < NC; c += 2) {
            round(c, std::integral_constant<int, 0>{});
            round(c + 1, std::integral_constant<int, 1>{});
        }
        if (c < NC) round(c, std::integral_constant<int, 0>{});
    }

    if (!live) return;
    // lane (ni, kb), value i of acc[t][f]: pair m0 + 16 t + 4 kb + i, weight row 64 j + 16 f + ni
    float bv[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int f = 0; f < 4; ++f)
        if (bias && f < live_tiles) bv[f] = BF16Traits::to_f32(bias[(size_t)e * N + 64 * j + 16 * f + ni]);
    // Neighbouring lanes hold neighbouring weight rows: the two lanes of a pair exchange their values (quad_perm
    // [1, 0, 3, 2]) and share the work - the even lane finishes pairs i = 0 and 2 of the four, the odd lane 1 and 3.
    const bool odd = ni & 1;
#pragma unroll
    for (int t = 0; t < MT; ++t)
#pragma unroll
        for (int f = 0; f < 4; ++f) {
            const int n = 64 * j + 16 * f + (ni & ~1);  // the lane pair's two weight rows: n, n + 1
            float mine[4], other[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                // rounded to bf16 as the projection's own output is (for the SwiGLU: what it would read)
                mine[i] = BF16Traits::to_f32(BF16Traits::from_f32(acc[t][f][i] + bv[f]));
                other[i] = __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, mine[i]), 0xB1, 0xF, 0xF, false));
            }
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                const int i = 2 * h + (odd ? 1 : 0);
                const int m = m0 + 16 * t + 4 * kb + i;
                const float lo = odd ? other[2 * h + 1] : mine[2 * h], hi = odd ? mine[2 * h + 1] : other[2 * h];  // rows n, n + 1
                if (m >= m_end || f >= live_tiles) continue;
                if (swiglu) {
                    // rows 2 c / 2 c + 1 are the gate / up of output c (moe.rs:152-173)
                    y[(size_t)m * (N >> 1) + (n >> 1)] = BF16Traits::from_f32(gpt_oss_swiglu_f32(lo, hi, limit));
                } else {
                    *(uint32_t *)(y + (size_t)m * N + n) = (uint32_t)BF16Traits::from_f32(lo) | ((uint32_t)BF16Traits::from_f32(hi) << 16);
                }
            }
        }
}

// Takes the grouped problem from three pairs an expert on average (below, the decode kernel's passes of four tokens
// read the weights once): 0 = not taken, else the rows of a tile.  The pairs of an expert are only known on the
// device, so the tile follows the average: small tiles waste fewer empty rows on experts with few pairs and, at two
// workgroups a CU, hide more latency; large tiles read the weights less often.  32 experts x (5760 + 2880) x 2880,
// tokens with top-4 of random logits, gate_up + down in us by tile rows 16 / 32 / 64 / 128:
//   128 pairs 77 / 85 / 125 / 211      512 pairs 124 / 90 / 129 / 214     2048 pairs 237 / 179 / 218 / 225
//   4096 pairs 365 / 298 / 287 / 373   8192 pairs 651 / 489 / 506 / 475   16384 pairs 1268 / 926 / 934 / 879
int mxfp4_gemm_form(const oxq_ctx *ctx, int64_t n_pairs, int64_t E, int64_t K, int64_t N) {
    const int64_t min_pairs = tune(ctx, OXQ_TUNE_MXFP4_GEMM_MIN_PAIRS, 3);
    if (min_pairs <= 0 || E <= 0 || n_pairs < min_pairs * E || N % 16 != 0 || K % 32 != 0) return 0;
    const int forced = tune(ctx, OXQ_TUNE_MXFP4_GEMM_ROWS, 0);
    if (forced == 16 || forced == 32 || forced == 64 || forced == 128) return forced;
    const int64_t avg = n_pairs / E;
    return avg <= 12 ? 16 : avg < 96 ? 32 : avg < 200 ? 64 : 128;
}

template <int MT>
static int mxfp4_gemm_go(hipStream_t s, dim3 grid, const Mxfp4Problem &p, int NC, int NG, uint32_t x_bytes) {
    static LdsGrant grant;  // one per instantiation
    const size_t lds = (size_t)2 * 16 * MT * 256;
    OXQ_HIP_CHECK(grant.ensure((const void *)mxfp4_gemm_kernel<MT>, lds));
    hipLaunchKernelGGL((mxfp4_gemm_kernel<MT>), grid, dim3(512), lds, s, (const uint16_t *)p.x, (const unsigned char *)p.blocks,
                       (const unsigned char *)p.scales, (const uint16_t *)p.bias, (uint16_t *)p.y, p.expert_offsets, p.token_ids,
                       (int)p.K, (int)p.N, NC, NG, (int)p.n_experts, x_bytes, p.swiglu, p.swiglu_limit);
    OXQ_HIP_CHECK(hipGetLastError());
    return OXQ_OK;
}

// p.blocks / p.scales hold the resident copy; grouped form only; p.M = rows of x
int launch_mxfp4_res_gemm(oxq_ctx *ctx, hipStream_t s, const Mxfp4Problem &p) {
    const int rows = mxfp4_gemm_form(ctx, p.n_pairs, p.n_experts, p.K, p.N);
    if (rows == 0) return fail(OXQ_ERR_UNSUPPORTED, "mxfp4 experts prefill: shape not taken");
    const int nb = (int)(p.K / 32), NC = (int)ceil_div(nb, 4), NG = (int)ceil_div(NC, 4);
    // sum over experts of ceil(pairs_e / rows) <= pairs / rows + experts
    const int64_t ytiles = p.n_pairs / rows + p.n_experts;
    if (ytiles > 65535) return fail(OXQ_ERR_UNSUPPORTED, "mxfp4 experts prefill: %lld row tiles exceed the grid limit of 65535", (long long)ytiles);
    dim3 grid((unsigned)ceil_div(p.N / 16, (int64_t)4 * MXG_WAVES), (unsigned)ytiles);
    char name[64];
    snprintf(name, sizeof name, "mxfp4_experts_gemm_bf16_r%dx8%s", rows, p.swiglu ? "_swiglu" : "");
    set_plan(ctx, name, grid, dim3(512), 1, 1, 0);
    if (ctx->plan_only) return OXQ_OK;
    const uint64_t x_bytes = (uint64_t)p.M * (uint64_t)p.K * 2u;
    if (x_bytes >= (1ull << 31)) return fail(OXQ_ERR_UNSUPPORTED, "mxfp4 experts prefill: x of %llu bytes exceeds 2 GiB", (unsigned long long)x_bytes);
    if ((uintptr_t)p.x & 15) return fail(OXQ_ERR_UNSUPPORTED, "mxfp4 experts prefill: x must be 16-byte aligned");
    if ((uintptr_t)p.y & 3) return fail(OXQ_ERR_UNSUPPORTED, "mxfp4 experts prefill: out must be 4-byte aligned");
    switch (rows) {
    case 16: return mxfp4_gemm_go<1>(s, grid, p, NC, NG, (uint32_t)x_bytes);
    case 32: return mxfp4_gemm_go<2>(s, grid, p, NC, NG, (uint32_t)x_bytes);
    case 64: return mxfp4_gemm_go<4>(s, grid, p, NC, NG, (uint32_t)x_bytes);
    default: return mxfp4_gemm_go<8>(s, grid, p, NC, NG, (uint32_t)x_bytes);
    }
}

}  // namespace oxq
