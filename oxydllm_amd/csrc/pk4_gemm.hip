// Resident layers at prefill sizes (linear.rs:494-509: m >= 64 takes the staged tile GEMM,
// mpp_gemm.metal:101-266): the tile arithmetic of pk4_mfma_kernel - B = T((q - z) * s) rounded once to the
// activation type, f32 accumulate - in a decomposition for many rows.
//
// pk4_mfma_kernel gives a workgroup one strip of 64 columns and 64 rows of x, and its 8 waves split K: every
// (row tile, strip) pair reads its 64 rows of x again, each wave for itself through the vector-memory unit.
// At 2048 rows of a 4096 x 14336 layer that is 7168 workgroups x 512 KB = 3.7 GB of activations out of L2 for
// 16.8 MB of x, and the kernel runs at the speed it has at 64 rows (0.6 PFLOP/s).  Here a workgroup takes 64
// rows and EIGHT strips: its waves share one copy of the rows in LDS (a block of 128 elements of K at a time,
// loaded from global memory straight into LDS - no registers, nothing for the compiler to sink behind the
// arithmetic - two buffers, one barrier a block), each wave owns a strip, streams its blocks with the
// one-block ring of pk4_mfma_kernel and keeps the whole K in its own accumulators - no partial tiles, no
// second launch.  x out of L2 falls to an eighth.  Workgroups are numbered so that 64 neighbours form a square
// of 8 row tiles x 8 strip groups, whose rows of x and weights the neighbours find in L2.
#include "oxq_device.hpp"
#include "oxq_internal.hpp"
#include "oxq_mfma.hpp"
#include "pk4_common.hpp"

#include <algorithm>
#include <cmath>
#include <type_traits>

namespace oxq {

constexpr int PK4G_STRIPS = 8;  // strips (= waves) of a workgroup

// KS = 1: eight strips a workgroup, a wave takes every block of its strip.  KS = 4 (the form for 65 to a few hundred
// rows, where workgroups of eight strips are too few to fill the chip): two strips a workgroup, the four waves of
// a strip take every fourth block; a round brings four blocks of x into LDS, each loaded by the two waves that use
// it; at the end the waves' partial tiles meet in LDS (where x was) and wave kq of a strip finishes row tile kq,
// adding the four partials in K order - the epilogue then runs on the accumulator layout as for KS = 1.
template <typename TT, int MT, int BITS, int KS>
__global__ __launch_bounds__(512) void pk4_gemm_kernel(const uint16_t *__restrict__ x, const uint32_t *__restrict__ pw,
                                                       const uint16_t *__restrict__ bias, uint16_t *__restrict__ y,
                                                       int M, int K, int N, int NG, int RT, int act) {
    typedef MfmaOps<TT> Ops;
    static_assert(KS == 1 || KS == MT, "wave kq of a strip finishes row tile kq");
    constexpr int SPW = PK4G_STRIPS / KS;  // strips a workgroup
    constexpr int ROWS = 16 * MT, BB = pk4_block_words(BITS) * 4, XBUF = KS * ROWS * 256;
    constexpr int WL = BITS / 4;          // 1 KB weight loads a step (8-bit: column pairs 0, 1 and 2, 3)
    constexpr int RING = 4 * WL + 1;      // ring loads of a block: younger than the block's loads of x
    constexpr bool BF = TT::DTYPE == BF16Traits::DTYPE;
    constexpr int XV = ROWS / 4 / SPW;  // loads of x a wave issues per round: 64 lanes x 16 bytes = 4 rows each
    extern __shared__ __attribute__((aligned(16))) unsigned char pk4_lds[];

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int ni = lane & 15, kb = lane >> 4;
    const int ws = wave % SPW, kq = wave / SPW;  // the wave's strip of the workgroup, and its share of K
    int rt, g;
    if constexpr (KS == 1) {
        pk4g_tile_of((int)blockIdx.x, RT, NG, rt, g);
        if (g >= NG) return;  // the whole workgroup, before any barrier: the ragged last column of squares
    } else {
        // a row tile's strip groups are neighbours: the eight XCDs share its rows of x, and with NG a multiple of 8
        // the row tiles of a strip group meet on one XCD, whose L2 then holds the group's weights
        rt = (int)blockIdx.x / NG, g = (int)blockIdx.x % NG;
    }
    const int j = g * SPW + ws;
    const bool live = j < (N >> 6);  // wave-uniform: the last group of a layer may have fewer strips
    const int m0 = rt * ROWS;
    const int NB = K >> 7, NR = (NB + KS - 1) / KS;  // blocks; rounds of KS blocks
    const int xrows = min(M - m0, ROWS);

    const __amdgpu_buffer_rsrc_t rs_none = make_rsrc(pw, 0u);
    const __amdgpu_buffer_rsrc_t rs_wl = make_rsrc(pw + (size_t)(live ? j : 0) * NB * (BB / 4), (uint32_t)NB * (uint32_t)BB);
    const __amdgpu_buffer_rsrc_t rs_w = live ? rs_wl : rs_none;
    const __amdgpu_buffer_rsrc_t rs_x = make_rsrc(x + (size_t)m0 * K, (uint32_t)xrows * (uint32_t)K * 2u);
    const int voff_w = lane * 16;
    const int voff_z = 1024 * WL * 4 + (ni * 4 + kb) * 4;
    // x: load q of a wave brings rows 4 (XV ws + q) .. + 3 of the wave's block of the round straight into LDS, lane l
    // the 16 bytes that belong at position l % 16 of row l / 16 - chunk (l % 16) ^ (row % 16) of the row, the
    // swizzle the fragment reads undo.  Rows past M lie beyond the descriptor: LDS receives zeros.
    int xo[XV];
#pragma unroll
    for (int q = 0; q < XV; ++q) {
        const int r = 4 * (ws * XV + q) + (lane >> 4);
        xo[q] = r * K * 2 + (((lane & 15) ^ (r & 15)) << 4);
    }
    int a_rd[4];  // fragment of step st, row tile mt (+ 4096 mt): row ni, chunk 8 (st / 2) + 2 kb + st % 2
#pragma unroll
    for (int st = 0; st < 4; ++st) a_rd[st] = ni * 256 + (((8 * (st >> 1) + 2 * kb + (st & 1)) ^ ni) << 4);
    const NibbleMasks nm = nibble_masks();

    u32x4_t wring[4][WL];
    uint32_t zring;
    // The compiler orders nothing against these loads: the wait for them (the ring loads of a block are
    // younger) is written out in front of the barrier that publishes the block.
    // round r: the wave's block is KS r + kq; its tile of x lies at kq ROWS 256 of the round's buffer
    auto dma_x = [&](int r) {
        const int i = KS * r + kq;
        const __amdgpu_buffer_rsrc_t rs = i < NB ? rs_x : rs_none;
#pragma unroll
        for (int q = 0; q < XV; ++q)
            pk4g_load_lds16(rs, pk4_lds + (r & 1) * XBUF + kq * (ROWS * 256) + (ws * XV + q) * 1024, xo[q], i * 256);
    };
    auto load_w = [&](int i, int st) {
        const __amdgpu_buffer_rsrc_t rs = i < NB ? rs_w : rs_none;
#pragma unroll
        for (int h = 0; h < WL; ++h) wring[st][h] = __builtin_amdgcn_raw_buffer_load_b128(rs, voff_w, i * BB + (st * WL + h) * 1024, 0);
    };
    auto load_z = [&](int i) {
        const __amdgpu_buffer_rsrc_t rs = i < NB ? rs_w : rs_none;
        zring = __builtin_amdgcn_raw_buffer_load_b32(rs, voff_z, i * BB, 0);
    };
    auto zs_words = [&](uint32_t z, uint32_t (&zv)[4]) {
        const auto p16 = __builtin_amdgcn_permlane16_swap(z, z, false, false);
        const uint32_t even = p16[0], odd = p16[1];
        const auto pe = __builtin_amdgcn_permlane32_swap(even, even, false, false);
        const auto po = __builtin_amdgcn_permlane32_swap(odd, odd, false, false);
        zv[0] = pe[0], zv[2] = pe[1], zv[1] = po[0], zv[3] = po[1];
    };

    dma_x(0);
    __builtin_amdgcn_sched_barrier(0);  // requests keep this order: the wait counts rely on it
    load_z(kq);
#pragma unroll
    for (int st = 0; st < 4; ++st) load_w(kq, st);
    __builtin_amdgcn_sched_barrier(0);
    float4_t acc[MT][4];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int f = 0; f < 4; ++f) acc[mt][f] = float4_t{0.f, 0.f, 0.f, 0.f};
    pk4g_wait_vmcnt<RING>();
    __syncthreads();

    for (int r = 0; r < NR; ++r) {
        const int i = KS * r + kq;  // past NB (a ragged last round): zeros from both streams
        // the other buffer was last read in the previous round, which every wave has left (the barrier below)
        dma_x(r + 1);
        __builtin_amdgcn_sched_barrier(0);
        const unsigned char *buf = pk4_lds + (r & 1) * XBUF + kq * (ROWS * 256);
        uint32_t zv[4], negzb[4], sp[4];
        Pk4gBf16 cb[4];
        zs_words(zring, zv);
#pragma unroll
        for (int f = 0; f < 4; ++f) {
            if constexpr (BF) {  // the pair word holds {-(bias + z), s}, bias = 128 for nibbles and 0 for bytes
                cb[f].set(__builtin_bit_cast(float, zv[f] & 0xFFFF0000u), __builtin_bit_cast(float, zv[f] << 16) + (BITS == 4 ? 128.0f : 0.0f));
            } else {
                Pk4T<TT>::prep(zv[f], negzb[f], sp[f]);
            }
        }
        load_z(i + KS);
#pragma unroll
        for (int st = 0; st < 4; ++st) {
            uint32_t wp[WL][4];
#pragma unroll
            for (int h = 0; h < WL; ++h) {
                const u32x4_t wv = wring[st][h];
                wp[h][0] = wv[0], wp[h][1] = wv[1], wp[h][2] = wv[2], wp[h][3] = wv[3];
            }
            uint32_t a[MT][4];
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) {
                const u32x4_t av = *(const u32x4_t *)(buf + mt * 4096 + a_rd[st]);
                a[mt][0] = av[0], a[mt][1] = av[1], a[mt][2] = av[2], a[mt][3] = av[3];
            }
            uint32_t tl[4], th[4];
            if constexpr (BF && BITS == 4) {
#pragma unroll
                for (int pp = 0; pp < 4; ++pp) pk4g_nibbles(wp[0][pp], tl[pp], th[pp]);
            }
#pragma unroll
            for (int f = 0; f < 4; ++f) {
                uint32_t b[4];
#pragma unroll
                for (int pp = 0; pp < 4; ++pp) {
                    if constexpr (BITS == 8) {
                        // word pp of half f / 2: bytes {row 2 pp, row 2 pp + 1} x {column 2 h, 2 h + 1}: the pair of
                        // column f in bytes f % 2 and f % 2 + 2
                        const uint32_t word = wp[f >> 1][pp];
                        if constexpr (BF) b[pp] = (f & 1) ? cb[f].template pair<1, false>(word) : cb[f].template pair<0, false>(word);
                        else b[pp] = Pk4T<TT>::deq(TT::unpack_bytes((f & 1) ? (word >> 8) : word), negzb[f], sp[f]);
                    } else {
                        // column f of word pp: nibble f of each 16-bit half = the low or high nibble of bytes f / 2 and 2 + f / 2
                        if constexpr (!BF) b[pp] = Pk4T<TT>::deq(TT::unpack1(wp[0][pp], f, nm), negzb[f], sp[f]);
                        else if (f == 0) b[pp] = cb[0].template pair<0, false>(tl[pp]);
                        else if (f == 1) b[pp] = cb[1].template pair<0, true>(th[pp]);
                        else if (f == 2) b[pp] = cb[2].template pair<1, false>(tl[pp]);
                        else b[pp] = cb[3].template pair<1, true>(th[pp]);
                    }
                }
#pragma unroll
                for (int mt = 0; mt < MT; ++mt) acc[mt][f] = Ops::mfma(a[mt], b, acc[mt][f]);
            }
            load_w(i + KS, st);  // into the registers this step has just left
        }
        __builtin_amdgcn_sched_barrier(0);
        pk4g_wait_vmcnt<RING>();  // this wave's part of the next round of x is in LDS; its ring loads may still fly
        __syncthreads();
    }

    // the finished tile rows of this wave: all of them (KS = 1), or row tile kq summed over the strip's waves
    float4_t fin[KS == 1 ? MT : 1][4];
    if constexpr (KS == 1) {
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
            for (int f = 0; f < 4; ++f) fin[mt][f] = acc[mt][f];
    } else {
        // slot of wave w: [mt][e][lane] x float4 (f = 0..3), 16 KB; the last round's barrier has freed the buffers
        float4_t *red = (float4_t *)pk4_lds;
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
            for (int e = 0; e < 4; ++e)
                red[((wave * MT + mt) * 4 + e) * 64 + lane] = float4_t{acc[mt][0][e], acc[mt][1][e], acc[mt][2][e], acc[mt][3][e]};
        __syncthreads();
#pragma unroll
        for (int f = 0; f < 4; ++f) fin[0][f] = float4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int k = 0; k < KS; ++k)  // K order: the same sum whatever the timing
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const float4_t v = red[(((k * SPW + ws) * MT + kq) * 4 + e) * 64 + lane];
                fin[0][0][e] += v[0], fin[0][1][e] += v[1], fin[0][2][e] += v[2], fin[0][3][e] += v[3];
            }
    }
    if (!live) return;
    constexpr int FT = KS == 1 ? MT : 1;  // row tiles this wave stores: fin[t] is row tile (KS == 1 ? t : kq)
    if (act) {
        // Fused gate|up layer (pk4_src_col): columns 0..31 of the strip are gate columns 32 j .. 32 j + 31, columns
        // 32..63 the up columns they meet - lane ni < 8 holds four gate columns, lane ni + 8 of the same row of 16
        // their up columns.  As in pk4_epilogue: both factors rounded to the layer type (what the projection's own
        // output would hold, ffn.rs:388-400), act(gate) * up in f32, one rounding; y is [M, N / 2].
        // The two lanes of a pair exchange all four values (row_ror:8) and share the work: lane ni takes outputs
        // 0 and 1 of its four columns, lane ni + 8 outputs 2 and 3.
        const int half = N >> 1, col = 32 * j + 4 * (ni & 7);
        const bool low = ni < 8;
        float bv[4] = {0.f, 0.f, 0.f, 0.f};
        if (bias) {
            const uint2 bw = *(const uint2 *)(bias + (low ? 0 : half) + col);
            bv[0] = TT::to_f32((uint16_t)(bw.x & 0xFFFFu)), bv[1] = TT::to_f32((uint16_t)(bw.x >> 16));
            bv[2] = TT::to_f32((uint16_t)(bw.y & 0xFFFFu)), bv[3] = TT::to_f32((uint16_t)(bw.y >> 16));
        }
#pragma unroll
        for (int t = 0; t < FT; ++t)
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int row = m0 + 16 * (KS == 1 ? t : kq) + 4 * kb + e;
                float mine[4], other[4];
#pragma unroll
                for (int f = 0; f < 4; ++f) {
                    mine[f] = TT::to_f32(TT::from_f32(fin[t][f][e] + bv[f]));
                    other[f] = __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, mine[f]), 0x128, 0xF, 0xF, false));
                }
                uint32_t o[2];
#pragma unroll
                for (int q = 0; q < 2; ++q) {
                    const float gq = low ? mine[q] : other[2 + q], uq = low ? other[q] : mine[2 + q];
                    o[q] = TT::from_f32(mul_f32_rn(act == 1 ? silu_f32(gq) : gelu_tanh_f32(gq), uq));
                }
                if (row < M) *(uint32_t *)(y + (size_t)row * half + col + (low ? 0 : 2)) = o[0] | (o[1] << 16);
            }
        return;
    }
    // row 16 mt + 4 kb + e, columns 64 j + 4 ni + f: four neighbours, one 8-byte store
    float bv[4] = {0.f, 0.f, 0.f, 0.f};
    if (bias) {
        const uint2 bw = *(const uint2 *)(bias + 64 * j + 4 * ni);
        bv[0] = TT::to_f32((uint16_t)(bw.x & 0xFFFFu)), bv[1] = TT::to_f32((uint16_t)(bw.x >> 16));
        bv[2] = TT::to_f32((uint16_t)(bw.y & 0xFFFFu)), bv[3] = TT::to_f32((uint16_t)(bw.y >> 16));
    }
#pragma unroll
    for (int t = 0; t < FT; ++t)
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const int row = m0 + 16 * (KS == 1 ? t : kq) + 4 * kb + e;
            if (row >= M) continue;
            const uint32_t o0 = TT::from_f32(fin[t][0][e] + bv[0]), o1 = TT::from_f32(fin[t][1][e] + bv[1]);
            const uint32_t o2 = TT::from_f32(fin[t][2][e] + bv[2]), o3 = TT::from_f32(fin[t][3][e] + bv[3]);
            *(uint2 *)(y + (size_t)row * N + 64 * j + 4 * ni) = uint2{o0 | (o1 << 16), o2 | (o3 << 16)};
        }
}

// The same decomposition on a layer stored in 16-column strips (the narrow layout of attention and down
// projections): a wave's 64 columns are four neighbouring strips, a strip's block is one 16-byte load a lane
// whose words are the block's four steps - so the ring holds whole blocks, two of them: the next block is
// requested into the other half when a block starts.  Lane (ni, kb) holds column 16 f + ni of strip f.
template <typename TT, int MT, int KS>
__global__ __launch_bounds__(512) void pk4n_gemm_kernel(const uint16_t *__restrict__ x, const uint32_t *__restrict__ pw,
                                                        const uint16_t *__restrict__ bias, uint16_t *__restrict__ y,
                                                        int M, int K, int N, int NG, int RT) {
    typedef MfmaOps<TT> Ops;
    static_assert(KS == 1 || KS == MT, "wave kq of a column group finishes row tile kq");
    constexpr int SPW = PK4G_STRIPS / KS;  // 64-column groups a workgroup
    constexpr int ROWS = 16 * MT, BB = PK4N_BW * 4, XBUF = KS * ROWS * 256, XV = ROWS / 4 / SPW;
    constexpr bool BF = TT::DTYPE == BF16Traits::DTYPE;
    extern __shared__ __attribute__((aligned(16))) unsigned char pk4_lds[];

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int ni = lane & 15, kb = lane >> 4;
    const int ws = wave % SPW, kq = wave / SPW;  // as in pk4_gemm_kernel
    int rt, g;
    if constexpr (KS == 1) {
        pk4g_tile_of((int)blockIdx.x, RT, NG, rt, g);
        if (g >= NG) return;  // the whole workgroup, before any barrier
    } else {
        rt = (int)blockIdx.x / NG, g = (int)blockIdx.x % NG;
    }
    const int j = g * SPW + ws;  // the wave's 64 columns: strips 4 j .. 4 j + 3
    const bool live = j < (N >> 6);
    const int m0 = rt * ROWS;
    const int NB = K >> 7, NR = (NB + KS - 1) / KS;
    const int xrows = min(M - m0, ROWS);

    const __amdgpu_buffer_rsrc_t rs_none = make_rsrc(pw, 0u);
    const __amdgpu_buffer_rsrc_t rs_wl =
        make_rsrc(pw + (size_t)(live ? 4 * j : 0) * NB * PK4N_BW, 4u * (uint32_t)NB * (uint32_t)BB);
    const __amdgpu_buffer_rsrc_t rs_w = live ? rs_wl : rs_none;
    const __amdgpu_buffer_rsrc_t rs_x = make_rsrc(x + (size_t)m0 * K, (uint32_t)xrows * (uint32_t)K * 2u);
    const int voff_w = lane * 16, voff_z = 1024 + ni * 4;
    int xo[XV];
#pragma unroll
    for (int q = 0; q < XV; ++q) {
        const int r = 4 * (ws * XV + q) + (lane >> 4);
        xo[q] = r * K * 2 + (((lane & 15) ^ (r & 15)) << 4);
    }
    int a_rd[4];
#pragma unroll
    for (int st = 0; st < 4; ++st) a_rd[st] = ni * 256 + (((8 * (st >> 1) + 2 * kb + (st & 1)) ^ ni) << 4);
    const NibbleMasks nm = nibble_masks();

    u32x4_t wring[2][4];
    uint32_t zring[4];
    // round r: the wave's block is KS r + kq, its tile of x at kq ROWS 256 of the round's buffer
    auto dma_x = [&](int r) {
        const int i = KS * r + kq;
        const __amdgpu_buffer_rsrc_t rs = i < NB ? rs_x : rs_none;
#pragma unroll
        for (int q = 0; q < XV; ++q)
            pk4g_load_lds16(rs, pk4_lds + (r & 1) * XBUF + kq * (ROWS * 256) + (ws * XV + q) * 1024, xo[q], i * 256);
    };
    auto load_w = [&](int i, u32x4_t (&w)[4]) {
        const __amdgpu_buffer_rsrc_t rs = i < NB ? rs_w : rs_none;
#pragma unroll
        for (int f = 0; f < 4; ++f) w[f] = __builtin_amdgcn_raw_buffer_load_b128(rs, voff_w, (f * NB + i) * BB, 0);
    };
    auto load_z = [&](int i) {
        const __amdgpu_buffer_rsrc_t rs = i < NB ? rs_w : rs_none;
#pragma unroll
        for (int f = 0; f < 4; ++f) zring[f] = __builtin_amdgcn_raw_buffer_load_b32(rs, voff_z, (f * NB + i) * BB, 0);
    };

    dma_x(0);
    __builtin_amdgcn_sched_barrier(0);  // requests keep this order: the wait counts rely on it
    load_z(kq);
    load_w(kq, wring[0]);
    __builtin_amdgcn_sched_barrier(0);
    float4_t acc[MT][4];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int f = 0; f < 4; ++f) acc[mt][f] = float4_t{0.f, 0.f, 0.f, 0.f};
    pk4g_wait_vmcnt<8>();
    __syncthreads();

    // one round, the block's weights in ring half CUR; eight ring loads are younger than the round's loads of x
    auto block = [&](int r, auto cur_c) {
        constexpr int CUR = decltype(cur_c)::value;
        const int i = KS * r + kq;  // past NB (a ragged last round): zeros from both streams
        dma_x(r + 1);
        __builtin_amdgcn_sched_barrier(0);
        load_w(i + KS, wring[CUR ^ 1]);
        __builtin_amdgcn_sched_barrier(0);  // not sunk to the block's end, where the next block would wait for them
        const unsigned char *buf = pk4_lds + (r & 1) * XBUF + kq * (ROWS * 256);
        Pk4N<TT> cst[4];
        Pk4gBf16 cb[4];
#pragma unroll
        for (int f = 0; f < 4; ++f) {
            if constexpr (BF) {  // the pair word holds {-z, s}
                cb[f].set(__builtin_bit_cast(float, zring[f] & 0xFFFF0000u), __builtin_bit_cast(float, zring[f] << 16));
            } else {
                cst[f].prep(zring[f]);
            }
        }
        load_z(i + KS);
#pragma unroll
        for (int st = 0; st < 4; ++st) {
            uint32_t a[MT][4];
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) {
                const u32x4_t av = *(const u32x4_t *)(buf + mt * 4096 + a_rd[st]);
                a[mt][0] = av[0], a[mt][1] = av[1], a[mt][2] = av[2], a[mt][3] = av[3];
            }
#pragma unroll
            for (int f = 0; f < 4; ++f) {
                const uint32_t w = wring[CUR][f][st];
                uint32_t b[4];
                if constexpr (BF) {  // row pair pp: nibble pp of each 16-bit half
                    uint32_t tl, th;
                    pk4g_nibbles(w, tl, th);
                    b[0] = cb[f].template pair<0, false>(tl), b[1] = cb[f].template pair<0, true>(th);
                    b[2] = cb[f].template pair<1, false>(tl), b[3] = cb[f].template pair<1, true>(th);
                } else {
#pragma unroll
                    for (int pp = 0; pp < 4; ++pp) b[pp] = cst[f].deq(TT::unpack1(w, pp, nm), pp);
                }
#pragma unroll
                for (int mt = 0; mt < MT; ++mt) acc[mt][f] = Ops::mfma(a[mt], b, acc[mt][f]);
            }
        }
        __builtin_amdgcn_sched_barrier(0);
        pk4g_wait_vmcnt<8>();  // this wave's part of the next round of x is in LDS
        __syncthreads();
    };
    {
        int r = 0;
        for (; r + 1 < NR; r += 2) {
            block(r, std::integral_constant<int, 0>{});
            block(r + 1, std::integral_constant<int, 1>{});
        }
        if (r < NR) block(r, std::integral_constant<int, 0>{});
    }

    // the finished tile rows of this wave, as in pk4_gemm_kernel
    float4_t fin[KS == 1 ? MT : 1][4];
    if constexpr (KS == 1) {
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
            for (int f = 0; f < 4; ++f) fin[mt][f] = acc[mt][f];
    } else {
        float4_t *red = (float4_t *)pk4_lds;
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
            for (int e = 0; e < 4; ++e)
                red[((wave * MT + mt) * 4 + e) * 64 + lane] = float4_t{acc[mt][0][e], acc[mt][1][e], acc[mt][2][e], acc[mt][3][e]};
        __syncthreads();
#pragma unroll
        for (int f = 0; f < 4; ++f) fin[0][f] = float4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int k = 0; k < KS; ++k)  // K order: the same sum whatever the timing
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const float4_t v = red[(((k * SPW + ws) * MT + kq) * 4 + e) * 64 + lane];
                fin[0][0][e] += v[0], fin[0][1][e] += v[1], fin[0][2][e] += v[2], fin[0][3][e] += v[3];
            }
    }
    if (!live) return;
    // row 16 mt + 4 kb + e, column 64 j + 16 f + ni
    float bv[4] = {0.f, 0.f, 0.f, 0.f};
    if (bias) {
#pragma unroll
        for (int f = 0; f < 4; ++f) bv[f] = TT::to_f32(bias[64 * j + 16 * f + ni]);
    }
    constexpr int FT = KS == 1 ? MT : 1;
#pragma unroll
    for (int t = 0; t < FT; ++t)
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const int row = m0 + 16 * (KS == 1 ? t : kq) + 4 * kb + e;
            if (row >= M) continue;
#pragma unroll
            for (int f = 0; f < 4; ++f) y[(size_t)row * N + 64 * j + 16 * f + ni] = TT::from_f32(fin[t][f][e] + bv[f]);
        }
}

// Which decomposition a resident layer runs at M rows: 0 = the split-K tiles of pk4_mfma_kernel /
// pk4n_mfma_kernel, else the rows of a workgroup here.  Costs are in units of a full round (one 64-row workgroup
// on every CU), fitted to sweeps over 128..8192 rows in both types (64-column strips: 4096 x 14336, 8192 x 28672;
// 16-column strips: 4096 x 4096, 4096 x 6144, 14336 x 4096, 8192 x 8192; 8-bit: 4096 x 14336, 5120 x 13824):
//   - 128-row workgroups (203..230 registers: one a CU) run in whole rounds; a round costs `full128`, a last
//     round that fills at most 0.7 of the CUs `part128`;
//   - 64-row workgroups of the 64-column layout (121..125 registers) share a CU in pairs: up to one a CU the launch
//     costs 1 (`part64` up to three quarters of the CUs), up to two a CU a64 + b64 w, beyond that slope64 w
//     (w = workgroups / CUs); those of the 16-column layout (144..145 registers) run in whole rounds;
//   - the split-K tiles cost `split_lo` (below one round) or `split_hi` times w at any M: small workgroups, no
//     ragged round, but the rate they have at 64 rows.
// OXQ_PK4_GEMM_ROWS = 64 | 128 takes the choice (tests, sweeps); OXQ_PK4_GEMM_MIN_M = 0 switches the kernels off.
// a round of the two-strip form (one workgroup a CU) against a full round of 64-row workgroups of eight strips:
// 19 - 24 us against 65 - 78 at K = 4096 over both widths and types
constexpr double PK4_MID_ROUND = 0.31;
// 16-column strips: the same for a whole round, 0.27 for a last round on at most half of the CUs (4096 x 4096,
// 4096 x 6144, 8192 x 8192, 14336 x 4096 over 65..2048 rows in both types: 18.7 - 24.4 us a round at K = 4096)
constexpr double PK4N_MID_ROUND = 0.31, PK4N_MID_PART = 0.27;

struct Pk4GemmCost {
    bool pairs64;
    double part64, a64, b64, slope64, full128, part128, split_lo, split_hi;
};
// rows of a workgroup (0: the split-K tiles) and the K split inside it (4: two strips a workgroup)
struct Pk4GemmForm {
    int rows, ks;
};
static Pk4GemmForm pk4_gemm_form(const oxq_ctx *ctx, const Pk4Problem &p) {
    const int64_t min_m = tune(ctx, OXQ_TUNE_PK4_GEMM_MIN_M, 65);
    if (min_m <= 0 || (p.w.bits != 4 && p.w.bits != 8) || (p.act && p.w.strip == 16) || p.M < min_m) return {0, 1};
    if (p.w.bits == 8 && p.w.strip == 16) return {0, 1};  // (16-column strips are a 4-bit layout)
    const int forced = tune(ctx, OXQ_TUNE_PK4_GEMM_ROWS, 0), forced_ks = tune(ctx, OXQ_TUNE_PK4_GEMM_KS, 0);
    if (forced_ks == 4) return {64, 4};
    if (forced == 64 || forced == 128) return {forced, 1};
    static const Pk4GemmCost WIDE_F16 = {true, 0.88, 1.20, 0.30, 0.97, 1.50, 1.27, 1.93, 1.50};
    static const Pk4GemmCost WIDE_BF16 = {true, 0.93, 1.29, 0.27, 0.98, 1.44, 1.35, 2.00, 1.53};
    static const Pk4GemmCost NARROW_F16 = {false, 0.86, 0, 0, 0, 1.64, 1.30, 1.60, 1.50};
    static const Pk4GemmCost NARROW_BF16 = {false, 0.94, 0, 0, 0, 1.51, 1.35, 1.60, 1.50};
    static const Pk4GemmCost WIDE8_F16 = {false, 0.88, 0, 0, 0, 1.47, 1.27, 1.92, 1.71};  // 8-bit: 137 registers at 64 rows
    static const Pk4GemmCost WIDE8_BF16 = {false, 0.91, 0, 0, 0, 1.47, 1.32, 2.00, 1.78};
    const bool f16 = p.w.dtype == OXQ_F16;
    const Pk4GemmCost &c = p.w.bits == 8      ? (f16 ? WIDE8_F16 : WIDE8_BF16)
                           : p.w.strip == 16 ? (f16 ? NARROW_F16 : NARROW_BF16)
                                             : (f16 ? WIDE_F16 : WIDE_BF16);
    const double cus = ctx->num_cus > 0 ? ctx->num_cus : 256;
    const int64_t groups = ceil_div(p.w.N / 64, (int64_t)PK4G_STRIPS);
    const double w64 = (double)(groups * ceil_div(p.M, (int64_t)64)) / cus, w128 = (double)(groups * ceil_div(p.M, (int64_t)128)) / cus;
    auto rounds = [](double w, double full, double part, double part_upto) {
        const double whole = std::floor(w), rest = w - whole;
        return whole * full + (rest <= 0.0 ? 0.0 : rest <= part_upto ? part : full);
    };
    const double c64 = !c.pairs64 || w64 <= 1.0 ? rounds(w64, 1.0, c.part64, 0.75) : w64 <= 2.0 ? c.a64 + c.b64 * w64 : c.slope64 * w64;
    const double c128 = rounds(w128, c.full128, c.part128, 0.7);
    // the split-K tiles of the 16-column layout are one workgroup a row tile and 64 columns, in whole rounds too
    const double c_split = (w64 < 1.0 ? c.split_lo : c.split_hi) * (p.w.strip == 16 ? std::ceil(8.0 * w64 - 1e-9) / 8.0 : w64);
    // two strips a workgroup (128 KB of LDS: one a CU), whole rounds of `PK4_MID_ROUND` each
    const double w_mid = (double)(ceil_div(p.w.N / 64, (int64_t)2) * ceil_div(p.M, (int64_t)64)) / cus;
    const double c_mid = forced_ks == 1        ? 1e30
                         : p.w.strip == 16 ? rounds(w_mid, PK4N_MID_ROUND, PK4N_MID_PART, 0.5)
                                           : std::ceil(w_mid) * PK4_MID_ROUND;
    if (c_split <= c64 && c_split <= c128 && c_split <= c_mid) return {0, 1};
    if (c_mid < c64 && c_mid < c128) return {64, 4};
    return {c128 < c64 ? 128 : 64, 1};
}
bool pk4_gemm_takes(const oxq_ctx *ctx, const Pk4Problem &p) { return pk4_gemm_form(ctx, p).rows != 0; }

template <typename TT, int MT, int LAYOUT, int KS>  // LAYOUT: 4 / 8 = bits of a layer in 64-column strips, 16 = 4-bit in 16-column strips
static int pk4_gemm_go(hipStream_t s, dim3 grid, const Pk4Problem &p, int NG, int RT) {
    static LdsGrant grant;  // one per instantiation
    const size_t lds = (size_t)2 * KS * 16 * MT * 256;
    if constexpr (LAYOUT == 16) {
        OXQ_HIP_CHECK(grant.ensure((const void *)pk4n_gemm_kernel<TT, MT, KS>, lds));
        hipLaunchKernelGGL((pk4n_gemm_kernel<TT, MT, KS>), grid, dim3(512), lds, s, (const uint16_t *)p.x, p.w.pw, (const uint16_t *)p.bias,
                           (uint16_t *)p.y, (int)p.M, (int)p.w.K, (int)p.w.N, NG, RT);
    } else {
        OXQ_HIP_CHECK(grant.ensure((const void *)pk4_gemm_kernel<TT, MT, LAYOUT, KS>, lds));
        hipLaunchKernelGGL((pk4_gemm_kernel<TT, MT, LAYOUT, KS>), grid, dim3(512), lds, s, (const uint16_t *)p.x, p.w.pw, (const uint16_t *)p.bias,
                           (uint16_t *)p.y, (int)p.M, (int)p.w.K, (int)p.w.N, NG, RT, p.act);
    }
    OXQ_HIP_CHECK(hipGetLastError());
    return OXQ_OK;
}
template <typename TT, int MT, int KS>
static int pk4_gemm_go_layout(hipStream_t s, dim3 grid, const Pk4Problem &p, int NG, int RT) {
    if (p.w.strip == 16) return pk4_gemm_go<TT, MT, 16, KS>(s, grid, p, NG, RT);
    return p.w.bits == 8 ? pk4_gemm_go<TT, MT, 8, KS>(s, grid, p, NG, RT) : pk4_gemm_go<TT, MT, 4, KS>(s, grid, p, NG, RT);
}

int launch_pk4_gemm(oxq_ctx *ctx, hipStream_t s, const Pk4Problem &p) {
    const Pk4GemmForm form = pk4_gemm_form(ctx, p);
    const int rows = form.rows, spw = PK4G_STRIPS / form.ks;
    const int64_t NG = ceil_div(p.w.N / 64, (int64_t)spw), RT = ceil_div(p.M, (int64_t)rows);
    // eight strips a workgroup: whole bands of 8 row tiles in squares of 64 workgroups, then the last RT % 8 row
    // tiles x NG groups; two strips: row tile by row tile
    const int64_t wgs = form.ks == 1 ? (RT / 8) * ceil_div(NG, (int64_t)8) * 64 + (RT % 8) * NG : RT * NG;
    if (wgs > 0x7FFFFFFF) return fail(OXQ_ERR_UNSUPPORTED, "repacked matmul: m = %lld exceeds the grid", (long long)p.M);
    dim3 grid((unsigned)wgs);
    char name[64];
    snprintf(name, sizeof name, "pk%d_gemm_%s_r%dx%d%s%s%s", p.w.bits, p.w.dtype == OXQ_F16 ? "f16" : "bf16", rows, spw,
             form.ks > 1 ? "k4" : "", p.w.strip == 16 ? "_n16" : "", p.act == 1 ? "_silu" : p.act == 2 ? "_gelu" : "");
    set_plan(ctx, name, grid, dim3(512), 1, 1, 0);
    if (ctx->plan_only) return OXQ_OK;
    if ((uint64_t)rows * (uint64_t)p.w.K * 2 >= (1ull << 31)) return fail(OXQ_ERR_UNSUPPORTED, "repacked matmul: K too large");
    if (((uintptr_t)p.x | (uintptr_t)p.y) & 15) return fail(OXQ_ERR_UNSUPPORTED, "repacked matmul: x and y must be 16-byte aligned");
    if (p.bias && ((uintptr_t)p.bias & 7)) return fail(OXQ_ERR_UNSUPPORTED, "repacked matmul: bias must be 8-byte aligned");
    const bool f16 = p.w.dtype == OXQ_F16;
    if (form.ks == 4)
        return f16 ? pk4_gemm_go_layout<F16Traits, 4, 4>(s, grid, p, (int)NG, (int)RT) : pk4_gemm_go_layout<BF16Traits, 4, 4>(s, grid, p, (int)NG, (int)RT);
    if (rows == 128)
        return f16 ? pk4_gemm_go_layout<F16Traits, 8, 1>(s, grid, p, (int)NG, (int)RT) : pk4_gemm_go_layout<BF16Traits, 8, 1>(s, grid, p, (int)NG, (int)RT);
    return f16 ? pk4_gemm_go_layout<F16Traits, 4, 1>(s, grid, p, (int)NG, (int)RT) : pk4_gemm_go_layout<BF16Traits, 4, 1>(s, grid, p, (int)NG, (int)RT);
}

}  // namespace oxq
