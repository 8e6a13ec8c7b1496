// Resident 4- and 8-bit layers in a tile-major layout: load-time repack + the
// matmul kernel that runs every batch size on it.
//
// Reference semantics: linear.rs:415-448 (PackedQuantLinear::new keeps the
// checkpoint tensors resident and converts the scales once at load) and
// linear.rs:482-533 (forward: fused GEMV for small m, staged tile GEMM above,
// f32 accumulation, result in the activation dtype).  The arithmetic per
// weight is the tile GEMM's (mpp_gemm.metal:101-266): B = T((q - z) * s)
// rounded once to the 16-bit activation type, f32 accumulate.
//
// Why a repack.  In the checkpoint layouts a [K x 64-column] strip is 32 bytes
// per row at a row pitch of N/2 bytes; a workgroup that owns such a strip reads
// narrow column stripes, which this memory system serves at less than half its
// streaming rate, so the raw-layout kernels give each workgroup a wide slab and
// split K across workgroups instead - and then pay for the partial sums in
// HBM.  Stored tile-major, a strip is one contiguous run: one workgroup per
// 64-column strip streams it with 1 KB wave loads, splits K across its own 8
// waves and reduces through LDS.  One launch, no workspace, no atomics.
//
// Kernels in this file: pk4_mfma_kernel (every row count; a wave rings one block of weights ahead),
// pk4_front_kernel (one row tile of a 4-bit layer with a short K slice: 16 waves, each requesting its
// whole share before it waits), pk4n_mfma_kernel / pk4n_front_kernel (the same pair for layers stored in
// 16-column strips), the load-time repacks and the dense dequants that pin them.
//
// Layout (K % 128 == 0, N % 64 == 0, group size a multiple of 128).  A strip is a run of
// K/128 self-contained blocks; a block covers 128 rows of K and holds its weights followed by the
// zeros and scales that apply to them:
//
//   pw  [N/64 strips][K/128 blocks]{ [4 steps][bits/4][64 lanes][4 words] , [16 column quads][4 words] }
//
// i.e. 4 KB (4-bit) or 8 KB (8-bit) of weights and 256 bytes of {-(bias_f + z), s} pairs, two 16-bit
// floats of the layer's dtype per column (z already includes GPTQ's +1; a group larger than 128 rows
// repeats its pair in each of its blocks).  With the pairs inside the stream a wave's loads for a
// block are one contiguous run, nothing is staged through LDS before the first multiply, and any
// wave can take any block.
//
// Step t = 4 * block + st covers 32 rows of K.  Lane l = (ni = l % 16, kb = l / 16)
// owns the 8 rows  kk = 64*(t/2) + 16*kb + 8*(t%2) .. +7  of the four columns
// 64*strip + 4*ni + f, f = 0..3: exactly one MFMA B fragment per f.  Word pp
// (0..3) holds rows kk+2pp (low 16 bits) and kk+2pp+1 (high 16 bits), four
// nibbles each, nibble f = column f.  Two consecutive steps therefore cover 16
// consecutive rows per lane group, so the matching activation loads are 32
// contiguous bytes per row.  One AND-OR per fragment register turns a row pair
// into two exact 16-bit floats (bias + q).  Lane (ni, any kb) reads the block's pairs for its
// four columns with one 16-byte load at word 4 * ni of the block's tail.

//
// 8-bit layers use the same scheme with two 1 KB loads per step: half h (0..1) of a step
// holds the column pair f = 2h, 2h+1; word pp = {q[kk+2pp][2h], q[kk+2pp][2h+1],
// q[kk+2pp+1][2h], q[kk+2pp+1][2h+1]} as bytes, so an AND-OR of bytes 0 and 2 (after a
// shift by 8 for the odd column) again yields a row pair as two exact 16-bit floats.

#include "oxq_device.hpp"
#include "oxq_internal.hpp"
#include "oxq_mfma.hpp"
#include "pk4_common.hpp"

#include <algorithm>
#include <type_traits>
#include <cstdlib>

namespace oxq {
// ---------------------------------------------------------------------------
// load-time repack
// ---------------------------------------------------------------------------

template <bool GPTQ, int BITS>
__device__ __forceinline__ uint32_t src_q(const uint32_t *__restrict__ qw, int k, int col, int N) {
    constexpr int PF = 32 / BITS;
    constexpr uint32_t MASK = (1u << BITS) - 1u;
    if (GPTQ) return (qw[(size_t)(k / PF) * N + col] >> (BITS * (k % PF))) & MASK;
    const int c = col % PF;
    // 4-bit AWQ interleaves the 8 columns of a word ([0,2,4,6,1,3,5,7]); 8-bit is in order
    const int slot = BITS == 4 ? ((c >> 1) | ((c & 1) << 2)) : c;
    return (qw[(size_t)k * (N / PF) + col / PF] >> (BITS * slot)) & MASK;
}

// one thread per word of the resident copy
template <typename TT, bool GPTQ, int BITS>
__global__ __launch_bounds__(256) void pk4_prepack_kernel(const uint32_t *__restrict__ qw,
                                                          const uint32_t *__restrict__ qz,
                                                          const uint16_t *__restrict__ sc,
                                                          uint32_t *__restrict__ pw, int K, int N, int gshift,
                                                          int half) {
    constexpr int PF = 32 / BITS, WL = BITS / 4, BW = pk4_block_words(BITS);
    const size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;
    const int NB = K >> 7;
    if (idx >= (size_t)(N >> 6) * NB * BW) return;
    const int w = (int)(idx % BW);
    const int b = (int)((idx / BW) % NB), j = (int)(idx / ((size_t)BW * NB));
    if (w < 1024 * WL) {
        const int pp = w & 3, l = (w >> 2) & 63, sh = w >> 8;
        const int h = sh % WL, st = sh / WL;
        const int ni = l & 15, kb = l >> 4;
        const int k = pk4_kk(4 * b + st, kb) + 2 * pp;
        uint32_t v = 0;
        if (BITS == 4) {
#pragma unroll
            for (int r = 0; r < 2; ++r)
#pragma unroll
                for (int f = 0; f < 4; ++f)
                    v |= src_q<GPTQ, BITS>(qw, k + r, pk4_src_col(64 * j + 4 * ni + f, half), N) << (16 * r + 4 * f);
        } else {
#pragma unroll
            for (int r = 0; r < 2; ++r)
#pragma unroll
                for (int c = 0; c < 2; ++c)
                    v |= src_q<GPTQ, BITS>(qw, k + r, pk4_src_col(64 * j + 4 * ni + 2 * h + c, half), N) << (16 * r + 8 * c);
        }
        pw[idx] = v;
    } else {
        const int q = w - 1024 * WL, ni = q >> 2, f = q & 3;
        const int g = (b << 7) >> gshift;
        const int col = pk4_src_col(64 * j + 4 * ni + f, half);
        const int c = col % PF;
        const int slot = (GPTQ || BITS == 8) ? c : ((c >> 1) | ((c & 1) << 2));
        const uint32_t z = ((qz[(size_t)g * (N / PF) + col / PF] >> (BITS * slot)) & ((1u << BITS) - 1u)) + (GPTQ ? 1u : 0u);
        const float bf = BITS == 4 ? TT::bias(f) : TT::BYTE_BIAS;
        const uint32_t nz = TT::from_f32(-((float)z + bf));
        pw[idx] = nz | ((uint32_t)sc[(size_t)g * N + col] << 16);
    }
}

// ---------------------------------------------------------------------------
// dense dequant of a resident layer -> [K, N] (linear.rs:510-523 fallback);
// the same arithmetic as the matmul kernel's B fragments.
// ---------------------------------------------------------------------------
template <typename TT, int BITS>
__global__ __launch_bounds__(256) void pk4_dequant_kernel(const uint32_t *__restrict__ pw,
                                                          uint16_t *__restrict__ out, int K, int N, int half) {
    constexpr int WL = BITS / 4, BW = pk4_block_words(BITS);
    const size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;  // over the weight words only
    const int NB = K >> 7;
    if (idx >= (size_t)(N >> 6) * NB * 1024 * WL) return;
    const int w = (int)(idx % (1024 * WL));
    const int b = (int)((idx / (1024 * WL)) % NB), j = (int)(idx / ((size_t)1024 * WL * NB));
    const uint32_t *blk = pw + ((size_t)j * NB + b) * BW;
    const int pp = w & 3, l = (w >> 2) & 63, sh = w >> 8;
    const int h = sh % WL, st = sh / WL;
    const int ni = l & 15, kb = l >> 4;
    const int k = pk4_kk(4 * b + st, kb) + 2 * pp;
    const uint32_t wd = blk[w];
    const NibbleMasks nm = nibble_masks();
#pragma unroll
    for (int c = 0; c < (BITS == 4 ? 4 : 2); ++c) {
        const int f = BITS == 4 ? c : 2 * h + c;
        const uint32_t zs = blk[1024 * WL + ni * 4 + f];
        uint32_t c0, c1;
        Pk4T<TT>::prep(zs, c0, c1);
        const uint32_t pair = BITS == 4 ? TT::unpack1(wd, f, nm) : TT::unpack_bytes(c ? (wd >> 8) : wd);
        const uint32_t d = Pk4T<TT>::deq(pair, c0, c1);
        const int col = pk4_src_col(64 * j + 4 * ni + f, half);
        out[(size_t)k * N + col] = (uint16_t)(d & 0xFFFFu);
        out[(size_t)(k + 1) * N + col] = (uint16_t)(d >> 16);
    }
}

// ---------------------------------------------------------------------------
// y[M, N] = x[M, K] . W   on the repacked layout
//
// grid.x = strip (64 output columns), grid.z = block of 16*MT rows of x,
// grid.y = K slice (1 unless the layer has few strips and a long K, see the
// launcher); the 8 waves deal the slice's blocks of 128 rows (4 MFMA steps) out
// round-robin, so that at any moment the workgroup reads one contiguous stretch of
// its strip (a plain read of the same bytes is 4 % faster that way than with one
// contiguous eighth per wave).  With more than one slice the workgroup writes its
// f32 partial tile to the workspace and a second launch adds the slices in order.
//
// Weights: one 1 KB wave load per step, issued one block (4 steps) ahead; the block's
// zero/scale pairs ride in the same ring (one 16-byte load per lane and block).
// Activations: the matrix-core fragment pattern (16 rows x 64 bytes per load)
// is served by L2 at a third of the rate of 256-byte row reads, so a wave
// fetches its next 16*MT x 128 block of x with 4-rows-x-256-bytes loads one
// block ahead, parks it in its private LDS slot (16-byte chunks XOR-swizzled by
// row, so both the row-wise write and the fragment read are conflict-free)
// and reads fragments from there.  Rows past M are never fetched (out-of-range
// lane offset: the buffer unit returns zero without touching memory).
// All vector loads are issued unconditionally - steps past the end of a
// wave's share also use the out-of-range offset - so the compiler can count
// exactly how many loads are younger than the one it waits for; a conditionally
// issued load makes it wait for all of them, which serialises the pipeline.
// The 8 partial 16*MT x 64 tiles meet in LDS (each wave's slot is its own
// activation slot) and are added in wave order, which fixes the summation order.
//
// Two arithmetic forms, both with f32 accumulation:
//  * GS = false (m > 16, the reference's tile-GEMM range): B = T((q - z) * s),
//    bit-identical to the dense dequant, fed to the matrix cores.
//  * GS = true (m <= 16, the reference's fused-GEMV range, which never rounds
//    the dequantized weight: quant_kernels.metal w4a16 GEMV keeps (q - z) * s in
//    f32): the matrix cores multiply x by the exact integers bias + q, one
//    extra MFMA against a fragment of ones yields the row sums of x in the
//    accumulator layout, and once per block
//        y += s * (acc_b - (bias + z) * rowsum_b(x))            (all f32).
// ---------------------------------------------------------------------------
// Ring depth: weights WD steps (1 KB wave loads).  One block of weights in flight per wave is
// the measured optimum (4096 x 14336, f16, M = 1 / 16): 2 steps equal, 8 steps 5 - 10 % slower,
// 16 steps 17 % slower.  A CU takes only so many vector loads in flight: what the first waves
// issue beyond their next block keeps the other waves' first loads waiting.
template <int MT, int BITS> struct Pk4Ring {
    static constexpr int WD = 4;
};

// XQ: activation loads per block and lane that can hold rows below M (4 rows each); the
// launcher passes 4 * MT, or fewer for a short single tile, whose other rows stay zero in LDS.
// NBLK > 0: every wave has exactly NBLK blocks and the block loop is straight-line code.
template <typename TT, int BITS, int MT, bool GS, int WD, int XQ, bool PLZ = false, int NBLK = 0>
__global__ __launch_bounds__(512) void pk4_mfma_kernel(const uint16_t *__restrict__ x,
                                                       const uint32_t *__restrict__ pw,
                                                       const uint16_t *__restrict__ bias,
                                                       uint16_t *__restrict__ y, float *__restrict__ ws,
                                                       int M, int K, int N, int bslice, int contiguous, int act) {
    typedef MfmaOps<TT> Ops;
    constexpr int NW = 8;                      // waves per workgroup (4 and 16 waves measured 30 % slower)
    constexpr int ROWS = 16 * MT;
    constexpr int AQ = XQ;                     // activation loads per block and lane
    constexpr int SLOT = ROWS * 256;           // bytes of one wave's LDS slot (= its partial tile)
    constexpr int OOB = 0x7FFFFF00;
    constexpr int WL = BITS / 4;               // 1 KB weight loads per step
    constexpr int BB = pk4_block_words(BITS) * 4;  // bytes of one block: weights, then the zero/scale pairs
    // Up to 48 rows there is one row tile, so every weight is read once per launch: nontemporal
    // loads (cache policy bit 1), which a bare read of the same 30 MB also gains 7 % from.
    // From 49 rows on several row tiles may share a strip through L2, so those keep the default - except the
    // forms that are only launched with one row-tile workgroup a strip (NBLK, PLZ).  64 rows, same box, default ->
    // nontemporal: 4096 x 14336 f16 15.93 -> 15.45 us, bf16 17.48 -> 17.02; 5120 x 13824 f16 19.33 -> 18.54, 8-bit 24.14 ->
    // 22.60; 8192 x 28672 51.7 -> 50.8.  (4096 x 11008 measures 14.44 -> 14.60: its 12 rotated copies, 270 MB, are
    // partly still in the 256 MB memory-side cache when their turn comes again, which a decoder's layers are not.)
    constexpr int WNT = (MT < 4 || NBLK > 0 || PLZ) ? 2 : 0;
    // Hand-placed memory operations (the three places marked PLACED below) instead of the compiler's own order,
    // where that measured faster - same box, 48 / 64 / 128 rows: 8-bit f16 5120 x 13824 21.8 / 27.3 / 42.5 ->
    // 20.6 / 24.3 / 41.0 us; 4-bit bf16 4096 x 14336 at 33 / 48 rows 16.4 / 16.7 -> 15.2 / 15.9 us.  The 4-bit f16
    // kernels and bf16 at four row tiles are as fast or faster as the compiler orders them (f16 at 64 / 128
    // rows 16.9 / 29.4 against 16.6 / 30.8; bf16 19.6 / 33.8 against 18.7 / 34.3).
    // PLZ: the 4-bit kernel at four row tiles when a strip has one row-tile workgroup and the tile is (nearly)
    // full, 57 - 64 rows: placed it is 1.5 - 5 % faster there (same box, 64 rows: f16 16.48 -> 16.24, bf16 19.39 ->
    // 18.43, 5120 x 13824 f16 20.3 -> 19.9 us), slower at 49 rows (f16 15.33 -> 15.71) and when two or more
    // row-tile workgroups share a strip's weights through L2 (128 rows: f16 29.4 -> 30.8).
    constexpr bool PLACED = PLZ || (MT >= 3 && (BITS == 8 || (TT::DTYPE == BF16Traits::DTYPE && MT == 3)));
    extern __shared__ __attribute__((aligned(16))) unsigned char pk4_lds[];

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int ni = lane & 15, kb = lane >> 4;
    const int j = blockIdx.x;
    const int m0 = blockIdx.z * ROWS;
    const int NB = K >> 7;
    // K slice of this workgroup: blocks [sb0, sb0 + SB).  The wave's blocks inside it, by local index
    // i: every 8th block starting at its own number (the default), or one contiguous run (a tuning
    // switch; the shares differ by at most one block either way).
    const int sb0 = blockIdx.y * bslice;
    const int SB = min(NB, sb0 + bslice) - sb0;
    const int cbase = SB / NW, crem = SB % NW;
    const int nloc = contiguous ? cbase + (wave < crem ? 1 : 0) : (SB > wave ? (SB - wave + NW - 1) / NW : 0);
    const int cb0 = sb0 + wave * cbase + min(wave, crem);
    auto blk_of = [&](int i) { return contiguous ? cb0 + i : sb0 + i * NW + wave; };
    unsigned char *slot = pk4_lds + wave * SLOT;

    const __amdgpu_buffer_rsrc_t rs_w = make_rsrc(pw + (size_t)j * NB * (BB / 4), (uint32_t)NB * (uint32_t)BB);
    const __amdgpu_buffer_rsrc_t rs_x = make_rsrc(x, (uint32_t)M * (uint32_t)K * 2u);
    const int voff_w = lane * 16;
    // The block's zero/scale pairs: lane (ni, kb) fetches word kb of column quad ni (one 4-byte load a lane,
    // 256 contiguous bytes a wave: a quarter of what a 16-byte load costs the address unit, which is the
    // busiest unit from 32 rows on) and the four lane groups then exchange their words (zs_words).
    const int voff_z = 1024 * WL * 4 + (ni * 4 + kb) * 4;
    // activation load q of a block: row 4q + lane/16, 16-byte chunk lane%16 of the row's 256 bytes; rows
    // past M get an offset beyond any buffer, for which the buffer unit returns zeros without touching
    // memory (the scalar offset of a buffer load is not part of its bounds check, so the lane offset
    // has to carry the row)
    // Up to two row tiles every load keeps its own offset register; the larger kernels are at their
    // register budget and derives them from the first one (a row past M then lies beyond the end of x by
    // its lane offset alone, which the bounds check does cover).
    constexpr bool VA1 = MT >= 3;
    int voff_a[VA1 ? 1 : AQ];
#pragma unroll
    for (int q = 0; q < (VA1 ? 1 : AQ); ++q) {
        const int r = m0 + 4 * q + kb;
        voff_a[q] = r < M ? (r * K * 2 + ni * 16) : OOB;
    }
    uint32_t rowstep = 4u * (uint32_t)K * 2u;
    // LDS position of (row = 4q + kb, chunk ni): chunk index XORed with row % 16 = kb | (q % 4) << 2
    int a_wr[4];
#pragma unroll
    for (int qq = 0; qq < 4; ++qq) a_wr[qq] = kb * 256 + (((ni ^ kb) ^ (qq << 2)) << 4);  // + 1024 q
    // fragment read of step s (0..3), row tile mt: row 16mt + ni, chunk 8*(s/2) + 2kb + (s%2)
    int a_rd[4];
#pragma unroll
    for (int st = 0; st < 4; ++st) a_rd[st] = ni * 256 + (((8 * (st >> 1) + 2 * kb + (st & 1)) ^ ni) << 4);
    const NibbleMasks nm = nibble_masks();
    // rows no load covers: zero once, no block writes them again
#pragma unroll
    for (int q = AQ; q < 4 * MT; ++q) {
        const int row = 4 * q + kb;
        *(u32x4_t *)(slot + row * 256 + ((ni ^ (row & 15)) << 4)) = u32x4_t{0u, 0u, 0u, 0u};
    }

    static_assert(WD == 4, "the ring holds exactly one block");
    u32x4_t aring[AQ], wring[WD][WL];
    uint32_t zring;
    // Past the end of the wave's share the loads go through an empty descriptor: a scalar select,
    // no vector instruction, and the buffer unit returns zero without touching memory.
    const __amdgpu_buffer_rsrc_t rs_none = make_rsrc(pw, 0u);
    auto load_a = [&](int i, u32x4_t (&a)[AQ]) {
        const __amdgpu_buffer_rsrc_t rs = i < nloc ? rs_x : rs_none;  // wave-uniform
        const int blk = blk_of(i);
#pragma unroll
        for (int q = 0; q < AQ; ++q) {
            if (VA1) {
                if (q == 0) asm volatile("" : "+s"(rowstep));  // recomputed per block: 15 registers less to hold
                // no wrap-around: 15 row steps stay below 2^31 (K <= 2^24, checked on the host), so a row
                // past M - from the first offset or by the steps - lies beyond x (< 2 GiB) and reads zeros
                a[q] = __builtin_amdgcn_raw_buffer_load_b128(rs, (int)((uint32_t)voff_a[0] + (uint32_t)q * rowstep), blk * 256, 0);
            } else {
                a[q] = __builtin_amdgcn_raw_buffer_load_b128(rs, voff_a[q], blk * 256, 0);
            }
        }
    };
    auto load_w = [&](int i, int st, u32x4_t (&w)[WL]) {
        const __amdgpu_buffer_rsrc_t rs = i < nloc ? rs_w : rs_none;
#pragma unroll
        for (int h = 0; h < WL; ++h)
            w[h] = __builtin_amdgcn_raw_buffer_load_b128(rs, voff_w, blk_of(i) * BB + (st * WL + h) * 1024, WNT);
    };
    auto load_z = [&](int i) {
        const __amdgpu_buffer_rsrc_t rs = i < nloc ? rs_w : rs_none;
        zring = __builtin_amdgcn_raw_buffer_load_b32(rs, voff_z, blk_of(i) * BB, WNT);
    };
    // zv[f] = the word that lane group f fetched, in every lane group: the lane-swap instructions
    // exchange 16-lane rows between two registers (odd rows of one with even rows of the other, then
    // the upper half of one with the lower half of the other).
    auto zs_words = [&](uint32_t z, uint32_t (&zv)[4]) {
        const auto p16 = __builtin_amdgcn_permlane16_swap(z, z, false, false);  // {r0 r0 r2 r2}, {r1 r1 r3 r3}
        const uint32_t even = p16[0], odd = p16[1];
        const auto pe = __builtin_amdgcn_permlane32_swap(even, even, false, false);  // {r0 x4}, {r2 x4}
        const auto po = __builtin_amdgcn_permlane32_swap(odd, odd, false, false);    // {r1 x4}, {r3 x4}
        zv[0] = pe[0], zv[2] = pe[1], zv[1] = po[0], zv[3] = po[1];
    };
    auto store_a = [&](const u32x4_t (&a)[AQ]) {
#pragma unroll
        for (int q = 0; q < AQ; ++q) *(u32x4_t *)(slot + q * 1024 + a_wr[q & 3]) = a[q];
    };

    // issue order = consumption order.  The tile form needs the pairs before its first B fragment,
    // the folded form after the block's last step.
    u32x4_t afirst[AQ];
    load_a(0, afirst);
    if (!GS) load_z(0);
#pragma unroll
    for (int g = 0; g < 4; ++g) load_w(0, g, wring[g]);
    if (GS) load_z(0);
    load_a(1, aring);

    float4_t acc[MT][4];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int f = 0; f < 4; ++f) acc[mt][f] = float4_t{0.f, 0.f, 0.f, 0.f};
    uint32_t negzb[4], sp[4];          // GS = false: the two Pk4T constants per column
    const uint32_t ones[4] = {TT::ONES, TT::ONES, TT::ONES, TT::ONES};
    const float4_t zero4 = float4_t{0.f, 0.f, 0.f, 0.f};

    store_a(afirst);

    // PLACED (1).  The counter a wave waits on counts its loads in issue order, and what the loop waits for at
    // its top is the stricter of what its two entries require.  From three row tiles on the compiler requests
    // the second x block before the first pairs and weights here, but after them inside the loop: coming from
    // here the pairs have 4 younger loads, so the loop would wait with "at most 4 outstanding" - that is, for
    // 12 of the 16 x loads it has just issued - in every iteration.  With block 0's pairs and weights
    // complete before the loop, only the loop's own order counts.
    if constexpr (PLACED) {
        asm volatile("" ::"v"(zring));
#pragma unroll
        for (int g = 0; g < 4; ++g)
#pragma unroll
            for (int h = 0; h < WL; ++h) asm volatile("" ::"v"(wring[g][h]));
    }
    // Two blocks an iteration where placed by hand: the ring registers a block loads are copied to the ones
    // the loop carries at the loop's end, which waits for those loads; twice as rarely this way.
    // With the block count known (NBLK) there is no loop at all (figures where it is launched).
    constexpr int UF = NBLK > 0 ? 1 : PLACED ? 2 : 1;
    const int trip = NBLK > 0 ? NBLK : nloc;
    constexpr int UNROLL = NBLK > 0 ? NBLK : 1;
#pragma unroll UNROLL
    for (int i0 = 0; i0 < trip; i0 += UF)
#pragma unroll
    for (int u = 0; u < UF; ++u) {
        const int i = i0 + u;
        if (u > 0 && i >= nloc) break;
        float4_t tmp[GS ? MT : 1][4], tmps[GS ? MT : 1];  // per-block integer sums of the GS form
        if (!GS) {
            uint32_t zv[4];
            zs_words(zring, zv);
#pragma unroll
            for (int f = 0; f < 4; ++f) Pk4T<TT>::prep(zv[f], negzb[f], sp[f]);
            load_z(i + 1);
        }
#pragma unroll
        for (int st = 0; st < 4; ++st) {
            u32x4_t wv[WL];
#pragma unroll
            for (int h = 0; h < WL; ++h) wv[h] = wring[st][h];
            uint32_t wp[WL][4];
#pragma unroll
            for (int h = 0; h < WL; ++h) {
                const uint32_t w0 = wv[h][0], w1 = wv[h][1], w2 = wv[h][2], w3 = wv[h][3];
                wp[h][0] = w0, wp[h][1] = w1, wp[h][2] = w2, wp[h][3] = w3;
            }
            // row pair pp of column f as two exact 16-bit floats bias + q
            auto pair = [&](int pp, int f) -> uint32_t {
                if (BITS == 4) return TT::unpack1(wp[0][pp], f, nm);
                const uint32_t word = wp[(f >> 1) % WL][pp];
                return TT::unpack_bytes((f & 1) ? (word >> 8) : word);
            };
            uint32_t a[MT][4];
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) {
                const u32x4_t av = *(const u32x4_t *)(slot + mt * 4096 + a_rd[st]);
                const uint32_t a0 = av[0], a1 = av[1], a2 = av[2], a3 = av[3];
                a[mt][0] = a0, a[mt][1] = a1, a[mt][2] = a2, a[mt][3] = a3;
            }
            if (GS) {
                const bool fresh = st == 0;  // the block's sums start from zero: no clearing
#pragma unroll
                for (int f = 0; f < 4; ++f) {
                    uint32_t b[4];
#pragma unroll
                    for (int pp = 0; pp < 4; ++pp) b[pp] = pair(pp, f);
#pragma unroll
                    for (int mt = 0; mt < MT; ++mt)
                        tmp[mt][f] = Ops::mfma(a[mt], b, fresh ? zero4 : tmp[mt][f]);
                }
#pragma unroll
                for (int mt = 0; mt < MT; ++mt) tmps[mt] = Ops::mfma(a[mt], ones, fresh ? zero4 : tmps[mt]);
            } else {
#pragma unroll
                for (int f = 0; f < 4; ++f) {
                    uint32_t b[4];
#pragma unroll
                    for (int pp = 0; pp < 4; ++pp) b[pp] = Pk4T<TT>::deq(pair(pp, f), negzb[f], sp[f]);
#pragma unroll
                    for (int mt = 0; mt < MT; ++mt) acc[mt][f] = Ops::mfma(a[mt], b, acc[mt][f]);
                }
            }
            // PLACED (2).  Vector-memory requests, LDS writes and MFMAs stay inside their step (vector and
            // scalar arithmetic and LDS reads may move across): the ring refill above is then issued a block
            // ahead of its use, as written, instead of at the block's end with the other three.
            // Refill this ring slot after its last use, so that the new block can land in the same registers
            // (requested while the old value is live it lands in others, copied at the loop's end behind a wait
            // for the request): 17 / 33 / 48 rows f16 9.96 / 12.76 / 13.57 -> 9.85 / 12.57 / 13.44 us.
            load_w(i + 1, st, wring[st]);
            if constexpr (PLACED) __builtin_amdgcn_sched_barrier(0x106);
        }
        if (GS) {  // fold the block in: y += s * (sum - (bias + z) * rowsum), all f32
            uint32_t zv[4];
            zs_words(zring, zv);
            load_z(i + 1);
#pragma unroll
            for (int f = 0; f < 4; ++f) {
                const float sf = TT::to_f32((uint16_t)(zv[f] >> 16));
                const float nszb = sf * TT::to_f32((uint16_t)(zv[f] & 0xFFFFu));  // -s * (bias_f + z)
#pragma unroll
                for (int mt = 0; mt < MT; ++mt)
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        acc[mt][f][e] = fmaf(sf, tmp[mt][f][e], fmaf(nszb, tmps[mt][e], acc[mt][f][e]));
            }
        }
        // the next block's activations replace this one's (same wave: LDS accesses stay in order)
        // PLACED (3).  The x block stays in its registers until here: hoisted to the block's start (with all 16
        // fragments of the current block held in registers instead), its reload comes late in the block and
        // is waited for at the next block's start.
        if constexpr (PLACED) __builtin_amdgcn_sched_barrier(0);
        store_a(aring);
        load_a(i + 2, aring);
        // two and four row tiles as straight-line code: the requests for the block after next stay at the block's
        // end (four tiles at 64 rows, same box: f16 16.54 -> 16.37 us, bf16 18.42 -> 17.90; three tiles the same
        // either way)
        if constexpr (NBLK > 0 && (MT == 2 || MT == 4)) __builtin_amdgcn_sched_barrier(0);
    }

    pk4_epilogue<TT, MT>(acc, bias, y, ws, M, N, j, m0, act, wave, lane);
}

// ---------------------------------------------------------------------------
// One row tile, a wave's whole share requested up front (folded form).
//
// With at most NBLK blocks a wave (K = 4096: 4) there is nothing to ring: every load of the wave - x, weights
// and pairs of all its blocks - is issued before the first one is waited for, in the order of use, and the
// blocks are then worked off as they arrive.  No loop, so no loop-carried ring registers for the compiler to
// copy (a copy waits for the load behind it) and no request that can sink below a use.
// ---------------------------------------------------------------------------
template <typename TT, int BITS, int NBLK, int XQ, int NW, int WIN = NBLK>
__global__ __launch_bounds__(NW * 64) void pk4_front_kernel(const uint16_t *__restrict__ x,
                                                        const uint32_t *__restrict__ pw,
                                                        const uint16_t *__restrict__ bias,
                                                        uint16_t *__restrict__ y, float *__restrict__ ws,
                                                        int M, int K, int N, int bslice, int act) {
    typedef MfmaOps<TT> Ops;
    constexpr int MT = 1, AQ = XQ, SLOT = 16 * 256, OOB = 0x7FFFFF00, WL = BITS / 4;
    constexpr int BB = pk4_block_words(BITS) * 4;
    extern __shared__ __attribute__((aligned(16))) unsigned char pk4_lds[];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int ni = lane & 15, kb = lane >> 4;
    const int j = blockIdx.x;
    const int NB = K >> 7;
    const int sb0 = blockIdx.y * bslice;
    const int SB = min(NB, sb0 + bslice) - sb0;
    const int cbase = SB / NW, crem = SB % NW;
    const int nloc = cbase + (wave < crem ? 1 : 0);
    const int cb0 = sb0 + wave * cbase + min(wave, crem);
    unsigned char *slot = pk4_lds + wave * SLOT;

    const __amdgpu_buffer_rsrc_t rs_w = make_rsrc(pw + (size_t)j * NB * (BB / 4), (uint32_t)NB * (uint32_t)BB);
    const __amdgpu_buffer_rsrc_t rs_x = make_rsrc(x, (uint32_t)M * (uint32_t)K * 2u);
    const __amdgpu_buffer_rsrc_t rs_none = make_rsrc(pw, 0u);
    const int voff_w = lane * 16;
    const int voff_z = 1024 * WL * 4 + (ni * 4 + kb) * 4;
    int voff_a[AQ];
#pragma unroll
    for (int q = 0; q < AQ; ++q) {
        const int r = 4 * q + kb;
        voff_a[q] = r < M ? (r * K * 2 + ni * 16) : OOB;
    }
    int a_wr[4];
#pragma unroll
    for (int qq = 0; qq < 4; ++qq) a_wr[qq] = kb * 256 + (((ni ^ kb) ^ (qq << 2)) << 4);
    int a_rd[4];
#pragma unroll
    for (int st = 0; st < 4; ++st) a_rd[st] = ni * 256 + (((8 * (st >> 1) + 2 * kb + (st & 1)) ^ ni) << 4);
    const NibbleMasks nm = nibble_masks();

    u32x4_t av[WIN][AQ], wv[WIN][4][WL];
    uint32_t zv[WIN];
    auto request = [&](int b, u32x4_t (&a)[AQ], u32x4_t (&w)[4][WL], uint32_t &z) {
        const bool live = b < nloc;  // wave-uniform
        const __amdgpu_buffer_rsrc_t rx = live ? rs_x : rs_none, rw = live ? rs_w : rs_none;
        const int blk = cb0 + b;
#pragma unroll
        for (int q = 0; q < AQ; ++q) a[q] = __builtin_amdgcn_raw_buffer_load_b128(rx, voff_a[q], blk * 256, 0);
#pragma unroll
        for (int st = 0; st < 4; ++st)
#pragma unroll
            for (int h = 0; h < WL; ++h)
                w[st][h] = __builtin_amdgcn_raw_buffer_load_b128(rw, voff_w, blk * BB + (st * WL + h) * 1024, 2);
        z = __builtin_amdgcn_raw_buffer_load_b32(rw, voff_z, blk * BB, 2);
        __builtin_amdgcn_sched_barrier(0);  // blocks are requested in the order they are used
    };
#pragma unroll
    for (int b = 0; b < WIN; ++b) request(b, av[b], wv[b], zv[b]);
    // rows no load covers: zero once
#pragma unroll
    for (int q = AQ; q < 4; ++q) {
        const int row = 4 * q + kb;
        *(u32x4_t *)(slot + row * 256 + ((ni ^ (row & 15)) << 4)) = u32x4_t{0u, 0u, 0u, 0u};
    }
    __builtin_amdgcn_sched_barrier(0);  // every request above, before anything below

    float4_t acc[MT][4];
#pragma unroll
    for (int f = 0; f < 4; ++f) acc[0][f] = float4_t{0.f, 0.f, 0.f, 0.f};
    const uint32_t ones[4] = {TT::ONES, TT::ONES, TT::ONES, TT::ONES};
    const float4_t zero4 = float4_t{0.f, 0.f, 0.f, 0.f};

#pragma unroll
    for (int b = 0; b < NBLK; ++b) {
        // No branch around a block past the wave's share (zeros times zeros): behind a branch the compiler
        // sinks the block's requests to their use.
        {
#pragma unroll
            for (int q = 0; q < AQ; ++q) *(u32x4_t *)(slot + q * 1024 + a_wr[q & 3]) = av[b % WIN][q];
            float4_t tmp[4], tmps;
#pragma unroll
            for (int st = 0; st < 4; ++st) {
                uint32_t wp[WL][4];
#pragma unroll
                for (int h = 0; h < WL; ++h) {
                    const u32x4_t t = wv[b % WIN][st][h];
                    wp[h][0] = t[0], wp[h][1] = t[1], wp[h][2] = t[2], wp[h][3] = t[3];
                }
                auto pair = [&](int pp, int f) -> uint32_t {
                    if (BITS == 4) return TT::unpack1(wp[0][pp], f, nm);
                    const uint32_t word = wp[(f >> 1) % WL][pp];
                    return TT::unpack_bytes((f & 1) ? (word >> 8) : word);
                };
                uint32_t a[4];
                {
                    const u32x4_t t = *(const u32x4_t *)(slot + a_rd[st]);
                    a[0] = t[0], a[1] = t[1], a[2] = t[2], a[3] = t[3];
                }
                const bool fresh = st == 0;
#pragma unroll
                for (int f = 0; f < 4; ++f) {
                    uint32_t bq[4];
#pragma unroll
                    for (int pp = 0; pp < 4; ++pp) bq[pp] = pair(pp, f);
                    tmp[f] = Ops::mfma(a, bq, fresh ? zero4 : tmp[f]);
                }
                tmps = Ops::mfma(a, ones, fresh ? zero4 : tmps);
            }
            // the pairs of the four columns: the four lane groups fetched one word each
            const auto p16 = __builtin_amdgcn_permlane16_swap(zv[b % WIN], zv[b % WIN], false, false);
            const uint32_t even = p16[0], odd = p16[1];
            const auto pe = __builtin_amdgcn_permlane32_swap(even, even, false, false);
            const auto po = __builtin_amdgcn_permlane32_swap(odd, odd, false, false);
            const uint32_t zq[4] = {pe[0], po[0], pe[1], po[1]};
#pragma unroll
            for (int f = 0; f < 4; ++f) {
                const float sf = TT::to_f32((uint16_t)(zq[f] >> 16));
                const float nszb = sf * TT::to_f32((uint16_t)(zq[f] & 0xFFFFu));
#pragma unroll
                for (int e = 0; e < 4; ++e) acc[0][f][e] = fmaf(sf, tmp[f][e], fmaf(nszb, tmps[e], acc[0][f][e]));
            }
        }
        if constexpr (WIN < NBLK) {
            // a window of WIN blocks in flight: the next one goes into the registers this block has left
            if (b + WIN < NBLK) request(b + WIN, av[b % WIN], wv[b % WIN], zv[b % WIN]);
        }
    }
    pk4_epilogue<TT, MT, NW>(acc, bias, y, ws, M, N, j, 0, act, wave, lane);
}

// ---------------------------------------------------------------------------
// Narrow layers: strips of 16 columns (4-bit).
//
// A layer with few 64-column strips (a down projection, an attention projection) fills the chip
// only when K is also cut into slices, whose partial tiles a second launch has to add.  Stored in
// strips of 16 columns the same layer has four times as many strips, so that at one to four rows of x
// a workgroup per strip fills the chip with K inside the workgroup: one launch.  With more rows a
// workgroup takes four neighbouring strips (every strip re-reads x, which then outweighs the weights)
// and the launch has the shape of the 64-column form.
//
//   pw  [N/16 strips][K/128 blocks]{ [64 lanes][4 words] , [16 columns] {-z, s} pairs }     1088 bytes a block
//
// Lane l = (ni = l % 16, kb = l / 16) of a block holds, in word t (= MFMA step t of the block), the 8 rows
// 128*b + 64*(t/2) + 16*kb + 8*(t%2) .. +7 (the wide form's order) of column 16*strip + ni: row 2pp in nibble pp of the low half, row 2pp+1 in
// nibble pp of the high half, so the same AND-OR as in the wide form yields row pair pp as two exact
// 16-bit floats.  One 1 KB wave load is a block: a strip's words span the block's four steps, so the ring
// holds whole blocks and a block is requested when an earlier one starts.
// The conversion bias now goes with the row pair, not with the column (f16: 1024 for even pp, 64 for
// odd pp; bf16: 128): the pairs hold -z alone, the folded form takes the biases out with a second row
// sum (x against a fragment of the biases), the tile form keeps one constant per bias and column.
// ---------------------------------------------------------------------------

template <typename TT, bool GPTQ>
__global__ __launch_bounds__(256) void pk4n_prepack_kernel(const uint32_t *__restrict__ qw,
                                                           const uint32_t *__restrict__ qz,
                                                           const uint16_t *__restrict__ sc,
                                                           uint32_t *__restrict__ pw, int K, int N, int gshift) {
    const size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;
    const int NB = K >> 7;
    if (idx >= (size_t)(N >> 4) * NB * PK4N_BW) return;
    const int w = (int)(idx % PK4N_BW);
    const int b = (int)((idx / PK4N_BW) % NB), j = (int)(idx / ((size_t)PK4N_BW * NB));
    if (w < 256) {
        const int t = w & 3, l = w >> 2, ni = l & 15, kb = l >> 4;
        const int k = pk4_kk(4 * b + t, kb), col = 16 * j + ni;  // the wide form's step -> row order
        uint32_t v = 0;
#pragma unroll
        for (int r = 0; r < 8; ++r) v |= src_q<GPTQ, 4>(qw, k + r, col, N) << (4 * (r >> 1) + 16 * (r & 1));
        pw[idx] = v;
    } else {
        const int col = 16 * j + (w - 256);
        const int g = (b << 7) >> gshift;
        const int c = col % 8;
        const int slot = GPTQ ? c : ((c >> 1) | ((c & 1) << 2));
        const uint32_t z = ((qz[(size_t)g * (N / 8) + col / 8] >> (4 * slot)) & 15u) + (GPTQ ? 1u : 0u);
        pw[idx] = (uint32_t)TT::from_f32(-(float)z) | ((uint32_t)sc[(size_t)g * N + col] << 16);
    }
}

template <typename TT>
__global__ __launch_bounds__(256) void pk4n_dequant_kernel(const uint32_t *__restrict__ pw,
                                                           uint16_t *__restrict__ out, int K, int N) {
    const size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;  // over the weight words only
    const int NB = K >> 7;
    if (idx >= (size_t)(N >> 4) * NB * 256) return;
    const int w = (int)(idx % 256);
    const int b = (int)((idx / 256) % NB), j = (int)(idx / ((size_t)256 * NB));
    const uint32_t *blk = pw + ((size_t)j * NB + b) * PK4N_BW;
    const int t = w & 3, l = w >> 2, ni = l & 15, kb = l >> 4;
    const int k = pk4_kk(4 * b + t, kb), col = 16 * j + ni;
    const uint32_t wd = blk[w];
    const NibbleMasks nm = nibble_masks();
    Pk4N<TT> c;
    c.prep(blk[256 + ni]);
#pragma unroll
    for (int pp = 0; pp < 4; ++pp) {
        const uint32_t d = c.deq(TT::unpack1(wd, pp, nm), pp);
        out[(size_t)(k + 2 * pp) * N + col] = (uint16_t)(d & 0xFFFFu);
        out[(size_t)(k + 2 * pp + 1) * N + col] = (uint16_t)(d >> 16);
    }
}

template <typename TT, int MT, bool GS, int NS, int XQ, int NW>
__global__ __launch_bounds__(NW * 64) void pk4n_mfma_kernel(const uint16_t *__restrict__ x,
                                                        const uint32_t *__restrict__ pw,
                                                        const uint16_t *__restrict__ bias,
                                                        uint16_t *__restrict__ y, float *__restrict__ ws,
                                                        int M, int K, int N, int bslice) {
    typedef MfmaOps<TT> Ops;
    constexpr bool DUAL = TT::DTYPE == F16Traits::DTYPE;  // two conversion biases (see the layout note)
    // A single f16 strip: the row sums would be two MFMAs a step beside the strip's one, so the zero and
    // the conversion bias are taken off the weights instead - (bias + q) - (bias + z) is an exact packed
    // f16 add - and the block folds in with its scale alone.
    constexpr bool EXACT = GS && DUAL && NS == 1;
    constexpr int ROWS = 16 * MT, AQ = XQ, SLOT = ROWS * 256, OOB = 0x7FFFFF00, BB = PK4N_BW * 4;
    constexpr int WNT = MT < 4 ? 2 : 0;  // (nontemporal at 49 - 64 rows measured slower here: 4096 x 4096 11.90 against 11.51 us)
    extern __shared__ __attribute__((aligned(16))) unsigned char pk4_lds[];

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int ni = lane & 15, kb = lane >> 4;
    const int j = blockIdx.x;
    const int m0 = blockIdx.z * ROWS;
    const int NB = K >> 7;
    const int sb0 = blockIdx.y * bslice;
    const int SB = min(NB, sb0 + bslice) - sb0;
    const int cbase = SB / NW, crem = SB % NW;
    const int nloc = cbase + (wave < crem ? 1 : 0);
    const int cb0 = sb0 + wave * cbase + min(wave, crem);
    unsigned char *slot = pk4_lds + wave * SLOT;

    const __amdgpu_buffer_rsrc_t rs_w =
        make_rsrc(pw + (size_t)j * NS * NB * PK4N_BW, (uint32_t)NS * (uint32_t)NB * (uint32_t)BB);
    const __amdgpu_buffer_rsrc_t rs_x = make_rsrc(x, (uint32_t)M * (uint32_t)K * 2u);
    const __amdgpu_buffer_rsrc_t rs_none = make_rsrc(pw, 0u);
    const int voff_w = lane * 16, voff_z = 1024 + ni * 4;
    constexpr bool VA1 = MT >= 3;
    int voff_a[VA1 ? 1 : AQ];
#pragma unroll
    for (int q = 0; q < (VA1 ? 1 : AQ); ++q) {
        const int r = m0 + 4 * q + kb;
        voff_a[q] = r < M ? (r * K * 2 + ni * 16) : OOB;
    }
    uint32_t rowstep = 4u * (uint32_t)K * 2u;
    int a_wr[4];
#pragma unroll
    for (int qq = 0; qq < 4; ++qq) a_wr[qq] = kb * 256 + (((ni ^ kb) ^ (qq << 2)) << 4);
    int a_rd[4];
#pragma unroll
    for (int st = 0; st < 4; ++st) a_rd[st] = ni * 256 + (((8 * (st >> 1) + 2 * kb + (st & 1)) ^ ni) << 4);
    const NibbleMasks nm = nibble_masks();
#pragma unroll
    for (int q = AQ; q < 4 * MT; ++q) {
        const int row = 4 * q + kb;
        *(u32x4_t *)(slot + row * 256 + ((ni ^ (row & 15)) << 4)) = u32x4_t{0u, 0u, 0u, 0u};
    }

    // ring of RD blocks: a workgroup of four strips keeps one block ahead (4 KB a wave in flight, as the
    // wide form), a single strip two (its blocks are 1 KB; measured 4096 x 4096 / 4096 x 6144 / 8192 x 4096
    // at one row: one ahead 4.11 / 4.82 / 6.19 us, two 3.89 / 4.84 / 5.78, three 3.93 / 5.13 / 5.97)
    constexpr int RD = NS == 1 ? 3 : 2;
    // The tile form turns a block's pairs into its constants at the block's start, so one set of pair
    // registers serves every block; the folded forms need the pairs at the block's end and ring them too.
    constexpr int ZD = (GS || EXACT) ? RD : 1;
    u32x4_t aring[AQ], wr[RD][NS];
    uint32_t zr[ZD][NS];
    auto load_a = [&](int i, u32x4_t (&a)[AQ]) {
        const __amdgpu_buffer_rsrc_t rs = i < nloc ? rs_x : rs_none;
        const int blk = cb0 + i;
#pragma unroll
        for (int q = 0; q < AQ; ++q) {
            if (VA1) {
                if (q == 0) asm volatile("" : "+s"(rowstep));
                // no wrap-around: 15 row steps stay below 2^31 (K <= 2^24, checked on the host), so a row
                // past M - from the first offset or by the steps - lies beyond x (< 2 GiB) and reads zeros
                a[q] = __builtin_amdgcn_raw_buffer_load_b128(rs, (int)((uint32_t)voff_a[0] + (uint32_t)q * rowstep), blk * 256, 0);
            } else {
                a[q] = __builtin_amdgcn_raw_buffer_load_b128(rs, voff_a[q], blk * 256, 0);
            }
        }
    };
    auto load_z = [&](int i, uint32_t (&z)[NS]) {
        const __amdgpu_buffer_rsrc_t rs = i < nloc ? rs_w : rs_none;
#pragma unroll
        for (int f = 0; f < NS; ++f)
            z[f] = __builtin_amdgcn_raw_buffer_load_b32(rs, voff_z, (f * NB + cb0 + i) * BB, WNT);
    };
    auto load_w = [&](int i, u32x4_t (&w)[NS], uint32_t (&z)[NS]) {
        const __amdgpu_buffer_rsrc_t rs = i < nloc ? rs_w : rs_none;
#pragma unroll
        for (int f = 0; f < NS; ++f) {
            const int so = (f * NB + cb0 + i) * BB;
            w[f] = __builtin_amdgcn_raw_buffer_load_b128(rs, voff_w, so, WNT);
            if constexpr (ZD == RD) z[f] = __builtin_amdgcn_raw_buffer_load_b32(rs, voff_z, so, WNT);
        }
    };
    auto store_a = [&](const u32x4_t (&a)[AQ]) {
#pragma unroll
        for (int q = 0; q < AQ; ++q) *(u32x4_t *)(slot + q * 1024 + a_wr[q & 3]) = a[q];
    };

    u32x4_t afirst[AQ];
    load_a(0, afirst);
#pragma unroll
    for (int d = 0; d + 1 < RD; ++d) load_w(d, wr[d], zr[d % ZD]);
    if constexpr (ZD == 1) load_z(0, zr[0]);
    load_a(1, aring);

    float4_t acc[MT][NS];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int f = 0; f < NS; ++f) acc[mt][f] = float4_t{0.f, 0.f, 0.f, 0.f};
    const uint32_t ones[4] = {TT::ONES, TT::ONES, TT::ONES, TT::ONES};
    // the biases of row pairs 0..3 as a B fragment (f16: 1024, 64, 1024, 64)
    const uint32_t biases[4] = {0x64006400u, 0x54005400u, 0x64006400u, 0x54005400u};
    const float4_t zero4 = float4_t{0.f, 0.f, 0.f, 0.f};

    store_a(afirst);

    // one block: its weights are in ring half CUR; the next block is requested into the other half first
    auto block = [&](int i, auto cur_c) {
        constexpr int CUR = decltype(cur_c)::value, NXT = (CUR + RD - 1) % RD;
        constexpr int ZC = CUR % ZD, ZN = NXT % ZD;
        load_w(i + RD - 1, wr[NXT], zr[ZN]);
        float4_t tmp[GS ? MT : 1][NS], tmp1[GS ? MT : 1], tmpb[(GS && DUAL) ? MT : 1];
        Pk4N<TT> cst[(GS && !EXACT) ? 1 : NS];
        if (!GS || EXACT) {
#pragma unroll
            for (int f = 0; f < NS; ++f) cst[f].prep(zr[ZC][f]);
        }
        if constexpr (ZD == 1) load_z(i + 1, zr[0]);
#pragma unroll
        for (int st = 0; st < 4; ++st) {
            uint32_t a[MT][4];
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) {
                const u32x4_t av = *(const u32x4_t *)(slot + mt * 4096 + a_rd[st]);
                const uint32_t a0 = av[0], a1 = av[1], a2 = av[2], a3 = av[3];
                a[mt][0] = a0, a[mt][1] = a1, a[mt][2] = a2, a[mt][3] = a3;
            }
            const bool fresh = st == 0;
#pragma unroll
            for (int f = 0; f < NS; ++f) {
                const uint32_t w = wr[CUR][f][st];
                uint32_t b[4];
                if constexpr (!GS && MT == 4) cst[f].odd_from_even();
#pragma unroll
                for (int pp = 0; pp < 4; ++pp) {
                    const uint32_t pr = TT::unpack1(w, pp, nm);
                    if constexpr (EXACT) b[pp] = cst[f].minus_zero(pr, pp);
                    else b[pp] = GS ? pr : cst[f].deq(pr, pp);
                }
#pragma unroll
                for (int mt = 0; mt < MT; ++mt) {
                    if (GS) tmp[mt][f] = Ops::mfma(a[mt], b, fresh ? zero4 : tmp[mt][f]);
                    else acc[mt][f] = Ops::mfma(a[mt], b, acc[mt][f]);
                }
            }
            if (GS && !EXACT) {
#pragma unroll
                for (int mt = 0; mt < MT; ++mt) {
                    tmp1[mt] = Ops::mfma(a[mt], ones, fresh ? zero4 : tmp1[mt]);
                    if (DUAL) tmpb[mt] = Ops::mfma(a[mt], biases, fresh ? zero4 : tmpb[mt]);
                }
            }
        }
        if (GS) {  // y += s * ((sum - biased row sum) - z * row sum), all f32
#pragma unroll
            for (int f = 0; f < NS; ++f) {
                const uint32_t zw = zr[ZC][f];
                const float sf = TT::to_f32((uint16_t)(zw >> 16));
                const float nz = TT::to_f32((uint16_t)(zw & 0xFFFFu)) - (DUAL ? 0.0f : 128.0f);
#pragma unroll
                for (int mt = 0; mt < MT; ++mt)
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        if constexpr (EXACT) {
                            acc[mt][f][e] = fmaf(sf, tmp[mt][f][e], acc[mt][f][e]);
                        } else {
                            const float d = DUAL ? tmp[mt][f][e] - tmpb[mt][e] : tmp[mt][f][e];
                            acc[mt][f][e] = fmaf(sf, fmaf(nz, tmp1[mt][e], d), acc[mt][f][e]);
                        }
                    }
            }
        }
        store_a(aring);
        load_a(i + 2, aring);
        // the requests for the block after next stay here: sunk to their use in the next block (which the
        // scheduler does in some single-tile instantiations to save registers) they would be waited for at
        // once (bf16, 16 rows, 14336 x 4096: 13.0 -> 10.7 us).  The larger tiles schedule better without.
        if constexpr (MT == 1) __builtin_amdgcn_sched_barrier(0);
    };
    {
        int i = 0;
        if constexpr (RD == 2) {
            for (; i + 1 < nloc; i += 2) {
                block(i, std::integral_constant<int, 0>{});
                block(i + 1, std::integral_constant<int, 1>{});
            }
            if (i < nloc) block(i, std::integral_constant<int, 0>{});
        } else {
            static_assert(RD == 3, "the loop below is unrolled for a ring of three");
            for (; i + 2 < nloc; i += 3) {
                block(i, std::integral_constant<int, 0>{});
                block(i + 1, std::integral_constant<int, 1>{});
                block(i + 2, std::integral_constant<int, 2>{});
            }
            if (i < nloc) block(i, std::integral_constant<int, 0>{});
            if (i + 1 < nloc) block(i + 1, std::integral_constant<int, 1>{});
        }
    }

    pk4n_epilogue<TT, MT, NS, NW>(acc, bias, y, ws, M, N, j, m0, wave, lane);
}

// A single strip, up to 16 rows, a wave's whole share (at most NBLK blocks of 1 KB) requested up front, or WIN
// blocks of it with the next requested into a block's registers when it is worked off: the 16-column
// counterpart of pk4_front_kernel, 16 waves.
template <typename TT, int NBLK, int XQ, int WIN = NBLK>
__global__ __launch_bounds__(1024) void pk4n_front_kernel(const uint16_t *__restrict__ x,
                                                          const uint32_t *__restrict__ pw,
                                                          const uint16_t *__restrict__ bias,
                                                          uint16_t *__restrict__ y, float *__restrict__ ws,
                                                          int M, int K, int N, int bslice) {
    typedef MfmaOps<TT> Ops;
    constexpr bool DUAL = TT::DTYPE == F16Traits::DTYPE;  // f16: zero and bias come off the weights exactly
    constexpr int NW = 16, MT = 1, AQ = XQ, SLOT = 16 * 256, OOB = 0x7FFFFF00, BB = PK4N_BW * 4;
    extern __shared__ __attribute__((aligned(16))) unsigned char pk4_lds[];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int ni = lane & 15, kb = lane >> 4;
    const int j = blockIdx.x;
    const int NB = K >> 7;
    const int sb0 = blockIdx.y * bslice;
    const int SB = min(NB, sb0 + bslice) - sb0;
    const int cbase = SB / NW, crem = SB % NW;
    const int nloc = cbase + (wave < crem ? 1 : 0);
    const int cb0 = sb0 + wave * cbase + min(wave, crem);
    unsigned char *slot = pk4_lds + wave * SLOT;

    const __amdgpu_buffer_rsrc_t rs_w = make_rsrc(pw + (size_t)j * NB * PK4N_BW, (uint32_t)NB * (uint32_t)BB);
    const __amdgpu_buffer_rsrc_t rs_x = make_rsrc(x, (uint32_t)M * (uint32_t)K * 2u);
    const __amdgpu_buffer_rsrc_t rs_none = make_rsrc(pw, 0u);
    const int voff_w = lane * 16, voff_z = 1024 + ni * 4;
    int voff_a[AQ];
#pragma unroll
    for (int q = 0; q < AQ; ++q) {
        const int r = 4 * q + kb;
        voff_a[q] = r < M ? (r * K * 2 + ni * 16) : OOB;
    }
    int a_wr[4];
#pragma unroll
    for (int qq = 0; qq < 4; ++qq) a_wr[qq] = kb * 256 + (((ni ^ kb) ^ (qq << 2)) << 4);
    int a_rd[4];
#pragma unroll
    for (int st = 0; st < 4; ++st) a_rd[st] = ni * 256 + (((8 * (st >> 1) + 2 * kb + (st & 1)) ^ ni) << 4);
    const NibbleMasks nm = nibble_masks();

    u32x4_t av[WIN][AQ], wv[WIN];
    uint32_t zv[WIN];
    auto request = [&](int b, u32x4_t (&a)[AQ], u32x4_t &w, uint32_t &z) {
        const bool live = b < nloc;  // wave-uniform
        const __amdgpu_buffer_rsrc_t rx = live ? rs_x : rs_none, rw = live ? rs_w : rs_none;
        const int blk = cb0 + b;
#pragma unroll
        for (int q = 0; q < AQ; ++q) a[q] = __builtin_amdgcn_raw_buffer_load_b128(rx, voff_a[q], blk * 256, 0);
        w = __builtin_amdgcn_raw_buffer_load_b128(rw, voff_w, blk * BB, 2);
        z = __builtin_amdgcn_raw_buffer_load_b32(rw, voff_z, blk * BB, 2);
        __builtin_amdgcn_sched_barrier(0);  // blocks are requested in the order they are used
    };
#pragma unroll
    for (int b = 0; b < WIN; ++b) request(b, av[b], wv[b], zv[b]);
#pragma unroll
    for (int q = AQ; q < 4; ++q) {
        const int row = 4 * q + kb;
        *(u32x4_t *)(slot + row * 256 + ((ni ^ (row & 15)) << 4)) = u32x4_t{0u, 0u, 0u, 0u};
    }
    __builtin_amdgcn_sched_barrier(0);

    float4_t acc[MT][1];
    acc[0][0] = float4_t{0.f, 0.f, 0.f, 0.f};
    const uint32_t ones[4] = {TT::ONES, TT::ONES, TT::ONES, TT::ONES};
    const float4_t zero4 = float4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int b = 0; b < NBLK; ++b) {
        // no branch around a block past the wave's share (zeros times zeros): behind one the compiler sinks
        // the block's requests to their use
#pragma unroll
        for (int q = 0; q < AQ; ++q) *(u32x4_t *)(slot + q * 1024 + a_wr[q & 3]) = av[b % WIN][q];
        Pk4N<TT> cst;
        if constexpr (DUAL) cst.prep(zv[b % WIN]);
        float4_t tmp, tmp1;
#pragma unroll
        for (int st = 0; st < 4; ++st) {
            uint32_t a[4];
            {
                const u32x4_t t = *(const u32x4_t *)(slot + a_rd[st]);
                a[0] = t[0], a[1] = t[1], a[2] = t[2], a[3] = t[3];
            }
            const uint32_t w = wv[b % WIN][st];
            uint32_t bq[4];
#pragma unroll
            for (int pp = 0; pp < 4; ++pp) {
                const uint32_t pr = TT::unpack1(w, pp, nm);
                bq[pp] = DUAL ? cst.minus_zero(pr, pp) : pr;
            }
            const bool fresh = st == 0;
            tmp = Ops::mfma(a, bq, fresh ? zero4 : tmp);
            if constexpr (!DUAL) tmp1 = Ops::mfma(a, ones, fresh ? zero4 : tmp1);
        }
        const uint32_t zw = zv[b % WIN];
        const float sf = TT::to_f32((uint16_t)(zw >> 16));
        if constexpr (DUAL) {
#pragma unroll
            for (int e = 0; e < 4; ++e) acc[0][0][e] = fmaf(sf, tmp[e], acc[0][0][e]);
        } else {
            const float nz = TT::to_f32((uint16_t)(zw & 0xFFFFu)) - 128.0f;
#pragma unroll
            for (int e = 0; e < 4; ++e) acc[0][0][e] = fmaf(sf, fmaf(nz, tmp1[e], tmp[e]), acc[0][0][e]);
        }
        if constexpr (WIN < NBLK)
            if (b + WIN < NBLK) request(b + WIN, av[b % WIN], wv[b % WIN], zv[b % WIN]);
    }
    pk4n_epilogue<TT, MT, 1, NW>(acc, bias, y, ws, M, N, j, 0, wave, lane);
}

// ---------------------------------------------------------------------------
// host side
// ---------------------------------------------------------------------------
size_t pk4_weight_bytes(int64_t K, int64_t N, int bits) {
    return (size_t)(N / 64) * (size_t)(K / 128) * (size_t)pk4_block_words(bits) * 4;
}
size_t pk4_zs_bytes(int64_t, int64_t, int) { return 0; }  // the pairs live inside the blocks

bool pk4_eligible(const Wna16Problem &p) {
    if (p.bits != 4 && p.bits != 8) return false;
    if (p.K % 128 != 0 || p.N % 64 != 0 || p.group_size % 128 != 0) return false;
    // 32-bit offsets inside a strip and in x; one launch of the repack covers the copy
    if ((uint64_t)(p.K / 128) * pk4_block_words(p.bits) * 4 >= (1ull << 31) || p.K > (1 << 24)) return false;
    if (pk4_weight_bytes(p.K, p.N, p.bits) / 4 >= (1ull << 31) * 256) return false;
    return true;
}

int launch_pk4_prepack(oxq_ctx *ctx, hipStream_t s, const Wna16Problem &src, const Pk4Weights &dst) {
    const int K = (int)src.K, N = (int)src.N;
    const size_t words = pk4_weight_bytes(K, N, src.bits) / 4;
    const bool gptq = src.pack_dim == OXQ_PACK_IN;
    dim3 grid((unsigned)ceil_div((int64_t)words, 256)), block(256);
    char name[64];
    snprintf(name, sizeof name, "pk%d_prepack_%s%s", src.bits, gptq ? "gptq" : "awq", dst.strip == 16 ? "_n16" : "");
    set_plan(ctx, name, grid, block, 1, 1, 0);
    if (ctx->plan_only) return OXQ_OK;
    if (dst.strip == 16) {
#define OXQ_PPN(TTv, Gv)                                                                                  \
    hipLaunchKernelGGL((pk4n_prepack_kernel<TTv, Gv>), grid, block, 0, s, src.qweight, src.qzeros,        \
                       (const uint16_t *)src.scales, dst.pw, K, N, src.group_shift)
        if (src.dtype == OXQ_F16) { if (gptq) OXQ_PPN(F16Traits, true); else OXQ_PPN(F16Traits, false); }
        else { if (gptq) OXQ_PPN(BF16Traits, true); else OXQ_PPN(BF16Traits, false); }
#undef OXQ_PPN
        OXQ_HIP_CHECK(hipGetLastError());
        return OXQ_OK;
    }
    const int half = (int)dst.gate_half;
#define OXQ_PP(TTv, Gv, Bv)                                                                                     \
    hipLaunchKernelGGL((pk4_prepack_kernel<TTv, Gv, Bv>), grid, block, 0, s, src.qweight, src.qzeros,           \
                       (const uint16_t *)src.scales, dst.pw, K, N, src.group_shift, half)
    if (src.dtype == OXQ_F16) {
        if (src.bits == 4) { if (gptq) OXQ_PP(F16Traits, true, 4); else OXQ_PP(F16Traits, false, 4); }
        else { if (gptq) OXQ_PP(F16Traits, true, 8); else OXQ_PP(F16Traits, false, 8); }
    } else {
        if (src.bits == 4) { if (gptq) OXQ_PP(BF16Traits, true, 4); else OXQ_PP(BF16Traits, false, 4); }
        else { if (gptq) OXQ_PP(BF16Traits, true, 8); else OXQ_PP(BF16Traits, false, 8); }
    }
#undef OXQ_PP
    OXQ_HIP_CHECK(hipGetLastError());
    return OXQ_OK;
}

int launch_pk4_dequant(oxq_ctx *ctx, hipStream_t s, const Pk4Weights &w, void *out_kn) {
    const size_t words = (size_t)w.K * w.N * w.bits / 32;
    dim3 grid((unsigned)ceil_div((int64_t)words, 256)), block(256);
    char name[64];
    snprintf(name, sizeof name, "pk%d_dequant_%s", w.bits, w.dtype == OXQ_F16 ? "f16" : "bf16");
    set_plan(ctx, name, grid, block, 1, 1, 0);
    if (ctx->plan_only) return OXQ_OK;
    if (w.strip == 16) {
        if (w.dtype == OXQ_F16)
            hipLaunchKernelGGL((pk4n_dequant_kernel<F16Traits>), grid, block, 0, s, w.pw, (uint16_t *)out_kn, (int)w.K, (int)w.N);
        else
            hipLaunchKernelGGL((pk4n_dequant_kernel<BF16Traits>), grid, block, 0, s, w.pw, (uint16_t *)out_kn, (int)w.K, (int)w.N);
        OXQ_HIP_CHECK(hipGetLastError());
        return OXQ_OK;
    }
#define OXQ_DQ(TTv, Bv)                                                                           \
    hipLaunchKernelGGL((pk4_dequant_kernel<TTv, Bv>), grid, block, 0, s, w.pw, (uint16_t *)out_kn, \
                       (int)w.K, (int)w.N, (int)w.gate_half)
    if (w.dtype == OXQ_F16) {
        if (w.bits == 4) OXQ_DQ(F16Traits, 4); else OXQ_DQ(F16Traits, 8);
    } else {
        if (w.bits == 4) OXQ_DQ(BF16Traits, 4); else OXQ_DQ(BF16Traits, 8);
    }
#undef OXQ_DQ
    OXQ_HIP_CHECK(hipGetLastError());
    return OXQ_OK;
}

template <typename TT, int BITS, int NBLK, int XQ, int NW, int WIN = NBLK>
static int pk4_front_go(hipStream_t s, dim3 grid, const Pk4Problem &p, int bslice) {
    const size_t lds = (size_t)NW * 4096;
    static LdsGrant lds_grant;
    OXQ_HIP_CHECK(lds_grant.ensure((const void *)pk4_front_kernel<TT, BITS, NBLK, XQ, NW, WIN>, lds));
    hipLaunchKernelGGL((pk4_front_kernel<TT, BITS, NBLK, XQ, NW, WIN>), grid, dim3(NW * 64), lds, s, (const uint16_t *)p.x, p.w.pw,
                       (const uint16_t *)p.bias, (uint16_t *)p.y, (float *)p.ws, (int)p.M, (int)p.w.K, (int)p.w.N,
                       bslice, p.act);
    OXQ_HIP_CHECK(hipGetLastError());
    return OXQ_OK;
}

// one instantiation of pk4_mfma_kernel: its LDS grant, the launch, the error check
template <typename TT, int BITS, int MT, bool GS, int WD, int XQ, bool PLZ = false, int NBLK = 0>
static int pk4_mfma_go(oxq_ctx *ctx, hipStream_t s, dim3 grid, const Pk4Problem &p, int bslice) {
    const size_t lds = (size_t)8 * MT * 4096;
    static LdsGrant lds_grant;
    OXQ_HIP_CHECK(lds_grant.ensure((const void *)pk4_mfma_kernel<TT, BITS, MT, GS, WD, XQ, PLZ, NBLK>, lds));
    hipLaunchKernelGGL((pk4_mfma_kernel<TT, BITS, MT, GS, WD, XQ, PLZ, NBLK>), grid, dim3(512), lds, s,
                       (const uint16_t *)p.x, p.w.pw, (const uint16_t *)p.bias, (uint16_t *)p.y, (float *)ctx->workspace,
                       (int)p.M, (int)p.w.K, (int)p.w.N, bslice, tune(ctx, OXQ_TUNE_PK4_CONTIGUOUS, 1), p.act);
    OXQ_HIP_CHECK(hipGetLastError());
    return OXQ_OK;
}

template <typename TT, int BITS, int MT, bool GS, int XQ>
static int pk4_go4(oxq_ctx *ctx, hipStream_t s, dim3 grid, const Pk4Problem &p, int bslice, int front) {
    if constexpr (MT == 1 && GS) {
        Pk4Problem q = p;
        q.ws = ctx->workspace;
        const int share8 = (bslice + 7) / 8;
        if (front == 2) {  // 8 waves, one or two blocks in flight: the ring, unrolled
            if constexpr (BITS == 4) {
                // two blocks in flight pay on a long chain: from 5 blocks a wave on at up to 4 rows, from 7 at any
                if constexpr (XQ == 1) {
                    if (share8 == 5) return pk4_front_go<TT, BITS, 5, XQ, 8, 2>(s, grid, q, bslice);
                    if (share8 == 6) return pk4_front_go<TT, BITS, 6, XQ, 8, 2>(s, grid, q, bslice);
                }
                if (share8 >= 7) return pk4_front_go<TT, BITS, 8, XQ, 8, 2>(s, grid, q, bslice);
            }
            switch (share8) {
            case 1: return pk4_front_go<TT, BITS, 1, XQ, 8, 1>(s, grid, q, bslice);
            case 2: return pk4_front_go<TT, BITS, 2, XQ, 8, 1>(s, grid, q, bslice);
            case 3: return pk4_front_go<TT, BITS, 3, XQ, 8, 1>(s, grid, q, bslice);
            case 4: return pk4_front_go<TT, BITS, 4, XQ, 8, 1>(s, grid, q, bslice);
            case 5: return pk4_front_go<TT, BITS, 5, XQ, 8, 1>(s, grid, q, bslice);
            case 6: return pk4_front_go<TT, BITS, 6, XQ, 8, 1>(s, grid, q, bslice);
            default: return pk4_front_go<TT, BITS, 8, XQ, 8, 1>(s, grid, q, bslice);
            }
        }
        if (front == 1) {  // 16 waves, two blocks each: all of it requested first (4-bit), one at a time (8-bit)
            if constexpr (BITS == 4) {
                if constexpr (XQ <= 2) return pk4_front_go<TT, BITS, 2, XQ, 16>(s, grid, q, bslice);
            } else {
                return pk4_front_go<TT, BITS, 2, XQ, 16, 1>(s, grid, q, bslice);
            }
        }
    }
    constexpr int WD = Pk4Ring<MT, BITS>::WD;
    // Two to four row tiles whose K slice is four or five blocks a wave (K = 4096, 5120 unsliced; 4-bit layers also six
    // and eight, K = 6144, 8192) with one row-tile workgroup a strip: the block loop as straight-line code.  Two row
    // tiles with the memory operations placed by hand and the block-end requests pinned (PLZ) - unrolled without the
    // pins they are slower than the loop.  Same box, loop -> straight line, 4096 x 14336: 17 / 32 rows f16 9.85 / 11.04 ->
    // 9.66 / 10.45 us, bf16 14.37 / 14.55 -> 12.04 / 12.48, 8-bit f16 14.00 / 14.71 -> 13.26 / 14.14; 48 / 64 rows 4-bit f16
    // 13.66 / 16.40 -> 13.06 / 16.29, bf16 15.74 / 18.70 -> 15.23 / 17.91, 8-bit f16 17.09 / 20.4 -> 16.65 / 19.85; 32 rows on
    // 6144 x 16384 / 8192 x 28672 f16 15.69 / 35.45 -> 14.88 / 33.73, bf16 20.54 / 49.01 -> 17.24 / 39.82.
    if constexpr (MT >= 2) {
        constexpr bool PLZ = MT == 2;
        if (grid.z == 1 && bslice % 8 == 0 && tune(ctx, OXQ_TUNE_PK4_FRONT, 1)) {
            switch (bslice / 8) {
            case 4: return pk4_mfma_go<TT, BITS, MT, GS, WD, XQ, PLZ, 4>(ctx, s, grid, p, bslice);
            case 5: return pk4_mfma_go<TT, BITS, MT, GS, WD, XQ, PLZ, 5>(ctx, s, grid, p, bslice);
            case 6: if constexpr (BITS == 4) return pk4_mfma_go<TT, BITS, MT, GS, WD, XQ, PLZ, 6>(ctx, s, grid, p, bslice); break;
            case 8: if constexpr (BITS == 4) return pk4_mfma_go<TT, BITS, MT, GS, WD, XQ, PLZ, 8>(ctx, s, grid, p, bslice); break;
            default: break;
            }
        }
    }
    // a (nearly) full fourth row tile of a 4-bit layer on its own strip: the loop with hand-placed memory operations
    if constexpr (MT == 4 && BITS == 4) {
        if (grid.z == 1 && p.M > 56 && tune(ctx, OXQ_TUNE_PK4_PLACE64, 1))
            return pk4_mfma_go<TT, BITS, MT, GS, WD, XQ, true>(ctx, s, grid, p, bslice);
    }
    return pk4_mfma_go<TT, BITS, MT, GS, WD, XQ>(ctx, s, grid, p, bslice);
}

template <typename TT, int BITS, int MT, bool GS>
static int pk4_go(oxq_ctx *ctx, hipStream_t s, dim3 grid, const Pk4Problem &p, int bslice, int front) {
    // A single short tile: rows past M are known at launch, so the loads that would only fetch them
    // are left out (M = 1: 8.8 instead of 9.1 us on 4096 x 14336).
    if constexpr (MT == 1) {
        const int xq = tune(ctx, OXQ_TUNE_PK4_XQ, 1) ? (int)ceil_div(p.M, 4) : 4;
        if (xq == 1) return pk4_go4<TT, BITS, MT, GS, 1>(ctx, s, grid, p, bslice, front);
        if (xq == 2) return pk4_go4<TT, BITS, MT, GS, 2>(ctx, s, grid, p, bslice, front);
    }
    return pk4_go4<TT, BITS, MT, GS, 4 * MT>(ctx, s, grid, p, bslice, front);
}

// Which form multiplies.  The folded form (exact integers through the matrix cores, scale and
// zero applied per block in f32: the weight is never rounded) is what the reference's fused GEMV
// computes, so it serves that kernel's range of m: 16 rows for AWQ, 32 for GPTQ (gemv_rows).
// Above, the reference's tile GEMM rounds the dequantized weight to the activation type: bf16
// layers keep that (tile form); for f16 the rounding is 2^-12 of a weight, far inside the
// tolerance either way, and the folded form is the faster one up to three row tiles
// (4096 x 14336 f16: 17 rows 10.8 -> 9.9 us, 48 rows 14.3 -> 13.5 us; bf16 GPTQ 17 rows 13.3 -> 10.1 us).
// At four row tiles the fold costs what the dequant costs and its extra accumulators do not fit.
static bool pk4_folds(const oxq_ctx *ctx, const Pk4Problem &p, int mt) {
    if (mt == 1) return true;
    if (mt > 3 || !tune(ctx, OXQ_TUNE_PK4_FOLD, 1)) return false;
    const int gemv_rows = p.w.gemv_rows ? p.w.gemv_rows : 16;
    if (p.w.dtype == OXQ_F16) return true;
    return mt == 2 && p.M <= gemv_rows;
}

template <typename TT, int BITS>
static int pk4_by_mt(oxq_ctx *ctx, hipStream_t s, dim3 grid, const Pk4Problem &p, int bslice, int mt, int front) {
    const bool fold = pk4_folds(ctx, p, mt);
    switch (mt) {
    case 1: return pk4_go<TT, BITS, 1, true>(ctx, s, grid, p, bslice, front);
    case 2: return fold ? pk4_go<TT, BITS, 2, true>(ctx, s, grid, p, bslice, 0) : pk4_go<TT, BITS, 2, false>(ctx, s, grid, p, bslice, 0);
    case 3: return fold ? pk4_go<TT, BITS, 3, true>(ctx, s, grid, p, bslice, 0) : pk4_go<TT, BITS, 3, false>(ctx, s, grid, p, bslice, 0);
    default: return pk4_go<TT, BITS, 4, false>(ctx, s, grid, p, bslice, 0);
    }
}

// Strip width of a layer's resident copy: 16 columns for 4-bit layers of at most 128 64-column strips and a
// K of 32 - 112 blocks, or at most 80 strips and 16 - 31 blocks (the shapes that otherwise leave CUs idle or need
// K slices and a second launch), 64 otherwise.
int pk4_choose_strip(const oxq_ctx *ctx, int64_t K, int64_t N, int bits, int64_t gate_half) {
    // Measured (f16; 64-column strips, with K slices where few -> 16-column strips, one launch up to 8 rows),
    // at 1 / 4 / 16 / 64 rows of x:
    //    4096 x  4096   5.85 / -    / -     / -      ->  3.64 /  3.95 /  5.24 / 11.5 us
    //    4096 x  8192   6.69 / 6.87 /  7.74 / 13.83  ->  5.01 /  5.53 /  8.29 / 14.13
    //    8192 x  8192   9.99 / 10.1 / 10.98 / 19.86  ->  7.82 /  8.77 / 11.58 / 20.27
    //   11008 x  4096   8.39 / 8.43 /  9.17 / 16.53  ->  5.94 /  6.62 /  9.44 / 16.86
    //   14336 x  4096   8.92 / 9.12 / 10.06 / 18.20  ->  7.00 /  7.75 / 10.47 / 18.73
    // one to eight rows gain 12 - 30 %, 16 rows and more lose 2 - 8 % (four strips share a workgroup there and
    // a strip's 1 KB blocks cost more per-block work than the wide form's 4 KB).  Layers that fill the chip
    // with 64-column strips gain nothing (4096 x 14336: 7.49 / 7.50 / 8.40 / 16.3 against 7.45 / 8.23 / 9.11 /
    // 16.4; 5120 x 13824 and 8192 x 28672 alike), and on a very long K every strip's pass over x outweighs
    // the saved launch from 4 rows on (28672 x 8192: 23.2 / 23.4 us wide, 21.3 / 26.6 narrow).
    const int mode = tune(ctx, OXQ_TUNE_PK4_STRIP16, 1);  // 0 never, 1 by shape, 2 wherever the layout applies
    if (!mode || bits != 4 || gate_half || N % 64 != 0) return 64;
    if (mode == 2) return 16;
    // Shorter K (16 - 31 blocks: hidden sizes of 2048 - 3968) gains on layers up to 5120 columns, whose 64-column
    // strips leave most CUs idle (3584 x 3584 at 1 / 8 / 16 / 64 rows 5.79 / 6.08 / 6.80 / 13.6 -> 3.57 / 4.08 / 5.05 /
    // 12.45 us; 3072 x 3072 4.99 -> 3.41, 2048 x 2048 3.95 -> 3.14, 3584 x 4608 5.87 -> 4.28 at one row), and loses
    // from 16 rows on at 8192 columns (3072 x 8192: 5.32 / 6.35 -> 4.66 / 7.06 at 1 / 16 rows).  A K beyond 112 blocks
    // gains at 1 - 4 rows only (18944 x 3584: 9.88 / 10.52 -> 8.18 / 11.64 at 1 / 8 rows).
    const int64_t nb = K / 128, wide = N / 64;
    return (N / 16 >= 128 && ((nb >= 32 && nb <= 112 && wide <= 128) || (nb >= 16 && nb < 32 && wide <= 80))) ? 16 : 64;
}

template <typename TT, int MT, bool GS, int NS, int XQ, int NW = 8>
static int pk4n_go4(oxq_ctx *ctx, hipStream_t s, dim3 grid, const Pk4Problem &p, int bslice) {
    const size_t lds = (size_t)NW * MT * 4096;
    static LdsGrant lds_grant;  // one per instantiation
    OXQ_HIP_CHECK(lds_grant.ensure((const void *)pk4n_mfma_kernel<TT, MT, GS, NS, XQ, NW>, lds));
    hipLaunchKernelGGL((pk4n_mfma_kernel<TT, MT, GS, NS, XQ, NW>), grid, dim3(NW * 64), lds, s, (const uint16_t *)p.x, p.w.pw,
                       (const uint16_t *)p.bias, (uint16_t *)p.y, (float *)ctx->workspace, (int)p.M, (int)p.w.K,
                       (int)p.w.N, bslice);
    OXQ_HIP_CHECK(hipGetLastError());
    return OXQ_OK;
}

template <typename TT, int NBLK, int XQ, int WIN = NBLK>
static int pk4n_front_go(oxq_ctx *ctx, hipStream_t s, dim3 grid, const Pk4Problem &p, int bslice) {
    const size_t lds = (size_t)16 * 4096;
    static LdsGrant lds_grant;
    OXQ_HIP_CHECK(lds_grant.ensure((const void *)pk4n_front_kernel<TT, NBLK, XQ, WIN>, lds));
    hipLaunchKernelGGL((pk4n_front_kernel<TT, NBLK, XQ, WIN>), grid, dim3(1024), lds, s, (const uint16_t *)p.x, p.w.pw,
                       (const uint16_t *)p.bias, (uint16_t *)p.y, (float *)ctx->workspace, (int)p.M, (int)p.w.K,
                       (int)p.w.N, bslice);
    OXQ_HIP_CHECK(hipGetLastError());
    return OXQ_OK;
}

template <typename TT>
static int pk4n_by_shape(oxq_ctx *ctx, hipStream_t s, dim3 grid, const Pk4Problem &p, int bslice, int mt, int ns,
                         bool fold, bool w16, bool nfront) {
    if (ns == 1) {
        const int share = (bslice + 15) / 16;
        if (nfront && p.M <= 4 && share <= 8) {
            switch (share) {
            case 1: case 2: return pk4n_front_go<TT, 2, 1>(ctx, s, grid, p, bslice);
            case 3: return pk4n_front_go<TT, 3, 1>(ctx, s, grid, p, bslice);
            case 4: return pk4n_front_go<TT, 4, 1>(ctx, s, grid, p, bslice);
            case 5: return pk4n_front_go<TT, 5, 1>(ctx, s, grid, p, bslice);
            case 6: return pk4n_front_go<TT, 6, 1>(ctx, s, grid, p, bslice);
            case 7: return pk4n_front_go<TT, 7, 1>(ctx, s, grid, p, bslice);
            default: return pk4n_front_go<TT, 8, 1>(ctx, s, grid, p, bslice);
            }
        }
        if (nfront && p.M > 8 && share <= 2) return pk4n_front_go<TT, 2, 4>(ctx, s, grid, p, bslice);
        if (nfront && p.M > 8 && share == 3) return pk4n_front_go<TT, 3, 4, 2>(ctx, s, grid, p, bslice);  // two in flight
        if (nfront && p.M > 8 && share == 4) return pk4n_front_go<TT, 4, 4, 2>(ctx, s, grid, p, bslice);
        if (nfront && p.M <= 8 && share <= 8) {
            switch (share) {
            case 1: case 2: return pk4n_front_go<TT, 2, 2>(ctx, s, grid, p, bslice);
            case 3: return pk4n_front_go<TT, 3, 2>(ctx, s, grid, p, bslice);
            case 4: return pk4n_front_go<TT, 4, 2>(ctx, s, grid, p, bslice);
            case 5: return pk4n_front_go<TT, 5, 2>(ctx, s, grid, p, bslice);
            case 6: return pk4n_front_go<TT, 6, 2>(ctx, s, grid, p, bslice);
            case 7: return pk4n_front_go<TT, 7, 2>(ctx, s, grid, p, bslice);
            default: return pk4n_front_go<TT, 8, 2>(ctx, s, grid, p, bslice);
            }
        }
        if (w16) return pk4n_go4<TT, 1, true, 1, 1, 16>(ctx, s, grid, p, bslice);
        if (p.M <= 4) return pk4n_go4<TT, 1, true, 1, 1>(ctx, s, grid, p, bslice);
        if (p.M <= 8) return pk4n_go4<TT, 1, true, 1, 2>(ctx, s, grid, p, bslice);
        return pk4n_go4<TT, 1, true, 1, 4>(ctx, s, grid, p, bslice);
    }
    switch (mt) {
    case 1: {
        const int xq = tune(ctx, OXQ_TUNE_PK4_XQ, 1) ? (int)ceil_div(p.M, 4) : 4;
        if (xq == 1) return pk4n_go4<TT, 1, true, 4, 1>(ctx, s, grid, p, bslice);
        if (xq == 2) return pk4n_go4<TT, 1, true, 4, 2>(ctx, s, grid, p, bslice);
        return pk4n_go4<TT, 1, true, 4, 4>(ctx, s, grid, p, bslice);
    }
    case 2: return fold ? pk4n_go4<TT, 2, true, 4, 8>(ctx, s, grid, p, bslice) : pk4n_go4<TT, 2, false, 4, 8>(ctx, s, grid, p, bslice);
    case 3: return pk4n_go4<TT, 3, false, 4, 12>(ctx, s, grid, p, bslice);
    default: return pk4n_go4<TT, 4, false, 4, 16>(ctx, s, grid, p, bslice);
    }
}

// forward on a layer stored in 16-column strips
static int launch_pk4n_forward(oxq_ctx *ctx, hipStream_t s, const Pk4Problem &p) {
    const int64_t M = p.M, N = p.w.N;
    const int mt = M > 48 ? 4 : (int)ceil_div(M, 16);
    const int NB = (int)(p.w.K / 128);
    // One workgroup per strip when that gives the chip enough workgroups and x is small: every strip
    // re-reads x (four rows against a strip's 16 columns are what 16 rows are against 64).  Measured, f16,
    // single strip against four strips with K slices: 4096 x 4096 at 8 / 16 rows 4.32 / 5.27 against 6.11 /
    // 6.47 us; 8192 x 4096 6.38 / 8.24 against 7.47 / 8.32; 4096 x 6144 (384 strips, more than one round of
    // workgroups) 6.21 / 8.04 against 7.11 / 7.80: up to 8 rows always, up to 16 on a single round and short K.
    // Also up to 16 on whole rounds of 256 strips and K <= 8192 (9 / 16 rows: 8192 x 4096 6.90 / 8.07 against
    // 7.87 / 8.31, 4096 x 8192 6.49 / 7.81 against 7.53 / 8.31); not beyond (14336 x 4096 at 12 / 16 rows 11.2 / 12.4
    // against 10.3 / 10.7) and not on half a round (8192 x 2048 at 16 rows 7.52 against 6.63).
    const int ns1_rows = tune(ctx, OXQ_TUNE_PK4N_NS1_ROWS, ((N / 16 <= 256 && NB <= 32) || ((N / 16) % 256 == 0 && NB <= 64)) ? 16 : 8);
    const int ns = (M <= ns1_rows && M <= 16 && N / 16 >= 128) ? 1 : 4;
    const int64_t tiles = (N / (16 * ns)) * ceil_div(M, 16 * mt);
    int ks = 1;
    if (tiles <= 96 && NB >= 32) ks = (int)std::max<int64_t>(1, std::min<int64_t>(256 / tiles, NB / 8));
    else if (ns == 4 && tiles <= 128 && NB >= 64) ks = 2;  // as in the wide form; 128 single strips are faster whole
                                                           // (8192 x 2048 at one row: 5.20 against 5.65 us)
    ks = tune(ctx, OXQ_TUNE_PK4_KS, ks);
    ks = std::max(1, std::min(ks, NB));
    if (p.no_split) ks = 1;
    while (ks > 1 && (size_t)ks * M * N * 4 > ctx->workspace_bytes) --ks;
    const int bslice = (int)ceil_div(NB, ks);
    ks = (int)ceil_div(NB, bslice);
    if (ceil_div(M, 16 * mt) > 65535)
        return fail(OXQ_ERR_UNSUPPORTED, "repacked matmul: m = %lld exceeds the grid limit (65535 row tiles)", (long long)M);
    if (p.act) return fail(OXQ_ERR_ARG, "repacked matmul: a fused activation on a layer in 16-column strips");
    const bool fold = mt <= 2 && pk4_folds(ctx, p, mt);  // three row tiles of folded sums do not fit beside the two-block ring
    dim3 grid((unsigned)(N / (16 * ns)), (unsigned)ks, (unsigned)ceil_div(M, 16 * mt));
    // One or two rows of a single strip on a long K: 16 waves, so that a wave's chain of blocks is half as
    // long (f16, one / two rows, 8 -> 16 waves: 14336 x 4096 7.44 / 7.55 -> 7.00 / 7.37 us, 8192 x 2048 at one
    // row 4.75 -> 4.39; from three rows on, and at K = 4096, 8 waves are as fast or faster).
    // Up to eight rows of a single strip whose K slice is at most 128 blocks: 16 waves that request their whole
    // share (at most 8 blocks of 1 KB) before waiting for anything (pk4n_front_kernel).  Measured, f16, 1 / 4 /
    // 8 rows, against the ring: 4096 x 4096 3.48 / 3.84 / 4.21 against 3.70 / 3.89 / 4.36 us, 8192 x 4096 4.78 /
    // 5.38 / 6.21 against 5.02 / 5.40 / 6.44, 14336 x 4096 6.76 / 7.57 / 9.33 against 6.96 / 7.70 / 9.49,
    // 4096 x 8192 4.72 / 5.26 / 6.10 against 5.02 / 5.53 / 6.56.  With at most two blocks a wave (K <= 4096) also
    // the 9 - 16 rows that a single strip takes there: 4096 x 4096 at 9 / 16 rows 4.37 / 5.12 against 4.71 / 5.28;
    // with three or four blocks a wave (K <= 8192) two of them in flight: 8192 x 4096 at 9 / 12 / 16 rows 6.90 /
    // 7.41 / 8.07 -> 6.67 / 7.16 / 7.96.
    const bool nfront = ns == 1 && ceil_div(bslice, 16) <= 8 && tune(ctx, OXQ_TUNE_PK4_FRONT, 1) &&
                        (M <= 8 || (M <= 16 && ceil_div(bslice, 16) <= 4));
    const bool w16 = nfront || (ns == 1 && M <= 2 && tune(ctx, OXQ_TUNE_PK4N_W16, NB >= 64));
    char name[64];
    snprintf(name, sizeof name, "pk4_mfma_%s_mt%d%s_n16x%d", p.w.dtype == OXQ_F16 ? "f16" : "bf16", mt,
             (fold || ns == 1) ? "_gs" : "", ns);
    set_plan(ctx, name, grid, dim3(w16 ? 1024 : 512), ks, 1, ks > 1 ? (size_t)ks * M * N * 4 : 0);
    if (ctx->plan_only) {
        if (ks > 1) add_launch(ctx);
        return OXQ_OK;
    }
    if ((uint64_t)M * (uint64_t)p.w.K * 2 >= (1ull << 31))
        return fail(OXQ_ERR_UNSUPPORTED, "repacked matmul: x larger than 2 GiB");
    if (((uintptr_t)p.x | (uintptr_t)p.y) & 15)
        return fail(OXQ_ERR_UNSUPPORTED, "repacked matmul: x and y must be 16-byte aligned");
    const int rc = p.w.dtype == OXQ_F16 ? pk4n_by_shape<F16Traits>(ctx, s, grid, p, bslice, mt, ns, fold, w16, nfront)
                                        : pk4n_by_shape<BF16Traits>(ctx, s, grid, p, bslice, mt, ns, fold, w16, nfront);
    if (rc != OXQ_OK || ks == 1) return rc;
    return launch_splitk_reduce(ctx, s, (const float *)ctx->workspace, p.bias, p.y, M, N, ks, p.w.dtype);
}

int launch_pk4_forward(oxq_ctx *ctx, hipStream_t s, const Pk4Problem &p) {
    if (p.act && (!p.w.gate_half || p.act > 2))
        return fail(OXQ_ERR_ARG, "repacked matmul: activation %d on a layer that is not a fused gate|up layer", p.act);
    if (pk4_gemm_takes(ctx, p)) return launch_pk4_gemm(ctx, s, p);  // prefill sizes, either layout
    if (p.w.strip == 16) return launch_pk4n_forward(ctx, s, p);
    const int64_t M = p.M;
    const int mt = M > 48 ? 4 : (int)ceil_div(M, 16);
    const int NB = (int)(p.w.K / 128);
    // Few column strips and a long K (a down projection: N = 4096 is 64 strips for 256 CUs):
    // K is also cut into slices, at least one block per wave, so that up to one workgroup per CU
    // runs; the slices' f32 partial tiles are added in slice order by a second launch.  Measured
    // (f16, M = 1 / 16): 14336 x 4096 16.9 / 19.1 us unsplit, 9.0 / 10.0 us in 4 slices, 9.5 - 10.2 /
    // 11.4 - 12.1 us in 3, 6 or 8; a 4096 x 4096 layer 6.4 / 7.4 us unsplit, 5.7 / 6.6 us in 4 slices.
    const int64_t tiles = (p.w.N / 64) * ceil_div(M, 16 * mt);
    int ks = 1;
    if (tiles <= 96 && NB >= 32) ks = (int)std::max<int64_t>(1, std::min<int64_t>(256 / tiles, NB / 8));
    // Half a round of workgroups and a long K: two slices.  Measured (f16, 1 / 16 / 64 rows): 8192 x 8192
    // 11.3 / 12.9 / 26.3 us unsplit, 9.9 / 10.9 / 20.0 us in two slices; 28672 x 8192 32.5 / 37.6 / 78.2
    // against 23.3 / 25.9 / 49.4 us (four slices: 23.4 / 26.8 / 54.2).  At K = 4096 or 5120 the second
    // launch costs more than the slices save (4096 x 8192: 6.7 / 7.8 / 13.5 against 7.0 / 8.0 / 14.9 us).
    else if (tiles <= 128 && NB >= 64) ks = 2;
    ks = tune(ctx, OXQ_TUNE_PK4_KS, ks);
    ks = std::max(1, std::min(ks, NB));
    if (p.act) ks = 1;  // the activation needs the whole sum: gate|up layers are wide, one slice fills the chip
    if (p.no_split) ks = 1;
    while (ks > 1 && (size_t)ks * M * p.w.N * 4 > ctx->workspace_bytes) --ks;
    const int bslice = (int)ceil_div(NB, ks);
    ks = (int)ceil_div(NB, bslice);  // no empty slice
    if (ceil_div(M, 16 * mt) > 65535)
        return fail(OXQ_ERR_UNSUPPORTED, "repacked matmul: m = %lld exceeds the grid limit (65535 row tiles)", (long long)M);
    dim3 grid((unsigned)(p.w.N / 64), (unsigned)ks, (unsigned)ceil_div(M, 16 * mt));
    char name[64];
    // A single row tile (up to 16 rows) runs straight-line kernels (pk4_front_kernel) where one exists for the
    // slice: no loop, so no loop-carried ring registers to copy (and wait for) at its end, and every request
    // placed where the source puts it.  Which form, measured side by side on one box (f16, us; "ring" is
    // pk4_mfma_kernel, "16w" 16 waves that request their whole share first, "8w1" / "8w2" 8 waves with one / two
    // blocks in flight, the next requested into a block's registers when it is worked off):
    //   4-bit          rows             ring                        16w                         8w1                         8w2
    //   2048 x 16384   1 / 4 / 16       5.15 / 5.25 / 5.96          5.00 / 5.08 / 5.55          4.91 / 5.04 / 5.36          4.93 / 5.12 / 5.64
    //   4096 x 14336   1 / 4 / 8 / 16   7.54 / 7.55 / 7.93 / 8.66   6.86 / 7.06 / 7.45 / 8.29   7.11 / 7.40 / 7.50 / 7.92   6.99 / 7.11 / 7.77 / 8.32
    //   5120 x 13824   1 / 4 / 8 / 16   8.90 / 8.96 / 9.31 / 10.4   8.51 / 8.76 / - / -         8.35 / 8.43 / 8.72 / 9.84   7.93 / 8.26 / 8.79 / 10.2
    //   6144 x 16384   1 / 4 / 8 / 16   10.5 / 10.6 / 11.0 / 12.3   10.2 / 10.3 / - / -         10.1 / 10.3 / 10.3 / 11.3   10.1 / 10.2 / 10.6 / 11.9
    //   8192 x 28672   1 / 4 / 8 / 16   22.7 / 23.2 / 24.8 / 27.3   21.6 / 22.2 / - / -         22.4 / 23.0 / 23.9 / 25.7   21.1 / 21.5 / 22.4 / 25.4
    //   8-bit                                                       (16 waves, one in flight)
    //   4096 x 14336   1 / 4 / 16       11.8 / 12.2 / 13.1          10.75 / 11.00 / 11.70       11.14 / 11.49 / 12.19       10.99 / 11.34 / 12.33
    //   5120 x 13824   1 / 4 / 16       12.96 / 13.3 / 15.0         -                           12.38 / 12.81 / 14.57       12.80 / 13.14 / 15.20
    //   6144 x 16384   1 / 4 / 16       17.75 / 17.95 / 18.65       17.20 / 17.40 / 18.26       17.29 / 17.49 / 18.00       17.32 / 17.53 / 19.03
    // (16 waves that request a whole 8-bit share first have twice the bytes in flight and lose: 5120 x 13824 at one
    // row 14.5 - 16.9 us.)  A wave whose share is short of the kernel's block count multiplies a block of zeros
    // through: 40 blocks over 16 waves (2 or 3 each) lose what 5 each over 8 waves do not.  The rule:
    //   4-bit  32 blocks, up to 8 rows: 16w.  Otherwise 8 waves for up to 8 blocks a wave (K <= 8192 unsliced), two
    //          in flight from 5 blocks a wave on at up to 4 rows and from 7 on at any, else one.
    //   8-bit  32 blocks in a single slice: 16 waves, one block in flight.  Otherwise 8w1 where every wave's share is
    //          whole and the kernel exists for it (1 - 6, 8).
    const int front_xq = tune(ctx, OXQ_TUNE_PK4_XQ, 1) ? (int)ceil_div(M, 4) : 4;
    const int front_mode = tune(ctx, OXQ_TUNE_PK4_FRONT, 1);  // 0: the ring kernel, 2: never 16 waves
    const int share8 = (bslice + 7) / 8;
    int front = 0;
    if (mt == 1 && front_mode != 0) {
        if (p.w.bits == 4)
            front = (front_mode != 2 && bslice == 32 && front_xq <= 2) ? 1 : share8 <= 8 ? 2 : 0;
        else
            front = (front_mode != 2 && bslice == 32 && ks == 1) ? 1 : (bslice % 8 == 0 && share8 <= 8 && share8 != 7) ? 2 : 0;
    }
    snprintf(name, sizeof name, "pk%d_mfma_%s_mt%d%s%s%s", p.w.bits, p.w.dtype == OXQ_F16 ? "f16" : "bf16", mt,
             pk4_folds(ctx, p, mt) ? "_gs" : "", front == 1 ? "_front" : front == 2 ? "_line" : "",
             p.act == 1 ? "_silu" : p.act == 2 ? "_gelu" : "");
    set_plan(ctx, name, grid, dim3(front == 1 ? 1024 : 512), ks, 1, ks > 1 ? (size_t)ks * M * p.w.N * 4 : 0);
    if (ctx->plan_only) {
        if (ks > 1) add_launch(ctx);
        return OXQ_OK;
    }
    if ((uint64_t)M * (uint64_t)p.w.K * 2 >= (1ull << 31))
        return fail(OXQ_ERR_UNSUPPORTED, "repacked matmul: x larger than 2 GiB");
    if (((uintptr_t)p.x | (uintptr_t)p.y) & 15)
        return fail(OXQ_ERR_UNSUPPORTED, "repacked matmul: x and y must be 16-byte aligned");
    const bool f16 = p.w.dtype == OXQ_F16;
    int rc;
    if (tune(ctx, OXQ_TUNE_PK4_T64, 1) && pk4_tile64_takes(p, ks)) {
        Pk4Problem q = p;
        q.ws = ctx->workspace;
        return launch_pk4_tile64(ctx, s, q);
    }
    if (p.w.bits == 4)
        rc = f16 ? pk4_by_mt<F16Traits, 4>(ctx, s, grid, p, bslice, mt, front)
                 : pk4_by_mt<BF16Traits, 4>(ctx, s, grid, p, bslice, mt, front);
    else
        rc = f16 ? pk4_by_mt<F16Traits, 8>(ctx, s, grid, p, bslice, mt, front)
                 : pk4_by_mt<BF16Traits, 8>(ctx, s, grid, p, bslice, mt, front);
    if (rc != OXQ_OK || ks == 1) return rc;
    return launch_splitk_reduce(ctx, s, (const float *)ctx->workspace, p.bias, p.y, M, p.w.N, ks, p.w.dtype);
}

}  // namespace oxq
