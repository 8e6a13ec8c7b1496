// Resident 4-bit layers in a tile-major layout: load-time repack + the
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
// Layout (K % 128 == 0, N % 64 == 0, group size a multiple of 128, at most 128 groups):
//
//   pw  [N/64 strips][K/32 steps][64 lanes][4 words]      4 bits per weight
//   pzs [N/64 strips][K/g groups][16 columns-of-4][4]     one word per column and group
//
// Step t of a strip covers 32 rows of K.  Lane l = (ni = l % 16, kb = l / 16)
// owns the 8 rows  kk = 64*(t/2) + 16*kb + 8*(t%2) .. +7  of the four columns
// 64*strip + 4*ni + f, f = 0..3: exactly one MFMA B fragment per f.  Word pp
// (0..3) holds rows kk+2pp (low 16 bits) and kk+2pp+1 (high 16 bits), four
// nibbles each, nibble f = column f.  Two consecutive steps therefore cover 16
// consecutive rows per lane group, so the matching activation loads are 32
// contiguous bytes per row.  One AND-OR per fragment register turns a row pair
// into two exact 16-bit floats (bias + q).  A pzs word is {-(bias_f + z), s} as
// two 16-bit floats of the layer's dtype (z already includes GPTQ's +1).

//
// 8-bit layers use the same scheme with two 1 KB loads per step: half h (0..1) of a step
// holds the column pair f = 2h, 2h+1; word pp = {q[kk+2pp][2h], q[kk+2pp][2h+1],
// q[kk+2pp+1][2h], q[kk+2pp+1][2h+1]} as bytes, so an AND-OR of bytes 0 and 2 (after a
// shift by 8 for the odd column) again yields a row pair as two exact 16-bit floats.

#include "oxq_device.hpp"
#include "oxq_internal.hpp"
#include "oxq_mfma.hpp"

#include <algorithm>
#include <cstdlib>

namespace oxq {

// B = T((q - z) * s) for a pair of weights, from one pzs word {-(bias_f + z), s}.
// prep() turns the word into two per-group registers, deq() applies them to a pair of
// (bias_f + q).  f16: packed add (exact) and packed multiply (one rounding).  bf16 has no
// packed arithmetic here: fma((bias + q), s, -(bias + z) * s) in f32 is exact (both
// products fit 16 bits, their sum is the 13-bit (q - z) * s), then one hardware
// round-to-nearest-even conversion of the pair.
typedef float float2_t __attribute__((ext_vector_type(2)));
template <typename TT> struct Pk4T;
template <> struct Pk4T<F16Traits> {
    __device__ static __forceinline__ void prep(uint32_t zs, uint32_t &c0, uint32_t &c1) {
        c0 = perm_b32(zs, zs, 0x01000100u);
        c1 = perm_b32(zs, zs, 0x03020302u);
    }
    __device__ static __forceinline__ uint32_t deq(uint32_t p, uint32_t c0, uint32_t c1) {
        return MfmaOps<F16Traits>::dequant_pair(p, c0, c1);
    }
};
template <> struct Pk4T<BF16Traits> {
    __device__ static __forceinline__ void prep(uint32_t zs, uint32_t &c0, uint32_t &c1) {
        const float sf = __builtin_bit_cast(float, zs & 0xFFFF0000u);
        const float nz = __builtin_bit_cast(float, zs << 16);
        c0 = __builtin_bit_cast(uint32_t, sf);
        c1 = __builtin_bit_cast(uint32_t, nz * sf);
    }
    __device__ static __forceinline__ uint32_t deq(uint32_t p, uint32_t c0, uint32_t c1) {
        const float sf = __builtin_bit_cast(float, c0), c = __builtin_bit_cast(float, c1);
        const float lo = __builtin_fmaf(__builtin_bit_cast(float, p << 16), sf, c);
        const float hi = __builtin_fmaf(__builtin_bit_cast(float, p & 0xFFFF0000u), sf, c);
        return __builtin_bit_cast(uint32_t, __builtin_convertvector(float2_t{lo, hi}, bf16x2_t));
    }
};

__device__ __forceinline__ int pk4_kk(int t, int kb) { return ((t >> 1) << 6) + (kb << 4) + ((t & 1) << 3); }

// Resident column -> checkpoint column.  A fused gate|up layer (half = N/2) keeps, in every strip
// of 64, 32 gate columns followed by the 32 up columns they are multiplied with, so that one
// workgroup holds both factors of its outputs.
__device__ __forceinline__ int pk4_src_col(int c, int half) {
    if (!half) return c;
    const int j = c >> 6, cc = c & 63;
    return cc < 32 ? 32 * j + cc : half + 32 * j + (cc - 32);
}

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

template <bool GPTQ, int BITS>
__global__ __launch_bounds__(256) void pk4_prepack_weights_kernel(const uint32_t *__restrict__ qw,
                                                                  uint32_t *__restrict__ pw, int K, int N,
                                                                  int half) {
    const size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;
    const size_t total = (size_t)K * N * BITS / 32;
    if (idx >= total) return;
    const int NS = K >> 5;
    const int pp = (int)(idx & 3), l = (int)((idx >> 2) & 63);
    const int h = BITS == 8 ? (int)((idx >> 8) & 1) : 0;
    const size_t st = idx >> (BITS == 8 ? 9 : 8);
    const int t = (int)(st % NS), j = (int)(st / NS);
    const int ni = l & 15, kb = l >> 4;
    const int k = pk4_kk(t, kb) + 2 * pp;
    uint32_t w = 0;
    if (BITS == 4) {
#pragma unroll
        for (int r = 0; r < 2; ++r)
#pragma unroll
            for (int f = 0; f < 4; ++f)
                w |= src_q<GPTQ, BITS>(qw, k + r, pk4_src_col(64 * j + 4 * ni + f, half), N) << (16 * r + 4 * f);
    } else {
#pragma unroll
        for (int r = 0; r < 2; ++r)
#pragma unroll
            for (int c = 0; c < 2; ++c)
                w |= src_q<GPTQ, BITS>(qw, k + r, pk4_src_col(64 * j + 4 * ni + 2 * h + c, half), N) << (16 * r + 8 * c);
    }
    pw[idx] = w;
}

template <typename TT, bool GPTQ, int BITS>
__global__ __launch_bounds__(256) void pk4_prepack_zs_kernel(const uint32_t *__restrict__ qz,
                                                             const uint16_t *__restrict__ sc,
                                                             uint32_t *__restrict__ pzs, int G, int N, int half) {
    constexpr int PF = 32 / BITS;
    const size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= (size_t)G * N) return;
    const int f = (int)(idx & 3), ni = (int)((idx >> 2) & 15);
    const size_t jg = idx >> 6;
    const int g = (int)(jg % G), j = (int)(jg / G);
    const int col = pk4_src_col(64 * j + 4 * ni + f, half);
    const int c = col % PF;
    const int slot = (GPTQ || BITS == 8) ? c : ((c >> 1) | ((c & 1) << 2));
    const uint32_t z = ((qz[(size_t)g * (N / PF) + col / PF] >> (BITS * slot)) & ((1u << BITS) - 1u)) + (GPTQ ? 1u : 0u);
    const float b = BITS == 4 ? TT::bias(f) : TT::BYTE_BIAS;
    const uint32_t nz = TT::from_f32(-((float)z + b));
    pzs[idx] = nz | ((uint32_t)sc[(size_t)g * N + col] << 16);
}

// ---------------------------------------------------------------------------
// dense dequant of a resident layer -> [K, N] (linear.rs:510-523 fallback);
// the same arithmetic as the matmul kernel's B fragments.
// ---------------------------------------------------------------------------
template <typename TT, int BITS>
__global__ __launch_bounds__(256) void pk4_dequant_kernel(const uint32_t *__restrict__ pw,
                                                          const uint32_t *__restrict__ pzs,
                                                          uint16_t *__restrict__ out, int K, int N, int gshift,
                                                          int half) {
    const size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= (size_t)K * N * BITS / 32) return;
    const int NS = K >> 5, G = K >> gshift;
    const int pp = (int)(idx & 3), l = (int)((idx >> 2) & 63);
    const int h = BITS == 8 ? (int)((idx >> 8) & 1) : 0;
    const size_t st = idx >> (BITS == 8 ? 9 : 8);
    const int t = (int)(st % NS), j = (int)(st / NS);
    const int ni = l & 15, kb = l >> 4;
    const int k = pk4_kk(t, kb) + 2 * pp;
    const int g = k >> gshift;
    const uint32_t w = pw[idx];
    const NibbleMasks nm = nibble_masks();
#pragma unroll
    for (int c = 0; c < (BITS == 4 ? 4 : 2); ++c) {
        const int f = BITS == 4 ? c : 2 * h + c;
        const uint32_t zs = pzs[(((size_t)j * G + g) * 16 + ni) * 4 + f];
        uint32_t c0, c1;
        Pk4T<TT>::prep(zs, c0, c1);
        const uint32_t pair = BITS == 4 ? TT::unpack1(w, f, nm) : TT::unpack_bytes(c ? (w >> 8) : w);
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
// launcher); 8 waves split the slice between them in blocks of 128 rows (4 MFMA
// steps).  With more than one slice the workgroup writes its f32 partial tile to
// the workspace and a second launch adds the slices in order.
//
// Weights: one 1 KB wave load per step, issued one block (4 steps) ahead.
// Activations: the matrix-core fragment pattern (16 rows x 64 bytes per load)
// is served by L2 at a third of the rate of 256-byte row reads, so a wave
// fetches its next 16*MT x 128 block of x with 4-rows-x-256-bytes loads one
// block ahead, parks it in its private LDS slot (16-byte chunks XOR-swizzled by
// row, so both the row-wise write and the fragment read are conflict-free)
// and reads fragments from there.  Rows past M are never fetched (out-of-range
// lane offset: the buffer unit returns zero without touching memory).
// All vector loads are issued unconditionally - steps past the end of a
// wave's slice also use the out-of-range offset - so the compiler can count
// exactly how many loads are younger than the one it waits for; a conditionally
// issued load makes it wait for all of them, which serialises the pipeline.
// Activation loads of block b+1 are issued before the weight loads of block
// b+2: loads retire in order, and this way waiting for the former leaves the
// latter in flight.  Zeros and scales are staged in LDS once (below).
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
//    accumulator layout, and once per group
//        y += s * (acc_g - (bias + z) * rowsum_g(x))            (all f32).
// ---------------------------------------------------------------------------
// The integers the GS form feeds the matrix cores: bias_f + q, the same AND-OR unpack as
// the other form (f16: 1024 + q or 64 + q by nibble position, bf16: 128 + q).
// Ring depths: weights WD steps (1 KB wave loads), activations AB 128-row blocks (registers; the
// current block's activations live in LDS).  One block of weights in flight per wave is the
// measured optimum (4096 x 14336, f16, M = 1 / 16 / 64): 4 steps 8.8 / 9.2 / 18.1 us, 8 steps
// 9.0 / 9.7 / 18.0 (8.9 / 9.9 / 18.5 with whole-block slots), 16 steps 9.6 at M = 1, 2 steps
// equal on this shape and 0.4 us slower on 4096 x 4096; 3 and 6 steps (a three-block loop body)
// cost 0.5 - 2 us.  A CU takes only so many vector loads in flight: what the first waves issue
// beyond their next block keeps the other waves' first loads waiting.
template <int MT, int BITS> struct Pk4Ring {
    static constexpr int AB = 1;
    static constexpr int WD = 4;
};

// BPG1: group size 128, i.e. every block is one group (no group bookkeeping).
// XQ: activation loads per block and lane that can hold rows below M (4 rows each); the
// launcher passes 4 * MT, or fewer for a short single tile, whose other rows stay zero in LDS.
// ZW: every wave stages the zeros and scales of its own groups (no barrier before the loop).
template <typename TT, int BITS, int MT, bool GS, bool BPG1, int AB, int WD, int XQ, bool ZW>
__global__ __launch_bounds__(512) void pk4_mfma_kernel(const uint16_t *__restrict__ x,
                                                       const uint32_t *__restrict__ pw,
                                                       const uint32_t *__restrict__ pzs,
                                                       const uint16_t *__restrict__ bias,
                                                       uint16_t *__restrict__ y, float *__restrict__ ws,
                                                       int M, int K, int N, int gshift, int gslice,
                                                       int interleave, int act) {
    typedef MfmaOps<TT> Ops;
    constexpr int NW = 8, NT = NW * 64;        // waves and threads per workgroup (4 and 16 waves measured 30 % slower)
    constexpr int ROWS = 16 * MT;
    constexpr int AQ = XQ;                     // activation loads per block and lane
    constexpr int SLOT = ROWS * 256;           // bytes of one wave's LDS slot (= its partial tile)
    constexpr int OOB = 0x7FFFFF00;
    constexpr int WL = BITS / 4;               // 1 KB weight loads per step
    // Up to 48 rows there is one row tile, so every weight is read once per launch: nontemporal
    // loads (cache policy bit 1), which a bare read of the same 30 MB also gains 7 % from.
    // From 49 rows on several row tiles may share a strip through L2, so those keep the default.
    constexpr int WNT = MT < 4 ? 2 : 0;
    extern __shared__ __attribute__((aligned(16))) unsigned char pk4_lds[];
    // the strip's zeros and scales, [G][16 column quads]: GS = false the four {-(bias+z), s} words,
    // GS = true already converted for the group fold: float4 s, float4 -s * (bias + z)
    u32x4_t *zs_lds = (u32x4_t *)(pk4_lds + NW * SLOT);
    float4_t *zs_ldsf = (float4_t *)(pk4_lds + NW * SLOT);

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int ni = lane & 15, kb = lane >> 4;
    const int j = blockIdx.x;
    const int m0 = blockIdx.z * ROWS;
    const int NS = K >> 5, G = K >> gshift;
    const int bpg_mask = (1 << (gshift - 7)) - 1;  // blocks per group - 1
    // K slice of this workgroup (grid.y slices of `gslice` whole groups; one slice = the
    // whole strip unless the grid would leave most CUs idle), then the wave's blocks inside
    // it, by local index i: either one contiguous run of whole groups, the groups dealt out
    // as evenly as 8 waves allow, or (jointly staged kernels only, a tuning switch that measured
    // equal) every 8th group, the 8 waves then sweeping the slice together, front to back.
    const int gs7 = gshift - 7;
    const int sg0 = blockIdx.y * gslice;                 // first group of the slice
    const int SG = min(G, sg0 + gslice) - sg0;           // groups in the slice (>= 1)
    const int gbase = SG / NW, grem = SG % NW;
    const int wg0 = sg0 + wave * gbase + min(wave, grem);  // the wave's first group
    const int wgn = gbase + (wave < grem ? 1 : 0);         // and how many
    const int b0 = wg0 << gs7;
    const int nloc = interleave ? (wave < SG ? ((SG - wave + NW - 1) / NW) << gs7 : 0) : wgn << gs7;
    auto blk_of = [&](int i) {
        return interleave ? ((((((i >> gs7) * NW) + wave) + sg0) << gs7) | (i & bpg_mask)) : b0 + i;
    };
    unsigned char *slot = pk4_lds + wave * SLOT;

    const __amdgpu_buffer_rsrc_t rs_w = make_rsrc(pw + (size_t)j * NS * 256 * WL, (uint32_t)NS * 1024u * WL);
    const __amdgpu_buffer_rsrc_t rs_z = make_rsrc(pzs + (size_t)j * G * 64, (uint32_t)G * 256u);
    const __amdgpu_buffer_rsrc_t rs_x = make_rsrc(x, (uint32_t)M * (uint32_t)K * 2u);
    const int voff_w = lane * 16;
    // activation load q of a block: row 4q + lane/16, 16-byte chunk lane%16 of the row's 256 bytes
    int voff_a[AQ], a_wr[AQ];
#pragma unroll
    for (int q = 0; q < AQ; ++q) {
        const int row = 4 * q + kb, r = m0 + row;
        voff_a[q] = r < M ? (r * K * 2 + ni * 16) : OOB;
        a_wr[q] = row * 256 + ((ni ^ (row & 15)) << 4);  // = kb*256 + ((ni^kb)<<4), xor (4q&15)<<4, + 1024q
    }
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

    // Zeros and scales go to LDS, [G][16 column quads].  ZW: every wave stages those of its own
    // groups, so no barrier stands before its loop (7.85 instead of 8.45 us at M = 1, 5 % at
    // M = 33..48 and at 256).  The four-tile kernels are at their register budget: they do so with
    // one 16-byte chunk per lane, i.e. up to four groups a wave, and otherwise stage the slice
    // together and meet at a barrier.
    constexpr bool ZWAVE = ZW;
    constexpr int ZCH = ZW && MT == 4 ? 1 : 4;  // 16-byte chunks per lane (4 groups each) or thread
    u32x4_t zstage[ZCH];
    const int ZT = ZWAVE ? 64 : NT, zt = ZWAVE ? lane : (int)threadIdx.x;
    const int zc0 = ZWAVE ? (wg0 - sg0) * 16 : 0, zchunks = (ZWAVE ? wgn : SG) * 16;  // within the slice
#pragma unroll
    for (int q = 0; q < ZCH; ++q)
        if (q * ZT < zchunks)  // uniform
            zstage[q] = __builtin_amdgcn_raw_buffer_load_b128(
                rs_z, !ZWAVE || zt + q * ZT < zchunks ? (zc0 + zt + q * ZT) * 16 : OOB, sg0 * 256, 0);

    // blocks per unrolled iteration: the ring slot of every step must be a constant, 4 * U % WD == 0
    constexpr int U = (WD % 4 == 0 ? WD / 4 : (WD % 2 == 0 ? WD / 2 : WD)) * AB;
    static_assert((4 * U) % WD == 0 && U % AB == 0, "ring slots must repeat with the unrolled loop");
    u32x4_t aring[AB][AQ], wring[WD][WL];
    // Past the end of the slice the loads go through an empty descriptor: a scalar select,
    // no vector instruction, and the buffer unit returns zero without touching memory.
    const __amdgpu_buffer_rsrc_t rs_none = make_rsrc(pw, 0u);
    auto load_a = [&](int i, u32x4_t (&a)[AQ]) {
        const __amdgpu_buffer_rsrc_t rs = i < nloc ? rs_x : rs_none;  // wave-uniform
        const int blk = blk_of(i);
#pragma unroll
        for (int q = 0; q < AQ; ++q) a[q] = __builtin_amdgcn_raw_buffer_load_b128(rs, voff_a[q], blk * 256, 0);
    };
    auto load_w = [&](int i, int st, u32x4_t (&w)[WL]) {
        const __amdgpu_buffer_rsrc_t rs = i < nloc ? rs_w : rs_none;
#pragma unroll
        for (int h = 0; h < WL; ++h)
            w[h] = __builtin_amdgcn_raw_buffer_load_b128(rs, voff_w, ((blk_of(i) * 4 + st) * WL + h) * 1024, WNT);
    };
    auto store_a = [&](const u32x4_t (&a)[AQ]) {
#pragma unroll
        for (int q = 0; q < AQ; ++q) *(u32x4_t *)(slot + a_wr[q]) = a[q];
    };

    // issue order = consumption order: A(b0), W(b0), A(b0+1), W(b0+1), ...
    u32x4_t afirst[AQ];
    load_a(0, afirst);
#pragma unroll
    for (int g = 0; g < (WD < 4 ? WD : 4); ++g) load_w(g >> 2, g & 3, wring[g]);
#pragma unroll
    for (int d = 1; d <= AB; ++d) load_a(d, aring[d % AB]);
#pragma unroll
    for (int g = 4; g < WD; ++g) load_w(g >> 2, g & 3, wring[g]);

    float4_t acc[MT][4];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int f = 0; f < 4; ++f) acc[mt][f] = float4_t{0.f, 0.f, 0.f, 0.f};
    uint32_t negzb[4], sp[4];          // GS = false: the two Pk4T constants per column
    float sf[4], nszb[4];              // GS = true: s and -s * (bias + z) in f32
    // per-group accumulators of the GS form; with one block per group they live inside one
    // loop iteration (tmpb below), otherwise across iterations
    float4_t tmpg[GS ? MT : 1][4], tmpsg[GS ? MT : 1];
    if (GS && !BPG1) {
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            tmpsg[mt] = float4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int f = 0; f < 4; ++f) tmpg[mt][f] = float4_t{0.f, 0.f, 0.f, 0.f};
        }
    }
    const uint32_t ones[4] = {TT::ONES, TT::ONES, TT::ONES, TT::ONES};
    const float4_t zero4 = float4_t{0.f, 0.f, 0.f, 0.f};

#pragma unroll
    for (int q = 0; q < ZCH; ++q) {
        const int c = zc0 + zt + q * ZT;
        if (zt + q * ZT < zchunks) {
            if (GS) {
                const uint32_t z0 = zstage[q][0], z1 = zstage[q][1], z2 = zstage[q][2], z3 = zstage[q][3];
                const uint32_t zv[4] = {z0, z1, z2, z3};
                float4_t s4, n4;
#pragma unroll
                for (int f = 0; f < 4; ++f) {
                    s4[f] = TT::to_f32((uint16_t)(zv[f] >> 16));
                    n4[f] = s4[f] * TT::to_f32((uint16_t)(zv[f] & 0xFFFFu));  // -s * (bias_f + z)
                }
                zs_ldsf[2 * c] = s4;
                zs_ldsf[2 * c + 1] = n4;
            } else {
                zs_lds[c] = zstage[q];
            }
        }
    }
    store_a(afirst);
    if (!ZWAVE) __syncthreads();

    for (int ib = 0; ib < nloc; ib += U) {
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int i = ib + u;
            const bool live = i < nloc;  // wave-uniform
            const int blk = blk_of(i);
            const bool gfirst = BPG1 || (blk & bpg_mask) == 0;
            const bool glast = BPG1 || (blk & bpg_mask) == bpg_mask;
            float4_t tmpb[(GS && BPG1) ? MT : 1][4], tmpsb[(GS && BPG1) ? MT : 1];  // written at step 0
            auto &tmp = *(BPG1 ? &tmpb : &tmpg);
            auto &tmps = *(BPG1 ? &tmpsb : &tmpsg);
            if (live && gfirst) {  // first block of a group
                if (GS) {
                    const float4_t s4 = zs_ldsf[(((blk >> gs7) - sg0) * 16 + ni) * 2];
                    const float4_t n4 = zs_ldsf[(((blk >> gs7) - sg0) * 16 + ni) * 2 + 1];
                    sf[0] = s4[0], sf[1] = s4[1], sf[2] = s4[2], sf[3] = s4[3];
                    nszb[0] = n4[0], nszb[1] = n4[1], nszb[2] = n4[2], nszb[3] = n4[3];
                } else {
                    const u32x4_t zq = zs_lds[((blk >> gs7) - sg0) * 16 + ni];
                    const uint32_t z0 = zq[0], z1 = zq[1], z2 = zq[2], z3 = zq[3];
                    const uint32_t zv[4] = {z0, z1, z2, z3};
#pragma unroll
                    for (int f = 0; f < 4; ++f) Pk4T<TT>::prep(zv[f], negzb[f], sp[f]);
                }
            }
#pragma unroll
            for (int st = 0; st < 4; ++st) {
                u32x4_t wv[WL];
#pragma unroll
                for (int h = 0; h < WL; ++h) wv[h] = wring[(4 * u + st) % WD][h];
                load_w(i + (st + WD) / 4, (st + WD) & 3, wring[(4 * u + st) % WD]);  // refill this ring slot
                if (live) {
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
                        // with one block per group the first step starts from zero: no clearing
                        const bool fresh = BPG1 && st == 0;
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
                            for (int pp = 0; pp < 4; ++pp)
                                b[pp] = Pk4T<TT>::deq(pair(pp, f), negzb[f], sp[f]);
#pragma unroll
                            for (int mt = 0; mt < MT; ++mt) acc[mt][f] = Ops::mfma(a[mt], b, acc[mt][f]);
                        }
                    }
                }
            }
            if (GS && live && glast) {  // last block of the group: fold it in
#pragma unroll
                for (int mt = 0; mt < MT; ++mt) {
#pragma unroll
                    for (int f = 0; f < 4; ++f) {
#pragma unroll
                        for (int i = 0; i < 4; ++i)
                            acc[mt][f][i] = fmaf(sf[f], tmp[mt][f][i], fmaf(nszb[f], tmps[mt][i], acc[mt][f][i]));
                        if (!BPG1) tmp[mt][f] = zero4;
                    }
                    if (!BPG1) tmps[mt] = zero4;
                }
            }
            // the next block's activations replace this one's (same wave: LDS accesses stay in order)
            store_a(aring[(u + 1) % AB]);
            load_a(i + 1 + AB, aring[(u + 1) % AB]);
        }
    }

    // the 8 partial tiles -> LDS (each wave into its own slot), float4 = the lane's four
    // columns of one row
    float4_t *red = (float4_t *)pk4_lds;  // [NW][MT][4 rows-in-quad][64 lanes] of float4 (f = 0..3)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int i = 0; i < 4; ++i)
            red[((wave * MT + mt) * 4 + i) * 64 + lane] =
                float4_t{acc[mt][0][i], acc[mt][1][i], acc[mt][2][i], acc[mt][3][i]};
    __syncthreads();

    if (act) {
        // Fused gate|up layer: columns 0..31 of the strip are gate, 32..63 the matching up columns.
        // thread -> (row, CG gate columns and their up columns); both factors are rounded to the
        // layer dtype first, as the projection's own output would be (ffn.rs:388-400 runs the
        // activation on that output), then act(gate) * up in f32 and one rounding.
        constexpr int CG = MT >= 3 ? 4 : 2;
        constexpr int TPG = 32 / CG;
        const int c0 = (threadIdx.x % TPG) * CG;
        for (int ml = threadIdx.x / TPG; ml < ROWS && m0 + ml < M; ml += NT / TPG) {
            const int mt = ml >> 4, r = ml & 15, rb = r >> 2, i = r & 3;
            const float *redf = (const float *)pk4_lds;
            float vg[CG], vu[CG];
#pragma unroll
            for (int c = 0; c < CG; ++c) vg[c] = vu[c] = 0.f;
#pragma unroll
            for (int s = 0; s < NW; ++s) {
                const float *src = redf + ((s * MT + mt) * 4 + i) * 256 + rb * 64 + c0;
#pragma unroll
                for (int c = 0; c < CG; ++c) vg[c] += src[c], vu[c] += src[32 + c];
            }
            const int half = N >> 1, n = 32 * j + c0;
            uint16_t o[CG];
#pragma unroll
            for (int c = 0; c < CG; ++c) {
                float g = vg[c], u = vu[c];
                if (bias) {
                    g += TT::to_f32(bias[n + c]);
                    u += TT::to_f32(bias[half + n + c]);
                }
                g = TT::to_f32(TT::from_f32(g));
                u = TT::to_f32(TT::from_f32(u));
                o[c] = TT::from_f32(mul_f32_rn(act == 1 ? silu_f32(g) : gelu_tanh_f32(g), u));
            }
            uint16_t *dst = y + (size_t)(m0 + ml) * half + n;
            if (CG == 2) *(uint32_t *)dst = (uint32_t)o[0] | ((uint32_t)o[1] << 16);
            else *(uint2 *)dst = uint2{(uint32_t)o[0] | ((uint32_t)o[1] << 16), (uint32_t)o[CG - 2] | ((uint32_t)o[CG - 1] << 16)};
        }
        return;
    }

    // thread -> (row, CP consecutive columns), every thread busy where the tile allows;
    // partials added in wave order.  A row of a partial tile is 64 consecutive floats.
    constexpr int CP = MT == 1 ? 2 : MT == 2 ? 4 : 8;  // columns per thread
    constexpr int TPR = 64 / CP;                        // threads per row
    const int c0 = (threadIdx.x % TPR) * CP;
    for (int ml = threadIdx.x / TPR; ml < ROWS && m0 + ml < M; ml += NT / TPR) {
        const int mt = ml >> 4, r = ml & 15, rb = r >> 2, i = r & 3;
        const float *redf = (const float *)pk4_lds;
        float v[CP];
#pragma unroll
        for (int c = 0; c < CP; ++c) v[c] = 0.f;
#pragma unroll
        for (int s = 0; s < NW; ++s) {
            const float *src = redf + ((s * MT + mt) * 4 + i) * 256 + rb * 64 + c0;
            if (CP == 2) {
                const float2 t = *(const float2 *)src;
                v[0] += t.x, v[1] += t.y;
            } else {
#pragma unroll
                for (int h = 0; h < CP / 4; ++h) {
                    const float4_t t = *(const float4_t *)(src + 4 * h);
#pragma unroll
                    for (int c = 0; c < 4; ++c) v[4 * h + c] += t[c];
                }
            }
        }
        const int n = 64 * j + c0;
        if (gridDim.y > 1) {  // this K slice's f32 partial; a second kernel adds the slices in order
            float *dst = ws + ((size_t)blockIdx.y * M + (m0 + ml)) * N + n;
            if (CP == 2) {
                *(float2 *)dst = float2{v[0], v[1]};
            } else {
#pragma unroll
                for (int h = 0; h < CP / 4; ++h)
                    *(float4_t *)(dst + 4 * h) = float4_t{v[4 * h], v[4 * h + 1], v[4 * h + 2], v[4 * h + 3]};
            }
            continue;
        }
        uint32_t o[CP / 2];
#pragma unroll
        for (int q = 0; q < CP / 2; ++q) {
            float lo = v[2 * q], hi = v[2 * q + 1];
            if (bias) {
                lo += TT::to_f32(bias[n + 2 * q]);
                hi += TT::to_f32(bias[n + 2 * q + 1]);
            }
            o[q] = (uint32_t)TT::from_f32(lo) | ((uint32_t)TT::from_f32(hi) << 16);
        }
        uint16_t *dst = y + (size_t)(m0 + ml) * N + n;
        if (CP == 2) *(uint32_t *)dst = o[0];
        else if (CP == 4) *(uint2 *)dst = uint2{o[0], o[1]};
        else *(u32x4_t *)dst = u32x4_t{o[0], o[1], o[2], o[3]};
    }
}

// ---------------------------------------------------------------------------
// host side
// ---------------------------------------------------------------------------
bool pk4_eligible(const Wna16Problem &p) {
    if (p.bits != 4 && p.bits != 8) return false;
    if (p.K % 128 != 0 || p.N % 64 != 0 || p.group_size % 128 != 0) return false;
    if ((uint64_t)p.K * (uint64_t)p.N * p.bits / 8 >= (1ull << 31)) return false;  // 32-bit offsets in a strip and in x
    if (p.K / p.group_size > 128) return false;  // a strip's zeros and scales must fit 32 KB of LDS
    return true;
}

size_t pk4_weight_bytes(int64_t K, int64_t N, int bits) { return (size_t)K * (size_t)N * bits / 8; }
size_t pk4_zs_bytes(int64_t K, int64_t N, int gshift) { return (size_t)(K >> gshift) * (size_t)N * 4; }

template <bool GPTQ, int BITS>
static void pk4_prepack_go(hipStream_t s, dim3 gw, dim3 gz, const Wna16Problem &src, const Pk4Weights &dst, int K,
                           int N, int G) {
    dim3 block(256);
    const int half = (int)dst.gate_half;
    hipLaunchKernelGGL((pk4_prepack_weights_kernel<GPTQ, BITS>), gw, block, 0, s, src.qweight, dst.pw, K, N, half);
    if (src.dtype == OXQ_F16)
        hipLaunchKernelGGL((pk4_prepack_zs_kernel<F16Traits, GPTQ, BITS>), gz, block, 0, s, src.qzeros,
                           (const uint16_t *)src.scales, dst.pzs, G, N, half);
    else
        hipLaunchKernelGGL((pk4_prepack_zs_kernel<BF16Traits, GPTQ, BITS>), gz, block, 0, s, src.qzeros,
                           (const uint16_t *)src.scales, dst.pzs, G, N, half);
}

int launch_pk4_prepack(oxq_ctx *ctx, hipStream_t s, const Wna16Problem &src, const Pk4Weights &dst) {
    const int K = (int)src.K, N = (int)src.N, G = (int)(src.K >> src.group_shift);
    const size_t words = (size_t)K * N * src.bits / 32, zsn = (size_t)G * N;
    const bool gptq = src.pack_dim == OXQ_PACK_IN;
    dim3 gw((unsigned)ceil_div((int64_t)words, 256)), gz((unsigned)ceil_div((int64_t)zsn, 256)), block(256);
    char name[64];
    snprintf(name, sizeof name, "pk%d_prepack_%s", src.bits, gptq ? "gptq" : "awq");
    set_plan(ctx, name, gw, block, 1, 2, 0);
    if (ctx->plan_only) return OXQ_OK;
    if (src.bits == 4) {
        if (gptq) pk4_prepack_go<true, 4>(s, gw, gz, src, dst, K, N, G);
        else pk4_prepack_go<false, 4>(s, gw, gz, src, dst, K, N, G);
    } else {
        if (gptq) pk4_prepack_go<true, 8>(s, gw, gz, src, dst, K, N, G);
        else pk4_prepack_go<false, 8>(s, gw, gz, src, dst, K, N, G);
    }
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
#define OXQ_DQ(TTv, Bv)                                                                                     \
    hipLaunchKernelGGL((pk4_dequant_kernel<TTv, Bv>), grid, block, 0, s, w.pw, w.pzs, (uint16_t *)out_kn, \
                       (int)w.K, (int)w.N, w.group_shift, (int)w.gate_half)
    if (w.dtype == OXQ_F16) {
        if (w.bits == 4) OXQ_DQ(F16Traits, 4); else OXQ_DQ(F16Traits, 8);
    } else {
        if (w.bits == 4) OXQ_DQ(BF16Traits, 4); else OXQ_DQ(BF16Traits, 8);
    }
#undef OXQ_DQ
    OXQ_HIP_CHECK(hipGetLastError());
    return OXQ_OK;
}

static int pk4_env(const char *name, int dflt) {
    const char *e = getenv(name);
    return e ? atoi(e) : dflt;
}

template <typename TT, int BITS, int MT, bool GS, bool BPG1, int XQ, bool ZW = (MT <= 3)>
static int pk4_go4(oxq_ctx *ctx, hipStream_t s, dim3 grid, const Pk4Problem &p, int gslice) {
    constexpr int AB = Pk4Ring<MT, BITS>::AB, WD = Pk4Ring<MT, BITS>::WD;
    const size_t lds = (size_t)8 * MT * 4096 + (size_t)gslice * 256 * (GS ? 2 : 1);
    static LdsGrant lds_grant;  // one per instantiation
    OXQ_HIP_CHECK(lds_grant.ensure((const void *)pk4_mfma_kernel<TT, BITS, MT, GS, BPG1, AB, WD, XQ, ZW>, lds));
    hipLaunchKernelGGL((pk4_mfma_kernel<TT, BITS, MT, GS, BPG1, AB, WD, XQ, ZW>), grid, dim3(512), lds, s,
                       (const uint16_t *)p.x, p.w.pw, p.w.pzs, (const uint16_t *)p.bias, (uint16_t *)p.y,
                       (float *)ctx->workspace, (int)p.M, (int)p.w.K, (int)p.w.N, p.w.group_shift, gslice,
                       ZW ? 0 : pk4_env("OXQ_PK4_INTERLEAVE", 0), p.act);
    OXQ_HIP_CHECK(hipGetLastError());
    return OXQ_OK;
}

template <typename TT, int BITS, int MT, bool GS, bool BPG1>
static int pk4_go3(oxq_ctx *ctx, hipStream_t s, dim3 grid, const Pk4Problem &p, int gslice) {
    // A single short tile: rows past M are known at launch, so the loads that would only fetch them
    // are left out (M = 1: 8.8 instead of 9.1 us on 4096 x 14336).
    if constexpr (MT == 1) {
        const int xq = pk4_env("OXQ_PK4_XQ", 1) ? (int)ceil_div(p.M, 4) : 4;
        if (xq == 1) return pk4_go4<TT, BITS, MT, GS, BPG1, 1>(ctx, s, grid, p, gslice);
        if (xq == 2) return pk4_go4<TT, BITS, MT, GS, BPG1, 2>(ctx, s, grid, p, gslice);
    }
    if constexpr (MT == 4) {  // at most four groups a wave: the single-chunk per-wave staging
        if (gslice <= 32 && pk4_env("OXQ_PK4_INTERLEAVE", 0) == 0)
            return pk4_go4<TT, BITS, MT, GS, BPG1, 4 * MT, true>(ctx, s, grid, p, gslice);
    }
    return pk4_go4<TT, BITS, MT, GS, BPG1, 4 * MT>(ctx, s, grid, p, gslice);
}

template <typename TT, int BITS, int MT, bool GS>
static int pk4_go(oxq_ctx *ctx, hipStream_t s, dim3 grid, const Pk4Problem &p, int gslice) {
    return p.w.group_shift == 7 ? pk4_go3<TT, BITS, MT, GS, true>(ctx, s, grid, p, gslice)
                                : pk4_go3<TT, BITS, MT, GS, false>(ctx, s, grid, p, gslice);
}

template <typename TT, int BITS>
static int pk4_by_mt(oxq_ctx *ctx, hipStream_t s, dim3 grid, const Pk4Problem &p, int gslice, int mt) {
    switch (mt) {
    case 1: return pk4_go<TT, BITS, 1, true>(ctx, s, grid, p, gslice);
    case 2: return pk4_go<TT, BITS, 2, false>(ctx, s, grid, p, gslice);
    case 3: return pk4_go<TT, BITS, 3, false>(ctx, s, grid, p, gslice);
    default: return pk4_go<TT, BITS, 4, false>(ctx, s, grid, p, gslice);
    }
}

int launch_pk4_forward(oxq_ctx *ctx, hipStream_t s, const Pk4Problem &p) {
    const int64_t M = p.M;
    const int mt = M > 48 ? 4 : (int)ceil_div(M, 16);
    const int G = (int)(p.w.K >> p.w.group_shift);
    // Few column strips and a long K (a down projection: N = 4096 is 64 strips for 256 CUs):
    // K is also cut into slices of whole groups, at least two groups per wave, so that up to
    // one workgroup per CU runs; the slices' f32 partial tiles are added in slice order by a
    // second launch.  Measured (f16, M = 1 / 64): 14336 x 4096 16.6 / 41.1 us unsplit,
    // 11.2 / 22.5 us in 4 slices, worse again in 5 or 7 (a second round of workgroups); a
    // 4096 x 4096 layer gains nothing (the extra launch costs what the split saves).
    const int64_t tiles = (p.w.N / 64) * ceil_div(M, 16 * mt);
    int ks = 1;
    if (tiles <= 96 && G >= 64) ks = (int)std::max<int64_t>(1, std::min<int64_t>(256 / tiles, G / 16));
    ks = pk4_env("OXQ_PK4_KS", ks);
    ks = std::max(1, std::min(ks, G));
    if (p.act) ks = 1;  // the activation needs the whole sum: gate|up layers are wide, one slice fills the chip
    if (p.no_split) ks = 1;
    while (ks > 1 && (size_t)ks * M * p.w.N * 4 > ctx->workspace_bytes) --ks;
    const int gslice = (int)ceil_div(G, ks);
    ks = (int)ceil_div(G, gslice);  // no empty slice
    if (ceil_div(M, 16 * mt) > 65535)
        return fail(OXQ_ERR_UNSUPPORTED, "repacked matmul: m = %lld exceeds the grid limit (65535 row tiles)", (long long)M);
    dim3 grid((unsigned)(p.w.N / 64), (unsigned)ks, (unsigned)ceil_div(M, 16 * mt));
    char name[64];
    if (p.act && (!p.w.gate_half || p.act > 2))
        return fail(OXQ_ERR_ARG, "repacked matmul: activation %d on a layer that is not a fused gate|up layer", p.act);
    snprintf(name, sizeof name, "pk%d_mfma_%s_mt%d%s%s", p.w.bits, p.w.dtype == OXQ_F16 ? "f16" : "bf16", mt,
             mt == 1 ? "_gs" : "", p.act == 1 ? "_silu" : p.act == 2 ? "_gelu" : "");
    set_plan(ctx, name, grid, dim3(512), ks, 1, ks > 1 ? (size_t)ks * M * p.w.N * 4 : 0);
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
    if (p.w.bits == 4)
        rc = f16 ? pk4_by_mt<F16Traits, 4>(ctx, s, grid, p, gslice, mt)
                 : pk4_by_mt<BF16Traits, 4>(ctx, s, grid, p, gslice, mt);
    else
        rc = f16 ? pk4_by_mt<F16Traits, 8>(ctx, s, grid, p, gslice, mt)
                 : pk4_by_mt<BF16Traits, 8>(ctx, s, grid, p, gslice, mt);
    if (rc != OXQ_OK || ks == 1) return rc;
    return launch_splitk_reduce(ctx, s, (const float *)ctx->workspace, p.bias, p.y, M, p.w.N, ks, p.w.dtype);
}

}  // namespace oxq
