// Resident GGUF layers (linear.rs:197-247 GgufFastPath::build keeps a copy of the block bytes for the
// life of the layer): a strip-major copy built once at load, and the decode GEMV that reads it.
//
// In the file layout a weight row is one run of blocks, so a kernel that gives a wave a row has to
// stage all of x for every workgroup behind a barrier and fetches blocks of 18, 34, 144 or 210 bytes
// that straddle every alignment.  The copy cuts the matrix into strips of 16 rows (output columns)
// and chunks of 128 elements of K; lane (col = l % 16, kq = l / 16) of a chunk owns unit kq (32
// consecutive elements) of row 16 strip + col:
//
//   block (CH chunks) = CH x { planes [64 lanes][16 B] (+ [64 lanes][8 B]) of quant bits,
//                              [64 lanes][2 B] unit header (if the format has one) }
//                       + [16 rows] block header (K-quants: the super-block's d / dmin / scales)
//
//   Q4_0  CH 1  16 B quants, unit header d                                                     1152 B
//   Q8_0  CH 1  32 B quants, unit header d                                                     2176 B
//   Q4_K  CH 2  16 B quants, block header = the super-block's first 16 bytes (d, dmin, 12
//               scale bytes)                                                                   2304 B
//   Q6_K  CH 2  16 B low nibbles + 8 B high bit pairs, unit header = the unit's two int8
//               scales, block header = d                                                       3360 B
//   Q4_1  CH 1  16 B quants, unit header d, m (4 B)                                            1280 B
//   Q5_0  CH 1  16 B low nibbles + 4 B high bits, unit header d                                1408 B
//   Q5_1  CH 1  16 B low nibbles + 4 B high bits, unit header d, m (4 B)                       1536 B
//   Q5_K  CH 2  16 B low nibbles + 4 B high bits, block header as Q4_K                         2816 B
//   Q2_K  CH 2  8 B bit pairs, unit header = the unit's two scale bytes, block header d, dmin  1344 B
//   Q3_K  CH 2  8 B low bit pairs + 4 B high bits, block header = the 12 scale bytes, d, 2 B
//               unused (the one format two bytes a super-block larger than the file)           1792 B
//
// Exactly the file's bytes per weight.  Inside a unit the 16 elements of each half are stored ROTATED
// by the lane's column: position n (0..15) of half h holds element 16 h + (col - n) mod 16 (4-bit
// formats: half 0 in the low nibbles of the 16 bytes, half 1 in the high ones, byte n = position n;
// Q8_0: byte 16 h + n; Q6_K: low nibbles likewise, the bit pair of position 16 h + 4 s + b in bits 2s
// of byte b of word h; 5-bit formats: low nibbles likewise, the high bit of position 16 h + n in bit
// 16 h + n of the fifth word; Q2_K / Q3_K: the bit pair of position 16 h + 4 s + b in bits 2s of byte b of
// word h, Q3_K's third bit as the fifth of the 5-bit formats).  That is what lets the activations stay in registers: lane col loads
// x[16 h + col] of its unit (two 4-byte loads, 64 contiguous bytes per 16 lanes), and a rotation of
// that register by n lanes inside the row of 16 (a DPP operand of the multiply-add, no instruction of
// its own) hands every lane the element its position n multiplies.  No LDS, no staging, no barrier
// before the arithmetic; the sums of x over 16 elements are four rotate-adds of the same register.
//
// The 16 (8) waves of a workgroup split the strip's chunks, the partial sums meet in LDS at the end
// in a fixed order.  The arithmetic is the staged GEMV's: raw integers converted once,
// y += a0 dot0 + a1 dot1 - b0 sum0 - b1 sum1 per unit (quant_kernels.metal:1097-1221, 1681-1838).
#include "gguf_decode.hpp"

namespace oxq {

template <int FMT> struct GgrFmt;
template <> struct GgrFmt<OXQ_GGUF_Q4_0> { static constexpr int CH = 1, QW = 4, UH = 2, BH = 0; };
template <> struct GgrFmt<OXQ_GGUF_Q8_0> { static constexpr int CH = 1, QW = 8, UH = 2, BH = 0; };
template <> struct GgrFmt<OXQ_GGUF_Q4_K> { static constexpr int CH = 2, QW = 4, UH = 0, BH = 16; };
template <> struct GgrFmt<OXQ_GGUF_Q6_K> { static constexpr int CH = 2, QW = 6, UH = 2, BH = 2; };
template <> struct GgrFmt<OXQ_GGUF_Q4_1> { static constexpr int CH = 1, QW = 4, UH = 4, BH = 0; };
template <> struct GgrFmt<OXQ_GGUF_Q5_0> { static constexpr int CH = 1, QW = 5, UH = 2, BH = 0; };
template <> struct GgrFmt<OXQ_GGUF_Q5_1> { static constexpr int CH = 1, QW = 5, UH = 4, BH = 0; };
template <> struct GgrFmt<OXQ_GGUF_Q5_K> { static constexpr int CH = 2, QW = 5, UH = 0, BH = 16; };
template <> struct GgrFmt<OXQ_GGUF_Q2_K> { static constexpr int CH = 2, QW = 2, UH = 2, BH = 4; };
template <> struct GgrFmt<OXQ_GGUF_Q3_K> { static constexpr int CH = 2, QW = 3, UH = 0, BH = 16; };
// formats with a scale per 16 elements: two multiply-add chains and two sums a unit
template <int FMT> constexpr bool ggr_two_scales = FMT == OXQ_GGUF_Q6_K || FMT == OXQ_GGUF_Q2_K || FMT == OXQ_GGUF_Q3_K;

template <int FMT> struct GgrLayout {
    typedef GgrFmt<FMT> F;
    static constexpr int P128 = F::QW / 4, P64 = (F::QW % 4) / 2, P32 = F::QW % 2;  // planes of 16, 8 and 4 bytes a lane
    static constexpr int UH_OFF = 64 * F::QW * 4;            // unit headers behind the planes
    static constexpr int CHB = 64 * (F::QW * 4 + F::UH);     // bytes of a chunk
    static constexpr int BH_OFF = F::CH * CHB;               // block header behind the chunks
    static constexpr int BLKB = F::CH * CHB + 16 * F::BH;    // bytes of a block
    // the file's bytes per weight, except Q3_K: its 12 scale bytes and d share one 16-byte header (112 for 110)
    static_assert(BLKB == 16 * (128 * F::CH / GgufFmt<FMT>::BE) * (GgufFmt<FMT>::BB + (FMT == OXQ_GGUF_Q3_K ? 2 : 0)),
                  "the copy has the file's size");
};

// ---------------------------------------------------------------------------
// repack: one thread per (strip, chunk, lane) = one unit of one row
// ---------------------------------------------------------------------------
template <int FMT>
__global__ __launch_bounds__(256) void ggr_repack_kernel(const uint8_t *__restrict__ w, uint8_t *__restrict__ pw,
                                                         int K, int N) {
    typedef GgrFmt<FMT> F;
    typedef GgrLayout<FMT> L;
    const int nch = K >> 7;
    const size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= (size_t)(N >> 4) * nch * 64) return;
    const int lane = (int)(idx & 63), c = (int)((idx >> 6) % nch), strip = (int)((idx >> 6) / nch);
    const int col = lane & 15, kq = lane >> 4;
    const int u = 4 * c + kq;
    const size_t row_bytes = (size_t)(K / GgufFmt<FMT>::BE) * GgufFmt<FMT>::BB;
    const uint8_t *row = w + (size_t)(16 * strip + col) * row_bytes;
    uint8_t *blk = pw + ((size_t)strip * (nch / F::CH) + c / F::CH) * L::BLKB;
    uint8_t *chunk = blk + (c % F::CH) * L::CHB;

    uint32_t qw[F::QW];
    uint32_t uh = 0;
    // position n of a half holds element (col - n) mod 16 of that half
    auto el = [&](int n) { return (col - n) & 15; };
    if constexpr (FMT == OXQ_GGUF_Q4_0) {
        const uint8_t *p = row + (size_t)u * 18;
        uh = ld16(p);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            uint32_t v = 0;
#pragma unroll
            for (int bb = 0; bb < 4; ++bb) v |= (uint32_t)p[2 + el(4 * i + bb)] << (8 * bb);  // byte e: elements e, e + 16
            qw[i] = v;
        }
    } else if constexpr (FMT == OXQ_GGUF_Q8_0) {
        const uint8_t *p = row + (size_t)u * 34;
        uh = ld16(p);
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            uint32_t v = 0;
#pragma unroll
            for (int bb = 0; bb < 4; ++bb) v |= (uint32_t)p[2 + 16 * (i >> 2) + el(4 * (i & 3) + bb)] << (8 * bb);
            qw[i] = v;
        }
    } else if constexpr (FMT == OXQ_GGUF_Q4_1 || FMT == OXQ_GGUF_Q5_0 || FMT == OXQ_GGUF_Q5_1) {
        constexpr bool MIN = FMT != OXQ_GGUF_Q5_0, FIVE = FMT != OXQ_GGUF_Q4_1;
        const uint8_t *p = row + (size_t)u * GgufFmt<FMT>::BB;
        uh = ld16(p) | (MIN ? ld16(p + 2) << 16 : 0u);
        const uint8_t *hp = p + (MIN ? 4 : 2), *qs = hp + (FIVE ? 4 : 0);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            uint32_t v = 0;
#pragma unroll
            for (int bb = 0; bb < 4; ++bb) v |= (uint32_t)qs[el(4 * i + bb)] << (8 * bb);  // byte e: elements e, e + 16
            qw[i] = v;
        }
        if constexpr (FIVE) {
            const uint32_t qh = ld16(hp) | (ld16(hp + 2) << 16);  // bit e: element e
            uint32_t v = 0;
#pragma unroll
            for (int nn = 0; nn < 16; ++nn) v |= (((qh >> el(nn)) & 1u) << nn) | (((qh >> (16 + el(nn))) & 1u) << (16 + nn));
            qw[4] = v;
        }
    } else if constexpr (FMT == OXQ_GGUF_Q4_K || FMT == OXQ_GGUF_Q5_K) {
        constexpr bool FIVE = FMT == OXQ_GGUF_Q5_K;
        const int b = u >> 3, sb = u & 7;
        const uint8_t *p = row + (size_t)b * (FIVE ? 176 : 144);
        const uint8_t *qs = p + (FIVE ? 48 : 16) + (sb >> 1) * 32;
        const int sh = (sb & 1) * 4;
        if constexpr (FIVE) {  // bit sb of byte e of qh (p + 16): element e of unit sb
            uint32_t v = 0;
#pragma unroll
            for (int nn = 0; nn < 16; ++nn)
                v |= ((((uint32_t)p[16 + el(nn)] >> sb) & 1u) << nn) | ((((uint32_t)p[32 + el(nn)] >> sb) & 1u) << (16 + nn));
            qw[4] = v;
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            uint32_t v = 0;
#pragma unroll
            for (int bb = 0; bb < 4; ++bb) {
                const int e = el(4 * i + bb);
                const uint32_t lo = ((uint32_t)qs[e] >> sh) & 0xFu, hi = ((uint32_t)qs[16 + e] >> sh) & 0xFu;
                v |= (lo | (hi << 4)) << (8 * bb);
            }
            qw[i] = v;
        }
        if (sb == 0) {
#pragma unroll
            for (int i = 0; i < 8; ++i) *(uint16_t *)(blk + L::BH_OFF + col * 16 + 2 * i) = (uint16_t)ld16(p + 2 * i);
        }
    } else if constexpr (FMT == OXQ_GGUF_Q2_K || FMT == OXQ_GGUF_Q3_K) {
        constexpr bool THREE = FMT == OXQ_GGUF_Q3_K;
        const int b = u >> 3, ub = u & 7;
        const uint8_t *p = row + (size_t)b * (THREE ? 110 : 84);
        const uint8_t *qs = p + (THREE ? 32 : 16) + (ub >> 2) * 32;  // element e: bits sh, sh + 1 of byte e
        const int sh = (ub & 3) * 2;
#pragma unroll
        for (int hs = 0; hs < 2; ++hs) {
            uint32_t v = 0;
#pragma unroll
            for (int s2 = 0; s2 < 4; ++s2)
#pragma unroll
                for (int bb = 0; bb < 4; ++bb)
                    v |= (((uint32_t)qs[16 * hs + el(4 * s2 + bb)] >> sh) & 3u) << (8 * bb + 2 * s2);
            qw[hs] = v;
        }
        if constexpr (THREE) {  // bit ub of byte e of hmask (p): the third bit of element e of unit ub
            uint32_t v = 0;
#pragma unroll
            for (int nn = 0; nn < 16; ++nn)
                v |= ((((uint32_t)p[el(nn)] >> ub) & 1u) << nn) | ((((uint32_t)p[16 + el(nn)] >> ub) & 1u) << (16 + nn));
            qw[2] = v;
            if (ub == 0) {
                uint16_t *h = (uint16_t *)(blk + L::BH_OFF + col * 16);
#pragma unroll
                for (int i = 0; i < 6; ++i) h[i] = (uint16_t)ld16(p + 96 + 2 * i);
                h[6] = (uint16_t)ld16(p + 108);
                h[7] = 0;
            }
        } else {
            uh = (uint32_t)p[2 * ub] | ((uint32_t)p[2 * ub + 1] << 8);
            if (ub == 0) *(uint32_t *)(blk + L::BH_OFF + col * 4) = ld16(p + 80) | (ld16(p + 82) << 16);
        }
    } else {  // Q6_K
        const int b = u >> 3, sub = u & 7;
        const int h = sub >> 2, quad = sub & 3;
        const uint8_t *p = row + (size_t)b * 210;
        const uint8_t *ql = p + 64 * h + (quad & 1) * 32;
        const uint8_t *qh = p + 128 + 32 * h;
        const int shl = (quad < 2) ? 0 : 4, shh = 2 * quad;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            uint32_t v = 0;
#pragma unroll
            for (int bb = 0; bb < 4; ++bb) {
                const int e = el(4 * i + bb);
                const uint32_t lo = ((uint32_t)ql[e] >> shl) & 0xFu, hi = ((uint32_t)ql[16 + e] >> shl) & 0xFu;
                v |= (lo | (hi << 4)) << (8 * bb);
            }
            qw[i] = v;
        }
#pragma unroll
        for (int hs = 0; hs < 2; ++hs) {
            uint32_t v = 0;
#pragma unroll
            for (int s = 0; s < 4; ++s)
#pragma unroll
                for (int bb = 0; bb < 4; ++bb)
                    v |= (((uint32_t)qh[16 * hs + el(4 * s + bb)] >> shh) & 3u) << (8 * bb + 2 * s);
            qw[4 + hs] = v;
        }
        uh = (uint32_t)p[192 + 2 * sub] | ((uint32_t)p[192 + 2 * sub + 1] << 8);
        if (sub == 0) *(uint16_t *)(blk + L::BH_OFF + col * 2) = (uint16_t)ld16(p + 208);
    }
#pragma unroll
    for (int pl = 0; pl < L::P128; ++pl)
        *(u32x4_t *)(chunk + pl * 1024 + lane * 16) = u32x4_t{qw[4 * pl], qw[4 * pl + 1], qw[4 * pl + 2], qw[4 * pl + 3]};
    if constexpr (L::P64) {
        uint32_t *d = (uint32_t *)(chunk + L::P128 * 1024 + lane * 8);
        d[0] = qw[4 * L::P128], d[1] = qw[4 * L::P128 + 1];
    }
    if constexpr (L::P32) *(uint32_t *)(chunk + L::P128 * 1024 + L::P64 * 512 + lane * 4) = qw[F::QW - 1];
    if constexpr (F::UH == 2) *(uint16_t *)(chunk + L::UH_OFF + lane * 2) = (uint16_t)uh;
    if constexpr (F::UH == 4) *(uint32_t *)(chunk + L::UH_OFF + lane * 4) = uh;
}

// ---------------------------------------------------------------------------
// A unit from the copy: the stored unsigned integers as floats and the four factors of
// a0*dot0 + a1*dot1 - b0*sum0 - b1*sum1 (as unit_ints does from the file layout).
//   qw: the unit's quant words; uh: its header; bh: the block header words of its row; sb: index of
//   the unit inside its block (K-quants).
// ---------------------------------------------------------------------------
__device__ __forceinline__ float f16_bits_to_f32(uint32_t v) { return (float)__builtin_bit_cast(_Float16, (uint16_t)v); }

template <int FMT>
__device__ __forceinline__ void ggr_factors(uint32_t uh, const uint32_t (&bh)[4], int sb, float &a0, float &a1,
                                            float &b0, float &b1) {
    if constexpr (FMT == OXQ_GGUF_Q4_0) {
        const float d = f16_bits_to_f32(uh);
        a0 = a1 = d, b0 = b1 = 8.0f * d;
    } else if constexpr (FMT == OXQ_GGUF_Q8_0) {
        const float d = f16_bits_to_f32(uh);
        a0 = a1 = d, b0 = b1 = 128.0f * d;
    } else if constexpr (FMT == OXQ_GGUF_Q4_1 || FMT == OXQ_GGUF_Q5_1) {
        a0 = a1 = f16_bits_to_f32(uh & 0xFFFFu);
        b0 = b1 = -f16_bits_to_f32(uh >> 16);
    } else if constexpr (FMT == OXQ_GGUF_Q5_0) {
        const float d = f16_bits_to_f32(uh);
        a0 = a1 = d, b0 = b1 = 16.0f * d;
    } else if constexpr (FMT == OXQ_GGUF_Q4_K || FMT == OXQ_GGUF_Q5_K) {
        const float d = f16_bits_to_f32(bh[0] & 0xFFFFu), dmin = f16_bits_to_f32(bh[0] >> 16);
        // get_scale_min_k4 (quant_kernels.metal:2438-2450) on the 12 scale bytes in bh[1..3]
        const uint32_t sft = 8u * (uint32_t)(sb & 3);
        const uint32_t a = (bh[1] >> sft) & 0xFFu, b = (bh[2] >> sft) & 0xFFu, c = (bh[3] >> sft) & 0xFFu;
        const uint32_t low = sb < 4 ? 0xFFFFFFFFu : 0u;
        const uint32_t scv = ((a & 63u) & low) | (((c & 0x0Fu) | ((a >> 6) << 4)) & ~low);
        const uint32_t mnv = ((b & 63u) & low) | (((c >> 4) | ((b >> 6) << 4)) & ~low);
        a0 = a1 = d * (float)scv;
        b0 = b1 = dmin * (float)mnv;
    } else if constexpr (FMT == OXQ_GGUF_Q2_K) {
        const float d = f16_bits_to_f32(bh[0] & 0xFFFFu), dmin = f16_bits_to_f32(bh[0] >> 16);
        a0 = d * (float)(uh & 0xFu);
        b0 = dmin * (float)((uh >> 4) & 0xFu);
        a1 = d * (float)((uh >> 8) & 0xFu);
        b1 = dmin * (float)(uh >> 12);
    } else if constexpr (FMT == OXQ_GGUF_Q3_K) {
        // q3k_scale (quant_kernels.metal:2594-2604) of sub-blocks 2 sb and 2 sb + 1 on the 12 scale bytes in bh[0..2]
        // (sub-blocks 2 sb and 2 sb + 1 share their group sb / 2 and sit in bytes k = 2 (sb % 2) and k + 1)
        const float d = f16_bits_to_f32(bh[3] & 0xFFFFu);
        const uint32_t group = (uint32_t)sb >> 1, k8 = 16u * ((uint32_t)sb & 1u);
        const uint32_t b0w = bh[0], b1w = bh[1], b2w = bh[2];
        const uint32_t lw = ((group & 1u) ? b1w : b0w) >> k8 >> (group < 2u ? 0u : 4u);  // bytes k, k + 1 in bits 0.., 8..
        const uint32_t hw = b2w >> k8 >> (2u * group);
        const int s0 = (int)((lw & 0xFu) | ((hw & 3u) << 4)) - 32;
        const int s1 = (int)(((lw >> 8) & 0xFu) | (((hw >> 8) & 3u) << 4)) - 32;
        a0 = d * (float)s0, a1 = d * (float)s1;
        b0 = 4.0f * a0, b1 = 4.0f * a1;
    } else {  // Q6_K
        const float d = f16_bits_to_f32(bh[0] & 0xFFFFu);
        a0 = d * (float)(int)(int8_t)(uh & 0xFFu);
        a1 = d * (float)(int)(int8_t)((uh >> 8) & 0xFFu);
        b0 = 32.0f * a0, b1 = 32.0f * a1;
    }
}

template <int FMT>
__device__ __forceinline__ void ggr_ints(const uint32_t (&qw)[GgrFmt<FMT>::QW], float q[32]) {
    if constexpr (FMT == OXQ_GGUF_Q8_0) {
#pragma unroll
        for (int i = 0; i < 8; ++i) bytes_to_f32(qw[i] ^ 0x80808080u, q + 4 * i);  // q + 128
    } else if constexpr (FMT == OXQ_GGUF_Q6_K) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            bytes_to_f32((qw[i] & 0x0F0F0F0Fu) | (((qw[4] >> (2 * i)) & 0x03030303u) << 4), q + 4 * i);  // q + 32
            bytes_to_f32(((qw[i] >> 4) & 0x0F0F0F0Fu) | (((qw[5] >> (2 * i)) & 0x03030303u) << 4), q + 16 + 4 * i);
        }
    } else if constexpr (FMT == OXQ_GGUF_Q2_K || FMT == OXQ_GGUF_Q3_K) {
#pragma unroll
        for (int h = 0; h < 2; ++h)
#pragma unroll
            for (int s2 = 0; s2 < 4; ++s2) {
                uint32_t v = (qw[h] >> (2 * s2)) & 0x03030303u;
                if constexpr (FMT == OXQ_GGUF_Q3_K) v |= spread4(qw[2] >> (16 * h + 4 * s2)) << 2;  // q + 4
                bytes_to_f32(v, q + 16 * h + 4 * s2);
            }
    } else if constexpr (GgrFmt<FMT>::QW == 5) {  // a fifth bit from word 4: bit 16 h + n for position n of half h
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            bytes_to_f32((qw[i] & 0x0F0F0F0Fu) | (spread4(qw[4] >> (4 * i)) << 4), q + 4 * i);
            bytes_to_f32(((qw[i] >> 4) & 0x0F0F0F0Fu) | (spread4(qw[4] >> (16 + 4 * i)) << 4), q + 16 + 4 * i);
        }
    } else {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            bytes_to_f32(qw[i] & 0x0F0F0F0Fu, q + 4 * i);
            bytes_to_f32((qw[i] >> 4) & 0x0F0F0F0Fu, q + 16 + 4 * i);
        }
    }
}

// dense [N, K] f32 from the copy, with the arithmetic of decode_unit (pins the repack bit for bit)
template <int FMT>
__global__ __launch_bounds__(256) void ggr_dequant_kernel(const uint8_t *__restrict__ pw, float *__restrict__ out,
                                                          int K, int N) {
    typedef GgrFmt<FMT> F;
    typedef GgrLayout<FMT> L;
    const int nch = K >> 7;
    const size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= (size_t)(N >> 4) * nch * 64) return;
    const int lane = (int)(idx & 63), c = (int)((idx >> 6) % nch), strip = (int)((idx >> 6) / nch);
    const int col = lane & 15, kq = lane >> 4;
    const uint8_t *blk = pw + ((size_t)strip * (nch / F::CH) + c / F::CH) * L::BLKB;
    const uint8_t *chunk = blk + (c % F::CH) * L::CHB;
    uint32_t qw[F::QW];
#pragma unroll
    for (int pl = 0; pl < L::P128; ++pl) {
        const u32x4_t v = *(const u32x4_t *)(chunk + pl * 1024 + lane * 16);
        qw[4 * pl] = v[0], qw[4 * pl + 1] = v[1], qw[4 * pl + 2] = v[2], qw[4 * pl + 3] = v[3];
    }
    if constexpr (L::P64) {
        const uint32_t *d = (const uint32_t *)(chunk + L::P128 * 1024 + lane * 8);
        qw[4 * L::P128] = d[0], qw[4 * L::P128 + 1] = d[1];
    }
    if constexpr (L::P32) qw[F::QW - 1] = *(const uint32_t *)(chunk + L::P128 * 1024 + L::P64 * 512 + lane * 4);
    uint32_t uh = 0, bh[4] = {0u, 0u, 0u, 0u};
    if constexpr (F::UH == 2) uh = *(const uint16_t *)(chunk + L::UH_OFF + lane * 2);
    if constexpr (F::UH == 4) uh = *(const uint32_t *)(chunk + L::UH_OFF + lane * 4);
    if constexpr (F::BH == 16) {
        const u32x4_t v = *(const u32x4_t *)(blk + L::BH_OFF + col * 16);
        bh[0] = v[0], bh[1] = v[1], bh[2] = v[2], bh[3] = v[3];
    } else if constexpr (F::BH == 4) {
        bh[0] = *(const uint32_t *)(blk + L::BH_OFF + col * 4);
    } else if constexpr (F::BH == 2) {
        bh[0] = *(const uint16_t *)(blk + L::BH_OFF + col * 2);
    }
    const int sb = 4 * (c % F::CH) + kq;
    float wf[32];
    if constexpr (FMT == OXQ_GGUF_Q4_0) {
        const float d = f16_bits_to_f32(uh);
#pragma unroll
        for (int e = 0; e < 16; ++e) {
            const uint32_t byte = (qw[e >> 2] >> (8 * (e & 3))) & 0xFFu;
            wf[e] = (float)((int)(byte & 0xF) - 8) * d;
            wf[e + 16] = (float)((int)(byte >> 4) - 8) * d;
        }
    } else if constexpr (FMT == OXQ_GGUF_Q8_0) {
        const float d = f16_bits_to_f32(uh);
#pragma unroll
        for (int e = 0; e < 32; ++e) wf[e] = (float)(int)(int8_t)((qw[e >> 2] >> (8 * (e & 3))) & 0xFFu) * d;
    } else if constexpr (FMT == OXQ_GGUF_Q4_K || FMT == OXQ_GGUF_Q5_K) {
        float sc_v, m_v, t0, t1;
        ggr_factors<FMT>(uh, bh, sb, sc_v, t0, m_v, t1);
#pragma unroll
        for (int e = 0; e < 16; ++e) {
            const uint32_t byte = (qw[e >> 2] >> (8 * (e & 3))) & 0xFFu;
            uint32_t lo = byte & 0xF, hi = byte >> 4;
            if constexpr (FMT == OXQ_GGUF_Q5_K) lo |= ((qw[4] >> e) & 1u) << 4, hi |= ((qw[4] >> (16 + e)) & 1u) << 4;
            wf[e] = sc_v * (float)lo - m_v;
            wf[e + 16] = sc_v * (float)hi - m_v;
        }
    } else if constexpr (FMT == OXQ_GGUF_Q4_1 || FMT == OXQ_GGUF_Q5_1) {
        const float d = f16_bits_to_f32(uh & 0xFFFFu), m = f16_bits_to_f32(uh >> 16);
#pragma unroll
        for (int e = 0; e < 16; ++e) {
            const uint32_t byte = (qw[e >> 2] >> (8 * (e & 3))) & 0xFFu;
            uint32_t lo = byte & 0xF, hi = byte >> 4;
            if constexpr (FMT == OXQ_GGUF_Q5_1) lo |= ((qw[4] >> e) & 1u) << 4, hi |= ((qw[4] >> (16 + e)) & 1u) << 4;
            wf[e] = (float)lo * d + m;
            wf[e + 16] = (float)hi * d + m;
        }
    } else if constexpr (FMT == OXQ_GGUF_Q2_K || FMT == OXQ_GGUF_Q3_K) {
        float s0, s1, m0, m1;
        ggr_factors<FMT>(uh, bh, sb, s0, s1, m0, m1);
#pragma unroll
        for (int e = 0; e < 16; ++e) {
            const int sft = 8 * (e & 3) + 2 * (e >> 2);
            const uint32_t lo = (qw[0] >> sft) & 3u, hi = (qw[1] >> sft) & 3u;
            if constexpr (FMT == OXQ_GGUF_Q2_K) {
                wf[e] = s0 * (float)lo - m0;
                wf[e + 16] = s1 * (float)hi - m1;
            } else {
                wf[e] = s0 * (float)((int)lo + (int)(((qw[2] >> e) & 1u) << 2) - 4);
                wf[e + 16] = s1 * (float)((int)hi + (int)(((qw[2] >> (16 + e)) & 1u) << 2) - 4);
            }
        }
    } else if constexpr (FMT == OXQ_GGUF_Q5_0) {
        const float d = f16_bits_to_f32(uh);
#pragma unroll
        for (int e = 0; e < 16; ++e) {
            const uint32_t byte = (qw[e >> 2] >> (8 * (e & 3))) & 0xFFu;
            const uint32_t lo = (byte & 0xF) | (((qw[4] >> e) & 1u) << 4), hi = (byte >> 4) | (((qw[4] >> (16 + e)) & 1u) << 4);
            wf[e] = (float)((int)lo - 16) * d;
            wf[e + 16] = (float)((int)hi - 16) * d;
        }
    } else {
        float s0, s1, t0, t1;
        ggr_factors<FMT>(uh, bh, sb, s0, s1, t0, t1);
#pragma unroll
        for (int e = 0; e < 16; ++e) {
            const uint32_t byte = (qw[e >> 2] >> (8 * (e & 3))) & 0xFFu;
            const uint32_t h0 = (qw[4] >> (8 * (e & 3) + 2 * (e >> 2))) & 3u, h1 = (qw[5] >> (8 * (e & 3) + 2 * (e >> 2))) & 3u;
            wf[e] = s0 * (float)((int)((byte & 0xF) | (h0 << 4)) - 32);
            wf[e + 16] = s1 * (float)((int)((byte >> 4) | (h1 << 4)) - 32);
        }
    }
    // wf is in stored order: position n of half h is element (col - n) mod 16 of that half
    float *o = out + (size_t)(16 * strip + col) * K + (size_t)(4 * c + kq) * 32;
#pragma unroll
    for (int i = 0; i < 32; ++i) o[(i & 16) + ((col - i) & 15)] = wf[i];
}

// ---------------------------------------------------------------------------
// Decode GEMV on the copy.  grid.x = workgroups that walk the strips; wave w takes a contiguous run
// of a strip's chunks with RD chunks (weights, headers and its lanes' two activations per row) in
// flight.  Nothing goes through LDS but the partial sums at the end.
// ---------------------------------------------------------------------------
// value of lane (l - n) mod 16 of the caller's row of 16 lanes (DPP row_ror: the compiler folds the
// move into the multiply-add that uses it)
template <int NROT>
__device__ __forceinline__ float row_ror(float v) {
    if constexpr (NROT == 0) return v;
    else return __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, v), 0x120 + NROT, 0xF, 0xF, true));
}
// dot += sum over n of q[n] * (xv of lane (l - n) mod 16).  Written out as v_fmac_f32 with a DPP source
// (the compiler keeps the rotation as a move of its own in front of every multiply-add otherwise).  A
// DPP source written by a vector instruction less than two wait states earlier reads stale data on this
// target, and the hazard pass does not look inside an asm block: hence the leading s_nop.
__device__ __forceinline__ void ggr_dot16(const float *q, float xv, float &dot) {
    asm("s_nop 1\n\t"
        "v_fmac_f32_e32 %0, %1, %2\n\t"
        "v_fmac_f32_dpp %0, %1, %3 row_ror:1 row_mask:0xf bank_mask:0xf bound_ctrl:1\n\t"
        "v_fmac_f32_dpp %0, %1, %4 row_ror:2 row_mask:0xf bank_mask:0xf bound_ctrl:1\n\t"
        "v_fmac_f32_dpp %0, %1, %5 row_ror:3 row_mask:0xf bank_mask:0xf bound_ctrl:1\n\t"
        "v_fmac_f32_dpp %0, %1, %6 row_ror:4 row_mask:0xf bank_mask:0xf bound_ctrl:1\n\t"
        "v_fmac_f32_dpp %0, %1, %7 row_ror:5 row_mask:0xf bank_mask:0xf bound_ctrl:1\n\t"
        "v_fmac_f32_dpp %0, %1, %8 row_ror:6 row_mask:0xf bank_mask:0xf bound_ctrl:1\n\t"
        "v_fmac_f32_dpp %0, %1, %9 row_ror:7 row_mask:0xf bank_mask:0xf bound_ctrl:1\n\t"
        "v_fmac_f32_dpp %0, %1, %10 row_ror:8 row_mask:0xf bank_mask:0xf bound_ctrl:1\n\t"
        "v_fmac_f32_dpp %0, %1, %11 row_ror:9 row_mask:0xf bank_mask:0xf bound_ctrl:1\n\t"
        "v_fmac_f32_dpp %0, %1, %12 row_ror:10 row_mask:0xf bank_mask:0xf bound_ctrl:1\n\t"
        "v_fmac_f32_dpp %0, %1, %13 row_ror:11 row_mask:0xf bank_mask:0xf bound_ctrl:1\n\t"
        "v_fmac_f32_dpp %0, %1, %14 row_ror:12 row_mask:0xf bank_mask:0xf bound_ctrl:1\n\t"
        "v_fmac_f32_dpp %0, %1, %15 row_ror:13 row_mask:0xf bank_mask:0xf bound_ctrl:1\n\t"
        "v_fmac_f32_dpp %0, %1, %16 row_ror:14 row_mask:0xf bank_mask:0xf bound_ctrl:1\n\t"
        "v_fmac_f32_dpp %0, %1, %17 row_ror:15 row_mask:0xf bank_mask:0xf bound_ctrl:1"
        : "+v"(dot)
        : "v"(xv), "v"(q[0]), "v"(q[1]), "v"(q[2]), "v"(q[3]), "v"(q[4]), "v"(q[5]), "v"(q[6]), "v"(q[7]), "v"(q[8]),
          "v"(q[9]), "v"(q[10]), "v"(q[11]), "v"(q[12]), "v"(q[13]), "v"(q[14]), "v"(q[15]));
}
// sum of the 16 lanes of a row, in every lane
__device__ __forceinline__ float row_sum16(float v) {
    v += row_ror<8>(v);
    v += row_ror<4>(v);
    v += row_ror<2>(v);
    v += row_ror<1>(v);
    return v;
}

template <int FMT, bool BF16X, int MB, int NW>
__global__ __launch_bounds__(NW * 64) void ggr_gemv_kernel(const void *__restrict__ x, const uint8_t *__restrict__ pw,
                                                       const void *__restrict__ bias, void *__restrict__ y, int M,
                                                       int K, int N) {
    typedef GgrFmt<FMT> F;
    typedef GgrLayout<FMT> L;
    constexpr int RD = NW == 8 ? 4 : 2, OOB = 0x7FFFFF00;
    constexpr int GR = 4;                                      // strips between two meetings of the workgroup
    constexpr int XB = BF16X ? 2 : 4;
    extern __shared__ __attribute__((aligned(16))) unsigned char gr_lds[];
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int col = lane & 15, kq = lane >> 4;
    int strip = blockIdx.x;
    const int nstrips = N >> 4;
    const int nch = K >> 7;
    const int cbase = nch / NW, crem = nch % NW;
    const int n = cbase + (wave < crem ? 1 : 0);               // this wave's chunks: [c0, c0 + n)
    const int c0 = wave * cbase + min(wave, crem);
    float *red0 = (float *)gr_lds;                             // 2 x GR x [MB][16][NW] partial sums

    const size_t strip_bytes = (size_t)(nch / F::CH) * L::BLKB;
    __amdgpu_buffer_rsrc_t rs_w = make_rsrc(pw + (size_t)strip * strip_bytes, (uint32_t)strip_bytes);
    const __amdgpu_buffer_rsrc_t rs_x = make_rsrc(x, (uint32_t)M * (uint32_t)K * (uint32_t)XB);
    const __amdgpu_buffer_rsrc_t rs_none = make_rsrc(pw, 0u);
    // lane (col, kq) holds x[16 h + col] of unit kq of a chunk, h = 0, 1; rows past M read nothing
    int voff_x[MB];
#pragma unroll
    for (int m = 0; m < MB; ++m) voff_x[m] = m < M ? (m * K + kq * 32 + col) * XB : OOB;

    struct Stage {
        uint32_t qw[F::QW];
        uint32_t uh;
        uint32_t bh[4];
        float xr[MB][2];
    };
    Stage ring[RD];
    auto load_x = [&](int i, Stage &st) {
        const __amdgpu_buffer_rsrc_t rs = i < n ? rs_x : rs_none;
        const int soff = (c0 + i) * 128 * XB;
#pragma unroll
        for (int m = 0; m < MB; ++m)
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                if constexpr (BF16X) {
                    const uint32_t v = (uint16_t)__builtin_amdgcn_raw_buffer_load_b16(rs, voff_x[m] + h * 16 * XB, soff, 0);
                    st.xr[m][h] = __builtin_bit_cast(float, v << 16);
                } else {
                    st.xr[m][h] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(rs, voff_x[m] + h * 16 * XB, soff, 0));
                }
            }
    };
    auto load_w = [&](int i, Stage &st) {  // chunk i of the wave; past its share through an empty descriptor
        const __amdgpu_buffer_rsrc_t rs = i < n ? rs_w : rs_none;
        const int c = c0 + i;
        const int boff = (c / F::CH) * L::BLKB, coff = boff + (c % F::CH) * L::CHB;
#pragma unroll
        for (int pl = 0; pl < L::P128; ++pl) {
            const u32x4_t v = __builtin_amdgcn_raw_buffer_load_b128(rs, lane * 16, coff + pl * 1024, 2);
            st.qw[4 * pl] = v[0], st.qw[4 * pl + 1] = v[1], st.qw[4 * pl + 2] = v[2], st.qw[4 * pl + 3] = v[3];
        }
        if constexpr (L::P64) {
            typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));
            const u32x2_t v = __builtin_amdgcn_raw_buffer_load_b64(rs, lane * 8, coff + L::P128 * 1024, 2);
            st.qw[4 * L::P128] = v[0], st.qw[4 * L::P128 + 1] = v[1];
        }
        if constexpr (L::P32)
            st.qw[F::QW - 1] = __builtin_amdgcn_raw_buffer_load_b32(rs, lane * 4, coff + L::P128 * 1024 + L::P64 * 512, 2);
        st.uh = 0;
        if constexpr (F::UH == 2) st.uh = (uint16_t)__builtin_amdgcn_raw_buffer_load_b16(rs, lane * 2, coff + L::UH_OFF, 2);
        if constexpr (F::UH == 4) st.uh = __builtin_amdgcn_raw_buffer_load_b32(rs, lane * 4, coff + L::UH_OFF, 2);
        st.bh[0] = st.bh[1] = st.bh[2] = st.bh[3] = 0;
        if constexpr (F::BH == 16) {
            const u32x4_t v = __builtin_amdgcn_raw_buffer_load_b128(rs, col * 16, boff + L::BH_OFF, 0);
            st.bh[0] = v[0], st.bh[1] = v[1], st.bh[2] = v[2], st.bh[3] = v[3];
        } else if constexpr (F::BH == 4) {
            st.bh[0] = __builtin_amdgcn_raw_buffer_load_b32(rs, col * 4, boff + L::BH_OFF, 0);
        } else if constexpr (F::BH == 2) {
            st.bh[0] = (uint16_t)__builtin_amdgcn_raw_buffer_load_b16(rs, col * 2, boff + L::BH_OFF, 0);
        }
    };
#pragma unroll
    for (int d = 0; d < RD; ++d) {
        load_x(d, ring[d]);
        load_w(d, ring[d]);
    }

    // a workgroup walks the strips blockIdx.x, + gridDim.x, ...
    for (int it = 0;; ++it) {
        const int r = it % GR, half = (it / GR) & 1;
        float *red = red0 + (half * GR + r) * (MB * 16 * NW);
        float acc[MB];
#pragma unroll
        for (int m = 0; m < MB; ++m) acc[m] = 0.0f;
        const int nround = (n + RD - 1) / RD * RD;
        const int strip_done = strip;
        strip += gridDim.x;
        const bool last = strip >= nstrips;
        for (int i0 = 0; i0 < nround; i0 += RD) {
#pragma unroll
            for (int d = 0; d < RD; ++d) {
                const int i = i0 + d;
                // The stage is unpacked before its slot is requested again: converting first delays the
                // request by a few dozen instructions and saves a register copy of the whole stage.
                float q[32], a0, a1, b0, b1, xr[MB][2];
                ggr_ints<FMT>(ring[d].qw, q);
                ggr_factors<FMT>(ring[d].uh, ring[d].bh, 4 * ((c0 + i) % F::CH) + kq, a0, a1, b0, b1);
#pragma unroll
                for (int m = 0; m < MB; ++m) xr[m][0] = ring[d].xr[m][0], xr[m][1] = ring[d].xr[m][1];
                // the ring runs on into the next strip (same chunks of x, the next strip's weights)
                if (i + RD < nround) {
                    load_x(i + RD, ring[d]);
                    load_w(i + RD, ring[d]);
                } else if (!last) {
                    if (d == 0 && i + RD == nround)
                        rs_w = make_rsrc(pw + (size_t)strip * strip_bytes, (uint32_t)strip_bytes);
                    load_x(i + RD - nround, ring[d]);
                    load_w(i + RD - nround, ring[d]);
                }
                // chunks past the share hold zeros (weights, headers and x alike)
#pragma unroll
                for (int m = 0; m < MB; ++m) {
                    if constexpr (ggr_two_scales<FMT>) {  // a scale per half unit
                        float dot0 = 0.0f, dot1 = 0.0f;
                        ggr_dot16(q, xr[m][0], dot0);
                        ggr_dot16(q + 16, xr[m][1], dot1);
                        const float sx0 = row_sum16(xr[m][0]), sx1 = row_sum16(xr[m][1]);
                        acc[m] += (a0 * dot0 + a1 * dot1) - (b0 * sx0 + b1 * sx1);
                    } else {                               // one scale a unit: one chain, one sum
                        float dot = 0.0f;
                        ggr_dot16(q, xr[m][0], dot);
                        ggr_dot16(q + 16, xr[m][1], dot);
                        acc[m] += a0 * dot - b0 * row_sum16(xr[m][0] + xr[m][1]);
                    }
                }
            }
        }
        // The four units of a column inside the wave (lanes l, l + 16, l + 32, l + 48), then the waves
        // through LDS: red [GR strips][MB][16 columns][NW waves], two such groups in turn.  The workgroup
        // meets once a group of GR strips (or at its last strip); the next group writes the other half, so
        // one barrier a group is enough.
#pragma unroll
        for (int m = 0; m < MB; ++m) {
            float v = acc[m];
            v += __shfl_xor(v, 16, 64);
            v += __shfl_xor(v, 32, 64);
            if (lane < 16) red[(m * 16 + lane) * NW + wave] = v;
        }
        if (r == GR - 1 || last) {
            __syncthreads();
            if (threadIdx.x < (r + 1) * 16 * MB) {
                const int rr = threadIdx.x / (16 * MB), m = (threadIdx.x >> 4) % MB, c = threadIdx.x & 15;
                if (m < M) {
                    const float4_t *r4 = (const float4_t *)(red0 + (half * GR + rr) * (MB * 16 * NW) + (m * 16 + c) * NW);
                    float tot = 0.0f;
#pragma unroll
                    for (int w = 0; w < NW / 4; ++w) {
                        const float4_t t = r4[w];
                        tot += (t[0] + t[1]) + (t[2] + t[3]);
                    }
                    const int nn = 16 * (strip_done - (r - rr) * (int)gridDim.x) + c;
                    if constexpr (BF16X) {
                        if (bias) tot += BF16Traits::to_f32(((const uint16_t *)bias)[nn]);
                        ((uint16_t *)y)[(size_t)m * N + nn] = BF16Traits::from_f32(tot);
                    } else {
                        if (bias) tot += ((const float *)bias)[nn];
                        ((float *)y)[(size_t)m * N + nn] = tot;
                    }
                }
            }
        }
        if (last) break;
    }
}

// ---------------------------------------------------------------------------
// host side
// ---------------------------------------------------------------------------
static bool ggr_format(int quant) {
    return quant == OXQ_GGUF_Q4_0 || quant == OXQ_GGUF_Q8_0 || quant == OXQ_GGUF_Q4_K || quant == OXQ_GGUF_Q6_K ||
           quant == OXQ_GGUF_Q4_1 || quant == OXQ_GGUF_Q5_0 || quant == OXQ_GGUF_Q5_1 || quant == OXQ_GGUF_Q5_K ||
           quant == OXQ_GGUF_Q2_K || quant == OXQ_GGUF_Q3_K;
}
static int ggr_chunks_per_block(int quant) {
    return (quant == OXQ_GGUF_Q4_K || quant == OXQ_GGUF_Q6_K || quant == OXQ_GGUF_Q5_K || quant == OXQ_GGUF_Q2_K ||
            quant == OXQ_GGUF_Q3_K) ? 2 : 1;
}

bool gguf_res_eligible(int quant, int64_t K, int64_t N) {
    if (!ggr_format(quant) || N <= 0 || N % 16 != 0 || K <= 0 || K % (128 * ggr_chunks_per_block(quant)) != 0) return false;
    int64_t be = 0, bb = 0;
    oxq_gguf_block_layout(quant, &be, &bb);
    // 32-bit offsets inside a strip and in x
    return (uint64_t)(K / be) * (uint64_t)bb * 16 < (1ull << 31) && K <= (1 << 22);
}
size_t gguf_res_bytes(int quant, int64_t K, int64_t N) {
    int64_t be = 0, bb = 0;
    oxq_gguf_block_layout(quant, &be, &bb);
    if (quant == OXQ_GGUF_Q3_K) bb += 2;  // the 16-byte header of the copy's super-block
    return (size_t)N * (size_t)(K / be) * (size_t)bb;
}

static int ggr_waves(const oxq_ctx *ctx, int64_t K) {
    const int w = tune(ctx, OXQ_TUNE_GGR_WAVES, 16);
    return (w == 8 || K / 128 < 16) ? 8 : 16;
}
static size_t ggr_lds_bytes(const oxq_ctx *ctx, int64_t K, int mb) { return (size_t)2 * 4 * ggr_waves(ctx, K) * mb * 16 * 4; }
// rows of x one launch of the resident GEMV takes (more go to the kernels on the file layout)
// (8 rows in one pass need more registers than a wave of a 16-wave workgroup has: measured 14.8 us on
// 4096 x 4096 Q4_0 against 6.3 us at 4 rows)
// f32 activations at 5 - 8 rows take two passes of four: the file layout has no staged kernel for them
// (4096 x 4096: 31 us), while bf16 rows go to the tile matmul there, which two passes only equal.
bool gguf_res_takes(int64_t, int64_t M, int act_dtype) { return M >= 1 && (M <= 4 || (M <= 8 && act_dtype == OXQ_F32)); }

static const char *ggr_name(int q) {
    switch (q) {
    case OXQ_GGUF_Q4_0: return "q4_0";
    case OXQ_GGUF_Q8_0: return "q8_0";
    case OXQ_GGUF_Q4_K: return "q4k";
    case OXQ_GGUF_Q4_1: return "q4_1";
    case OXQ_GGUF_Q5_0: return "q5_0";
    case OXQ_GGUF_Q5_1: return "q5_1";
    case OXQ_GGUF_Q5_K: return "q5k";
    case OXQ_GGUF_Q2_K: return "q2k";
    case OXQ_GGUF_Q3_K: return "q3k";
    default: return "q6k";
    }
}

int launch_gguf_res_repack(oxq_ctx *ctx, hipStream_t s, int quant, const uint8_t *w, void *pw, int64_t K, int64_t N) {
    const size_t threads = (size_t)(N / 16) * (K / 128) * 64;
    dim3 grid((unsigned)ceil_div((int64_t)threads, 256)), block(256);
    char name[64];
    snprintf(name, sizeof name, "gguf_%s_repack", ggr_name(quant));
    set_plan(ctx, name, grid, block, 1, 1, 0);
    if (ctx->plan_only) return OXQ_OK;
#define OXQ_GR(F) \
    case F: hipLaunchKernelGGL((ggr_repack_kernel<F>), grid, block, 0, s, w, (uint8_t *)pw, (int)K, (int)N); break
    switch (quant) {
        OXQ_GR(OXQ_GGUF_Q4_0);
        OXQ_GR(OXQ_GGUF_Q8_0);
        OXQ_GR(OXQ_GGUF_Q4_K);
        OXQ_GR(OXQ_GGUF_Q6_K);
        OXQ_GR(OXQ_GGUF_Q4_1);
        OXQ_GR(OXQ_GGUF_Q5_0);
        OXQ_GR(OXQ_GGUF_Q5_1);
        OXQ_GR(OXQ_GGUF_Q5_K);
        OXQ_GR(OXQ_GGUF_Q2_K);
        OXQ_GR(OXQ_GGUF_Q3_K);
    default: return fail(OXQ_ERR_UNSUPPORTED, "gguf repack: format %d has no resident layout", quant);
    }
#undef OXQ_GR
    OXQ_HIP_CHECK(hipGetLastError());
    return OXQ_OK;
}

int launch_gguf_res_dequant(oxq_ctx *ctx, hipStream_t s, int quant, const void *pw, int64_t K, int64_t N, float *out_nk) {
    const size_t threads = (size_t)(N / 16) * (K / 128) * 64;
    dim3 grid((unsigned)ceil_div((int64_t)threads, 256)), block(256);
    char name[64];
    snprintf(name, sizeof name, "gguf_%s_res_dequant", ggr_name(quant));
    set_plan(ctx, name, grid, block, 1, 1, 0);
    if (ctx->plan_only) return OXQ_OK;
#define OXQ_GR(F) \
    case F: hipLaunchKernelGGL((ggr_dequant_kernel<F>), grid, block, 0, s, (const uint8_t *)pw, out_nk, (int)K, (int)N); break
    switch (quant) {
        OXQ_GR(OXQ_GGUF_Q4_0);
        OXQ_GR(OXQ_GGUF_Q8_0);
        OXQ_GR(OXQ_GGUF_Q4_K);
        OXQ_GR(OXQ_GGUF_Q6_K);
        OXQ_GR(OXQ_GGUF_Q4_1);
        OXQ_GR(OXQ_GGUF_Q5_0);
        OXQ_GR(OXQ_GGUF_Q5_1);
        OXQ_GR(OXQ_GGUF_Q5_K);
        OXQ_GR(OXQ_GGUF_Q2_K);
        OXQ_GR(OXQ_GGUF_Q3_K);
    default: return fail(OXQ_ERR_UNSUPPORTED, "gguf dequant: format %d has no resident layout", quant);
    }
#undef OXQ_GR
    OXQ_HIP_CHECK(hipGetLastError());
    return OXQ_OK;
}

template <int FMT, bool BF16X, int MB, int NW>
static int ggr_go(hipStream_t s, dim3 grid, const GgufProblem &p, size_t lds) {
    static LdsGrant lds_grant;  // one per instantiation
    OXQ_HIP_CHECK(lds_grant.ensure((const void *)ggr_gemv_kernel<FMT, BF16X, MB, NW>, lds));
    hipLaunchKernelGGL((ggr_gemv_kernel<FMT, BF16X, MB, NW>), grid, dim3(NW * 64), lds, s, p.x, p.w, p.bias, p.y,
                       (int)p.M, (int)p.K, (int)p.N);
    OXQ_HIP_CHECK(hipGetLastError());
    return OXQ_OK;
}
template <int FMT, int NW>
static int ggr_by_rows(hipStream_t s, dim3 grid, const GgufProblem &p, size_t lds, int mb) {
    const bool bf = p.act_dtype == OXQ_BF16;
    if (mb == 1) return bf ? ggr_go<FMT, true, 1, NW>(s, grid, p, lds) : ggr_go<FMT, false, 1, NW>(s, grid, p, lds);
    if (mb == 2) return bf ? ggr_go<FMT, true, 2, NW>(s, grid, p, lds) : ggr_go<FMT, false, 2, NW>(s, grid, p, lds);
    return bf ? ggr_go<FMT, true, 4, NW>(s, grid, p, lds) : ggr_go<FMT, false, 4, NW>(s, grid, p, lds);
}

// p.w is the resident copy
int launch_gguf_res_gemv(oxq_ctx *ctx, hipStream_t s, const GgufProblem &p0) {
    const int64_t rows0 = std::min<int64_t>(p0.M, 4);
    const int mb = rows0 <= 1 ? 1 : rows0 <= 2 ? 2 : 4;
    const int nw = ggr_waves(ctx, p0.K);
    const size_t lds = ggr_lds_bytes(ctx, p0.K, mb);
    const int64_t cap = tune(ctx, OXQ_TUNE_GGR_GRID, nw == 8 ? 512 : 256);
    dim3 grid((unsigned)std::min<int64_t>(p0.N / 16, cap > 0 ? cap : p0.N / 16));
    char name[64];
    snprintf(name, sizeof name, "gguf_%s_res_gemv_%s_m%d", ggr_name(p0.quant), p0.act_dtype == OXQ_BF16 ? "bf16" : "f32", mb);
    set_plan(ctx, name, grid, dim3(nw * 64), 1, (uint32_t)ceil_div(p0.M, 4), 0);
    if (ctx->plan_only) return OXQ_OK;
    if (!gguf_res_takes(p0.K, p0.M, p0.act_dtype)) return fail(OXQ_ERR_UNSUPPORTED, "gguf resident gemv: m = %lld", (long long)p0.M);
    if ((uintptr_t)p0.x & 3) return fail(OXQ_ERR_UNSUPPORTED, "gguf resident gemv: x must be 4-byte aligned");
    const size_t xb = p0.act_dtype == OXQ_BF16 ? 2 : 4;
    if ((uint64_t)p0.M * (uint64_t)p0.K * 4 >= (1ull << 31)) return fail(OXQ_ERR_UNSUPPORTED, "gguf resident gemv: x larger than 2 GiB");
    for (int64_t m0 = 0; m0 < p0.M; m0 += 4) {  // rows of x four at a time
        GgufProblem p = p0;
        p.M = std::min<int64_t>(4, p0.M - m0);
        p.x = (const uint8_t *)p0.x + (size_t)m0 * p0.K * xb;
        p.y = (uint8_t *)p0.y + (size_t)m0 * p0.N * xb;
        int rc;
        switch (p.quant) {
        case OXQ_GGUF_Q4_0: rc = nw == 8 ? ggr_by_rows<OXQ_GGUF_Q4_0, 8>(s, grid, p, lds, mb) : ggr_by_rows<OXQ_GGUF_Q4_0, 16>(s, grid, p, lds, mb); break;
        case OXQ_GGUF_Q8_0: rc = nw == 8 ? ggr_by_rows<OXQ_GGUF_Q8_0, 8>(s, grid, p, lds, mb) : ggr_by_rows<OXQ_GGUF_Q8_0, 16>(s, grid, p, lds, mb); break;
        case OXQ_GGUF_Q4_K: rc = nw == 8 ? ggr_by_rows<OXQ_GGUF_Q4_K, 8>(s, grid, p, lds, mb) : ggr_by_rows<OXQ_GGUF_Q4_K, 16>(s, grid, p, lds, mb); break;
        case OXQ_GGUF_Q6_K: rc = nw == 8 ? ggr_by_rows<OXQ_GGUF_Q6_K, 8>(s, grid, p, lds, mb) : ggr_by_rows<OXQ_GGUF_Q6_K, 16>(s, grid, p, lds, mb); break;
        case OXQ_GGUF_Q4_1: rc = nw == 8 ? ggr_by_rows<OXQ_GGUF_Q4_1, 8>(s, grid, p, lds, mb) : ggr_by_rows<OXQ_GGUF_Q4_1, 16>(s, grid, p, lds, mb); break;
        case OXQ_GGUF_Q5_0: rc = nw == 8 ? ggr_by_rows<OXQ_GGUF_Q5_0, 8>(s, grid, p, lds, mb) : ggr_by_rows<OXQ_GGUF_Q5_0, 16>(s, grid, p, lds, mb); break;
        case OXQ_GGUF_Q5_1: rc = nw == 8 ? ggr_by_rows<OXQ_GGUF_Q5_1, 8>(s, grid, p, lds, mb) : ggr_by_rows<OXQ_GGUF_Q5_1, 16>(s, grid, p, lds, mb); break;
        case OXQ_GGUF_Q5_K: rc = nw == 8 ? ggr_by_rows<OXQ_GGUF_Q5_K, 8>(s, grid, p, lds, mb) : ggr_by_rows<OXQ_GGUF_Q5_K, 16>(s, grid, p, lds, mb); break;
        case OXQ_GGUF_Q2_K: rc = nw == 8 ? ggr_by_rows<OXQ_GGUF_Q2_K, 8>(s, grid, p, lds, mb) : ggr_by_rows<OXQ_GGUF_Q2_K, 16>(s, grid, p, lds, mb); break;
        case OXQ_GGUF_Q3_K: rc = nw == 8 ? ggr_by_rows<OXQ_GGUF_Q3_K, 8>(s, grid, p, lds, mb) : ggr_by_rows<OXQ_GGUF_Q3_K, 16>(s, grid, p, lds, mb); break;
        default: return fail(OXQ_ERR_UNSUPPORTED, "gguf resident gemv: format %d", p.quant);
        }
        if (rc != OXQ_OK) return rc;
    }
    return OXQ_OK;
}

}  // namespace oxq
