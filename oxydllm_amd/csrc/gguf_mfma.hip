// Resident GGUF layers for 16-bit activations: a copy of the blocks laid out for the matrix cores, and the
// matmul that reads it at any number of rows (linear.rs:197-284 GgufFastPath: forward_decode up to 8 rows,
// forward_prefill above; kernels quant_kernels.metal:792-870, 1097-1221 and the mul_mm strips).
//
// The rotated copy of gguf_res.hip gives a lane one unit of 32 elements and multiplies on the vector ALU: the
// work grows with every row of x.  Here a strip of 16 output columns and a unit of 32 elements of K are one
// v_mfma_f32_16x16x32_bf16 whose 16 rows are rows of x, so 1 to 16 rows cost the same instructions:
//
//   strip j (16 columns), chunk c (128 elements of K = 4 units), lane l = (ni = l % 16, kb = l / 16):
//   word t of the lane's quants = elements 8 kb .. 8 kb + 7 of unit 4 c + t of column 16 j + ni, which is the B
//   operand of the unit's MFMA once the integers are 16-bit floats; A = the same 8 elements of row ni of x.
//
//   Q4_0  chunk = [64 lanes][16 B] nibbles (element 2 pp in nibble pp, 2 pp + 1 in nibble pp + 4 of word t, so
//                 that one AND-OR per pair yields 128 + q as two bf16) + [16 columns][4 units] f16 d    1152 B
//   Q8_0  chunk = 2 x [64 lanes][16 B] (plane h = units 2 h, 2 h + 1; bytes of a word: elements 0, 2, 1, 3 of
//                 its four, stored as q + 128) + [16 columns][4 units] f16 d                             2176 B
//   Q4_1  as Q4_0, the unit headers are {d, m} pairs                                                     1280 B
//   Q5_0  as Q4_0 + [64 lanes][4 B] of fifth bits: the bit of element 2 pp (2 pp + 1) of unit t in bit
//         4 t + pp (16 + 4 t + pp), so that one shift puts a pair's bits at positions 4 and 20           1408 B
//   Q5_1  as Q5_0 with {d, m} pairs                                                                      1536 B
//   Q5_K  as Q4_K with the plane of fifth bits in every chunk                                            2816 B
//   Q4_K  block = 2 chunks of [64 lanes][16 B] nibbles as Q4_0 + [16 columns] the super-block's first 16
//                 bytes (d, dmin, 12 scale bytes)                                                        2304 B
//   Q6_K  block = 2 chunks of { [64 lanes][16 B] low nibbles, [64 lanes][8 B] high bit pairs, [16 columns][8]
//                 int8 scales } + [16 columns] f16 d.  A scale covers 16 elements, so a step is a sub-block of 16
//                 and v_mfma_f32_16x16x16_bf16: step s of the chunk takes elements 16 s + 4 kb .. + 3; their
//                 nibbles sit in word s / 2 as Q4_0's pairs 2 (s % 2) and 2 (s % 2) + 1, their bit pairs in
//                 word s / 4 of the second plane, field 2 (s % 4) + pair of each 16-bit half              3360 B
//
// Exactly the file's bytes per weight.  The integers stay integers: the MFMA accumulates x * (bias + q) in f32
// (products of 8-bit significands are exact), a second MFMA against the constant -(bias + offset) takes the
// bias and the format's offset out in the same accumulator, and the unit's scale multiplies the sum once per
// output, in f32, as the reference's GEMV does (d * sum of q * x, quant_kernels.metal:1097-1221).
//
// A workgroup is one strip; its 16 (8) waves split the strip's chunks and stage their own rows of x through
// LDS (no barrier before the epilogue); the partial tiles meet in LDS in wave order.
#include "gguf_decode.hpp"
#include "pk4_common.hpp"

namespace oxq {

template <int FMT> struct GgmFmt;
// WQ: 16-byte quant planes a chunk; CH: chunks a block; UH: bytes of unit headers a chunk and column;
// BH: bytes of block header a column; NEG: the constant that takes bias and offset out (as a bf16 pair)
template <> struct GgmFmt<OXQ_GGUF_Q4_0> { static constexpr int WQ = 1, CH = 1, UH = 8, BH = 0; static constexpr uint32_t NEG = 0xC308C308u; };  // -136
template <> struct GgmFmt<OXQ_GGUF_Q8_0> { static constexpr int WQ = 2, CH = 1, UH = 8, BH = 0; static constexpr uint32_t NEG = 0xC300C300u; };  // -128
template <> struct GgmFmt<OXQ_GGUF_Q4_1> { static constexpr int WQ = 1, CH = 1, UH = 16, BH = 0; static constexpr uint32_t NEG = 0xC300C300u; };  // -128
template <> struct GgmFmt<OXQ_GGUF_Q5_0> { static constexpr int WQ = 1, CH = 1, UH = 8, BH = 0; static constexpr uint32_t NEG = 0xC310C310u; };  // -144
template <> struct GgmFmt<OXQ_GGUF_Q5_1> { static constexpr int WQ = 1, CH = 1, UH = 16, BH = 0; static constexpr uint32_t NEG = 0xC300C300u; };  // -128
template <> struct GgmFmt<OXQ_GGUF_Q5_K> { static constexpr int WQ = 1, CH = 2, UH = 0, BH = 16; static constexpr uint32_t NEG = 0xC300C300u; };  // -128
template <> struct GgmFmt<OXQ_GGUF_Q4_K> { static constexpr int WQ = 1, CH = 2, UH = 0, BH = 16; static constexpr uint32_t NEG = 0xC300C300u; };  // -128
template <> struct GgmFmt<OXQ_GGUF_Q6_K> { static constexpr int WQ = 1, CH = 2, UH = 8, BH = 2; static constexpr uint32_t NEG = 0xC320C320u; };  // -160

// formats with a fifth bit; with a minimum beside the scale
template <int FMT> constexpr bool ggm_fifth_bit = FMT == OXQ_GGUF_Q5_0 || FMT == OXQ_GGUF_Q5_1 || FMT == OXQ_GGUF_Q5_K;
template <int FMT> constexpr bool ggm_has_min = FMT == OXQ_GGUF_Q4_K || FMT == OXQ_GGUF_Q5_K || FMT == OXQ_GGUF_Q4_1 || FMT == OXQ_GGUF_Q5_1;

template <int FMT> struct GgmLayout {
    typedef GgmFmt<FMT> F;
    static constexpr int H_OFF = F::WQ * 1024;                                  // Q6_K: the plane of bit pairs; fifth bits
    static constexpr int UH_OFF = F::WQ * 1024 + (FMT == OXQ_GGUF_Q6_K ? 512 : ggm_fifth_bit<FMT> ? 256 : 0);
    static constexpr int CHB = UH_OFF + 16 * F::UH;
    static constexpr int BH_OFF = F::CH * CHB;
    static constexpr int BLKB = F::CH * CHB + 16 * F::BH;
    static_assert(BLKB == 16 * (128 * F::CH / GgufFmt<FMT>::BE) * GgufFmt<FMT>::BB, "the copy has the file's size");
};

// ---------------------------------------------------------------------------
// repack: one thread per (strip, chunk, lane)
// ---------------------------------------------------------------------------
// Resident column -> row of the file.  A fused gate|up layer (half = N / 2 gate rows followed by as many up rows)
// keeps, in every strip of 16, 8 gate columns followed by the 8 up columns they are multiplied with, so that one
// workgroup holds both factors of its outputs.
__device__ __forceinline__ int ggm_src_row(int c, int half) {
    if (!half) return c;
    const int j = c >> 4, cc = c & 15;
    return cc < 8 ? 8 * j + cc : half + 8 * j + (cc - 8);
}

template <int FMT>
__global__ __launch_bounds__(256) void ggm_repack_kernel(const uint8_t *__restrict__ w, uint8_t *__restrict__ pw, int K,
                                                         int N, int half) {
    typedef GgmFmt<FMT> F;
    typedef GgmLayout<FMT> L;
    const int nch = K >> 7;
    const size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= (size_t)(N >> 4) * nch * 64) return;
    const int lane = (int)(idx & 63), c = (int)((idx >> 6) % nch), strip = (int)((idx >> 6) / nch);
    const int ni = lane & 15, kb = lane >> 4;
    const size_t row_bytes = (size_t)(K / GgufFmt<FMT>::BE) * GgufFmt<FMT>::BB;
    const uint8_t *row = w + (size_t)ggm_src_row(16 * strip + ni, half) * row_bytes;
    uint8_t *blk = pw + ((size_t)strip * (nch / F::CH) + c / F::CH) * L::BLKB;
    uint8_t *chunk = blk + (c % F::CH) * L::CHB;
    if constexpr (FMT == OXQ_GGUF_Q4_0) {
        uint32_t q[4];
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            const uint8_t *p = row + (size_t)(4 * c + t) * 18;
            uint32_t v = 0;
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const int e = 8 * kb + i;  // element e of the unit: low nibble of byte e (e < 16), high of byte e - 16
                const uint32_t nib = e < 16 ? (p[2 + e] & 0xFu) : (p[2 + e - 16] >> 4);
                v |= nib << (4 * (i >> 1) + 16 * (i & 1));
            }
            q[t] = v;
            if (t == kb) *(uint16_t *)(chunk + L::UH_OFF + ni * 8 + t * 2) = ld16(p);
        }
        *(u32x4_t *)(chunk + lane * 16) = u32x4_t{q[0], q[1], q[2], q[3]};
    } else if constexpr (FMT == OXQ_GGUF_Q8_0) {
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            uint32_t q[4];
#pragma unroll
            for (int tt = 0; tt < 2; ++tt) {
                const int t = 2 * h + tt;
                const uint8_t *p = row + (size_t)(4 * c + t) * 34;
#pragma unroll
                for (int d = 0; d < 2; ++d) {  // word d of the step: elements 4 d .. 4 d + 3 of the lane's 8
                    const uint8_t *e = p + 2 + 8 * kb + 4 * d;
                    q[2 * tt + d] = ((uint32_t)(e[0] ^ 0x80u)) | ((uint32_t)(e[2] ^ 0x80u) << 8) |
                                    ((uint32_t)(e[1] ^ 0x80u) << 16) | ((uint32_t)(e[3] ^ 0x80u) << 24);
                }
                if (t == kb) *(uint16_t *)(chunk + L::UH_OFF + ni * 8 + t * 2) = ld16(p);
            }
            *(u32x4_t *)(chunk + h * 1024 + lane * 16) = u32x4_t{q[0], q[1], q[2], q[3]};
        }
    } else if constexpr (FMT == OXQ_GGUF_Q4_1 || FMT == OXQ_GGUF_Q5_0 || FMT == OXQ_GGUF_Q5_1) {
        // quant_kernels.metal:709-790, 872-1036: {d (, m)} (, 32 fifth bits), 16 bytes of nibbles as Q4_0
        constexpr bool MIN = FMT != OXQ_GGUF_Q5_0, FIFTH = FMT != OXQ_GGUF_Q4_1;
        constexpr int BB = GgufFmt<FMT>::BB, QS = (MIN ? 4 : 2) + (FIFTH ? 4 : 0);
        uint32_t q[4], hb = 0;
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            const uint8_t *p = row + (size_t)(4 * c + t) * BB;
            const uint32_t qh = FIFTH ? (ld16(p + QS - 4) | (ld16(p + QS - 2) << 16)) : 0u;
            uint32_t v = 0;
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const int e = 8 * kb + i;
                const uint32_t nib = e < 16 ? (p[QS + e] & 0xFu) : (p[QS + e - 16] >> 4);
                v |= nib << (4 * (i >> 1) + 16 * (i & 1));
                hb |= ((qh >> e) & 1u) << (4 * t + (i >> 1) + 16 * (i & 1));
            }
            q[t] = v;
            if (t == kb) {
                if constexpr (MIN) *(uint32_t *)(chunk + L::UH_OFF + ni * 16 + t * 4) = ld16(p) | (ld16(p + 2) << 16);
                else *(uint16_t *)(chunk + L::UH_OFF + ni * 8 + t * 2) = ld16(p);
            }
        }
        *(u32x4_t *)(chunk + lane * 16) = u32x4_t{q[0], q[1], q[2], q[3]};
        if constexpr (FIFTH) *(uint32_t *)(chunk + L::H_OFF + lane * 4) = hb;
    } else if constexpr (FMT == OXQ_GGUF_Q4_K || FMT == OXQ_GGUF_Q5_K) {
        // quant_kernels.metal:2438-2482: sub-block sb of the super-block reads byte (sb / 2) * 32 + e of qs, low
        // nibble if sb is even; Q5_K (1438-1680): its fifth bit is bit sb of byte e of qh
        constexpr bool FIFTH = FMT == OXQ_GGUF_Q5_K;
        const uint8_t *p = row + (size_t)(c >> 1) * GgufFmt<FMT>::BB;
        const uint8_t *qs = p + (FIFTH ? 48 : 16);
        uint32_t q[4], hb = 0;
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            const int sb = 4 * (c & 1) + t;
            uint32_t v = 0;
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const uint32_t byte = qs[(sb >> 1) * 32 + 8 * kb + i];
                v |= ((sb & 1) ? (byte >> 4) : (byte & 0xFu)) << (4 * (i >> 1) + 16 * (i & 1));
                if constexpr (FIFTH) hb |= (((uint32_t)p[16 + 8 * kb + i] >> sb) & 1u) << (4 * t + (i >> 1) + 16 * (i & 1));
            }
            q[t] = v;
        }
        *(u32x4_t *)(chunk + lane * 16) = u32x4_t{q[0], q[1], q[2], q[3]};
        if constexpr (FIFTH) *(uint32_t *)(chunk + L::H_OFF + lane * 4) = hb;
        if ((c & 1) == 0 && kb < 4) *(uint32_t *)(blk + L::BH_OFF + ni * 16 + kb * 4) = ld32a2(p + 4 * kb);
    } else if constexpr (FMT == OXQ_GGUF_Q6_K) {
        // quant_kernels.metal:2518-2554: element j of the super-block, h = j / 128, q = (j % 128) / 32, l = j % 32:
        // low nibble from ql[64 h + (q & 1) * 32 + l] (high nibble of the byte if q >= 2), bit pair 2 q of qh[32 h + l]
        const uint8_t *p = row + (size_t)(c >> 1) * 210;
        const int h = c & 1;
        uint32_t lw[4] = {0u, 0u, 0u, 0u}, hw[2] = {0u, 0u};
#pragma unroll
        for (int s2 = 0; s2 < 8; ++s2)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int jj = 16 * s2 + 4 * kb + i;  // element of this half of the super-block
                const int qq = jj >> 5, l = jj & 31;
                const uint32_t lb = p[64 * h + (qq & 1) * 32 + l];
                const uint32_t lo = qq < 2 ? (lb & 0xFu) : (lb >> 4);
                const uint32_t hi = (p[128 + 32 * h + l] >> (2 * qq)) & 3u;
                const int pair = i >> 1, half = i & 1;
                lw[s2 >> 1] |= lo << (4 * (2 * (s2 & 1) + pair) + 16 * half);
                hw[s2 >> 2] |= hi << (2 * (2 * (s2 & 3) + pair) + 16 * half);
            }
        *(u32x4_t *)(chunk + lane * 16) = u32x4_t{lw[0], lw[1], lw[2], lw[3]};
        *(uint2 *)(chunk + L::H_OFF + lane * 8) = uint2{hw[0], hw[1]};
        if (kb < 2) *(uint32_t *)(chunk + L::UH_OFF + ni * 8 + kb * 4) = ld32a2(p + 192 + 8 * h + 4 * kb);
        if (h == 0 && kb == 0) *(uint16_t *)(blk + L::BH_OFF + ni * 2) = ld16(p + 208);
    }
}

// dense [N, K] f32 from the copy, with the arithmetic of the file-layout dequant (pins the repack bit for bit)
template <int FMT>
__global__ __launch_bounds__(256) void ggm_dequant_kernel(const uint8_t *__restrict__ pw, float *__restrict__ out, int K,
                                                          int N, int half) {
    typedef GgmFmt<FMT> F;
    typedef GgmLayout<FMT> L;
    const int nch = K >> 7;
    const size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= (size_t)(N >> 4) * nch * 64) return;
    const int lane = (int)(idx & 63), c = (int)((idx >> 6) % nch), strip = (int)((idx >> 6) / nch);
    const int ni = lane & 15, kb = lane >> 4;
    const uint8_t *blk = pw + ((size_t)strip * (nch / F::CH) + c / F::CH) * L::BLKB;
    const uint8_t *chunk = blk + (c % F::CH) * L::CHB;
    const size_t orow = (size_t)ggm_src_row(16 * strip + ni, half);
    float *o = out + orow * K + (size_t)c * 128 + 8 * kb;
    if constexpr (FMT == OXQ_GGUF_Q4_0) {
        const u32x4_t q = *(const u32x4_t *)(chunk + lane * 16);
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            const float d = (float)__builtin_bit_cast(_Float16, *(const uint16_t *)(chunk + L::UH_OFF + ni * 8 + t * 2));
#pragma unroll
            for (int i = 0; i < 8; ++i)
                o[32 * t + i] = (float)((int)((q[t] >> (4 * (i >> 1) + 16 * (i & 1))) & 0xFu) - 8) * d;
        }
    } else if constexpr (FMT == OXQ_GGUF_Q8_0) {
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const u32x4_t q = *(const u32x4_t *)(chunk + h * 1024 + lane * 16);
#pragma unroll
            for (int tt = 0; tt < 2; ++tt) {
                const int t = 2 * h + tt;
                const float d = (float)__builtin_bit_cast(_Float16, *(const uint16_t *)(chunk + L::UH_OFF + ni * 8 + t * 2));
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    const int byte = ((i & 3) >> 1) | ((i & 1) << 1);  // elements 0, 2, 1, 3 in bytes 0 .. 3
                    o[32 * t + i] = (float)((int)((q[2 * tt + (i >> 2)] >> (8 * byte)) & 0xFFu) - 128) * d;
                }
            }
        }
    } else if constexpr (FMT == OXQ_GGUF_Q4_1 || FMT == OXQ_GGUF_Q5_0 || FMT == OXQ_GGUF_Q5_1) {
        constexpr bool MIN = FMT != OXQ_GGUF_Q5_0, FIFTH = FMT != OXQ_GGUF_Q4_1;
        const u32x4_t q = *(const u32x4_t *)(chunk + lane * 16);
        const uint32_t hb = FIFTH ? *(const uint32_t *)(chunk + L::H_OFF + lane * 4) : 0u;
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            const uint8_t *uh = chunk + L::UH_OFF + ni * (MIN ? 16 : 8) + t * (MIN ? 4 : 2);
            const float d = (float)__builtin_bit_cast(_Float16, *(const uint16_t *)uh);
            const float m = MIN ? (float)__builtin_bit_cast(_Float16, *(const uint16_t *)(uh + 2)) : 0.0f;
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const uint32_t v = ((q[t] >> (4 * (i >> 1) + 16 * (i & 1))) & 0xFu) |
                                   (((hb >> (4 * t + (i >> 1) + 16 * (i & 1))) & 1u) << 4);
                o[32 * t + i] = MIN ? (float)v * d + m : (float)((int)v - 16) * d;
            }
        }
    } else if constexpr (FMT == OXQ_GGUF_Q4_K || FMT == OXQ_GGUF_Q5_K) {
        const u32x4_t q = *(const u32x4_t *)(chunk + lane * 16);
        const uint32_t hb = FMT == OXQ_GGUF_Q5_K ? *(const uint32_t *)(chunk + L::H_OFF + lane * 4) : 0u;
        const uint8_t *hd = blk + L::BH_OFF + ni * 16;
        const float d = (float)__builtin_bit_cast(_Float16, *(const uint16_t *)hd);
        const float dmin = (float)__builtin_bit_cast(_Float16, *(const uint16_t *)(hd + 2));
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            uint32_t scv, mnv;
            k4_scale_min(hd + 4, 4 * (c & 1) + t, scv, mnv);
            const float d1 = d * (float)scv, m1 = dmin * (float)mnv;
#pragma unroll
            for (int i = 0; i < 8; ++i)
                o[32 * t + i] = d1 * (float)(((q[t] >> (4 * (i >> 1) + 16 * (i & 1))) & 0xFu) |
                                             (((hb >> (4 * t + (i >> 1) + 16 * (i & 1))) & 1u) << 4)) - m1;
        }
    } else if constexpr (FMT == OXQ_GGUF_Q6_K) {
        const u32x4_t lw = *(const u32x4_t *)(chunk + lane * 16);
        const uint2 hw = *(const uint2 *)(chunk + L::H_OFF + lane * 8);
        const float d = (float)__builtin_bit_cast(_Float16, *(const uint16_t *)(blk + L::BH_OFF + ni * 2));
        float *o6 = out + orow * K + (size_t)c * 128 + 4 * kb;
#pragma unroll
        for (int s2 = 0; s2 < 8; ++s2) {
            const float ds = d * (float)(int)*(const int8_t *)(chunk + L::UH_OFF + ni * 8 + s2);
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int pair = i >> 1, half = i & 1;
                const uint32_t lo = (lw[s2 >> 1] >> (4 * (2 * (s2 & 1) + pair) + 16 * half)) & 0xFu;
                const uint32_t hi = ((s2 < 4 ? hw.x : hw.y) >> (2 * (2 * (s2 & 3) + pair) + 16 * half)) & 3u;
                o6[16 * s2 + i] = ds * (float)((int)(lo | (hi << 4)) - 32);
            }
        }
    }
}

// ---------------------------------------------------------------------------
// the matmul
// ---------------------------------------------------------------------------
// bytes 0 and 2 (1 and 3) of a word as a pair of bf16: through f32, exact for 0 .. 255
__device__ __forceinline__ uint32_t ggm_bytes02(uint32_t w) {
    const float lo = (float)(w & 0xFFu), hi = (float)((w >> 16) & 0xFFu);
    return pack_hi16(__builtin_bit_cast(uint32_t, lo), __builtin_bit_cast(uint32_t, hi));
}
__device__ __forceinline__ uint32_t ggm_bytes13(uint32_t w) {
    const float lo = (float)((w >> 8) & 0xFFu), hi = (float)(w >> 24);
    return pack_hi16(__builtin_bit_cast(uint32_t, lo), __builtin_bit_cast(uint32_t, hi));
}
typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));
__device__ __forceinline__ float ggm_f16(uint32_t bits) { return (float)__builtin_bit_cast(_Float16, (uint16_t)bits); }

// The registers of one chunk: its quants and headers as requested, and what turns them into MFMA operands and
// the factors of a step.  A step's sum t = sum over the step's elements of x * q', q' = q minus the format's
// offset (exact integers); y += f0(step) * t + f1(step) * (sum of x) where the format has a minimum.
template <int FMT> struct GgmChunk {
    typedef GgmFmt<FMT> F;
    typedef GgmLayout<FMT> L;
    static constexpr int NSTEP = FMT == OXQ_GGUF_Q6_K ? 8 : 4;
    static constexpr bool HAS_MIN = ggm_has_min<FMT>;
    // vector loads of one request()
    static constexpr int LOADS = (F::UH ? 1 : 0) + (F::BH ? 1 : 0) + F::WQ + ((FMT == OXQ_GGUF_Q6_K || ggm_fifth_bit<FMT>) ? 1 : 0);
    u32x4_t q[F::WQ];
    uint32_t qh[FMT == OXQ_GGUF_Q6_K ? 2 : 1];
    uint32_t uh[F::UH == 16 ? 4 : F::UH ? 2 : 1];   // unit headers of the column: four f16 d or {d, m} pairs, eight int8 scales (Q6_K)
    uint32_t bh[F::BH == 16 ? 4 : 1];  // block header of the column

    // c: the chunk's index in its strip
    template <typename RS>
    __device__ __forceinline__ void request(const RS &rs, int lane, int ni, int c, int strip_off) {
        const int blk = strip_off + (c / F::CH) * L::BLKB, soff = blk + (c % F::CH) * L::CHB;
        // headers first: the factors and the minimum's term are worked out while the quants are on their way
        if constexpr (F::UH == 8) {
            const u32x2_t v = __builtin_amdgcn_raw_buffer_load_b64(rs, ni * 8, soff + L::UH_OFF, 2);
            uh[0] = v[0], uh[1] = v[1];
        } else if constexpr (F::UH == 16) {
            const u32x4_t v = __builtin_amdgcn_raw_buffer_load_b128(rs, ni * 16, soff + L::UH_OFF, 2);
            uh[0] = v[0], uh[1] = v[1], uh[2] = v[2], uh[3] = v[3];
        }
        if constexpr (F::BH == 16) {
            const u32x4_t v = __builtin_amdgcn_raw_buffer_load_b128(rs, ni * 16, blk + L::BH_OFF, 0);
            bh[0] = v[0], bh[1] = v[1], bh[2] = v[2], bh[3] = v[3];
        } else if constexpr (F::BH == 2) {
            bh[0] = __builtin_amdgcn_raw_buffer_load_b32(rs, (ni >> 1) * 4, blk + L::BH_OFF, 0);
        }
#pragma unroll
        for (int pl = 0; pl < F::WQ; ++pl) q[pl] = __builtin_amdgcn_raw_buffer_load_b128(rs, lane * 16, soff + pl * 1024, 2);
        if constexpr (FMT == OXQ_GGUF_Q6_K) {
            const u32x2_t v = __builtin_amdgcn_raw_buffer_load_b64(rs, lane * 8, soff + L::H_OFF, 2);
            qh[0] = v[0], qh[1] = v[1];
        } else if constexpr (ggm_fifth_bit<FMT>) {
            qh[0] = __builtin_amdgcn_raw_buffer_load_b32(rs, lane * 4, soff + L::H_OFF, 2);
        }
    }
    // The factors of the chunk's steps, once per chunk when its registers have arrived; half = c % 2 (wave-uniform).
    // f0[st] multiplies the step's sum, f1[st] (formats with a minimum) the bias term -128 sum(x).
    __device__ __forceinline__ void factors(int half, int ni, float (&f0)[NSTEP], float (&f1)[NSTEP]) const {
        if constexpr (FMT == OXQ_GGUF_Q4_K || FMT == OXQ_GGUF_Q5_K) {
            // get_scale_min_k4 (quant_kernels.metal:2438-2450) for the chunk's four sub-blocks at once, a byte each
            // (selected by mask: as a branch on the chunk's parity the two sides kept twice the registers alive)
            const uint32_t hm = half ? 0xFFFFFFFFu : 0u;
            const uint32_t sc4 = (((bh[3] & 0x0F0F0F0Fu) | ((bh[1] >> 2) & 0x30303030u)) & hm) | (bh[1] & 0x3F3F3F3Fu & ~hm);
            const uint32_t mn4 = ((((bh[3] >> 4) & 0x0F0F0F0Fu) | ((bh[2] >> 2) & 0x30303030u)) & hm) | (bh[2] & 0x3F3F3F3Fu & ~hm);
            const float d = ggm_f16(bh[0] & 0xFFFFu), dm = ggm_f16(bh[0] >> 16) * 0.0078125f;  // dmin / 128
#pragma unroll
            for (int t = 0; t < 4; ++t) {
                f0[t] = d * (float)((sc4 >> (8 * t)) & 0xFFu);
                f1[t] = dm * (float)((mn4 >> (8 * t)) & 0xFFu);
            }
        } else if constexpr (FMT == OXQ_GGUF_Q6_K) {
            const float d = ggm_f16((ni & 1) ? (bh[0] >> 16) : (bh[0] & 0xFFFFu));
#pragma unroll
            for (int st = 0; st < 8; ++st) f0[st] = d * (float)(int)(int8_t)((uh[st >> 2] >> (8 * (st & 3))) & 0xFFu), f1[st] = 0.f;
        } else if constexpr (F::UH == 16) {  // w = d q + m: the minimum times sum(x) = -m / 128 times the bias term
#pragma unroll
            for (int st = 0; st < 4; ++st) f0[st] = ggm_f16(uh[st] & 0xFFFFu), f1[st] = ggm_f16(uh[st] >> 16) * -0.0078125f;
        } else {
#pragma unroll
            for (int st = 0; st < 4; ++st) f0[st] = ggm_f16((st & 1) ? (uh[st >> 1] >> 16) : (uh[st >> 1] & 0xFFFFu)), f1[st] = 0.f;
        }
    }
    // B operand of step st: bias + q as bf16 pairs (four for a step of 32 elements, two for one of 16)
    __device__ __forceinline__ void operand(int st, uint32_t (&b)[4], const NibbleMasks &nm) const {
        if constexpr (FMT == OXQ_GGUF_Q4_0 || FMT == OXQ_GGUF_Q4_K || FMT == OXQ_GGUF_Q4_1) {
#pragma unroll
            for (int pp = 0; pp < 4; ++pp) b[pp] = BF16Traits::unpack1(q[0][st], pp, nm);
        } else if constexpr (ggm_fifth_bit<FMT>) {  // nibble | fifth bit << 4; m1: the bits' mask, in a register
#pragma unroll
            for (int pp = 0; pp < 4; ++pp) {
                const int sft = 4 * st + pp - 4;
                const uint32_t hs = sft < 0 ? (qh[0] << -sft) : (qh[0] >> sft);
                b[pp] = (hs & nm.m1) | BF16Traits::unpack1(q[0][st], pp, nm);
            }
        } else if constexpr (FMT == OXQ_GGUF_Q8_0) {
            const uint32_t w0 = q[st >> 1][2 * (st & 1)], w1 = q[st >> 1][2 * (st & 1) + 1];
            b[0] = ggm_bytes02(w0), b[1] = ggm_bytes13(w0), b[2] = ggm_bytes02(w1), b[3] = ggm_bytes13(w1);
        } else {  // Q6_K: nibble | bit pair << 4, 128 + (0 .. 63) is exact in bf16
            const uint32_t lw = q[0][st >> 1], hw = qh[st >> 2];
#pragma unroll
            for (int pr = 0; pr < 2; ++pr) {
                const int f = 2 * (st & 3) + pr;
                const uint32_t hs = f < 2 ? (hw << (4 - 2 * f)) : (hw >> (2 * f - 4));
                b[pr] = (hs & nm.m1) | BF16Traits::unpack1(lw, 2 * (st & 1) + pr, nm);  // m1: the bit pairs' mask, in a register
            }
            b[2] = b[3] = 0u;
        }
    }
};

typedef short short4_t __attribute__((ext_vector_type(4)));
__device__ __forceinline__ float4_t ggm_mfma16(uint32_t a0, uint32_t a1, uint32_t b0, uint32_t b1, float4_t c) {
    return __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(__builtin_bit_cast(short4_t, u32x2_t{a0, a1}),
                                                     __builtin_bit_cast(short4_t, u32x2_t{b0, b1}), c, 0, 0, 0);
}

// Epilogue of a fused gate|up layer (ffn.rs:386-400 runs gated_silu_fused / gated_gelu_tanh_fused on the fused
// projection's output): the waves' partial tiles meet in LDS as in pk4n_epilogue; a thread then owns (row, gate
// column p of a strip and its up column p + 8), adds the waves in order, rounds both factors to bf16 as the
// projection's own output would be, and writes act(gate) * up to y [M, N / 2].
template <int MT, int NS, int NW>
__device__ __forceinline__ void ggm_epilogue_act(const float4_t (&acc)[MT][NS], const uint16_t *__restrict__ bias,
                                                 uint16_t *__restrict__ y, int M, int N, int j, int m0, int act,
                                                 int wave, int lane) {
    typedef BF16Traits TT;
    constexpr int NT = NW * 64, ROWS = 16 * MT;
    extern __shared__ __attribute__((aligned(16))) unsigned char pk4_lds[];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            float *dst = (float *)(pk4_lds + (size_t)wave * MT * 4096) + ((mt * 4 + e) * 64 + lane) * NS;
#pragma unroll
            for (int f = 0; f < NS; ++f) dst[f] = acc[mt][f][e];
        }
    __syncthreads();
    const int half = N >> 1;
    for (int t = threadIdx.x; t < ROWS * 8 * NS; t += NT) {
        const int p = t & 7, f = (t >> 3) % NS, ml = t / (8 * NS);
        if (m0 + ml >= M) continue;
        const int mt = ml >> 4, r = ml & 15, kb = r >> 2, e = r & 3;
        float g = 0.f, u = 0.f;
#pragma unroll
        for (int s = 0; s < NW; ++s) {
            const float *src = (const float *)(pk4_lds + (size_t)s * MT * 4096) + ((mt * 4 + e) * 64 + kb * 16 + p) * NS + f;
            g += src[0];
            u += src[8 * NS];
        }
        const int n = 8 * (NS * j + f) + p;
        if (bias) {
            g += TT::to_f32(bias[n]);
            u += TT::to_f32(bias[half + n]);
        }
        g = TT::to_f32(TT::from_f32(g));
        u = TT::to_f32(TT::from_f32(u));
        y[(size_t)(m0 + ml) * half + n] = TT::from_f32(mul_f32_rn(act == 1 ? silu_f32(g) : gelu_tanh_f32(g), u));
    }
}

template <int FMT, int MT, int XQ, int NW, int NS>
__global__ __launch_bounds__(NW * 64) void ggm_kernel(const uint16_t *__restrict__ x, const uint8_t *__restrict__ pw,
                                                      const uint16_t *__restrict__ bias, uint16_t *__restrict__ y,
                                                      float *__restrict__ ws, int M, int K, int N, int cslice, int act) {
    typedef BF16Traits TT;
    typedef MfmaOps<TT> Ops;
    typedef GgmFmt<FMT> F;
    typedef GgmLayout<FMT> L;
    typedef GgmChunk<FMT> C;
    constexpr int ROWS = 16 * MT, AQ = XQ, SLOT = ROWS * 256, OOB = 0x7FFFFF00, NSTEP = C::NSTEP;
    // chunks in flight a wave: three (4096 x 4096 at one row, Q8_0: 5.06 us with three, 5.87 with two); two
    // where a workgroup takes four strips, whose quants are four times the registers
    constexpr int RD = NS > 1 ? 2 : 3;
    constexpr bool K16 = NSTEP == 8;  // steps of 16 elements
    extern __shared__ __attribute__((aligned(16))) unsigned char pk4_lds[];

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int ni = lane & 15, kb = lane >> 4;
    const int j = blockIdx.x;
    const int m0 = blockIdx.z * ROWS;
    const int NC = K >> 7;
    const int sc0 = blockIdx.y * cslice;
    const int SC = min(NC, sc0 + cslice) - sc0;
    const int cbase = SC / NW, crem = SC % NW;
    const int nloc = cbase + (wave < crem ? 1 : 0);
    const int cc0 = sc0 + wave * cbase + min(wave, crem);
    unsigned char *slot = pk4_lds + wave * SLOT;

    // the workgroup's NS neighbouring strips behind one descriptor (NS * strip_bytes < 2^31: checked on the host)
    const uint32_t strip_bytes = (uint32_t)(NC / F::CH) * (uint32_t)L::BLKB;
    const __amdgpu_buffer_rsrc_t rs_w = make_rsrc(pw + (size_t)j * NS * strip_bytes, NS * strip_bytes);
    const int xrows = min(M - m0, ROWS);
    const __amdgpu_buffer_rsrc_t rs_x = make_rsrc(x + (size_t)m0 * K, (uint32_t)xrows * (uint32_t)K * 2u);
    const __amdgpu_buffer_rsrc_t rs_none = make_rsrc(pw, 0u);
    int voff_a[AQ];
#pragma unroll
    for (int q = 0; q < AQ; ++q) {
        const int r = 4 * q + kb;
        voff_a[q] = r < xrows ? (r * K * 2 + ni * 16) : OOB;
    }
    // x in LDS: row r of the tile at r * 256, its sixteen 16-byte pieces XOR-swizzled by the row
    int a_wr[4];
#pragma unroll
    for (int qq = 0; qq < 4; ++qq) a_wr[qq] = kb * 256 + (((ni ^ kb) ^ (qq << 2)) << 4);
    // step st of the chunk: elements 32 st + 8 kb .. + 7 of row ni (16 st + 4 kb .. + 3 for steps of 16)
    int a_rd[NSTEP];
#pragma unroll
    for (int st = 0; st < NSTEP; ++st)
        a_rd[st] = K16 ? ni * 256 + (((2 * st + (kb >> 1)) ^ ni) << 4) + (kb & 1) * 8 : ni * 256 + (((4 * st + kb) ^ ni) << 4);
    // both masks in registers: v_and_or_b32 takes one literal, and the exponent pattern is it
    const NibbleMasks nm = FMT == OXQ_GGUF_Q6_K ? NibbleMasks{vgpr_const(0x000F000Fu), vgpr_const(0x00300030u)}
                           : ggm_fifth_bit<FMT> ? NibbleMasks{vgpr_const(0x000F000Fu), vgpr_const(0x00100010u)} : nibble_masks();
#pragma unroll
    for (int q = AQ; q < 4 * MT; ++q) {  // rows no call of this instantiation brings stay zero
        const int row = 4 * q + kb;
        *(u32x4_t *)(slot + row * 256 + ((ni ^ (row & 15)) << 4)) = u32x4_t{0u, 0u, 0u, 0u};
    }

    C wr[RD][NS];
    u32x4_t ar[RD][AQ];
    auto request = [&](int i, C (&w)[NS], u32x4_t (&a)[AQ]) {
        const bool live = i < nloc;  // wave-uniform
        const __amdgpu_buffer_rsrc_t rx = live ? rs_x : rs_none, rw = live ? rs_w : rs_none;
        const int c = cc0 + i;
#pragma unroll
        for (int q = 0; q < AQ; ++q) a[q] = __builtin_amdgcn_raw_buffer_load_b128(rx, voff_a[q], c * 256, 0);
#pragma unroll
        for (int f = 0; f < NS; ++f) w[f].request(rw, lane, ni, c, (int)(f * strip_bytes));
        __builtin_amdgcn_sched_barrier(0);  // chunks are requested in the order they are used
    };
#pragma unroll
    for (int d = 0; d < RD; ++d) request(d, wr[d], ar[d]);

    float4_t acc[MT][NS];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int f = 0; f < NS; ++f) acc[mt][f] = float4_t{0.f, 0.f, 0.f, 0.f};
    const uint32_t neg[4] = {F::NEG, F::NEG, F::NEG, F::NEG};
    const float4_t zero4 = float4_t{0.f, 0.f, 0.f, 0.f};

    // A operand of step st, row tile mt
    auto load_a = [&](int st, int mt, uint32_t (&a)[4]) {
        if constexpr (K16) {
            const uint2 av = *(const uint2 *)(slot + mt * 4096 + a_rd[st]);
            a[0] = av.x, a[1] = av.y, a[2] = 0u, a[3] = 0u;
        } else {
            const u32x4_t av = *(const u32x4_t *)(slot + mt * 4096 + a_rd[st]);
            a[0] = av[0], a[1] = av[1], a[2] = av[2], a[3] = av[3];
        }
    };
    auto mma = [&](const uint32_t (&a)[4], const uint32_t (&b)[4], float4_t c) -> float4_t {
        if constexpr (K16) return ggm_mfma16(a[0], a[1], b[0], b[1], c);
        else return Ops::mfma(a, b, c);
    };

    auto chunk = [&](int i, auto cur_c, bool more) {
        constexpr int CUR = decltype(cur_c)::value;
#pragma unroll
        for (int q = 0; q < AQ; ++q) *(u32x4_t *)(slot + q * 1024 + a_wr[q & 3]) = ar[CUR][q];
        float f0[NSTEP], f1[NSTEP];
        if constexpr (MT == 1) {
            // what depends on x alone first (x is requested ahead of the chunk's quants): the operands and the
            // bias term of four steps, so that one MFMA a step and strip is left when the quants arrive
#pragma unroll
            for (int g = 0; g < NSTEP; g += 4) {
                uint32_t a[4][4];
                float4_t tn[4];
#pragma unroll
                for (int s4 = 0; s4 < 4; ++s4) {
                    load_a(g + s4, 0, a[s4]);
                    tn[s4] = mma(a[s4], neg, zero4);
                }
#pragma unroll
                for (int f = 0; f < NS; ++f) {
                    const C &w = wr[CUR][f];
                    if (g == 0 || NS > 1) w.factors((cc0 + i) & 1, ni, f0, f1);
                    if constexpr (C::HAS_MIN) {
#pragma unroll
                        for (int s4 = 0; s4 < 4; ++s4)
#pragma unroll
                            for (int e = 0; e < 4; ++e) acc[0][f][e] = fmaf(f1[g + s4], tn[s4][e], acc[0][f][e]);
                    }
#pragma unroll
                    for (int s4 = 0; s4 < 4; ++s4) {
                        uint32_t b[4];
                        w.operand(g + s4, b, nm);
                        const float4_t t = mma(a[s4], b, tn[s4]);
#pragma unroll
                        for (int e = 0; e < 4; ++e) acc[0][f][e] = fmaf(f0[g + s4], t[e], acc[0][f][e]);
                    }
                    if constexpr (NS > 1) __builtin_amdgcn_sched_barrier(0);  // one strip's operands at a time
                }
            }
        } else {  // more row tiles: step by step, the registers do not hold a chunk's operands
#pragma unroll
            for (int f = 0; f < NS; ++f) {
                const C &w = wr[CUR][f];
                w.factors((cc0 + i) & 1, ni, f0, f1);
#pragma unroll
                for (int st = 0; st < NSTEP; ++st) {
                    uint32_t b[4];
                    w.operand(st, b, nm);
#pragma unroll
                    for (int mt = 0; mt < MT; ++mt) {
                        uint32_t a[4];
                        load_a(st, mt, a);
                        const float4_t tn = mma(a, neg, zero4);
                        const float4_t t = mma(a, b, tn);
#pragma unroll
                        for (int e = 0; e < 4; ++e) {
                            acc[mt][f][e] = fmaf(f0[st], t[e], acc[mt][f][e]);
                            if constexpr (C::HAS_MIN) acc[mt][f][e] = fmaf(f1[st], tn[e], acc[mt][f][e]);
                        }
                    }
                }
                if constexpr (NS > 1) __builtin_amdgcn_sched_barrier(0);  // one strip's operands at a time
            }
        }
        if (more) request(i + RD, wr[CUR], ar[CUR]);
        __builtin_amdgcn_sched_barrier(0);  // one chunk's operands in the registers at a time
    };
    {
        int i = 0;
        if constexpr (RD == 2) {
            for (; i + 1 < nloc; i += 2) {
                chunk(i, std::integral_constant<int, 0>{}, true);
                chunk(i + 1, std::integral_constant<int, 1>{}, true);
            }
            if (i < nloc) chunk(i, std::integral_constant<int, 0>{}, false);
        } else {
            for (; i + 2 < nloc; i += 3) {
                chunk(i, std::integral_constant<int, 0>{}, true);
                chunk(i + 1, std::integral_constant<int, 1>{}, true);
                chunk(i + 2, std::integral_constant<int, 2>{}, true);
            }
            if (i < nloc) chunk(i, std::integral_constant<int, 0>{}, false);
            if (i + 1 < nloc) chunk(i + 1, std::integral_constant<int, 1>{}, false);
        }
    }
    if (act) ggm_epilogue_act<MT, NS, NW>(acc, bias, y, M, N, j, m0, act, wave, lane);
    else pk4n_epilogue<TT, MT, NS, NW>(acc, bias, y, ws, M, N, j, m0, wave, lane);
}

// ---------------------------------------------------------------------------
// prefill: the decomposition of pk4n_gemm_kernel on the matrix-core copy
// ---------------------------------------------------------------------------
// More rows than the integer kernel above should take (every 32 of them read the weights again, and the scale is
// applied per unit and output) run the tile arithmetic of the reference's mul_mm (quant_kernels.metal strips,
// linear.rs:270-284 forward_prefill): B = the dequantized weight rounded once to bf16, f32 accumulation.  A
// workgroup takes 64 rows of x and eight waves x four neighbouring strips (512 columns); a chunk (128 elements of
// K) of the rows goes from global memory straight into LDS once for all eight waves (two buffers, one barrier a
// chunk); a wave rings its four strips' chunks in two halves, turns a step's integers into the weight with one
// fma each (two where a five-bit format has a minimum) from the integer kernel's own factors, and keeps the whole
// K in its accumulators: one launch, no partial tiles.
// KS = 4: two waves of 64 columns a workgroup and the four waves of a column group take every fourth chunk, as in
// pk4_gemm_kernel - the form for 33 to a few hundred rows of a wide layer.
template <int FMT, int MT, int KS>
__global__ __launch_bounds__(512) void ggm_gemm_kernel(const uint16_t *__restrict__ x, const uint8_t *__restrict__ pw,
                                                       const uint16_t *__restrict__ bias, uint16_t *__restrict__ y,
                                                       int M, int K, int N, int NG, int RT, int act) {
    typedef BF16Traits TT;
    typedef MfmaOps<TT> Ops;
    typedef GgmFmt<FMT> F;
    typedef GgmLayout<FMT> L;
    typedef GgmChunk<FMT> C;
    static_assert(KS == 1 || KS == MT, "wave kq of a column group finishes row tile kq");
    constexpr int SPW = 8 / KS;  // waves of 64 columns a workgroup
    constexpr int ROWS = 16 * MT, XBUF = KS * ROWS * 256, XV = ROWS / 4 / SPW, NSTEP = C::NSTEP;
    constexpr bool K16 = NSTEP == 8;
    constexpr int RING = 4 * C::LOADS;  // vector loads of a chunk's weights: younger than the chunk's loads of x
    extern __shared__ __attribute__((aligned(16))) unsigned char pk4_lds[];

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int ni = lane & 15, kb = lane >> 4;
    const int ws = wave % SPW, kq = wave / SPW;  // the wave's column group of the workgroup, and its share of K
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
    const int NC = K >> 7, NR = (NC + KS - 1) / KS;  // chunks; rounds of KS chunks
    const int xrows = min(M - m0, ROWS);

    const uint32_t strip_bytes = (uint32_t)(NC / F::CH) * (uint32_t)L::BLKB;
    const __amdgpu_buffer_rsrc_t rs_none = make_rsrc(pw, 0u);
    const __amdgpu_buffer_rsrc_t rs_wl = make_rsrc(pw + (size_t)(live ? 4 * j : 0) * strip_bytes, 4u * strip_bytes);
    const __amdgpu_buffer_rsrc_t rs_w = live ? rs_wl : rs_none;
    const __amdgpu_buffer_rsrc_t rs_x = make_rsrc(x + (size_t)m0 * K, (uint32_t)xrows * (uint32_t)K * 2u);
    // x: load q of a wave brings rows 4 (XV wave + q) .. + 3 of the chunk, lane l the 16 bytes that belong at
    // position l % 16 of row l / 16 (piece (l % 16) ^ (row % 16): the swizzle the fragment reads undo); rows past
    // M lie beyond the descriptor and arrive as zeros
    int xo[XV];
#pragma unroll
    for (int q = 0; q < XV; ++q) {
        const int r = 4 * (ws * XV + q) + (lane >> 4);
        xo[q] = r * K * 2 + (((lane & 15) ^ (r & 15)) << 4);
    }
    int a_rd[NSTEP];
#pragma unroll
    for (int st = 0; st < NSTEP; ++st)
        a_rd[st] = K16 ? ni * 256 + (((2 * st + (kb >> 1)) ^ ni) << 4) + (kb & 1) * 8 : ni * 256 + (((4 * st + kb) ^ ni) << 4);
    const NibbleMasks nm = FMT == OXQ_GGUF_Q6_K ? NibbleMasks{vgpr_const(0x000F000Fu), vgpr_const(0x00300030u)}
                           : ggm_fifth_bit<FMT> ? NibbleMasks{vgpr_const(0x000F000Fu), vgpr_const(0x00100010u)} : nibble_masks();
    constexpr float NEGF = __builtin_bit_cast(float, (F::NEG & 0xFFFFu) << 16);
    constexpr bool NIB = FMT == OXQ_GGUF_Q4_0 || FMT == OXQ_GGUF_Q4_1 || FMT == OXQ_GGUF_Q4_K;

    C wr[2][4];
    auto dma_x = [&](int r) {  // round r: the wave's chunk is KS r + kq, its tile of x at kq ROWS 256 of the round's buffer
        const int i = KS * r + kq;
        const __amdgpu_buffer_rsrc_t rs = i < NC ? rs_x : rs_none;
#pragma unroll
        for (int q = 0; q < XV; ++q)
            pk4g_load_lds16(rs, pk4_lds + (r & 1) * XBUF + kq * (ROWS * 256) + (ws * XV + q) * 1024, xo[q], i * 256);
    };
    auto request = [&](int i, C (&w)[4]) {
        const __amdgpu_buffer_rsrc_t rs = i < NC ? rs_w : rs_none;
#pragma unroll
        for (int f = 0; f < 4; ++f) w[f].request(rs, lane, ni, i, (int)(f * strip_bytes));
    };

    dma_x(0);
    __builtin_amdgcn_sched_barrier(0);  // requests keep this order: the wait counts rely on it
    request(kq, wr[0]);
    __builtin_amdgcn_sched_barrier(0);
    float4_t acc[MT][4];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int f = 0; f < 4; ++f) acc[mt][f] = float4_t{0.f, 0.f, 0.f, 0.f};
    pk4g_wait_vmcnt<RING>();
    __syncthreads();

    auto chunk = [&](int r, auto cur_c) {
        constexpr int CUR = decltype(cur_c)::value;
        const int i = KS * r + kq;  // past NC (a ragged last round): zeros from both streams
        dma_x(r + 1);
        __builtin_amdgcn_sched_barrier(0);
        request(i + KS, wr[CUR ^ 1]);
        __builtin_amdgcn_sched_barrier(0);  // not sunk to the chunk's end, where the next chunk would wait for them
        const unsigned char *buf = pk4_lds + (r & 1) * XBUF + kq * (ROWS * 256);
        // w = f0 q' + c2 with q' = q minus the format's offset and c2 = -(minimum): exact products, one rounding -
        // the bits of the dense dequant (ggm_dequant_kernel), so the tile the matrix cores see is the reference's
        float f0[4][NSTEP], c2[4][C::HAS_MIN ? NSTEP : 1];
#pragma unroll
        for (int f = 0; f < 4; ++f) {
            float f1[NSTEP];
            wr[CUR][f].factors(i & 1, ni, f0[f], f1);
            if constexpr (C::HAS_MIN) {
#pragma unroll
                for (int st = 0; st < NSTEP; ++st) c2[f][st] = -128.0f * f1[st];
            }
        }
#pragma unroll
        for (int st = 0; st < NSTEP; ++st) {
            uint32_t a[MT][4];
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) {
                if constexpr (K16) {
                    const uint2 av = *(const uint2 *)(buf + mt * 4096 + a_rd[st]);
                    a[mt][0] = av.x, a[mt][1] = av.y, a[mt][2] = 0u, a[mt][3] = 0u;
                } else {
                    const u32x4_t av = *(const u32x4_t *)(buf + mt * 4096 + a_rd[st]);
                    a[mt][0] = av[0], a[mt][1] = av[1], a[mt][2] = av[2], a[mt][3] = av[3];
                }
            }
#pragma unroll
            for (int f = 0; f < 4; ++f) {
                uint32_t b[4];
                const float sc = f0[f][st];
                if constexpr (NIB) {
                    // plain nibbles (pair pp = nibble pp of each 16-bit half): masked in place a byte holds q or 16 q,
                    // which v_cvt_f32_ubyteN widens; one fma a weight
                    uint32_t tl, th;
                    pk4g_nibbles(wr[CUR][f].q[0][st], tl, th);
                    Pk4gBf16 cv;
                    cv.s = sc, cv.s16 = sc * 0.0625f, cv.c = C::HAS_MIN ? c2[f][st] : (NEGF + 128.0f) * sc;
                    b[0] = cv.template pair<0, false>(tl), b[1] = cv.template pair<0, true>(th);
                    b[2] = cv.template pair<1, false>(tl), b[3] = cv.template pair<1, true>(th);
                } else if constexpr (FMT == OXQ_GGUF_Q8_0) {
                    // bytes q + 128, elements 0, 2, 1, 3 of a word's four: pairs in bytes (0, 2) and (1, 3)
                    const uint32_t w0 = wr[CUR][f].q[st >> 1][2 * (st & 1)], w1 = wr[CUR][f].q[st >> 1][2 * (st & 1) + 1];
                    Pk4gBf16 cv;
                    cv.s = sc, cv.s16 = 0.f, cv.c = -128.0f * sc;
                    b[0] = cv.template pair<0, false>(w0), b[1] = cv.template pair<1, false>(w0);
                    b[2] = cv.template pair<0, false>(w1), b[3] = cv.template pair<1, false>(w1);
                } else {
                    // bias + q as bf16 (the integer kernel's operand): f0 (bias + q) + NEG f0 is exact in one fma
                    wr[CUR][f].operand(st, b, nm);
                    const float c = NEGF * sc;
#pragma unroll
                    for (int pp = 0; pp < (K16 ? 2 : 4); ++pp) {
                        float lo = __builtin_fmaf(__builtin_bit_cast(float, b[pp] << 16), sc, c);
                        float hi = __builtin_fmaf(__builtin_bit_cast(float, b[pp] & 0xFFFF0000u), sc, c);
                        if constexpr (C::HAS_MIN) lo += c2[f][st], hi += c2[f][st];
                        b[pp] = __builtin_bit_cast(uint32_t, __builtin_convertvector(float2_t{lo, hi}, bf16x2_t));
                    }
                }
#pragma unroll
                for (int mt = 0; mt < MT; ++mt) {
                    if constexpr (K16) acc[mt][f] = ggm_mfma16(a[mt][0], a[mt][1], b[0], b[1], acc[mt][f]);
                    else acc[mt][f] = Ops::mfma(a[mt], b, acc[mt][f]);
                }
            }
        }
        __builtin_amdgcn_sched_barrier(0);
        pk4g_wait_vmcnt<RING>();  // this wave's part of the next chunk of x is in LDS
        __syncthreads();
    };
    {
        int r = 0;
        for (; r + 1 < NR; r += 2) {
            chunk(r, std::integral_constant<int, 0>{});
            chunk(r + 1, std::integral_constant<int, 1>{});
        }
        if (r < NR) chunk(r, std::integral_constant<int, 0>{});
    }

    // the finished tile rows of this wave: all of them (KS = 1), or row tile kq summed over the column group's waves
    constexpr int FT = KS == 1 ? MT : 1;
    float4_t fin[FT][4];
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
    if (act) {
        // Fused gate|up layer (ggm_src_row): strip 4 j + f holds gate columns 8 (4 j + f) .. + 7 in lanes ni < 8 and
        // the up columns they meet in lanes ni + 8.  The two lanes of a pair exchange their four values (row_ror:8)
        // and finish two outputs each; both factors rounded to bf16 first, as in ggm_epilogue_act.  y is [M, N / 2].
        const int half = N >> 1, p = ni & 7;
        const bool low = ni < 8;
        float bv[4] = {0.f, 0.f, 0.f, 0.f};
        if (bias) {
#pragma unroll
            for (int f = 0; f < 4; ++f) bv[f] = TT::to_f32(bias[(low ? 0 : half) + 8 * (4 * j + f) + p]);
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
#pragma unroll
                for (int q = 0; q < 2; ++q) {
                    const int f = low ? q : 2 + q;
                    const float gq = low ? mine[q] : other[2 + q], uq = low ? other[q] : mine[2 + q];
                    const uint16_t o = TT::from_f32(mul_f32_rn(act == 1 ? silu_f32(gq) : gelu_tanh_f32(gq), uq));
                    if (row < M) y[(size_t)row * half + 8 * (4 * j + f) + p] = o;
                }
            }
        return;
    }
    // row 16 mt + 4 kb + e, column 64 j + 16 f + ni
    float bv[4] = {0.f, 0.f, 0.f, 0.f};
    if (bias) {
#pragma unroll
        for (int f = 0; f < 4; ++f) bv[f] = TT::to_f32(bias[64 * j + 16 * f + ni]);
    }
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

// ---------------------------------------------------------------------------
// host side
// ---------------------------------------------------------------------------
static bool ggm_format(int quant) {
    return quant == OXQ_GGUF_Q4_0 || quant == OXQ_GGUF_Q8_0 || quant == OXQ_GGUF_Q4_K || quant == OXQ_GGUF_Q6_K ||
           quant == OXQ_GGUF_Q4_1 || quant == OXQ_GGUF_Q5_0 || quant == OXQ_GGUF_Q5_1 || quant == OXQ_GGUF_Q5_K;
}
static const char *ggm_name(int q) {
    switch (q) {
    case OXQ_GGUF_Q4_0: return "q4_0";
    case OXQ_GGUF_Q8_0: return "q8_0";
    case OXQ_GGUF_Q4_K: return "q4k";
    case OXQ_GGUF_Q4_1: return "q4_1";
    case OXQ_GGUF_Q5_0: return "q5_0";
    case OXQ_GGUF_Q5_1: return "q5_1";
    case OXQ_GGUF_Q5_K: return "q5k";
    default: return "q6k";
    }
}

bool gguf_mfma_eligible(const oxq_ctx *ctx, int quant, int64_t K, int64_t N) {
    if (!ggm_format(quant) || tune(ctx, OXQ_TUNE_GGUF_MFMA, 1) == 0) return false;
    return gguf_res_eligible(quant, K, N);  // the same strips, chunks and 32-bit offsets
}

int launch_gguf_mfma_repack(oxq_ctx *ctx, hipStream_t s, int quant, const uint8_t *w, void *pw, int64_t K, int64_t N,
                            int64_t gate_half) {
    const size_t threads = (size_t)(N / 16) * (K / 128) * 64;
    dim3 grid((unsigned)ceil_div((int64_t)threads, 256)), block(256);
    char name[64];
    snprintf(name, sizeof name, "gguf_%s_mfma_repack", ggm_name(quant));
    set_plan(ctx, name, grid, block, 1, 1, 0);
    if (ctx->plan_only) return OXQ_OK;
    switch (quant) {
    case OXQ_GGUF_Q4_0: hipLaunchKernelGGL((ggm_repack_kernel<OXQ_GGUF_Q4_0>), grid, block, 0, s, w, (uint8_t *)pw, (int)K, (int)N, (int)gate_half); break;
    case OXQ_GGUF_Q8_0: hipLaunchKernelGGL((ggm_repack_kernel<OXQ_GGUF_Q8_0>), grid, block, 0, s, w, (uint8_t *)pw, (int)K, (int)N, (int)gate_half); break;
    case OXQ_GGUF_Q4_K: hipLaunchKernelGGL((ggm_repack_kernel<OXQ_GGUF_Q4_K>), grid, block, 0, s, w, (uint8_t *)pw, (int)K, (int)N, (int)gate_half); break;
    case OXQ_GGUF_Q6_K: hipLaunchKernelGGL((ggm_repack_kernel<OXQ_GGUF_Q6_K>), grid, block, 0, s, w, (uint8_t *)pw, (int)K, (int)N, (int)gate_half); break;
    case OXQ_GGUF_Q4_1: hipLaunchKernelGGL((ggm_repack_kernel<OXQ_GGUF_Q4_1>), grid, block, 0, s, w, (uint8_t *)pw, (int)K, (int)N, (int)gate_half); break;
    case OXQ_GGUF_Q5_0: hipLaunchKernelGGL((ggm_repack_kernel<OXQ_GGUF_Q5_0>), grid, block, 0, s, w, (uint8_t *)pw, (int)K, (int)N, (int)gate_half); break;
    case OXQ_GGUF_Q5_1: hipLaunchKernelGGL((ggm_repack_kernel<OXQ_GGUF_Q5_1>), grid, block, 0, s, w, (uint8_t *)pw, (int)K, (int)N, (int)gate_half); break;
    case OXQ_GGUF_Q5_K: hipLaunchKernelGGL((ggm_repack_kernel<OXQ_GGUF_Q5_K>), grid, block, 0, s, w, (uint8_t *)pw, (int)K, (int)N, (int)gate_half); break;
    default: return fail(OXQ_ERR_UNSUPPORTED, "gguf repack: format %d has no matrix-core layout", quant);
    }
    OXQ_HIP_CHECK(hipGetLastError());
    return OXQ_OK;
}

int launch_gguf_mfma_dequant(oxq_ctx *ctx, hipStream_t s, int quant, const void *pw, int64_t K, int64_t N, float *out_nk,
                             int64_t gate_half) {
    const size_t threads = (size_t)(N / 16) * (K / 128) * 64;
    dim3 grid((unsigned)ceil_div((int64_t)threads, 256)), block(256);
    char name[64];
    snprintf(name, sizeof name, "gguf_%s_mfma_dequant", ggm_name(quant));
    set_plan(ctx, name, grid, block, 1, 1, 0);
    if (ctx->plan_only) return OXQ_OK;
    switch (quant) {
    case OXQ_GGUF_Q4_0: hipLaunchKernelGGL((ggm_dequant_kernel<OXQ_GGUF_Q4_0>), grid, block, 0, s, (const uint8_t *)pw, out_nk, (int)K, (int)N, (int)gate_half); break;
    case OXQ_GGUF_Q8_0: hipLaunchKernelGGL((ggm_dequant_kernel<OXQ_GGUF_Q8_0>), grid, block, 0, s, (const uint8_t *)pw, out_nk, (int)K, (int)N, (int)gate_half); break;
    case OXQ_GGUF_Q4_K: hipLaunchKernelGGL((ggm_dequant_kernel<OXQ_GGUF_Q4_K>), grid, block, 0, s, (const uint8_t *)pw, out_nk, (int)K, (int)N, (int)gate_half); break;
    case OXQ_GGUF_Q6_K: hipLaunchKernelGGL((ggm_dequant_kernel<OXQ_GGUF_Q6_K>), grid, block, 0, s, (const uint8_t *)pw, out_nk, (int)K, (int)N, (int)gate_half); break;
    case OXQ_GGUF_Q4_1: hipLaunchKernelGGL((ggm_dequant_kernel<OXQ_GGUF_Q4_1>), grid, block, 0, s, (const uint8_t *)pw, out_nk, (int)K, (int)N, (int)gate_half); break;
    case OXQ_GGUF_Q5_0: hipLaunchKernelGGL((ggm_dequant_kernel<OXQ_GGUF_Q5_0>), grid, block, 0, s, (const uint8_t *)pw, out_nk, (int)K, (int)N, (int)gate_half); break;
    case OXQ_GGUF_Q5_1: hipLaunchKernelGGL((ggm_dequant_kernel<OXQ_GGUF_Q5_1>), grid, block, 0, s, (const uint8_t *)pw, out_nk, (int)K, (int)N, (int)gate_half); break;
    case OXQ_GGUF_Q5_K: hipLaunchKernelGGL((ggm_dequant_kernel<OXQ_GGUF_Q5_K>), grid, block, 0, s, (const uint8_t *)pw, out_nk, (int)K, (int)N, (int)gate_half); break;
    default: return fail(OXQ_ERR_UNSUPPORTED, "gguf dequant: format %d has no matrix-core layout", quant);
    }
    OXQ_HIP_CHECK(hipGetLastError());
    return OXQ_OK;
}

template <int FMT, int MT, int XQ, int NW, int NS>
static int ggm_go(hipStream_t s, dim3 grid, const GgufProblem &p, float *ws, int cslice) {
    static LdsGrant lds_grant;  // one per instantiation
    const size_t lds = (size_t)NW * MT * 4096;
    OXQ_HIP_CHECK(lds_grant.ensure((const void *)ggm_kernel<FMT, MT, XQ, NW, NS>, lds));
    hipLaunchKernelGGL((ggm_kernel<FMT, MT, XQ, NW, NS>), grid, dim3(NW * 64), lds, s, (const uint16_t *)p.x, p.w,
                       (const uint16_t *)p.bias, (uint16_t *)p.y, ws, (int)p.M, (int)p.K, (int)p.N, cslice, p.act);
    OXQ_HIP_CHECK(hipGetLastError());
    return OXQ_OK;
}
template <int FMT>
static int ggm_by_shape(hipStream_t s, dim3 grid, const GgufProblem &p, float *ws, int cslice, int mt, int xq, int nw, int ns) {
    if (ns == 4) {  // 8 waves: four strips' quants in flight take the registers of two waves of a 16-wave workgroup
        if (mt == 2) return ggm_go<FMT, 2, 8, 8, 4>(s, grid, p, ws, cslice);
        if (xq == 1) return ggm_go<FMT, 1, 1, 8, 4>(s, grid, p, ws, cslice);
        if (xq == 2) return ggm_go<FMT, 1, 2, 8, 4>(s, grid, p, ws, cslice);
        return ggm_go<FMT, 1, 4, 8, 4>(s, grid, p, ws, cslice);
    }
    if (mt == 2) return ggm_go<FMT, 2, 8, 8, 1>(s, grid, p, ws, cslice);
    if (nw == 8) {
        if (xq == 1) return ggm_go<FMT, 1, 1, 8, 1>(s, grid, p, ws, cslice);
        if (xq == 2) return ggm_go<FMT, 1, 2, 8, 1>(s, grid, p, ws, cslice);
        return ggm_go<FMT, 1, 4, 8, 1>(s, grid, p, ws, cslice);
    }
    if (xq == 1) return ggm_go<FMT, 1, 1, 16, 1>(s, grid, p, ws, cslice);
    if (xq == 2) return ggm_go<FMT, 1, 2, 16, 1>(s, grid, p, ws, cslice);
    return ggm_go<FMT, 1, 4, 16, 1>(s, grid, p, ws, cslice);
}

// A wide layer (768 strips or more) gives a workgroup four neighbouring strips: every strip of a workgroup re-reads
// the rows of x, which outweighs the weights from a few rows on, and 224 workgroups of 64 columns fill the chip
// as 896 of 16 do not (three and a half rounds).
static int ggm_strips(const oxq_ctx *ctx, int64_t N) {
    const int v = tune(ctx, OXQ_TUNE_GGUF_MFMA_NS, 0);
    if (v == 1 || v == 4) return (N / 16) % v == 0 ? v : 1;
    return (N / 16 >= 768 && (N / 16) % 4 == 0) ? 4 : 1;
}

// rows of x a launch of the matrix-core kernel takes (more go to the tile matmul on the file layout)
bool gguf_mfma_takes(const oxq_ctx *ctx, int64_t M, int64_t, int act_dtype) {
    return act_dtype == OXQ_BF16 && M >= 1 && M <= std::min<int64_t>(32, tune(ctx, OXQ_TUNE_GGUF_MFMA_MAX_M, 32));
}

// p.w is the matrix-core copy; p.act: 0, or 1 + the gated activation of a fused gate|up layer, whose y is [M, N / 2].
// More rows than gguf_mfma_takes allows run as row tiles of the grid (every tile reads the weights again: the
// callers send such calls elsewhere where they can).

int launch_gguf_mfma(oxq_ctx *ctx, hipStream_t s, const GgufProblem &p) {
    const int ns = ggm_strips(ctx, p.N);
    const int mt = p.M > 16 ? 2 : 1;
    const int rows = (int)std::min<int64_t>(p.M, 16 * mt);
    const int xq = rows <= 4 ? 1 : rows <= 8 ? 2 : 4;
    // 16 waves split a strip's chunks where that leaves a wave two to three of them; from 64 chunks on 8 waves with
    // twice the run each measured 3 - 8 % faster (8192 x 4096 at one row, Q4_0 / Q4_K / Q6_K: 5.38 / 5.89 / 7.61
    // against 5.87 / 6.30 / 8.11 us).  Two row tiles or four strips need more than the 128 registers a wave of a
    // 16-wave workgroup has.
    const int64_t chunks = p.K / 128;
    const int nw = (chunks < 16 || chunks >= 64 || mt == 2 || ns == 4 || tune(ctx, OXQ_TUNE_GGR_WAVES, 16) == 8) ? 8 : 16;
    dim3 grid((unsigned)(p.N / (16 * ns)), 1, (unsigned)ceil_div(p.M, (int64_t)16 * mt));
    char name[64];
    snprintf(name, sizeof name, "gguf_%s_mfma_bf16_mt%d%s%s", ggm_name(p.quant), mt, ns == 4 ? "_n64" : "", p.act ? "_act" : "");
    set_plan(ctx, name, grid, dim3(nw * 64), 1, 1, 0);
    if (ctx->plan_only) return OXQ_OK;
    if (p.act_dtype != OXQ_BF16) return fail(OXQ_ERR_UNSUPPORTED, "gguf matrix-core matmul: activations must be BF16");
    if ((uintptr_t)p.x & 15) return fail(OXQ_ERR_UNSUPPORTED, "gguf matrix-core matmul: x must be 16-byte aligned");
    if ((uint64_t)16 * mt * (uint64_t)p.K * 2 >= (1ull << 31)) return fail(OXQ_ERR_UNSUPPORTED, "gguf matrix-core matmul: K too large");
    if (gguf_res_bytes(p.quant, p.K, 16) * (uint64_t)ns >= (1ull << 31)) return fail(OXQ_ERR_UNSUPPORTED, "gguf matrix-core matmul: K too large");
    const int cslice = (int)(p.K / 128);
    switch (p.quant) {
    case OXQ_GGUF_Q4_0: return ggm_by_shape<OXQ_GGUF_Q4_0>(s, grid, p, nullptr, cslice, mt, xq, nw, ns);
    case OXQ_GGUF_Q8_0: return ggm_by_shape<OXQ_GGUF_Q8_0>(s, grid, p, nullptr, cslice, mt, xq, nw, ns);
    case OXQ_GGUF_Q4_K: return ggm_by_shape<OXQ_GGUF_Q4_K>(s, grid, p, nullptr, cslice, mt, xq, nw, ns);
    case OXQ_GGUF_Q6_K: return ggm_by_shape<OXQ_GGUF_Q6_K>(s, grid, p, nullptr, cslice, mt, xq, nw, ns);
    case OXQ_GGUF_Q4_1: return ggm_by_shape<OXQ_GGUF_Q4_1>(s, grid, p, nullptr, cslice, mt, xq, nw, ns);
    case OXQ_GGUF_Q5_0: return ggm_by_shape<OXQ_GGUF_Q5_0>(s, grid, p, nullptr, cslice, mt, xq, nw, ns);
    case OXQ_GGUF_Q5_1: return ggm_by_shape<OXQ_GGUF_Q5_1>(s, grid, p, nullptr, cslice, mt, xq, nw, ns);
    case OXQ_GGUF_Q5_K: return ggm_by_shape<OXQ_GGUF_Q5_K>(s, grid, p, nullptr, cslice, mt, xq, nw, ns);
    default: return fail(OXQ_ERR_UNSUPPORTED, "gguf matrix-core matmul: format %d", p.quant);
    }
}

// Rows from which a bf16 layer's matrix-core copy runs the prefill kernel instead of the tile matmul on the file
// layout (gguf_mm: a workgroup of 64 rows x 64 columns with K slices), and in which form: 1 = eight waves of 64
// columns a workgroup, 4 = two, with K split across the waves inside (0: the file layout).  Costs in rounds of 256
// workgroups of 64 rows x 512 columns (one a CU: 154 - 210 registers), as for the packed layers (pk4_gemm_form): a
// last round that fills at most three quarters of the CUs costs 0.95; a round of the two-wave form GGM_MID_ROUND
// (25 - 35 us against 82 - 120 at K = 4096); the file-layout tile matmul 0.17 + 1.45 w (1.3 w for the five- and
// six-bit formats, whose conversion weighs on the prefill kernel too): two launches or a latency floor, then about
// two thirds of a full round's rate.  Fitted to 4096 x 4096, 4096 x 14336 and 14336 x 4096 at
// 64 - 4096 rows.  OXQ_GGUF_GEMM_MIN_M: unset = by cost, 0 = never, n = the eight-wave form from n rows on whatever
// the cost; OXQ_GGUF_GEMM_KS = 4 | 1: always | never the two-wave form.
constexpr double GGM_MID_ROUND = 0.31;
static int gguf_gemm_form(const oxq_ctx *ctx, int quant, int64_t M, int64_t N, int act_dtype) {
    const int64_t v = tune(ctx, OXQ_TUNE_GGUF_GEMM_MIN_M, -1);
    if (v == 0 || act_dtype != OXQ_BF16 || !ggm_format(quant) || M <= 32 || N % 64 != 0) return 0;
    const int ks = tune(ctx, OXQ_TUNE_GGUF_GEMM_KS, 0);
    if (ks == 4) return 4;
    if (v > 0) return M >= v ? 1 : 0;
    const bool light = quant == OXQ_GGUF_Q4_0 || quant == OXQ_GGUF_Q4_1 || quant == OXQ_GGUF_Q4_K || quant == OXQ_GGUF_Q8_0;
    const double cus = ctx->num_cus > 0 ? ctx->num_cus : 256;
    const int64_t row_tiles = ceil_div(M, (int64_t)64);
    const double w64 = (double)(ceil_div(N / 64, (int64_t)8) * row_tiles) / cus;
    const double whole = std::floor(w64), rest = w64 - whole;
    const double c64 = whole + (rest <= 0.0 ? 0.0 : rest <= 0.75 ? 0.95 : 1.0);
    const double c_mid = ks == 1 ? 1e30 : std::ceil((double)(ceil_div(N / 64, (int64_t)2) * row_tiles) / cus) * GGM_MID_ROUND;
    // (Q8_0's 34-byte blocks make the file layout's matmul 1.2 - 1.35 x the 4-bit formats' at the same shape)
    const double c_file = 0.17 + (quant == OXQ_GGUF_Q8_0 ? 1.75 : light ? 1.45 : 1.3) * w64;
    if (c_file <= c64 && c_file <= c_mid) return 0;
    return c_mid < c64 ? 4 : 1;
}
bool gguf_gemm_takes(const oxq_ctx *ctx, int quant, int64_t M, int64_t K, int64_t N, int act_dtype) {
    (void)K;
    return gguf_gemm_form(ctx, quant, M, N, act_dtype) != 0;
}

template <int FMT, int KS>
static int ggm_gemm_go(hipStream_t s, dim3 grid, const GgufProblem &p, int NG, int RT) {
    static LdsGrant grant;  // one per instantiation
    constexpr int MT = 4;
    const size_t lds = (size_t)2 * KS * 16 * MT * 256;
    OXQ_HIP_CHECK(grant.ensure((const void *)ggm_gemm_kernel<FMT, MT, KS>, lds));
    hipLaunchKernelGGL((ggm_gemm_kernel<FMT, MT, KS>), grid, dim3(512), lds, s, (const uint16_t *)p.x, p.w, (const uint16_t *)p.bias,
                       (uint16_t *)p.y, (int)p.M, (int)p.K, (int)p.N, NG, RT, p.act);
    OXQ_HIP_CHECK(hipGetLastError());
    return OXQ_OK;
}
template <int FMT>
static int ggm_gemm_go_form(hipStream_t s, dim3 grid, const GgufProblem &p, int NG, int RT, int ks) {
    return ks == 4 ? ggm_gemm_go<FMT, 4>(s, grid, p, NG, RT) : ggm_gemm_go<FMT, 1>(s, grid, p, NG, RT);
}

// p.w is the matrix-core copy; p.act as for launch_gguf_mfma
int launch_gguf_gemm(oxq_ctx *ctx, hipStream_t s, const GgufProblem &p) {
    const int rows = 64;
    int ks = gguf_gemm_form(ctx, p.quant, p.M, p.N, p.act_dtype);
    if (ks == 0) ks = 1;  // a caller that asks for this kernel gets it
    const int spw = 8 / ks;
    const int64_t NG = ceil_div(p.N / 64, (int64_t)spw), RT = ceil_div(p.M, (int64_t)rows);
    const int64_t wgs = ks == 1 ? (RT / 8) * ceil_div(NG, (int64_t)8) * 64 + (RT % 8) * NG : RT * NG;
    if (wgs > 0x7FFFFFFF) return fail(OXQ_ERR_UNSUPPORTED, "gguf prefill matmul: m = %lld exceeds the grid", (long long)p.M);
    dim3 grid((unsigned)wgs);
    char name[64];
    snprintf(name, sizeof name, "gguf_%s_gemm_bf16_r%dx%d%s%s", ggm_name(p.quant), rows, spw, ks > 1 ? "k4" : "",
             p.act == 1 ? "_silu" : p.act == 2 ? "_gelu" : "");
    set_plan(ctx, name, grid, dim3(512), 1, 1, 0);
    if (ctx->plan_only) return OXQ_OK;
    if (p.act_dtype != OXQ_BF16) return fail(OXQ_ERR_UNSUPPORTED, "gguf prefill matmul: activations must be BF16");
    if ((uint64_t)rows * (uint64_t)p.K * 2 >= (1ull << 31)) return fail(OXQ_ERR_UNSUPPORTED, "gguf prefill matmul: K too large");
    if (((uintptr_t)p.x & 15) || ((uintptr_t)p.y & 1)) return fail(OXQ_ERR_UNSUPPORTED, "gguf prefill matmul: x must be 16-byte aligned");
    switch (p.quant) {
    case OXQ_GGUF_Q4_0: return ggm_gemm_go_form<OXQ_GGUF_Q4_0>(s, grid, p, (int)NG, (int)RT, ks);
    case OXQ_GGUF_Q8_0: return ggm_gemm_go_form<OXQ_GGUF_Q8_0>(s, grid, p, (int)NG, (int)RT, ks);
    case OXQ_GGUF_Q4_K: return ggm_gemm_go_form<OXQ_GGUF_Q4_K>(s, grid, p, (int)NG, (int)RT, ks);
    case OXQ_GGUF_Q6_K: return ggm_gemm_go_form<OXQ_GGUF_Q6_K>(s, grid, p, (int)NG, (int)RT, ks);
    case OXQ_GGUF_Q4_1: return ggm_gemm_go_form<OXQ_GGUF_Q4_1>(s, grid, p, (int)NG, (int)RT, ks);
    case OXQ_GGUF_Q5_0: return ggm_gemm_go_form<OXQ_GGUF_Q5_0>(s, grid, p, (int)NG, (int)RT, ks);
    case OXQ_GGUF_Q5_1: return ggm_gemm_go_form<OXQ_GGUF_Q5_1>(s, grid, p, (int)NG, (int)RT, ks);
    case OXQ_GGUF_Q5_K: return ggm_gemm_go_form<OXQ_GGUF_Q5_K>(s, grid, p, (int)NG, (int)RT, ks);
    default: return fail(OXQ_ERR_UNSUPPORTED, "gguf prefill matmul: format %d has no matrix-core layout", p.quant);
    }
}

}  // namespace oxq
