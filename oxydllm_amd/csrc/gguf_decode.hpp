// Decoders of the ggml block formats shared by the GGUF kernels: unit `u` (32 consecutive
// elements of one weight row) -> 32 floats, each computed exactly as the reference's
// dequant strips compute it (quant_kernels.metal:2315-2640, one strip per format; block
// structs at 709-713, 792-795, 872-876, 954-959, 1100-1103, 1228-1233, 1439-1445,
// 1681-1686, 1841-1846, 2032-2037).  All field offsets inside a block are even, so bytes
// are fetched as 16-bit words.
#pragma once

#include "oxq_device.hpp"
#include "oxq_internal.hpp"

namespace oxq {

__device__ __forceinline__ uint32_t ld16(const uint8_t *p) { return *(const uint16_t *)p; }
__device__ __forceinline__ float ld_f16(const uint8_t *p) {
    return (float)__builtin_bit_cast(_Float16, *(const uint16_t *)p);
}

template <int FMT> struct GgufFmt;
template <> struct GgufFmt<OXQ_GGUF_Q4_0> { static constexpr int BE = 32, BB = 18; };
template <> struct GgufFmt<OXQ_GGUF_Q8_0> { static constexpr int BE = 32, BB = 34; };
template <> struct GgufFmt<OXQ_GGUF_Q4_K> { static constexpr int BE = 256, BB = 144; };
template <> struct GgufFmt<OXQ_GGUF_Q6_K> { static constexpr int BE = 256, BB = 210; };
template <> struct GgufFmt<OXQ_GGUF_Q4_1> { static constexpr int BE = 32, BB = 20; };
template <> struct GgufFmt<OXQ_GGUF_Q5_0> { static constexpr int BE = 32, BB = 22; };
template <> struct GgufFmt<OXQ_GGUF_Q5_1> { static constexpr int BE = 32, BB = 24; };
template <> struct GgufFmt<OXQ_GGUF_Q2_K> { static constexpr int BE = 256, BB = 84; };
template <> struct GgufFmt<OXQ_GGUF_Q3_K> { static constexpr int BE = 256, BB = 110; };
template <> struct GgufFmt<OXQ_GGUF_Q5_K> { static constexpr int BE = 256, BB = 176; };

// NDW consecutive dwords from an even address.  Blocks of 18, 22, 34, 110 or 210 bytes put every other
// block at an address that is 2 mod 4; a 16-byte LDS read from such an address is served in short
// pieces (Q6_K, four such reads per unit: waves spent a third of their time waiting on LDS).  Aligned
// dword reads and one funnel shift per dword cost the same LDS cycles as an aligned wide read.
// Reads one dword past the span when the address is aligned (its value is shifted out).
template <int NDW>
__device__ __forceinline__ void ld_span(const uint8_t *p, uint32_t (&out)[NDW]) {
    const uint32_t mis = (uint32_t)(uintptr_t)p & 2u;
    const uint32_t *q = (const uint32_t *)(p - mis);
    uint32_t d[NDW + 1];
#pragma unroll
    for (int i = 0; i <= NDW; ++i) d[i] = q[i];
#pragma unroll
    for (int i = 0; i < NDW; ++i) out[i] = __builtin_amdgcn_alignbit(d[i + 1], d[i], mis * 8u);
}

// 16-bit pieces of a span of NDW dwords that starts at an even address: read one by one (any memory),
// or - SPAN, LDS only, since it reads up to four bytes past the span - fetched at once with ld_span.
template <int NDW, bool SPAN> struct Halves {
    uint32_t d[SPAN ? NDW : 1];
    const uint8_t *p;
    __device__ __forceinline__ explicit Halves(const uint8_t *p_) : p(p_) {
        if constexpr (SPAN) ld_span<NDW>(p_, d);
    }
    __device__ __forceinline__ uint32_t h(int i) const {
        if constexpr (SPAN) return (d[i >> 1] >> (16 * (i & 1))) & 0xFFFFu;
        else return ld16(p + 2 * i);
    }
};

// get_scale_min_k4 (quant_kernels.metal:2438-2450): the 6-bit scale and minimum of
// sub-block sb of a Q4_K / Q5_K super-block.
__device__ __forceinline__ void k4_scale_min(const uint8_t *sc, int sb, uint32_t &scv, uint32_t &mnv) {
    // three byte reads and selects for every sub-block: lanes of one wave hold both kinds, and a
    // branch would run both sides one after the other
    const int j = sb & 3;
    const uint32_t a = sc[j], b = sc[j + 4], c = sc[j + 8];
    const uint32_t low = sb < 4 ? 0xFFFFFFFFu : 0u;  // bit select, so that no branch comes back
    scv = ((a & 63u) & low) | (((c & 0x0Fu) | ((a >> 6) << 4)) & ~low);
    mnv = ((b & 63u) & low) | (((c >> 4) | ((b >> 6) << 4)) & ~low);
}

// Signed 6-bit scale of sub-block `sub` (0..15) of a Q3_K super-block
// (quant_kernels.metal:2594-2604).
__device__ __forceinline__ int q3k_scale(const uint8_t *scales, int sub) {
    const int k = sub & 3, group = sub >> 2;
    const uint32_t low = ((uint32_t)scales[k + 4 * (group & 1)] >> (group < 2 ? 0 : 4)) & 0x0Fu;
    const uint32_t high = ((uint32_t)scales[8 + k] >> (2 * group)) & 3u;
    return (int)(low | (high << 4)) - 32;
}

// The four low bits of v, one per byte of the result (bit b -> bit 0 of byte b).
__device__ __forceinline__ uint32_t spread4(uint32_t v) { return ((v & 0xFu) * 0x00204081u) & 0x01010101u; }

// Decode unit `u` (32 elements) of the row starting at `row` into w[0..31].
template <int FMT, bool SPAN = false>
__device__ __forceinline__ void decode_unit(const uint8_t *__restrict__ row, int u, float w[32]) {
    if constexpr (FMT == OXQ_GGUF_Q4_0) {
        const uint8_t *p = row + (size_t)u * 18;
        const float d = ld_f16(p);
        const Halves<4, SPAN> qs(p + 2);
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const uint32_t q = qs.h(i);  // bytes 2i, 2i+1
            w[2 * i] = (float)((int)(q & 0xF) - 8) * d;
            w[2 * i + 16] = (float)((int)((q >> 4) & 0xF) - 8) * d;
            w[2 * i + 1] = (float)((int)((q >> 8) & 0xF) - 8) * d;
            w[2 * i + 17] = (float)((int)((q >> 12) & 0xF) - 8) * d;
        }
    } else if constexpr (FMT == OXQ_GGUF_Q8_0) {
        const uint8_t *p = row + (size_t)u * 34;
        const float d = ld_f16(p);
        const Halves<8, SPAN> qs(p + 2);
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const uint32_t q = qs.h(i);
            w[2 * i] = (float)(int)(int8_t)(q & 0xFF) * d;
            w[2 * i + 1] = (float)(int)(int8_t)(q >> 8) * d;
        }
    } else if constexpr (FMT == OXQ_GGUF_Q4_K) {
        const int b = u >> 3, sb = u & 7;
        const uint8_t *p = row + (size_t)b * 144;
        const float d = ld_f16(p), dmin = ld_f16(p + 2);
        const uint8_t *sc = p + 4;
        uint32_t scv, mnv;
        if (sb < 4) {  // get_scale_min_k4
            scv = sc[sb] & 63u;
            mnv = sc[sb + 4] & 63u;
        } else {
            scv = (sc[sb + 4] & 0x0Fu) | ((uint32_t)(sc[sb - 4] >> 6) << 4);
            mnv = ((uint32_t)sc[sb + 4] >> 4) | ((uint32_t)(sc[sb] >> 6) << 4);
        }
        const float sc_v = d * (float)scv;
        const float m_v = dmin * (float)mnv;
        const uint8_t *qs = p + 16 + (sb >> 1) * 32;
        const int sh = (sb & 1) * 4;
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const uint32_t q = ld16(qs + 2 * i);
            w[2 * i] = sc_v * (float)((q >> sh) & 0xF) - m_v;
            w[2 * i + 1] = sc_v * (float)((q >> (8 + sh)) & 0xF) - m_v;
        }
    } else if constexpr (FMT == OXQ_GGUF_Q4_1) {
        const uint8_t *p = row + (size_t)u * 20;
        const float d = ld_f16(p), m = ld_f16(p + 2);
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const uint32_t q = ld16(p + 4 + 2 * i);
            w[2 * i] = (float)(q & 0xF) * d + m;
            w[2 * i + 16] = (float)((q >> 4) & 0xF) * d + m;
            w[2 * i + 1] = (float)((q >> 8) & 0xF) * d + m;
            w[2 * i + 17] = (float)((q >> 12) & 0xF) * d + m;
        }
    } else if constexpr (FMT == OXQ_GGUF_Q5_0 || FMT == OXQ_GGUF_Q5_1) {
        constexpr bool MIN = FMT == OXQ_GGUF_Q5_1;
        const uint8_t *p = row + (size_t)u * (MIN ? 24 : 22);
        const float d = ld_f16(p), m = MIN ? ld_f16(p + 2) : 0.0f;
        const uint8_t *hp = p + (MIN ? 4 : 2);
        const Halves<5, SPAN> hq(hp);
        const uint32_t qh = hq.h(0) | (hq.h(1) << 16);
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const uint32_t q = hq.h(2 + i);
#pragma unroll
            for (int e = 0; e < 2; ++e) {
                const int j = 2 * i + e;
                const uint32_t lo = ((q >> (8 * e)) & 0xF) | (((qh >> j) & 1u) << 4);
                const uint32_t hi = ((q >> (8 * e + 4)) & 0xF) | (((qh >> (j + 16)) & 1u) << 4);
                if constexpr (MIN) {
                    w[j] = (float)lo * d + m;
                    w[j + 16] = (float)hi * d + m;
                } else {
                    w[j] = (float)((int)lo - 16) * d;
                    w[j + 16] = (float)((int)hi - 16) * d;
                }
            }
        }
    } else if constexpr (FMT == OXQ_GGUF_Q2_K) {
        const int b = u >> 3, ub = u & 7;
        const uint8_t *p = row + (size_t)b * 84;
        const float d = ld_f16(p + 80), dmin = ld_f16(p + 82);
        const uint8_t *qs = p + 16 + (ub >> 2) * 32;
        const int sh = (ub & 3) * 2;
        const uint32_t sc0 = p[2 * ub], sc1 = p[2 * ub + 1];
        const float dl0 = d * (float)(sc0 & 0xF), ml0 = dmin * (float)(sc0 >> 4);
        const float dl1 = d * (float)(sc1 & 0xF), ml1 = dmin * (float)(sc1 >> 4);
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const uint32_t q = ld16(qs + 2 * i);
            const float dl = (i < 8) ? dl0 : dl1, ml = (i < 8) ? ml0 : ml1;
            w[2 * i] = dl * (float)((q >> sh) & 3) - ml;
            w[2 * i + 1] = dl * (float)((q >> (8 + sh)) & 3) - ml;
        }
    } else if constexpr (FMT == OXQ_GGUF_Q3_K) {
        const int b = u >> 3, ub = u & 7;
        const uint8_t *p = row + (size_t)b * 110;
        const float d = ld_f16(p + 108);
        const uint8_t *qs = p + 32 + (ub >> 2) * 32;
        const int sh = (ub & 3) * 2;
        const float s0 = d * (float)q3k_scale(p + 96, 2 * ub);
        const float s1 = d * (float)q3k_scale(p + 96, 2 * ub + 1);
        const Halves<8, SPAN> lq(qs), hq(p);
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const uint32_t q = lq.h(i), hm = hq.h(i) >> ub;
            const float sv = (i < 8) ? s0 : s1;
            w[2 * i] = sv * (float)((int)((q >> sh) & 3) + (int)((hm & 1) << 2) - 4);
            w[2 * i + 1] = sv * (float)((int)((q >> (8 + sh)) & 3) + (int)(((hm >> 8) & 1) << 2) - 4);
        }
    } else if constexpr (FMT == OXQ_GGUF_Q5_K) {
        const int b = u >> 3, sb = u & 7;
        const uint8_t *p = row + (size_t)b * 176;
        const float d = ld_f16(p), dmin = ld_f16(p + 2);
        uint32_t scv, mnv;
        k4_scale_min(p + 4, sb, scv, mnv);
        const float sc_v = d * (float)scv;
        const float m_v = dmin * (float)mnv;
        const uint8_t *qs = p + 48 + (sb >> 1) * 32;
        const int sh = (sb & 1) * 4;
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const uint32_t q = ld16(qs + 2 * i), hb = ld16(p + 16 + 2 * i) >> sb;
            w[2 * i] = sc_v * (float)(((q >> sh) & 0xF) | ((hb & 1) << 4)) - m_v;
            w[2 * i + 1] = sc_v * (float)(((q >> (8 + sh)) & 0xF) | (((hb >> 8) & 1) << 4)) - m_v;
        }
    } else {  // Q6_K
        const int b = u >> 3, sub = u & 7;
        const int h = sub >> 2, quad = sub & 3;
        const uint8_t *p = row + (size_t)b * 210;
        const uint8_t *ql = p + 64 * h + (quad & 1) * 32;
        const uint8_t *qh = p + 128 + 32 * h;
        const int8_t *scales = (const int8_t *)(p + 192);
        const float d = ld_f16(p + 208);
        const float s0 = d * (float)scales[8 * h + 2 * quad];
        const float s1 = d * (float)scales[8 * h + 2 * quad + 1];
        const int shl = (quad < 2) ? 0 : 4;
        const int shh = 2 * quad;
        const Halves<8, SPAN> lq(ql), hq(qh);
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const uint32_t l16 = lq.h(i);
            const uint32_t h16 = hq.h(i);
            const int q0 = (int)(((l16 >> shl) & 0xF) | (((h16 >> shh) & 3) << 4)) - 32;
            const int q1 = (int)(((l16 >> (8 + shl)) & 0xF) | (((h16 >> (8 + shh)) & 3) << 4)) - 32;
            const float sv = (i < 8) ? s0 : s1;  // elements 0..15 / 16..31
            w[2 * i] = sv * (float)q0;
            w[2 * i + 1] = sv * (float)q1;
        }
    }
}

// ---------------------------------------------------------------------------
// The same units as raw integers plus factors, for kernels that hold the block bytes in LDS
// (the staged GEMV, the tile matmul): reads through ld_span / 16-byte chunks, LDS only.
// ---------------------------------------------------------------------------
struct __attribute__((packed, aligned(2))) U32A2 { uint32_t v; };
__device__ __forceinline__ uint32_t ld32a2(const uint8_t *p) { return ((const U32A2 *)p)->v; }

// The empty asm keeps the caller's shift-and-mask of the whole dword apart from the four conversions:
// merged, the compiler extracts every byte by itself (v_bfe + v_cvt_f32_ubyte0, two instructions a
// weight); apart, each conversion is one v_cvt_f32_ubyteN.
__device__ __forceinline__ void bytes_to_f32(uint32_t w, float *o) {
    asm volatile("" : "+v"(w));
    o[0] = (float)(w & 0xFFu);
    o[1] = (float)((w >> 8) & 0xFFu);
    o[2] = (float)((w >> 16) & 0xFFu);
    o[3] = (float)(w >> 24);
}

// Unit `u` of a row: q[0..31] = the stored unsigned integers as floats, and the four
// numbers that turn (dot over elements 0..15, dot over 16..31, sum x over 0..15, sum x
// over 16..31) into the unit's contribution: a0*dot0 + a1*dot1 - b0*sx0 - b1*sx1.
template <int FMT>
__device__ __forceinline__ void unit_ints(const uint8_t *__restrict__ row, int u, float q[32], float &a0,
                                          float &a1, float &b0, float &b1) {
    if constexpr (FMT == OXQ_GGUF_Q4_0) {
        const uint8_t *p = row + (size_t)u * 18;
        const float d = ld_f16(p);
        uint32_t qs[4];
        ld_span<4>(p + 2, qs);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const uint32_t w = qs[i];
            bytes_to_f32(w & 0x0F0F0F0Fu, q + 4 * i);
            bytes_to_f32((w >> 4) & 0x0F0F0F0Fu, q + 16 + 4 * i);
        }
        a0 = a1 = d;
        b0 = b1 = 8.0f * d;
    } else if constexpr (FMT == OXQ_GGUF_Q8_0) {
        const uint8_t *p = row + (size_t)u * 34;
        const float d = ld_f16(p);
        uint32_t qs[8];
        ld_span<8>(p + 2, qs);
#pragma unroll
        for (int i = 0; i < 8; ++i) bytes_to_f32(qs[i] ^ 0x80808080u, q + 4 * i);  // q + 128
        a0 = a1 = d;
        b0 = b1 = 128.0f * d;
    } else if constexpr (FMT == OXQ_GGUF_Q4_K) {
        const int b = u >> 3, sb = u & 7;
        const uint8_t *p = row + (size_t)b * 144;
        const float d = ld_f16(p), dmin = ld_f16(p + 2);
        uint32_t scv, mnv;
        k4_scale_min(p + 4, sb, scv, mnv);
        // 144-byte blocks in rows that start at a multiple of 16: the 32 bytes are two aligned chunks
        const u32x4_t *qs = (const u32x4_t *)(p + 16 + (sb >> 1) * 32);
        const u32x4_t q0 = qs[0], q1 = qs[1];
        const uint32_t qw[8] = {q0[0], q0[1], q0[2], q0[3], q1[0], q1[1], q1[2], q1[3]};
        const int sh = (sb & 1) * 4;
#pragma unroll
        for (int i = 0; i < 8; ++i) bytes_to_f32((qw[i] >> sh) & 0x0F0F0F0Fu, q + 4 * i);
        a0 = a1 = d * (float)scv;
        b0 = b1 = dmin * (float)mnv;
    } else if constexpr (FMT == OXQ_GGUF_Q4_1) {
        const uint8_t *p = row + (size_t)u * 20;
        const float d = ld_f16(p), m = ld_f16(p + 2);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const uint32_t w = ld32a2(p + 4 + 4 * i);
            bytes_to_f32(w & 0x0F0F0F0Fu, q + 4 * i);
            bytes_to_f32((w >> 4) & 0x0F0F0F0Fu, q + 16 + 4 * i);
        }
        a0 = a1 = d;
        b0 = b1 = -m;
    } else if constexpr (FMT == OXQ_GGUF_Q5_0 || FMT == OXQ_GGUF_Q5_1) {
        constexpr bool MIN = FMT == OXQ_GGUF_Q5_1;
        const uint8_t *p = row + (size_t)u * (MIN ? 24 : 22);
        const float d = ld_f16(p);
        const uint8_t *hp = p + (MIN ? 4 : 2);
        uint32_t hq[5];
        ld_span<5>(hp, hq);
        const uint32_t qh = hq[0];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const uint32_t w = hq[1 + i];
            bytes_to_f32((w & 0x0F0F0F0Fu) | (spread4(qh >> (4 * i)) << 4), q + 4 * i);
            bytes_to_f32(((w >> 4) & 0x0F0F0F0Fu) | (spread4(qh >> (16 + 4 * i)) << 4), q + 16 + 4 * i);
        }
        a0 = a1 = d;
        b0 = b1 = MIN ? -ld_f16(p + 2) : 16.0f * d;
    } else if constexpr (FMT == OXQ_GGUF_Q2_K) {
        const int b = u >> 3, ub = u & 7;
        const uint8_t *p = row + (size_t)b * 84;
        const float d = ld_f16(p + 80), dmin = ld_f16(p + 82);
        const uint8_t *qs = p + 16 + (ub >> 2) * 32;
        const int sh = (ub & 3) * 2;
        const uint32_t sc = ld16(p + 2 * ub);
#pragma unroll
        for (int i = 0; i < 8; ++i) bytes_to_f32((ld32a2(qs + 4 * i) >> sh) & 0x03030303u, q + 4 * i);
        a0 = d * (float)(sc & 0xF);
        b0 = dmin * (float)((sc >> 4) & 0xF);
        a1 = d * (float)((sc >> 8) & 0xF);
        b1 = dmin * (float)(sc >> 12);
    } else if constexpr (FMT == OXQ_GGUF_Q3_K) {
        const int b = u >> 3, ub = u & 7;
        const uint8_t *p = row + (size_t)b * 110;
        const float d = ld_f16(p + 108);
        const uint8_t *qs = p + 32 + (ub >> 2) * 32;
        const int sh = (ub & 3) * 2;
        uint32_t lw[8], hw[8];
        ld_span<8>(qs, lw);
        ld_span<8>(p, hw);
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const uint32_t lo = (lw[i] >> sh) & 0x03030303u;
            const uint32_t hi = ((hw[i] >> ub) & 0x01010101u) << 2;
            bytes_to_f32(lo | hi, q + 4 * i);  // q + 4
        }
        a0 = d * (float)q3k_scale(p + 96, 2 * ub);
        a1 = d * (float)q3k_scale(p + 96, 2 * ub + 1);
        b0 = 4.0f * a0;
        b1 = 4.0f * a1;
    } else if constexpr (FMT == OXQ_GGUF_Q5_K) {
        const int b = u >> 3, sb = u & 7;
        const uint8_t *p = row + (size_t)b * 176;
        const float d = ld_f16(p), dmin = ld_f16(p + 2);
        uint32_t scv, mnv;
        k4_scale_min(p + 4, sb, scv, mnv);
        const uint8_t *qs = p + 48 + (sb >> 1) * 32;
        const int sh = (sb & 1) * 4;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const uint32_t lo = (ld32a2(qs + 4 * i) >> sh) & 0x0F0F0F0Fu;
            const uint32_t hi = ((ld32a2(p + 16 + 4 * i) >> sb) & 0x01010101u) << 4;
            bytes_to_f32(lo | hi, q + 4 * i);
        }
        a0 = a1 = d * (float)scv;
        b0 = b1 = dmin * (float)mnv;
    } else {  // Q6_K
        const int b = u >> 3, sub = u & 7;
        const int h = sub >> 2, quad = sub & 3;
        const uint8_t *p = row + (size_t)b * 210;
        const uint8_t *ql = p + 64 * h + (quad & 1) * 32;
        const uint8_t *qh = p + 128 + 32 * h;
        const int8_t *scales = (const int8_t *)(p + 192);
        const float d = ld_f16(p + 208);
        const int shl = (quad < 2) ? 0 : 4;
        const int shh = 2 * quad;
        uint32_t lw[8], hw[8];
        ld_span<8>(ql, lw);
        ld_span<8>(qh, hw);
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const uint32_t lo = (lw[i] >> shl) & 0x0F0F0F0Fu;
            const uint32_t hi = ((hw[i] >> shh) & 0x03030303u) << 4;
            bytes_to_f32(lo | hi, q + 4 * i);  // q + 32
        }
        a0 = d * (float)scales[8 * h + 2 * quad];
        a1 = d * (float)scales[8 * h + 2 * quad + 1];
        b0 = 32.0f * a0;
        b1 = 32.0f * a1;
    }
}

}  // namespace oxq
