/*
 * oxq_oracle.c - CPU restatement of oxydLLM's quantized-weight matmul path.
 *
 * TEST INFRASTRUCTURE ONLY.  This file is the checker the HIP kernels are
 * compared against and the "port" CPU baseline bench.py times.  Nothing in the
 * shipped library links, loads or calls it; the product path has no CPU
 * fallback.
 *
 * Every function restates one piece of the reference and cites it
 * (paths relative to the reference tree):
 *
 *   orc_dequantize_awq        src/common/awq.rs:325-440, 612-633   (AWQ 4-bit)
 *   orc_dequantize_awq8       src/common/metal_ops.rs:3960-4009 +
 *                             src/common/quant_kernels.metal:40-48, 188-215
 *                             (AWQ-layout 8-bit, identity slot order)
 *   orc_dequantize_gptq       src/common/awq.rs:442-590            (GPTQ 4/8-bit)
 *   orc_dequantize_mxfp4_f32  src/common/mxfp4.rs:13-64
 *   orc_dequantize_gguf       src/common/quant_kernels.metal:709-713, 792-795, 872-876,
 *                             954-959, 1100-1103, 1228-1233, 1439-1445, 1681-1686,
 *                             1841-1846, 2032-2037 (block structs) and 2315-2640
 *                             (one dequant formula per format)
 *   orc_f8e4m3_to_f32, orc_f8_block_dequant_bf16
 *                             src/common/metal_ops.rs:2942-2955 (spec decode),
 *                             src/common/quant_kernels.metal:3877-3911 (cast chain)
 *   orc_compressed_to_awq     src/common/awq.rs:187-254
 *   orc_rtn_quantize_awq      src/common/awq.rs:637-742
 *   orc_matmul_nt_f32         src/common/linear.rs:40-79  (x . W^T + bias, f32)
 *   orc_moe_route             src/common/moe.rs:466-499 + linear.rs:160-171
 *   orc_moe_group             src/common/moe.rs:563-607  (dispatch_sparse lists)
 *   orc_gpt_oss_swiglu        src/common/moe.rs:152-173
 *   orc_gated_silu / _gelu_tanh src/common/ffn_kernels.metal:5-17, 23-36, 115-128
 *   orc_moe_combine           src/common/moe.rs:592-605 (index_add of gate-weighted rows)
 *   orc_f32_to_f16 / bf16     `half` crate from_f32 (IEEE round-to-nearest-even),
 *                             used by awq.rs:421-431
 *
 * Pinning (what fixes each function besides its own formula) is listed in
 * tests/test_oracle_kat.py: the reference's hand-packed known-answer tests for
 * AWQ-4 (awq.rs:954-1011), GPTQ-4/8 (awq.rs:1170-1283), the compressed-tensors
 * closed form (awq.rs:754-800), W8 generator (metal_ops.rs:3975-4009), MXFP4
 * code table and dot (mxfp4.rs:178-214), the GPT-OSS expert scalar test
 * (moe.rs:705-788), numpy's IEEE float16 cast for the conversions, and an
 * independent numpy restatement of the ggml block formats for GGUF.
 * GGUF has no golden vector in the reference (its tests compare against the
 * third-party candle-core 0.11.0 QTensor::dequantize, which is absent here), so
 * bit-level agreement with candle for the ten block formats is "parity unpinned"
 * by fixtures; it is pinned by the public ggml block specification, which the
 * reference restates in the cited Metal strips.
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define ORC_OK 0
#define ORC_ERR_SHAPE -1
#define ORC_ERR_ARG -2

/* ------------------------------------------------------------------ */
/* 16-bit float conversions (round-to-nearest-even, IEEE 754)          */
/* ------------------------------------------------------------------ */

static inline uint32_t f32_bits(float f) {
    uint32_t u;
    memcpy(&u, &f, 4);
    return u;
}
static inline float bits_f32(uint32_t u) {
    float f;
    memcpy(&f, &u, 4);
    return f;
}

uint16_t orc_f32_to_bf16(float f) {
    uint32_t u = f32_bits(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) { /* NaN: keep quiet bit set */
        return (uint16_t)((u >> 16) | 0x0040u);
    }
    uint32_t lsb = (u >> 16) & 1u;
    u += 0x7fffu + lsb;
    return (uint16_t)(u >> 16);
}

float orc_bf16_to_f32(uint16_t h) { return bits_f32(((uint32_t)h) << 16); }

uint16_t orc_f32_to_f16(float f) {
    uint32_t x = f32_bits(f);
    uint32_t sign = (x >> 16) & 0x8000u;
    uint32_t ax = x & 0x7fffffffu;
    if (ax >= 0x7f800000u) { /* inf / nan */
        if (ax > 0x7f800000u) return (uint16_t)(sign | 0x7e00u | ((ax >> 13) & 0x3ffu));
        return (uint16_t)(sign | 0x7c00u);
    }
    if (ax >= 0x477ff000u) { /* rounds to >= 65520 -> inf */
        return (uint16_t)(sign | 0x7c00u);
    }
    if (ax < 0x33000001u) { /* < 2^-25 (or exactly 2^-25 which ties to 0) */
        return (uint16_t)sign;
    }
    int32_t exp = (int32_t)(ax >> 23) - 127;
    uint32_t man = (ax & 0x7fffffu) | 0x800000u;
    uint32_t shift;
    uint32_t half_exp;
    if (exp < -14) { /* subnormal half */
        shift = (uint32_t)(13 + (-14 - exp));
        half_exp = 0;
    } else {
        shift = 13;
        half_exp = (uint32_t)(exp + 15);
    }
    uint32_t q = man >> shift;
    uint32_t rem = man & ((1u << shift) - 1u);
    uint32_t halfway = 1u << (shift - 1);
    if (rem > halfway || (rem == halfway && (q & 1u))) q++;
    uint32_t out;
    if (half_exp == 0) {
        out = q; /* carry into exponent 1 is the right encoding */
    } else {
        out = ((half_exp - 1) << 10) + q; /* q has the implicit bit at 0x400 */
    }
    return (uint16_t)(sign | out);
}

float orc_f16_to_f32(uint16_t h) {
    uint32_t sign = ((uint32_t)h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1fu;
    uint32_t man = h & 0x3ffu;
    if (exp == 0) {
        if (man == 0) return bits_f32(sign);
        float v = ldexpf((float)man, -24);
        return sign ? -v : v;
    }
    if (exp == 31) return bits_f32(sign | 0x7f800000u | (man << 13));
    return bits_f32(sign | ((exp + 112u) << 23) | (man << 13));
}

/* dtype codes shared with the tests: 0 = f32, 1 = f16, 2 = bf16 */
void orc_convert_f32(const float *in, void *out, size_t n, int dtype) {
    if (dtype == 0) {
        memcpy(out, in, n * sizeof(float));
    } else if (dtype == 1) {
        uint16_t *o = (uint16_t *)out;
        for (size_t i = 0; i < n; ++i) o[i] = orc_f32_to_f16(in[i]);
    } else {
        uint16_t *o = (uint16_t *)out;
        for (size_t i = 0; i < n; ++i) o[i] = orc_f32_to_bf16(in[i]);
    }
}

void orc_widen_to_f32(const void *in, float *out, size_t n, int dtype) {
    if (dtype == 0) {
        memcpy(out, in, n * sizeof(float));
    } else if (dtype == 1) {
        const uint16_t *p = (const uint16_t *)in;
        for (size_t i = 0; i < n; ++i) out[i] = orc_f16_to_f32(p[i]);
    } else {
        const uint16_t *p = (const uint16_t *)in;
        for (size_t i = 0; i < n; ++i) out[i] = orc_bf16_to_f32(p[i]);
    }
}

/* ------------------------------------------------------------------ */
/* AWQ 4-bit: awq.rs:325-440 (checks + zero unpack), 612-633 (fill)    */
/* ------------------------------------------------------------------ */

static const int AWQ_PACK_ORDER[8] = {0, 2, 4, 6, 1, 3, 5, 7}; /* awq.rs:23 */

/* out: [N, K] row-major f32, W[n,k] = (nibble - zero) * scale[k/g, n]. */
int orc_dequantize_awq(const uint32_t *qweight, /* [K, N/8] */
                       const uint32_t *qzeros,  /* [K/g, N/8] */
                       const float *scales,     /* [K/g, N] */
                       int64_t K, int64_t N, int64_t group_size, float *out) {
    if (K <= 0 || N <= 0 || group_size <= 0) return ORC_ERR_ARG;
    if (N % 8 != 0) return ORC_ERR_SHAPE; /* awq.rs:332-336 */
    if (K % group_size != 0) return ORC_ERR_SHAPE;
    const int64_t groups = K / group_size;
    const int64_t packed_out = N / 8;

    /* awq.rs:390-401: expand qzeros to one byte per (group, column). */
    uint8_t *zeros = (uint8_t *)malloc((size_t)(groups * N));
    if (!zeros) return ORC_ERR_ARG;
    for (int64_t g = 0; g < groups; ++g)
        for (int64_t j = 0; j < packed_out; ++j) {
            uint32_t packed = qzeros[g * packed_out + j];
            for (int k = 0; k < 8; ++k) {
                uint8_t nib = (uint8_t)((packed >> (4 * k)) & 0xF);
                zeros[g * N + j * 8 + AWQ_PACK_ORDER[k]] = nib;
            }
        }
    /* awq.rs:403-406: inverse permutation, column offset -> slot. */
    uint32_t inv[8];
    for (int k = 0; k < 8; ++k) inv[AWQ_PACK_ORDER[k]] = (uint32_t)k;

    /* awq.rs:612-633: parallel over output rows. */
#pragma omp parallel for schedule(static)
    for (int64_t n = 0; n < N; ++n) {
        const int64_t j = n / 8;
        const uint32_t shift = 4 * inv[n % 8];
        float *row = out + n * K;
        for (int64_t i = 0; i < K; ++i) {
            const int64_t g = i / group_size;
            const uint32_t packed = qweight[i * packed_out + j];
            const int32_t nib = (int32_t)((packed >> shift) & 0xF);
            const int32_t zero = (int32_t)zeros[g * N + n];
            row[i] = (float)(nib - zero) * scales[g * N + n];
        }
    }
    free(zeros);
    return ORC_OK;
}

/* AWQ-layout 8-bit: slot k of word (i, j) is column 4j + k (identity order,
 * quant_kernels.metal:45-48); value (q - z) * s (metal_ops.rs:4001-4009). */
int orc_dequantize_awq8(const uint32_t *qweight, /* [K, N/4] */
                        const uint32_t *qzeros,  /* [K/g, N/4] */
                        const float *scales,     /* [K/g, N] */
                        int64_t K, int64_t N, int64_t group_size, float *out) {
    if (K <= 0 || N <= 0 || group_size <= 0) return ORC_ERR_ARG;
    if (N % 4 != 0 || K % group_size != 0) return ORC_ERR_SHAPE;
    const int64_t packed_out = N / 4;
#pragma omp parallel for schedule(static)
    for (int64_t n = 0; n < N; ++n) {
        const int64_t j = n / 4;
        const uint32_t shift = 8 * (uint32_t)(n % 4);
        float *row = out + n * K;
        for (int64_t i = 0; i < K; ++i) {
            const int64_t g = i / group_size;
            const int32_t q = (int32_t)((qweight[i * packed_out + j] >> shift) & 0xFF);
            const int32_t z = (int32_t)((qzeros[g * packed_out + j] >> shift) & 0xFF);
            row[i] = (float)(q - z) * scales[g * N + n];
        }
    }
    return ORC_OK;
}

/* ------------------------------------------------------------------ */
/* GPTQ: awq.rs:442-590                                                */
/* ------------------------------------------------------------------ */

/* qzeros may be NULL (=> symmetric).  out: [N, K] f32,
 * W[n,k] = (q - (zero + 1)) * scale[k/g, n]. */
int orc_dequantize_gptq(const uint32_t *qweight, /* [K/pf, N] */
                        const uint32_t *qzeros,  /* [K/g, N/pf] or NULL */
                        const float *scales,     /* [K/g, N] */
                        int bits, int sym, int64_t K, int64_t N, int64_t group_size,
                        float *out) {
    if (bits != 4 && bits != 8) return ORC_ERR_ARG; /* awq.rs:451-453 */
    if (K <= 0 || N <= 0 || group_size <= 0) return ORC_ERR_ARG;
    const int64_t pf = 32 / bits;
    if (K % pf != 0 || K % group_size != 0) return ORC_ERR_SHAPE;
    if (N % pf != 0) return ORC_ERR_SHAPE; /* awq.rs:475-479 */
    const int64_t packed_out = N / pf;
    const uint32_t mask = (1u << bits) - 1u;
    const int use_sym = (qzeros == NULL) || sym; /* awq.rs:518 */
    /* awq.rs:567: (1 << (bits-1)) - 1, then +1 in the formula. */
    const uint32_t sym_zero = (1u << (bits - 1)) - 1u;
#pragma omp parallel for schedule(static)
    for (int64_t n = 0; n < N; ++n) {
        const int64_t o_word = n / pf;
        const uint32_t o_shift = (uint32_t)((n % pf) * bits);
        float *row = out + n * K;
        for (int64_t i = 0; i < K; ++i) {
            const int64_t g = i / group_size;
            const int64_t i_word = i / pf;
            const uint32_t i_shift = (uint32_t)((i % pf) * bits);
            const uint32_t q = (qweight[i_word * N + n] >> i_shift) & mask;
            const uint32_t zero =
                use_sym ? sym_zero : ((qzeros[g * packed_out + o_word] >> o_shift) & mask);
            row[i] = (float)((int32_t)q - ((int32_t)zero + 1)) * scales[g * N + n];
        }
    }
    return ORC_OK;
}

/* Transpose [N,K] f32 -> [K,N] in `dtype`: the layout and element type of the
 * reference's GPU dequant ops (quant_kernels.metal:188-215, 508-545), whose
 * per-element value T((q - z) * s) is the same single rounding of the same
 * exact product as convert((nib - zero) as f32 * scale) above. */
void orc_transpose_convert(const float *w_nk, int64_t N, int64_t K, void *out_kn, int dtype) {
#pragma omp parallel for schedule(static)
    for (int64_t k = 0; k < K; ++k) {
        for (int64_t n = 0; n < N; ++n) {
            float v = w_nk[n * K + k];
            if (dtype == 0)
                ((float *)out_kn)[k * N + n] = v;
            else if (dtype == 1)
                ((uint16_t *)out_kn)[k * N + n] = orc_f32_to_f16(v);
            else
                ((uint16_t *)out_kn)[k * N + n] = orc_f32_to_bf16(v);
        }
    }
}

/* ------------------------------------------------------------------ */
/* MXFP4: mxfp4.rs:13-64                                               */
/* ------------------------------------------------------------------ */

static const float MXFP4_LUT[8] = {0.0f, 0.5f, 1.0f, 1.5f, 2.0f, 3.0f, 4.0f, 6.0f};

static inline float mxfp4_decode(uint8_t nibble) { /* mxfp4.rs:19-22 */
    float v = MXFP4_LUT[nibble & 7];
    return (nibble & 8) ? -v : v;
}

static inline float e8m0_scale(uint8_t s) { /* mxfp4.rs:25-31 */
    if (s == 0xFF) return NAN;
    return exp2f((float)s - 127.0f);
}

int orc_dequantize_mxfp4_f32(const uint8_t *blocks, size_t blocks_len, const uint8_t *scales,
                             size_t scales_len, int64_t rows, int64_t cols, float *out) {
    if (cols % 32 != 0) return ORC_ERR_SHAPE; /* mxfp4.rs:41-43 */
    const int64_t nb = cols / 32;
    if (blocks_len != (size_t)(rows * nb * 16) || scales_len != (size_t)(rows * nb))
        return ORC_ERR_SHAPE; /* mxfp4.rs:45-51 */
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < rows; ++r) {
        for (int64_t b = 0; b < nb; ++b) {
            const float scale = e8m0_scale(scales[r * nb + b]);
            const uint8_t *bytes = blocks + (r * nb + b) * 16;
            float *o = out + r * cols + b * 32;
            for (int i = 0; i < 16; ++i) {
                o[2 * i] = mxfp4_decode(bytes[i] & 0xF) * scale;
                o[2 * i + 1] = mxfp4_decode(bytes[i] >> 4) * scale;
            }
        }
    }
    return ORC_OK;
}

/* ------------------------------------------------------------------ */
/* Block-scaled F8E4M3 (fn variant)                                    */
/* ------------------------------------------------------------------ */

/* metal_ops.rs:2942-2955 (e4m3_decode): 1 sign, 4 exponent (bias 7), 3 mantissa;
 * S.1111.111 is NaN, there is no infinity. */
float orc_f8e4m3_to_f32(uint8_t v) {
    const uint32_t s = v >> 7, e = (v >> 3) & 0xFu, m = v & 0x7u;
    float val;
    if (e == 0) val = ldexpf((float)m * 0.125f, -6);
    else if (e == 15 && m == 7) val = NAN;
    else val = ldexpf(1.0f + (float)m * 0.125f, (int)e - 7);
    return s ? -val : val;
}

void orc_cast_f8e4m3_to_f32(const uint8_t *in, float *out, size_t n) {
    for (size_t i = 0; i < n; ++i) out[i] = orc_f8e4m3_to_f32(in[i]);
}

/* quant_kernels.metal:3877-3911 / metal_ops.rs:4310-4345: F8 -> F32 -> BF16, F32 block
 * scale fold, -> BF16.  bytes [rows, cols], scales [s_rows, s_cols]; out = bf16 bits. */
int orc_f8_block_dequant_bf16(const uint8_t *bytes, const float *scales, int64_t rows, int64_t cols,
                              int64_t s_rows, int64_t s_cols, uint16_t *out) {
    if (s_rows <= 0 || s_cols <= 0 || rows % s_rows != 0 || cols % s_cols != 0) return ORC_ERR_SHAPE;
    const int64_t block_r = rows / s_rows, block_c = cols / s_cols;
    for (int64_t r = 0; r < rows; ++r)
        for (int64_t c = 0; c < cols; ++c) {
            const float w = orc_bf16_to_f32(orc_f32_to_bf16(orc_f8e4m3_to_f32(bytes[r * cols + c])));
            out[r * cols + c] = orc_f32_to_bf16(w * scales[(r / block_r) * s_cols + c / block_c]);
        }
    return ORC_OK;
}

/* ------------------------------------------------------------------ */
/* Load-time transforms into the AWQ layout                            */
/* ------------------------------------------------------------------ */

static const int ORC_AWQ_ORDER[8] = {0, 2, 4, 6, 1, 3, 5, 7}; /* awq.rs:23 */

/* awq.rs:187-254.  ct [out, in/8]: word (o, c) nibble k = column 8c+k (q+8);
 * scale_ct [out, groups] f32 -> qweight [in, out/8], qzeros [groups, out/8],
 * scales [groups, out] f32. */
int orc_compressed_to_awq(const uint32_t *ct, const float *scale_ct, int64_t out_f, int64_t in_f,
                          int64_t groups, uint32_t *qweight, uint32_t *qzeros, float *scales) {
    if (in_f % 8 != 0 || out_f % 8 != 0 || groups == 0 || in_f % groups != 0) return ORC_ERR_SHAPE;
    const int64_t packed_out = out_f / 8, packed_in = in_f / 8;
    for (int64_t i = 0; i < in_f; ++i) {
        const int64_t c = i / 8;
        const uint32_t sh = 4u * (uint32_t)(i % 8);
        for (int64_t jw = 0; jw < packed_out; ++jw) {
            uint32_t w = 0;
            for (int k = 0; k < 8; ++k) {
                const int64_t o = jw * 8 + ORC_AWQ_ORDER[k];
                w |= ((ct[o * packed_in + c] >> sh) & 0xFu) << (4 * k);
            }
            qweight[i * packed_out + jw] = w;
        }
    }
    for (int64_t z = 0; z < groups * packed_out; ++z) qzeros[z] = 0x88888888u;
    for (int64_t o = 0; o < out_f; ++o)
        for (int64_t g = 0; g < groups; ++g) scales[g * out_f + o] = scale_ct[o * groups + g];
    return ORC_OK;
}

/* awq.rs:637-742.  weight [out, in] f32 -> AWQ 4-bit tensors, scales f32 [groups, out]. */
int orc_rtn_quantize_awq(const float *w, int64_t out_f, int64_t in_f, int64_t group_size,
                         uint32_t *qweight, uint32_t *qzeros, float *scales) {
    if (out_f % 8 != 0 || group_size <= 0 || in_f % group_size != 0) return ORC_ERR_SHAPE;
    const int64_t groups = in_f / group_size, packed_out = out_f / 8;
    uint8_t *qnib = (uint8_t *)malloc((size_t)(out_f * in_f));
    uint8_t *znib = (uint8_t *)malloc((size_t)(out_f * groups));
    if (!qnib || !znib) {
        free(qnib);
        free(znib);
        return ORC_ERR_ARG;
    }
    for (int64_t o = 0; o < out_f; ++o) {
        const float *w_row = w + o * in_f;
        for (int64_t g = 0; g < groups; ++g) {
            const float *grp = w_row + g * group_size;
            float xmin = grp[0], xmax = grp[0];
            for (int64_t i = 0; i < group_size; ++i) {
                xmin = fminf(xmin, grp[i]);
                xmax = fmaxf(xmax, grp[i]);
            }
            xmin = fminf(xmin, 0.0f); /* the representable range always spans 0 */
            xmax = fmaxf(xmax, 0.0f);
            if (xmax - xmin < 1e-12f) {
                scales[g * out_f + o] = xmin;
                znib[o * groups + g] = 0;
                for (int64_t i = 0; i < group_size; ++i) qnib[o * in_f + g * group_size + i] = 1;
            } else {
                const float scale = (xmax - xmin) / 15.0f;
                const float zero = fminf(fmaxf(roundf(-xmin / scale), 0.0f), 15.0f);
                scales[g * out_f + o] = scale;
                znib[o * groups + g] = (uint8_t)zero;
                for (int64_t i = 0; i < group_size; ++i)
                    qnib[o * in_f + g * group_size + i] =
                        (uint8_t)fminf(fmaxf(roundf(grp[i] / scale + zero), 0.0f), 15.0f);
            }
        }
    }
    memset(qweight, 0, (size_t)(in_f * packed_out) * 4);
    memset(qzeros, 0, (size_t)(groups * packed_out) * 4);
    for (int64_t j = 0; j < packed_out; ++j)
        for (int k = 0; k < 8; ++k) {
            const int64_t o = j * 8 + ORC_AWQ_ORDER[k];
            for (int64_t i = 0; i < in_f; ++i) qweight[i * packed_out + j] |= (uint32_t)qnib[o * in_f + i] << (4 * k);
            for (int64_t g = 0; g < groups; ++g) qzeros[g * packed_out + j] |= (uint32_t)znib[o * groups + g] << (4 * k);
        }
    free(qnib);
    free(znib);
    return ORC_OK;
}

/* ------------------------------------------------------------------ */
/* GGUF block formats (ggml): 0..3 = Q4_0, Q8_0, Q4_K, Q6_K,            */
/* 4..9 = Q4_1, Q5_0, Q5_1, Q2_K, Q3_K, Q5_K                           */
/* ------------------------------------------------------------------ */

enum { ORC_Q4_0 = 0, ORC_Q8_0 = 1, ORC_Q4_K = 2, ORC_Q6_K = 3,
       ORC_Q4_1 = 4, ORC_Q5_0 = 5, ORC_Q5_1 = 6, ORC_Q2_K = 7, ORC_Q3_K = 8, ORC_Q5_K = 9 };

int orc_gguf_block_layout(int fmt, int *elems, int *bytes) { /* metal_ops.rs:5228-5241 */
    switch (fmt) {
    case ORC_Q4_0: *elems = 32; *bytes = 18; return ORC_OK;
    case ORC_Q8_0: *elems = 32; *bytes = 34; return ORC_OK;
    case ORC_Q4_K: *elems = 256; *bytes = 144; return ORC_OK;
    case ORC_Q6_K: *elems = 256; *bytes = 210; return ORC_OK;
    case ORC_Q4_1: *elems = 32; *bytes = 20; return ORC_OK;
    case ORC_Q5_0: *elems = 32; *bytes = 22; return ORC_OK;
    case ORC_Q5_1: *elems = 32; *bytes = 24; return ORC_OK;
    case ORC_Q2_K: *elems = 256; *bytes = 84; return ORC_OK;
    case ORC_Q3_K: *elems = 256; *bytes = 110; return ORC_OK;
    case ORC_Q5_K: *elems = 256; *bytes = 176; return ORC_OK;
    default: return ORC_ERR_ARG;
    }
}

static inline float rd_f16(const uint8_t *p) {
    uint16_t h = (uint16_t)(p[0] | ((uint16_t)p[1] << 8));
    return orc_f16_to_f32(h);
}

/* quant_kernels.metal:2438-2450 (get_scale_min_k4) */
static inline void q4k_scale_min(int j, const uint8_t *q, uint32_t *sc, uint32_t *mn) {
    if (j < 4) {
        *sc = q[j] & 63u;
        *mn = q[j + 4] & 63u;
    } else {
        *sc = (q[j + 4] & 0x0Fu) | ((uint32_t)(q[j - 4] >> 6) << 4);
        *mn = ((uint32_t)q[j + 4] >> 4) | ((uint32_t)(q[j] >> 6) << 4);
    }
}

static inline uint32_t rd_u32(const uint8_t *p) {
    return (uint32_t)p[0] | ((uint32_t)p[1] << 8) | ((uint32_t)p[2] << 16) | ((uint32_t)p[3] << 24);
}

/* quant_kernels.metal:2594-2604: signed 6-bit scale of sub-block 0..15, low four bits in
 * scales[0..7] (nibbles), high two bits in scales[8..11], offset -32. */
static inline int q3k_scale(int sub, const uint8_t *scales) {
    const int k = sub % 4, group = sub / 4;
    const int low_byte = (group < 2) ? (k + 4 * group) : (k + 4 * (group - 2));
    const int low_shift = (group < 2) ? 0 : 4;
    const uint32_t low = ((uint32_t)scales[low_byte] >> low_shift) & 0x0Fu;
    const uint32_t high = ((uint32_t)scales[8 + k] >> (2 * group)) & 0x03u;
    return (int)(low | (high << 4)) - 32;
}

static void dequant_block(int fmt, const uint8_t *blk, float *o) {
    switch (fmt) {
    case ORC_Q4_0: { /* {f16 d; u8 qs[16]}  quant_kernels.metal:2364-2384 */
        const float d = rd_f16(blk);
        const uint8_t *qs = blk + 2;
        for (int j = 0; j < 32; ++j) {
            const uint32_t qp = (j < 16) ? (qs[j] & 0x0Fu) : (uint32_t)(qs[j - 16] >> 4);
            o[j] = (float)((int)qp - 8) * d;
        }
    } break;
    case ORC_Q8_0: { /* {f16 d; i8 qs[32]}  quant_kernels.metal:2342-2362 */
        const float d = rd_f16(blk);
        const int8_t *qs = (const int8_t *)(blk + 2);
        for (int j = 0; j < 32; ++j) o[j] = (float)qs[j] * d;
    } break;
    case ORC_Q4_K: { /* {f16 d, dmin; u8 scales[12]; u8 qs[128]}  2452-2482 */
        const float d = rd_f16(blk), dmin = rd_f16(blk + 2);
        const uint8_t *scales = blk + 4, *qs = blk + 16;
        for (int j = 0; j < 256; ++j) {
            const int sb = j / 32, elem = j % 32;
            uint32_t sc, mn;
            q4k_scale_min(sb, scales, &sc, &mn);
            const float sc_v = d * (float)sc;
            const float m_v = dmin * (float)mn;
            const int iq = sb / 2, lo = sb % 2;
            const uint32_t nib =
                (lo == 0) ? (qs[iq * 32 + elem] & 0x0Fu) : (uint32_t)(qs[iq * 32 + elem] >> 4);
            o[j] = sc_v * (float)nib - m_v;
        }
    } break;
    case ORC_Q6_K: { /* {u8 ql[128]; u8 qh[64]; i8 scales[16]; f16 d}  2518-2554 */
        const uint8_t *ql = blk, *qh = blk + 128;
        const int8_t *scales = (const int8_t *)(blk + 192);
        const float d = rd_f16(blk + 208);
        for (int j = 0; j < 256; ++j) {
            const int h = j / 128, pos = j % 128, quad = pos / 32, l = pos % 32;
            const uint8_t *ql_base = ql + 64 * h, *qh_base = qh + 32 * h;
            const int ql_idx = (quad & 1) ? (l + 32) : l;
            const int shift_ql = (quad < 2) ? 0 : 4;
            const uint32_t nib = ((uint32_t)ql_base[ql_idx] >> shift_ql) & 0x0Fu;
            const uint32_t hb = ((uint32_t)qh_base[l] >> (2 * quad)) & 3u;
            const int qv = (int)(nib | (hb << 4)) - 32;
            const float sc_v = d * (float)scales[8 * h + 2 * quad + l / 16];
            o[j] = sc_v * (float)qv;
        }
    } break;
    case ORC_Q4_1: { /* {f16 d, m; u8 qs[16]}  quant_kernels.metal:872-876, 2386-2408 */
        const float d = rd_f16(blk), m = rd_f16(blk + 2);
        const uint8_t *qs = blk + 4;
        for (int j = 0; j < 32; ++j) {
            const uint32_t qp = (j < 16) ? (qs[j] & 0x0Fu) : (uint32_t)(qs[j - 16] >> 4);
            o[j] = (float)qp * d + m;
        }
    } break;
    case ORC_Q5_0: { /* {f16 d; u8 qh[4]; u8 qs[16]}  709-713, 2315-2340 */
        const float d = rd_f16(blk);
        const uint32_t qh = rd_u32(blk + 2);
        const uint8_t *qs = blk + 6;
        for (int j = 0; j < 32; ++j) {
            const int hi = j / 16, jj = j % 16;
            const uint32_t xh = ((qh >> (jj + hi * 16)) & 1u) << 4;
            const uint32_t qp = (hi == 0) ? (qs[jj] & 0x0Fu) : (uint32_t)(qs[jj] >> 4);
            o[j] = (float)((int)(qp | xh) - 16) * d;
        }
    } break;
    case ORC_Q5_1: { /* {f16 d, m; u8 qh[4]; u8 qs[16]}  954-959, 2410-2436 */
        const float d = rd_f16(blk), m = rd_f16(blk + 2);
        const uint32_t qh = rd_u32(blk + 4);
        const uint8_t *qs = blk + 8;
        for (int j = 0; j < 32; ++j) {
            const int hi = j / 16, jj = j % 16;
            const uint32_t xh = ((qh >> (jj + hi * 16)) & 1u) << 4;
            const uint32_t qp = (hi == 0) ? (qs[jj] & 0x0Fu) : (uint32_t)(qs[jj] >> 4);
            o[j] = (float)(qp | xh) * d + m;
        }
    } break;
    case ORC_Q2_K: { /* {u8 scales[16]; u8 qs[64]; f16 d, dmin}  1841-1846, 2556-2592 */
        const uint8_t *scales = blk, *qs = blk + 16;
        const float d = rd_f16(blk + 80), dmin = rd_f16(blk + 82);
        for (int j = 0; j < 256; ++j) {
            const int half = j / 128, pos = j % 128, sub = pos / 32, in_sub = pos % 32;
            const int second = in_sub / 16, elem = in_sub % 16;
            const uint32_t q = ((uint32_t)qs[half * 32 + second * 16 + elem] >> (2 * sub)) & 3u;
            const uint32_t sc = scales[half * 8 + sub * 2 + second];
            const float dl = d * (float)(sc & 0x0Fu);
            const float ml = dmin * (float)((sc >> 4) & 0x0Fu);
            o[j] = dl * (float)q - ml;
        }
    } break;
    case ORC_Q3_K: { /* {u8 hmask[32]; u8 qs[64]; u8 scales[12]; f16 d}  2032-2037, 2594-2640 */
        const uint8_t *hmask = blk, *qs = blk + 32, *scales = blk + 96;
        const float d = rd_f16(blk + 108);
        for (int j = 0; j < 256; ++j) {
            const int half = j / 128, shift_idx = (j % 128) / 32, e = j % 32;
            const uint32_t low2 = ((uint32_t)qs[half * 32 + e] >> (2 * shift_idx)) & 3u;
            const uint32_t hbit = ((uint32_t)hmask[e] >> (half * 4 + shift_idx)) & 1u;
            const int q = (int)low2 - (hbit ? 0 : 4);
            o[j] = d * (float)q3k_scale(j / 16, scales) * (float)q;
        }
    } break;
    case ORC_Q5_K: { /* {f16 d, dmin; u8 scales[12]; u8 qh[32]; u8 qs[128]}  1439-1445, 2484-2516 */
        const float d = rd_f16(blk), dmin = rd_f16(blk + 2);
        const uint8_t *scales = blk + 4, *qh = blk + 16, *qs = blk + 48;
        for (int j = 0; j < 256; ++j) {
            const int sb = j / 32, elem = j % 32;
            uint32_t sc, mn;
            q4k_scale_min(sb, scales, &sc, &mn);
            const float sc_v = d * (float)sc;
            const float m_v = dmin * (float)mn;
            const int iq = sb / 2, lo = sb % 2;
            const uint32_t low4 =
                (lo == 0) ? (qs[iq * 32 + elem] & 0x0Fu) : (uint32_t)(qs[iq * 32 + elem] >> 4);
            const uint32_t hb = ((uint32_t)qh[elem] >> (2 * iq + lo)) & 1u;
            o[j] = sc_v * (float)(low4 | (hb << 4)) - m_v;
        }
    } break;
    }
}

/* bytes: N rows of K/elems consecutive blocks; out: [N, K] f32. */
int orc_dequantize_gguf(int fmt, const uint8_t *bytes, size_t bytes_len, int64_t N, int64_t K,
                        float *out) {
    int elems, bbytes;
    if (orc_gguf_block_layout(fmt, &elems, &bbytes) != ORC_OK) return ORC_ERR_ARG;
    if (K % elems != 0) return ORC_ERR_SHAPE;
    const int64_t nb = K / elems;
    if (bytes_len != (size_t)(N * nb * bbytes)) return ORC_ERR_SHAPE;
#pragma omp parallel for schedule(static)
    for (int64_t n = 0; n < N; ++n)
        for (int64_t b = 0; b < nb; ++b)
            dequant_block(fmt, bytes + (n * nb + b) * bbytes, out + n * K + b * elems);
    return ORC_OK;
}

/* ------------------------------------------------------------------ */
/* y = x . W^T (+ bias): linear.rs:40-79, f32 accumulate               */
/* ------------------------------------------------------------------ */

void orc_matmul_nt_f32(const float *x, /* [M,K] */ const float *w, /* [N,K] */
                       const float *bias /* [N] or NULL */, float *y /* [M,N] */, int64_t M,
                       int64_t K, int64_t N) {
#pragma omp parallel for schedule(static)
    for (int64_t n = 0; n < N; ++n) {
        const float *wr = w + n * K;
        for (int64_t m = 0; m < M; ++m) {
            const float *xr = x + m * K;
            float acc = 0.0f;
            for (int64_t k = 0; k < K; ++k) acc += xr[k] * wr[k];
            y[m * N + n] = bias ? acc + bias[n] : acc;
        }
    }
}

/* Same contraction accumulated in f64, rounded once to f32: used by tests to
 * tell kernel error from the f32 oracle's own accumulation-order noise. */
void orc_matmul_nt_f64acc(const float *x, const float *w, const float *bias, float *y, int64_t M,
                          int64_t K, int64_t N) {
#pragma omp parallel for schedule(static)
    for (int64_t n = 0; n < N; ++n) {
        const float *wr = w + n * K;
        for (int64_t m = 0; m < M; ++m) {
            const float *xr = x + m * K;
            double acc = 0.0;
            for (int64_t k = 0; k < K; ++k) acc += (double)xr[k] * (double)wr[k];
            if (bias) acc += (double)bias[n];
            y[m * N + n] = (float)acc;
        }
    }
}

/* ------------------------------------------------------------------ */
/* MoE routing: moe.rs:466-499 and dispatch_sparse lists 563-590       */
/* ------------------------------------------------------------------ */

/* logits [T,E] f32 -> softmax (max-subtracted, linear.rs:160-171) -> indices of
 * the top_k largest probabilities in descending order (stable for ties) ->
 * gathered probabilities, renormalised to sum 1 when norm_topk != 0. */
int orc_moe_route(const float *logits, int64_t T, int64_t E, int64_t top_k, int norm_topk,
                  uint32_t *top_idx /* [T,top_k] */, float *top_vals /* [T,top_k] */) {
    if (top_k <= 0 || top_k > E) return ORC_ERR_ARG;
    float *probs = (float *)malloc((size_t)E * sizeof(float));
    uint32_t *order = (uint32_t *)malloc((size_t)E * sizeof(uint32_t));
    if (!probs || !order) return ORC_ERR_ARG;
    for (int64_t t = 0; t < T; ++t) {
        const float *l = logits + t * E;
        float mx = l[0];
        for (int64_t e = 1; e < E; ++e) mx = l[e] > mx ? l[e] : mx;
        float sum = 0.0f;
        for (int64_t e = 0; e < E; ++e) {
            probs[e] = expf(l[e] - mx);
            sum += probs[e];
        }
        for (int64_t e = 0; e < E; ++e) probs[e] /= sum;
        for (int64_t e = 0; e < E; ++e) order[e] = (uint32_t)e;
        /* stable insertion sort, descending */
        for (int64_t i = 1; i < E; ++i) {
            uint32_t cur = order[i];
            int64_t j = i - 1;
            while (j >= 0 && probs[order[j]] < probs[cur]) {
                order[j + 1] = order[j];
                --j;
            }
            order[j + 1] = cur;
        }
        float denom = 0.0f;
        for (int64_t s = 0; s < top_k; ++s) {
            top_idx[t * top_k + s] = order[s];
            top_vals[t * top_k + s] = probs[order[s]];
            denom += probs[order[s]];
        }
        if (norm_topk)
            for (int64_t s = 0; s < top_k; ++s) top_vals[t * top_k + s] /= denom;
    }
    free(probs);
    free(order);
    return ORC_OK;
}

/* Token lists per expert in dispatch_sparse order (token-major, slot-minor):
 * offsets [E+1], tokens [T*top_k], weights [T*top_k]. */
int orc_moe_group(const uint32_t *top_idx, const float *top_vals, int64_t T, int64_t E,
                  int64_t top_k, int64_t *offsets, uint32_t *tokens, float *weights) {
    for (int64_t e = 0; e <= E; ++e) offsets[e] = 0;
    for (int64_t i = 0; i < T * top_k; ++i) {
        if (top_idx[i] >= (uint32_t)E) return ORC_ERR_ARG;
        offsets[top_idx[i] + 1]++;
    }
    for (int64_t e = 0; e < E; ++e) offsets[e + 1] += offsets[e];
    int64_t *cursor = (int64_t *)malloc((size_t)E * sizeof(int64_t));
    if (!cursor) return ORC_ERR_ARG;
    for (int64_t e = 0; e < E; ++e) cursor[e] = offsets[e];
    for (int64_t t = 0; t < T; ++t)
        for (int64_t s = 0; s < top_k; ++s) {
            const uint32_t e = top_idx[t * top_k + s];
            tokens[cursor[e]] = (uint32_t)t;
            weights[cursor[e]] = top_vals[t * top_k + s];
            cursor[e]++;
        }
    free(cursor);
    return ORC_OK;
}

/* GPT-OSS clamped SwiGLU on an interleaved gate/up row: moe.rs:152-173.
 * gu [M, 2I] (even = gate, odd = up) -> h [M, I]. */
void orc_gpt_oss_swiglu(const float *gu, int64_t M, int64_t I, float limit, float *h) {
    for (int64_t m = 0; m < M; ++m)
        for (int64_t k = 0; k < I; ++k) {
            float gate = gu[m * 2 * I + 2 * k];
            float up = gu[m * 2 * I + 2 * k + 1];
            gate = gate < limit ? gate : limit;
            up = up < -limit ? -limit : (up > limit ? limit : up);
            const float sig = 1.0f / (1.0f + expf(-(gate * 1.702f)));
            h[m * I + k] = (up + 1.0f) * (gate * sig);
        }
}

/* Fused gated activations over [.., gate | up]: ffn_kernels.metal:5-17 (scalar functions),
 * 23-36 and 115-128 (the f32 kernels).  gu [M, 2I] -> out [M, I], f32 math. */
void orc_gated_silu(const float *gu, int64_t M, int64_t I, float *out) {
    for (int64_t m = 0; m < M; ++m)
        for (int64_t k = 0; k < I; ++k) {
            const float g = gu[m * 2 * I + k], u = gu[m * 2 * I + I + k];
            out[m * I + k] = (g / (1.0f + expf(-g))) * u;
        }
}

void orc_gated_gelu_tanh(const float *gu, int64_t M, int64_t I, float *out) {
    const float k0 = 0.7978845608028654f, k1 = 0.044715f;
    for (int64_t m = 0; m < M; ++m)
        for (int64_t k = 0; k < I; ++k) {
            const float g = gu[m * 2 * I + k], u = gu[m * 2 * I + I + k];
            const float inner = k0 * (g + k1 * g * g * g);
            out[m * I + k] = (0.5f * g * (1.0f + tanhf(inner))) * u;
        }
}

/* dispatch_sparse's scatter, moe.rs:592-605: experts in ascending order, each adding
 * weight * expert_out for its tokens.  Restated in f32 (the reference accumulates in the
 * activation dtype; the caller rounds as needed).  expert_out is in grouped pair order. */
void orc_moe_combine(const float *expert_out, const int64_t *offsets, const uint32_t *tokens,
                     const float *weights, int64_t E, int64_t T, int64_t H, float *out) {
    for (int64_t i = 0; i < T * H; ++i) out[i] = 0.0f;
    for (int64_t e = 0; e < E; ++e)
        for (int64_t p = offsets[e]; p < offsets[e + 1]; ++p) {
            const int64_t t = tokens[p];
            for (int64_t h = 0; h < H; ++h) out[t * H + h] += weights[p] * expert_out[p * H + h];
        }
}
