// MXFP4 (E2M1 values, one E8M0 scale per 32) expert GEMV and dense dequant.
//
// Reference semantics: mxfp4.rs:13-64 (code table, low nibble first,
// scale 2^(s-127), 0xFF -> NaN) and quant_kernels.metal:3104-3173
// (mxfp4_gemv_batch_bf16: bf16 x/y, f32 accumulation).  The grouped form runs
// every active expert of one MoE projection in a single launch; it replaces
// the per-expert loop of moe.rs:593-605.
//
// One wave per output row; a lane owns whole 32-element blocks (one aligned
// 128-bit load each) and strides over the row.  HBM-bound.

#include "oxq_device.hpp"
#include "oxq_internal.hpp"

#include <cstdlib>

namespace oxq {

// E2M1 code -> f32: sign | exponent e (2 bits) | mantissa m (1 bit);
// e == 0 is the subnormal {0, 0.5}; else (1 + m/2) * 2^(e-1).
__device__ __forceinline__ float fp4_to_f32(uint32_t c) {
    const uint32_t e = (c >> 1) & 3u, m = c & 1u;
    uint32_t bits = e ? (((126u + e) << 23) | (m << 22)) : (m ? 0x3F000000u : 0u);
    bits |= (c & 8u) << 28;
    return __builtin_bit_cast(float, bits);
}

__device__ __forceinline__ void decode_block(const u32x4_t q, float scale, float w[32]) {
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int b = 0; b < 4; ++b) {
            const uint32_t byte = (q[i] >> (8 * b)) & 0xFFu;
            w[8 * i + 2 * b] = fp4_to_f32(byte & 0xFu) * scale;
            w[8 * i + 2 * b + 1] = fp4_to_f32(byte >> 4) * scale;
        }
}

// Block dot product on the gfx950 conversion path: v_cvt_scalef32_pk_bf16_fp4
// turns one byte (two E2M1 codes, low nibble first) into a bf16 pair - every
// E2M1 value is exact in bf16 - and v_dot2_f32_bf16 multiplies it with the
// matching activation pair into an f32 accumulator.  One conversion and one
// dot per two weights; the E8M0 scale multiplies the block sum once.
// The activation pair is taken as a by-value uint32_t: bit-casting an element
// of a vector lvalue directly made the compiler read element 0 every time.
__device__ __forceinline__ float dot2_fp4(float acc, uint32_t xpair, bf16x2_t wpair) {
    return __builtin_amdgcn_fdot2_f32_bf16(wpair, __builtin_bit_cast(bf16x2_t, xpair), acc, false);
}

__device__ __forceinline__ float block_dot_bf16(const u32x4_t q, const uint16_t *__restrict__ xr) {
    const u32x4_t *xp = (const u32x4_t *)xr;
    float acc = 0.0f;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const u32x4_t xv = xp[i];
        const uint32_t w = q[i], x0 = xv[0], x1 = xv[1], x2 = xv[2], x3 = xv[3];
        acc = dot2_fp4(acc, x0, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(w, 1.0f, 0));
        acc = dot2_fp4(acc, x1, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(w, 1.0f, 1));
        acc = dot2_fp4(acc, x2, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(w, 1.0f, 2));
        acc = dot2_fp4(acc, x3, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(w, 1.0f, 3));
    }
    return acc;
}

// Same, with the block's activations stored as four 16-byte chunks `pitch` chunks apart
// (LDS layout of the staged kernel: consecutive lanes read consecutive chunks, no bank conflicts).
__device__ __forceinline__ float block_dot_bf16_chunked(const u32x4_t q, const unsigned char *xb, int pitch) {
    float acc = 0.0f;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const u32x4_t xv = *(const u32x4_t *)(xb + (size_t)i * pitch * 16);
        const uint32_t w = q[i], x0 = xv[0], x1 = xv[1], x2 = xv[2], x3 = xv[3];
        acc = dot2_fp4(acc, x0, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(w, 1.0f, 0));
        acc = dot2_fp4(acc, x1, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(w, 1.0f, 1));
        acc = dot2_fp4(acc, x2, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(w, 1.0f, 2));
        acc = dot2_fp4(acc, x3, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(w, 1.0f, 3));
    }
    return acc;
}

// grid.x = row quads, grid.y = expert (1 for the plain form).
// offsets == nullptr: plain form, rows 0..M-1 of x / y.
template <int MB>
__global__ __launch_bounds__(256) void mxfp4_gemv_kernel(
    const uint16_t *__restrict__ x, const uint8_t *__restrict__ blocks,
    const uint8_t *__restrict__ scales, const uint16_t *__restrict__ bias,
    uint16_t *__restrict__ y, const int32_t *__restrict__ offsets,
    const int32_t *__restrict__ token_ids, int M, int K, int N) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int n = blockIdx.x * 4 + wave;
    if (n >= N) return;
    const int e = blockIdx.y;
    int p0 = 0, p1 = M;
    if (offsets) {
        p0 = offsets[e];
        p1 = offsets[e + 1];
        if (p1 <= p0) return;
    }
    const int nb = K >> 5;
    const size_t row = (size_t)e * N + n;
    const u32x4_t *brow = (const u32x4_t *)blocks + row * nb;
    const uint8_t *srow = scales + row * nb;
    const float bv = bias ? BF16Traits::to_f32(bias[row]) : 0.0f;

    for (int pbase = p0; pbase < p1; pbase += MB) {
        const int rows = min(MB, p1 - pbase);
        const uint16_t *xrow[MB];
#pragma unroll
        for (int m = 0; m < MB; ++m) {
            const int p = pbase + (m < rows ? m : 0);
            const int src = token_ids ? token_ids[p] : p;
            xrow[m] = x + (size_t)src * K;
        }
        float acc[MB];
#pragma unroll
        for (int m = 0; m < MB; ++m) acc[m] = 0.0f;
        for (int b = lane; b < nb; b += 64) {
            const u32x4_t q = brow[b];
            const float scale = e8m0_to_f32(srow[b]);
#pragma unroll
            for (int m = 0; m < MB; ++m)
                if (m < rows) acc[m] = fmaf(scale, block_dot_bf16(q, xrow[m] + (size_t)b * 32), acc[m]);
        }
#pragma unroll
        for (int m = 0; m < MB; ++m) {
            if (m < rows) {
                const float tot = wave_sum_xor<64>(acc[m]);
                if (lane == 0) y[(size_t)(pbase + m) * N + n] = BF16Traits::from_f32(tot + bv);
            }
        }
    }
}

// Activations in LDS, several rows per wave.  With one wave per output row every wave
// re-reads its tokens' activations (K * 2 bytes each) from L2, four times the bytes of
// the weight row itself, and that traffic - not HBM - sets the pace.  Here a workgroup
// stages the expert's tokens once (up to MB at a time) and its 4 waves then stream RW rows
// each, all of a row's loads in flight before the first dot product.
// grid.x = blocks of 4*RW rows, grid.y = expert (1 for the plain form).
template <int MB, int RW>
__global__ __launch_bounds__(256) void mxfp4_gemv_lds_kernel(
    const uint16_t *__restrict__ x, const uint8_t *__restrict__ blocks,
    const uint8_t *__restrict__ scales, const uint16_t *__restrict__ bias,
    uint16_t *__restrict__ y, const int32_t *__restrict__ offsets,
    const int32_t *__restrict__ token_ids, int M, int K, int N) {
    // [MB] token rows; chunk c (0..3) of block b at ((c * (nb + 1)) + b) * 16 bytes
    extern __shared__ __attribute__((aligned(16))) unsigned char mx_lds[];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int e = blockIdx.y;
    int p0 = 0, p1 = M;
    if (offsets) {
        p0 = offsets[e];
        p1 = offsets[e + 1];
        if (p1 <= p0) return;  // block-uniform
    }
    const int nb = K >> 5;
    const int n0 = (blockIdx.x * 4 + wave) * RW;
    const int cpr = K >> 3;  // 16-byte chunks per activation row
    const int pitch = nb + 1;
    const size_t xrow_bytes = (size_t)4 * pitch * 16;
    constexpr int PASSES = 2;  // blocks per lane and row held in registers (K <= 4096)

    for (int pbase = p0; pbase < p1; pbase += MB) {
        const int rows = min(MB, p1 - pbase);
        if (pbase > p0) __syncthreads();  // everyone is done with the previous tokens
        for (int c = threadIdx.x; c < rows * cpr; c += 256) {
            const int m = c / cpr, cc = c - m * cpr;
            const int p = pbase + m;
            const int src = token_ids ? token_ids[p] : p;
            *(u32x4_t *)(mx_lds + m * xrow_bytes + ((size_t)(cc & 3) * pitch + (cc >> 2)) * 16) =
                *(const u32x4_t *)(x + (size_t)src * K + (size_t)cc * 8);
        }
        __syncthreads();

#pragma unroll 1
        for (int r0 = 0; r0 < RW; r0 += 2) {
            // two rows at a time: 2 x PASSES weight blocks and scale bytes in flight per lane
            u32x4_t q[2][PASSES];
            uint32_t sb[2][PASSES];
#pragma unroll
            for (int r = 0; r < 2; ++r) {
                const int n = n0 + r0 + r;
                const size_t row = (size_t)e * N + (n < N ? n : N - 1);
#pragma unroll
                for (int ps = 0; ps < PASSES; ++ps) {
                    const int b = lane + 64 * ps;
                    const int bc = b < nb ? b : nb - 1;
                    q[r][ps] = ((const u32x4_t *)blocks)[row * nb + bc];
                    sb[r][ps] = scales[row * nb + bc];
                }
            }
#pragma unroll
            for (int r = 0; r < 2; ++r) {
                const int n = n0 + r0 + r;
                float acc[MB];
#pragma unroll
                for (int m = 0; m < MB; ++m) acc[m] = 0.0f;
#pragma unroll
                for (int ps = 0; ps < PASSES; ++ps) {
                    const int b = lane + 64 * ps;
                    if (b < nb) {
                        const float scale = e8m0_to_f32(sb[r][ps]);
#pragma unroll
                        for (int m = 0; m < MB; ++m)
                            if (m < rows)
                                acc[m] = fmaf(scale,
                                              block_dot_bf16_chunked(q[r][ps], mx_lds + m * xrow_bytes + (size_t)b * 16, pitch),
                                              acc[m]);
                    }
                }
                // blocks past 2 x 64 (K > 4096): stream the rest
                for (int b = lane + 64 * PASSES; b < nb; b += 64) {
                    const size_t row = (size_t)e * N + (n < N ? n : N - 1);
                    const u32x4_t qq = ((const u32x4_t *)blocks)[row * nb + b];
                    const float scale = e8m0_to_f32(scales[row * nb + b]);
#pragma unroll
                    for (int m = 0; m < MB; ++m)
                        if (m < rows)
                            acc[m] = fmaf(scale, block_dot_bf16_chunked(qq, mx_lds + m * xrow_bytes + (size_t)b * 16, pitch), acc[m]);
                }
                if (n < N) {  // wave-uniform
                    const float bv = bias ? BF16Traits::to_f32(bias[(size_t)e * N + n]) : 0.0f;
#pragma unroll
                    for (int m = 0; m < MB; ++m) {
                        if (m < rows) {
                            const float tot = wave_sum_xor<64>(acc[m]);
                            if (lane == 0) y[(size_t)(pbase + m) * N + n] = BF16Traits::from_f32(tot + bv);
                        }
                    }
                }
            }
        }
    }
}

// ---------------------------------------------------------------------------
// Expert GEMV on the matrix cores: the tokens are the M tile (<= 16 rows of
// v_mfma_f32_16x16x32_bf16), 16 weight rows are one N tile.
//
// An MXFP4 block is 32 consecutive k of one row = exactly one MFMA K step for that row, and
// v_cvt_scalef32_pk_bf16_fp4 converts two E2M1 codes to bf16 *and* applies the block's E8M0
// scale (a per-lane operand) in one instruction: 4 conversions build a B fragment, exactly.
// The k index inside an MFMA step only has to agree between A and B, so lane (ni = row,
// kb = lane / 16) takes four whole consecutive blocks 16T + 4kb + j (j = 0..3, 64 contiguous
// bytes, four 16-byte loads) and spends them over 16 steps (block j, quarter s = bytes
// 4s..4s+3); the matching activation fragment is the 16-byte chunk 4*(16T+4kb+j) + s of the
// token row, read from LDS where the tokens are staged once per workgroup (chunk-major,
// token fastest).  Rows of the M tile past the expert's token count compute garbage that is
// never stored (MFMA rows are independent).  One conversion per two weights and one MFMA per
// 512 weights replace the dot2 chain, the per-row wave reduction and the 70 % lane use of
// the one-wave-per-row form at 90 blocks per row.
// grid.x = blocks of 4 waves x FR x 16 rows, grid.y = expert (1 for the plain form).
// ---------------------------------------------------------------------------
template <int MTOK, int FR>
__global__ __launch_bounds__(256) void mxfp4_mfma_kernel(
    const uint16_t *__restrict__ x, const uint8_t *__restrict__ blocks,
    const uint8_t *__restrict__ scales, const uint16_t *__restrict__ bias,
    uint16_t *__restrict__ y, const int32_t *__restrict__ offsets,
    const int32_t *__restrict__ token_ids, int M, int K, int N, int swiglu, float limit) {
    // [K/8 chunks][MTOK] x 16 B of tokens, then per wave the scale bytes of its 16*FR rows
    extern __shared__ __attribute__((aligned(16))) unsigned char mm_lds[];
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int ni = lane & 15, kb = lane >> 4;
    const int e = blockIdx.y;
    int p0 = 0, p1 = M;
    if (offsets) {
        p0 = offsets[e];
        p1 = offsets[e + 1];
        if (p1 <= p0) return;  // block-uniform
    }
    const int nb = K >> 5, cpr = K >> 3;
    const int NT = (nb + 15) >> 4;  // tiles of 16 blocks
    const int n_base = (blockIdx.x * 4 + wave) * (16 * FR);
    const int nrows = min(16 * FR, N - n_base);  // rows of this wave inside the matrix (<= 0: none)
    const bool active = nrows > 0;               // wave-uniform
    // Loads are issued row-major: lane (lr = lane / 4, lc = lane % 4) fetches block 16T + 4j + lc of
    // row lr, so four neighbouring lanes read 64 contiguous bytes (16 separate 16-byte requests per
    // row would reach 4.8 TB/s where this reaches 5.5).  The matrix core wants lane (ni, kb) to hold
    // row ni: a 4 x 16 lane transpose (ds_bpermute, no LDS memory) at the point of use gives lane
    // (ni, kb) the block 16T + 4j + kb of row ni.
    const int lr = lane >> 2, lc = lane & 3;
    const int tr_src = (4 * ni + kb) * 4;  // byte index of the lane whose register this lane needs
    // Buffer loads relative to the wave's first row: a tile past the row's end is requested from beyond the
    // descriptor (zeros, no memory access), so that every request is unconditional - behind a condition the
    // compiler joins the paths with and without new requests and waits as if there were none, i.e. for the
    // tile just requested.
    const __amdgpu_buffer_rsrc_t rs_w = make_rsrc((const u32x4_t *)blocks + ((size_t)e * N + (active ? n_base : 0)) * nb,
                                                  active ? (uint32_t)nrows * (uint32_t)nb * 16u : 0u);
    int wrow[FR];  // byte offset of the lane's row (clamped to the wave's last valid row)
#pragma unroll
    for (int f = 0; f < FR; ++f) wrow[f] = min(16 * f + lr, max(nrows, 1) - 1) * nb * 16;
    const int a_tok = (ni & (MTOK - 1)) * 16;
    // token chunks in LDS: quarter sq (16 bytes of every token) of block b
    auto tok_chunk = [](int b, int sq) { return (b * 4 + sq) * (MTOK * 16); };

    constexpr int D = 2;  // weight tiles in registers: one in use, D - 1 in flight (3 measured the same)
    u32x4_t wq[D][FR][4];
    auto load_tile = [&](int T, u32x4_t (&w)[FR][4]) {
#pragma unroll
        for (int f = 0; f < FR; ++f)
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int b = 16 * T + 4 * j + lc;
                w[f][j] = __builtin_amdgcn_raw_buffer_load_b128(rs_w, T < NT ? wrow[f] + (b < nb ? b : nb - 1) * 16 : 0x7FFFFF00, 0, 0);
            }
    };
    // the first weight tiles do not depend on the tokens: they are requested before those are staged
    if (active) {
#pragma unroll
        for (int d = 0; d < D - 1; ++d) load_tile(d, wq[d]);
    }

    // The wave's scale bytes (rows n_base .. n_base + nrows - 1 are contiguous, nb bytes each): one
    // coalesced pass of aligned 32-bit loads into LDS instead of four single-byte loads per lane and
    // tile.  The first and last word may reach up to 3 bytes outside the range; an aligned word that
    // holds a byte of the tensor lies in the same page as that byte.
    unsigned char *sc_lds = mm_lds + (size_t)MTOK * K * 2 + (size_t)wave * (16 * FR * nb + 16);
    int sc_mis = 0;
    if (active) {
        const uint8_t *s0 = scales + ((size_t)e * N + n_base) * nb;
        sc_mis = (int)((uintptr_t)s0 & 3);
        const uint32_t *s32 = (const uint32_t *)(s0 - sc_mis);
        const int words = (sc_mis + nrows * nb + 3) >> 2;
        for (int i = lane; i < words; i += 64) ((uint32_t *)sc_lds)[i] = s32[i];
    }
    // per fragment: where this lane's row (clamped to the wave's last valid row) starts in sc_lds
    int sc_row[FR];
#pragma unroll
    for (int f = 0; f < FR; ++f) sc_row[f] = sc_mis + min(16 * f + ni, max(nrows, 1) - 1) * nb;

    for (int pbase = p0; pbase < p1; pbase += MTOK) {
        const int rows = min(MTOK, p1 - pbase);
        if (pbase > p0) {
            __syncthreads();  // everyone is done with the previous tokens
            if (active) {
#pragma unroll
                for (int d = 0; d < D - 1; ++d) load_tile(d, wq[d]);
            }
        }
        for (int c = threadIdx.x; c < rows * cpr; c += 256) {
            const int m = c / cpr, cc = c - m * cpr;
            const int p = pbase + m;
            const int src = token_ids ? token_ids[p] : p;
            *(u32x4_t *)(mm_lds + tok_chunk(cc >> 2, cc & 3) + m * 16) = *(const u32x4_t *)(x + (size_t)src * K + (size_t)cc * 8);
        }
        __syncthreads();
        if (!active) continue;  // wave-uniform; the barriers above are reached by every wave

        float4_t acc[FR];
#pragma unroll
        for (int f = 0; f < FR; ++f) acc[f] = float4_t{0.f, 0.f, 0.f, 0.f};
        auto tile = [&](int T, int par) {
            load_tile(T + D - 1, wq[(par + D - 1) % D]);  // past the end: zeros, no memory access
            // Lane transposes and scale reads in batches of two blocks, activation reads in batches
            // of one block: a wave waits for LDS six times a tile, not once per fragment.
            const bool ragged = T == NT - 1 && (nb & 15);  // wave-uniform: only the last tile can be
#pragma unroll
            for (int jh = 0; jh < 4; jh += 2) {
                uint32_t wp[FR][2][4];
                float scf[FR][2];
                int bcl[2];
#pragma unroll
                for (int jj = 0; jj < 2; ++jj) {
                    const int b = 16 * T + 4 * (jh + jj) + kb;
                    bcl[jj] = b < nb ? b : nb - 1;  // blocks past the row: a finite chunk, weights zeroed below
                }
#pragma unroll
                for (int f = 0; f < FR; ++f)
#pragma unroll
                    for (int jj = 0; jj < 2; ++jj) {
                        const u32x4_t t = wq[par][f][jh + jj];
#pragma unroll
                        for (int q = 0; q < 4; ++q)
                            wp[f][jj][q] = (uint32_t)__builtin_amdgcn_ds_bpermute(tr_src, (int)t[q]);
                        scf[f][jj] = e8m0_to_f32(sc_lds[sc_row[f] + bcl[jj]]);
                    }
                if (ragged) {
#pragma unroll
                    for (int jj = 0; jj < 2; ++jj) {
                        const bool valid = 16 * T + 4 * (jh + jj) + kb < nb;
#pragma unroll
                        for (int f = 0; f < FR; ++f)
#pragma unroll
                            for (int q = 0; q < 4; ++q) wp[f][jj][q] = valid ? wp[f][jj][q] : 0u;
                    }
                }
#pragma unroll
                for (int jj = 0; jj < 2; ++jj) {
                    u32x4_t av[4];
#pragma unroll
                    for (int sq = 0; sq < 4; ++sq)
                        av[sq] = *(const u32x4_t *)(mm_lds + tok_chunk(bcl[jj], sq) + a_tok);
#pragma unroll
                    for (int sq = 0; sq < 4; ++sq) {
#pragma unroll
                        for (int f = 0; f < FR; ++f) {
                            const uint32_t w = wp[f][jj][sq];
                            u32x4_t bv;
                            bv[0] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(w, scf[f][jj], 0));
                            bv[1] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(w, scf[f][jj], 1));
                            bv[2] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(w, scf[f][jj], 2));
                            bv[3] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(w, scf[f][jj], 3));
                            acc[f] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, av[sq]),
                                                                            __builtin_bit_cast(bf16x8_t, bv), acc[f], 0, 0, 0);
                        }
                    }
                }
            }
        };
        // (as straight-line code for a known tile count this kernel is slower: 59.7 against 53.5 us a decode step)
        for (int T0 = 0; T0 < NT; T0 += D) {
#pragma unroll
            for (int par = 0; par < D; ++par)
                if (T0 + par < NT) tile(T0 + par, par);  // block-uniform
        }
        // D[m][n]: lane (n = ni, m = 4*kb + i): token 4*kb + i of weight row n_base + 16 f + ni
#pragma unroll
        for (int f = 0; f < FR; ++f) {
            const int n = n_base + 16 * f + ni;
            const float bv = (bias && n < N) ? BF16Traits::to_f32(bias[(size_t)e * N + n]) : 0.0f;
            if (swiglu) {
                // rows 2c / 2c + 1 are the gate / up of output c (moe.rs:152-173) and sit in neighbouring
                // lanes: each is rounded to bf16 as the projection's own output would be, the even lane
                // fetches its neighbour's value and stores the activation
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const int m = 4 * kb + i;
                    const float v = BF16Traits::to_f32(BF16Traits::from_f32(acc[f][i] + bv));
                    const float other = __shfl_xor(v, 1, 64);
                    if (!(ni & 1) && n + 1 < N && m < rows)
                        y[(size_t)(pbase + m) * (N >> 1) + (n >> 1)] = BF16Traits::from_f32(gpt_oss_swiglu_f32(v, other, limit));
                }
            } else if (n < N) {
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const int m = 4 * kb + i;
                    if (m < rows) y[(size_t)(pbase + m) * N + n] = BF16Traits::from_f32(acc[f][i] + bv);
                }
            }
        }
    }
}

__global__ __launch_bounds__(256) void mxfp4_dequant_kernel(const uint8_t *__restrict__ blocks,
                                                            const uint8_t *__restrict__ scales,
                                                            float *__restrict__ out, size_t nblocks) {
    const size_t b = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (b >= nblocks) return;
    float w[32];
    decode_block(((const u32x4_t *)blocks)[b], e8m0_to_f32(scales[b]), w);
    float *o = out + b * 32;
#pragma unroll
    for (int i = 0; i < 32; ++i) o[i] = w[i];
}

// ---------------------------------------------------------------------------
// Resident experts (moe.rs:366-417 keeps the stacked expert tensors of a projection for the life of
// the model): a tile-major copy built once at load, read by the decode GEMV below.
//
// In the checkpoint layout the 16 weight rows a wave feeds the matrix cores with are 16 runs of
// K/2 bytes, and a wave load is sixteen 64-byte pieces, most of them split over two cache lines.
// The copy stores, per expert and tile of 16 rows, chunks of 1 KB in operand order:
//
//   pw [E][N/16 tiles][K/32 blocks][16 rows][16 bytes]    = NC chunks of [64 lanes][16 bytes], NC = ceil(K/32 / 4),
//                                                           the last one cut off after the row's last block
//   ps [E][N/16 tiles][ceil(NC/4)][64 lanes][4 bytes]     the E8M0 bytes, byte c % 4 = chunk c
//
// Chunk c, lane (ni = lane % 16, kb = lane / 16) holds block 4c + kb of row 16 tile + ni.  Blocks past
// the row are not stored: their lanes load from beyond the tile's buffer descriptor, which returns
// zero weights without touching memory (K = 2880 is 22.5 chunks: 2.2 % of the bytes).  A wave's weights are one contiguous run read front to back
// with 1 KB loads - nontemporal, nothing is read twice - and land in matrix-core operand order: no
// lane transpose, no scale staging.  The four 4-byte words of a lane's block serve four MFMA steps.
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(256) void mxfp4_repack_kernel(const uint8_t *__restrict__ blocks,
                                                           const uint8_t *__restrict__ scales,
                                                           u32x4_t *__restrict__ pw, uint8_t *__restrict__ ps,
                                                           int E, int N, int nb, int NC, int NG) {
    // one thread per (expert, tile, chunk, lane)
    const size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;
    const int ntiles = N >> 4;
    if (idx >= (size_t)E * ntiles * NC * 64) return;
    const int lane = (int)(idx & 63);
    const int c = (int)((idx >> 6) % NC);
    const size_t et = (idx >> 6) / NC;  // expert * ntiles + tile
    const int ni = lane & 15, kb = lane >> 4;
    const int b = 4 * c + kb;
    const size_t row = et * 16 + ni;  // = expert * N + 16 tile + ni
    const bool valid = b < nb;
    if (valid) pw[et * nb * 16 + c * 64 + lane] = ((const u32x4_t *)blocks)[row * nb + b];
    ps[((et * NG + (c >> 2)) * 64 + lane) * 4 + (c & 3)] = valid ? scales[row * nb + b] : (uint8_t)127;
    // the tail of the last scale word (chunks past NC) is never read as a scale of a real block; keep it defined
    if (c == NC - 1)
        for (int cc = (c & 3) + 1; cc < 4; ++cc) ps[((et * NG + (c >> 2)) * 64 + lane) * 4 + cc] = 127;
}

// dense [N, K] f32 of one expert, from the resident copy (pins the repack bit for bit)
__global__ __launch_bounds__(256) void mxfp4_res_dequant_kernel(const u32x4_t *__restrict__ pw,
                                                                const uint8_t *__restrict__ ps,
                                                                float *__restrict__ out, int N, int nb, int NC,
                                                                int NG) {
    const size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;  // (tile, chunk, lane) of this expert
    const int ntiles = N >> 4;
    if (idx >= (size_t)ntiles * NC * 64) return;
    const int lane = (int)(idx & 63), c = (int)((idx >> 6) % NC), tile = (int)((idx >> 6) / NC);
    const int ni = lane & 15, kb = lane >> 4;
    const int b = 4 * c + kb;
    if (b >= nb) return;
    float w[32];
    decode_block(pw[(size_t)tile * nb * 16 + c * 64 + lane], e8m0_to_f32(ps[(((size_t)tile * NG + (c >> 2)) * 64 + lane) * 4 + (c & 3)]), w);
    float *o = out + ((size_t)(16 * tile + ni) * nb + b) * 32;
#pragma unroll
    for (int i = 0; i < 32; ++i) o[i] = w[i];
}

// Decode GEMV on the resident copy.  grid.x = groups of 4 tiles (one wave each), grid.y = expert.
// The expert's tokens (MTOK per pass) are staged in LDS once per workgroup; every wave then streams its
// tile: WR chunks in flight, one scale word per four chunks, four MFMA steps per chunk with the tokens
// as the M tile.  Token chunks of one block lie 64 bytes further apart than they are long, which
// spreads the four lane groups (four consecutive blocks) over all banks.
template <int MTOK, int WR, int NWV, int NCT>
__global__ __launch_bounds__(NWV * 64) void mxfp4_res_kernel(const uint16_t *__restrict__ x,
                                                        const u32x4_t *__restrict__ pw,
                                                        const uint8_t *__restrict__ ps,
                                                        const uint16_t *__restrict__ bias, uint16_t *__restrict__ y,
                                                        const int32_t *__restrict__ offsets,
                                                        const int32_t *__restrict__ token_ids, int K, int N, int NC,
                                                        int NG, int swiglu, float limit) {
    extern __shared__ __attribute__((aligned(16))) unsigned char mr_lds[];
    // WR: weight chunks in flight per wave (1 KB each); NWV: waves (tiles of 16 rows) per workgroup
    constexpr int BSTR = 4 * MTOK * 16 + 64;    // bytes of one block's token chunks, padded
    constexpr int OOB = 0x7FFFFF00;
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int ni = lane & 15, kb = lane >> 4;
    const int e = blockIdx.y;
    const int p0 = offsets[e], p1 = offsets[e + 1];
    if (p1 <= p0) return;  // block-uniform: an expert without tokens
    const int nb = K >> 5, cpr = K >> 3;
    const int ntiles = N >> 4;
    const int tile = blockIdx.x * NWV + wave;
    const bool active = tile < ntiles;  // wave-uniform
    const size_t et = (size_t)e * ntiles + (active ? tile : 0);
    const __amdgpu_buffer_rsrc_t rs_w = make_rsrc(pw + et * nb * 16, active ? (uint32_t)nb * 256u : 0u);
    const __amdgpu_buffer_rsrc_t rs_s = make_rsrc(ps + et * NG * 256, active ? (uint32_t)NG * 256u : 0u);
    const int voff_w = lane * 16, voff_s = lane * 4;
    const int a_tok = (ni & (MTOK - 1)) * 16;

    u32x4_t wring[WR];
    uint32_t sring[WR / 4];
    // blocks past the row get an offset beyond the descriptor: zeros, no memory access (the range check
    // looks at the lane's offset only, not at the scalar one, so the lane has to carry it)
    auto load_w = [&](int c) {
        return __builtin_amdgcn_raw_buffer_load_b128(rs_w, 4 * c + kb < nb ? voff_w : OOB, c * 1024, 2);
    };
    auto load_s = [&](int g) { return __builtin_amdgcn_raw_buffer_load_b32(rs_s, g < NG ? voff_s : OOB, g * 256, 2); };

    for (int pbase = p0; pbase < p1; pbase += MTOK) {
        const int rows = min(MTOK, p1 - pbase);
        // the first weights do not depend on the tokens: they are requested before those are staged
#pragma unroll
        for (int u = 0; u < WR; ++u) {
            if ((u & 3) == 0) sring[u >> 2] = load_s(u >> 2);
            wring[u] = load_w(u);
        }
        if (pbase > p0) __syncthreads();  // everyone is done with the previous tokens
        for (int c = threadIdx.x; c < rows * cpr; c += NWV * 64) {
            const int m = c / cpr, cc = c - m * cpr;
            const int p = pbase + m;
            const int src = token_ids ? token_ids[p] : p;
            *(u32x4_t *)(mr_lds + (cc >> 2) * BSTR + (cc & 3) * (MTOK * 16) + m * 16) =
                *(const u32x4_t *)(x + (size_t)src * K + (size_t)cc * 8);
        }
        __syncthreads();
        if (!active) continue;  // wave-uniform; the barriers above are reached by every wave

        float4_t acc = float4_t{0.f, 0.f, 0.f, 0.f};
        auto chunk = [&](int c, int u, const u32x4_t w, const uint32_t sw) {
            const float scale = e8m0_to_f32((sw >> (8 * (u & 3))) & 0xFFu);
            const int b = min(4 * c + kb, nb - 1);  // blocks past the row: a finite chunk times zero weights
            const unsigned char *xb = mr_lds + b * BSTR + a_tok;
            const uint32_t w0 = w[0], w1 = w[1], w2 = w[2], w3 = w[3];
            const uint32_t wq[4] = {w0, w1, w2, w3};
#pragma unroll
            for (int sq = 0; sq < 4; ++sq) {
                const u32x4_t av = *(const u32x4_t *)(xb + sq * (MTOK * 16));
                u32x4_t bv;
                bv[0] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(wq[sq], scale, 0));
                bv[1] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(wq[sq], scale, 1));
                bv[2] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(wq[sq], scale, 2));
                bv[3] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(wq[sq], scale, 3));
                acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, av),
                                                             __builtin_bit_cast(bf16x8_t, bv), acc, 0, 0, 0);
            }
        };
        // A slot is requested again only after its last use, so that the new chunk can land in the same registers:
        // requested before (while the old value is still live) it lands in others, and the copies into the loop's
        // registers at the loop's end wait for every request just made - the ring drained once a round.
        if constexpr (NCT > 0) {
            // the chunk count is known: straight-line code, every request a value of its own
#pragma unroll
            for (int c = 0; c < NCT; ++c) {
                const int u = c % WR;
                chunk(c, u, wring[u], sring[u >> 2]);
                if (c + WR < NCT) wring[u] = load_w(c + WR);
                if ((u & 3) == 3 && c + WR - 3 < NCT) sring[u >> 2] = load_s((c + WR) >> 2);  // chunks c + WR - 3 .. c + WR
                __builtin_amdgcn_sched_barrier(0);
            }
        } else {
            for (int c0 = 0; c0 < NC; c0 += WR) {
#pragma unroll
                for (int u = 0; u < WR; ++u) {
                    const int c = c0 + u;
                    if (c < NC) chunk(c, u, wring[u], sring[u >> 2]);  // wave-uniform
                    wring[u] = load_w(c + WR);
                    if ((u & 3) == 3) sring[u >> 2] = load_s((c + WR) >> 2);
                }
            }
        }
        // D[m][n]: lane (n = ni, m = 4*kb + i): token 4*kb + i of weight row 16 tile + ni
        const int n = 16 * tile + ni;
        const float bvv = bias ? BF16Traits::to_f32(bias[(size_t)e * N + n]) : 0.0f;
        if (swiglu) {
            // rows 2c / 2c + 1 are the gate / up of output c (moe.rs:152-173) and sit in neighbouring lanes:
            // each is rounded to bf16 as the projection's own output would be, the even lane fetches its
            // neighbour's value and stores the activation
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int m = 4 * kb + i;
                const float v = BF16Traits::to_f32(BF16Traits::from_f32(acc[i] + bvv));
                const float other = __shfl_xor(v, 1, 64);
                if (!(ni & 1) && m < rows)
                    y[(size_t)(pbase + m) * (N >> 1) + (n >> 1)] = BF16Traits::from_f32(gpt_oss_swiglu_f32(v, other, limit));
            }
        } else {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int m = 4 * kb + i;
                if (m < rows) y[(size_t)(pbase + m) * N + n] = BF16Traits::from_f32(acc[i] + bvv);
            }
        }
    }
}

bool mxfp4_res_eligible(int64_t K, int64_t N) {
    // whole tiles of 16 rows; the staged tokens (4 per pass) must fit LDS; 32-bit offsets inside a tile
    return K % 32 == 0 && N % 16 == 0 && N > 0 && (K / 32) * (4 * 4 * 16 + 64) <= 96 * 1024 && K <= (1 << 24);
}
size_t mxfp4_res_weight_bytes(int64_t E, int64_t K, int64_t N) {
    return (size_t)E * (size_t)(N / 16) * (size_t)(K / 32) * 256;
}
size_t mxfp4_res_scale_bytes(int64_t E, int64_t K, int64_t N) {
    return (size_t)E * (size_t)(N / 16) * (size_t)ceil_div(ceil_div(K / 32, 4), 4) * 256;
}

int launch_mxfp4_repack(oxq_ctx *ctx, hipStream_t s, const uint8_t *blocks, const uint8_t *scales, void *pw, void *ps,
                        int64_t E, int64_t K, int64_t N) {
    const int nb = (int)(K / 32), NC = (int)ceil_div(nb, 4), NG = (int)ceil_div(NC, 4);
    const size_t threads = (size_t)E * (N / 16) * NC * 64;
    dim3 grid((unsigned)ceil_div((int64_t)threads, 256)), block(256);
    set_plan(ctx, "mxfp4_repack", grid, block, 1, 1, 0);
    if (ctx->plan_only) return OXQ_OK;
    if ((uintptr_t)blocks & 15) return fail(OXQ_ERR_UNSUPPORTED, "mxfp4 repack: blocks must be 16-byte aligned");
    hipLaunchKernelGGL(mxfp4_repack_kernel, grid, block, 0, s, blocks, scales, (u32x4_t *)pw, (uint8_t *)ps, (int)E,
                       (int)N, nb, NC, NG);
    OXQ_HIP_CHECK(hipGetLastError());
    return OXQ_OK;
}

int launch_mxfp4_res_dequant(oxq_ctx *ctx, hipStream_t s, const void *pw, const void *ps, int64_t expert, int64_t K,
                             int64_t N, float *out_nk) {
    const int nb = (int)(K / 32), NC = (int)ceil_div(nb, 4), NG = (int)ceil_div(NC, 4);
    const size_t threads = (size_t)(N / 16) * NC * 64;
    dim3 grid((unsigned)ceil_div((int64_t)threads, 256)), block(256);
    set_plan(ctx, "mxfp4_res_dequant", grid, block, 1, 1, 0);
    if (ctx->plan_only) return OXQ_OK;
    const u32x4_t *w = (const u32x4_t *)pw + (size_t)expert * (N / 16) * nb * 16;
    const uint8_t *sc = (const uint8_t *)ps + (size_t)expert * (N / 16) * NG * 256;
    hipLaunchKernelGGL(mxfp4_res_dequant_kernel, grid, block, 0, s, w, sc, out_nk, (int)N, nb, NC, NG);
    OXQ_HIP_CHECK(hipGetLastError());
    return OXQ_OK;
}

template <int MTOK, int WR, int NWV, int NCT>
static int mxfp4_res_go(hipStream_t s, dim3 grid, dim3 block, size_t lds, const Mxfp4Problem &p, int NC, int NG) {
    static LdsGrant lds_grant;  // one per instantiation
    OXQ_HIP_CHECK(lds_grant.ensure((const void *)mxfp4_res_kernel<MTOK, WR, NWV, NCT>, lds));
    hipLaunchKernelGGL((mxfp4_res_kernel<MTOK, WR, NWV, NCT>), grid, block, lds, s, (const uint16_t *)p.x,
                       (const u32x4_t *)p.blocks, p.scales, (const uint16_t *)p.bias, (uint16_t *)p.y, p.expert_offsets,
                       p.token_ids, (int)p.K, (int)p.N, NC, NG, p.swiglu, p.swiglu_limit);
    OXQ_HIP_CHECK(hipGetLastError());
    return OXQ_OK;
}

// p.blocks / p.scales hold the resident copy; grouped form only
int launch_mxfp4_res_gemv(oxq_ctx *ctx, hipStream_t s, const Mxfp4Problem &p) {
    const int nb = (int)(p.K / 32), NC = (int)ceil_div(nb, 4), NG = (int)ceil_div(NC, 4);
    constexpr int MTOK = 4;
    const size_t lds = (size_t)nb * (4 * MTOK * 16 + 64);
    // 8 chunks in flight per wave and 4 waves per workgroup measured best on 32 experts x (5760 + 2880) x 2880
    // (44.7 us a decode step; 4 / 12 / 16 chunks: 45.8 / 48.7 / 51.6 us; 8 / 2 waves: 46.5 / 54.2 us).  The same
    // step with the chunk loop kept as a loop: 45.6 us; with its slots requested before their last use: 47.7)
    constexpr int WR = 8, NWV = 4;
    dim3 grid((unsigned)ceil_div(p.N / 16, NWV), (unsigned)p.n_experts), block(NWV * 64);
    char name[64];
    snprintf(name, sizeof name, "mxfp4_experts_gemv_bf16_t%d%s", MTOK, p.swiglu ? "_swiglu" : "");
    set_plan(ctx, name, grid, block, 1, 1, 0);
    if (ctx->plan_only) return OXQ_OK;
    if ((uintptr_t)p.x & 15) return fail(OXQ_ERR_UNSUPPORTED, "mxfp4 experts: x must be 16-byte aligned");
    switch (NC) {  // K = 2048, 2880, 3072, 4096: the chunk loop as straight-line code
    case 16: return mxfp4_res_go<MTOK, WR, NWV, 16>(s, grid, block, lds, p, NC, NG);
    case 23: return mxfp4_res_go<MTOK, WR, NWV, 23>(s, grid, block, lds, p, NC, NG);
    case 24: return mxfp4_res_go<MTOK, WR, NWV, 24>(s, grid, block, lds, p, NC, NG);
    case 32: return mxfp4_res_go<MTOK, WR, NWV, 32>(s, grid, block, lds, p, NC, NG);
    default: return mxfp4_res_go<MTOK, WR, NWV, 0>(s, grid, block, lds, p, NC, NG);
    }
}

template <int MB, int RW>
static int mxfp4_lds_go(hipStream_t s, dim3 grid, const Mxfp4Problem &p, size_t lds) {
    static LdsGrant lds_grant;  // one per instantiation
    OXQ_HIP_CHECK(lds_grant.ensure((const void *)mxfp4_gemv_lds_kernel<MB, RW>, lds));
    hipLaunchKernelGGL((mxfp4_gemv_lds_kernel<MB, RW>), grid, dim3(256), lds, s, (const uint16_t *)p.x, p.blocks,
                       p.scales, (const uint16_t *)p.bias, (uint16_t *)p.y, p.expert_offsets, p.token_ids,
                       (int)p.M, (int)p.K, (int)p.N);
    OXQ_HIP_CHECK(hipGetLastError());
    return OXQ_OK;
}

template <int MTOK, int FR>
static int mxfp4_mfma_go(hipStream_t s, dim3 grid, const Mxfp4Problem &p, size_t lds) {
    static LdsGrant lds_grant;  // one per instantiation
    OXQ_HIP_CHECK(lds_grant.ensure((const void *)mxfp4_mfma_kernel<MTOK, FR>, lds));
    hipLaunchKernelGGL((mxfp4_mfma_kernel<MTOK, FR>), grid, dim3(256), lds, s, (const uint16_t *)p.x, p.blocks,
                       p.scales, (const uint16_t *)p.bias, (uint16_t *)p.y, p.expert_offsets, p.token_ids,
                       (int)p.M, (int)p.K, (int)p.N, p.swiglu, p.swiglu_limit);
    OXQ_HIP_CHECK(hipGetLastError());
    return OXQ_OK;
}

int launch_mxfp4_gemv(oxq_ctx *ctx, hipStream_t s, const Mxfp4Problem &p) {
    const bool grouped = p.n_experts > 0;
    bool force_rows = false;
    {
        // prefill sizes go to the tile matmul, which converts a weight once per 64 tokens
        // instead of once per pass of 16 (4 grouped) tokens
        const int mm_mode = tune(ctx, OXQ_TUNE_MXFP4_MM, -1);  // 0 = never, 1 = always, default by size
        // plain form, measured on one expert's gate_up: m = 8 9.3 / 8.6 us, m = 16 11.8 / 8.7 us
        const bool big = grouped ? p.n_pairs >= 8 * p.n_experts : p.M >= 8;
        if ((mm_mode == 1 || (mm_mode != 0 && big)) && p.K % 32 == 0)
            return p.swiglu ? OXQ_DECLINED : launch_mxfp4_mm(ctx, s, p);  // the tile matmul has no fused epilogue
    }
    {
        // matrix-core form: tokens staged in LDS (MTOK per pass), 4 waves x FR x 16 rows per workgroup
        const int variant = tune(ctx, OXQ_TUNE_MXFP4_VARIANT, 0);  // 0 = matrix cores, 1 = dot2 with staged tokens, 2 = one wave per row
        const int mtok = (grouped || p.M <= 4) ? 4 : 16;
        int FR = tune(ctx, OXQ_TUNE_MXFP4_FR, 1);
        FR = FR >= 4 ? 4 : FR >= 2 ? 2 : 1;  // the instantiated fragment counts
        // tokens, then the four waves' scale bytes (16 * FR rows of K / 32 bytes, + alignment slack)
        const size_t lds = (size_t)mtok * (size_t)p.K * 2 + 4 * ((size_t)16 * FR * (size_t)(p.K >> 5) + 16);
        if (variant == 0 && lds <= 128 * 1024 && p.K % 32 == 0) {
            dim3 grid((unsigned)ceil_div(p.N, 4 * 16 * FR), grouped ? (unsigned)p.n_experts : 1u), block(256);
            char name[64];
            snprintf(name, sizeof name, "%s_mfma_t%d%s", grouped ? "mxfp4_moe_gemv_bf16" : "mxfp4_gemv_bf16", mtok,
                     p.swiglu ? "_swiglu" : "");
            set_plan(ctx, name, grid, block, 1, 1, 0);
            if (ctx->plan_only) return OXQ_OK;
            if (((uintptr_t)p.blocks & 15) || ((uintptr_t)p.x & 15))
                return fail(OXQ_ERR_UNSUPPORTED, "mxfp4 gemv: blocks and x must be 16-byte aligned");
            if (FR == 1) return mtok == 4 ? mxfp4_mfma_go<4, 1>(s, grid, p, lds) : mxfp4_mfma_go<16, 1>(s, grid, p, lds);
            if (FR == 4) return mtok == 4 ? mxfp4_mfma_go<4, 4>(s, grid, p, lds) : mxfp4_mfma_go<16, 4>(s, grid, p, lds);
            return mtok == 4 ? mxfp4_mfma_go<4, 2>(s, grid, p, lds) : mxfp4_mfma_go<16, 2>(s, grid, p, lds);
        }
        force_rows = variant == 2;
    }
    if (p.swiglu) return OXQ_DECLINED;  // only the matrix-core form carries the activation
    const int64_t rows_hint = grouped ? 4 : p.M;  // tokens per expert are few in decode
    const int mb = rows_hint <= 1 ? 1 : rows_hint <= 2 ? 2 : rows_hint <= 4 ? 4 : 8;
    constexpr int RW = 8;
    const size_t lds = (size_t)mb * 4 * (size_t)((p.K >> 5) + 1) * 16;
    const bool use_lds = lds <= 96 * 1024 && !tune(ctx, OXQ_TUNE_FORCE_GENERIC, 0) && !force_rows;
    if (use_lds) {
        dim3 grid((unsigned)ceil_div(p.N, 4 * RW), grouped ? (unsigned)p.n_experts : 1u), block(256);
        char name[64];
        snprintf(name, sizeof name, "%s_lds_m%d", grouped ? "mxfp4_moe_gemv_bf16" : "mxfp4_gemv_bf16", mb);
        set_plan(ctx, name, grid, block, 1, 1, 0);
        if (ctx->plan_only) return OXQ_OK;
        if (((uintptr_t)p.blocks & 15) || ((uintptr_t)p.x & 15) || (p.K % 8))
            return fail(OXQ_ERR_UNSUPPORTED, "mxfp4 gemv: blocks and x must be 16-byte aligned");
        switch (mb) {
        case 1: return mxfp4_lds_go<1, RW>(s, grid, p, lds);
        case 2: return mxfp4_lds_go<2, RW>(s, grid, p, lds);
        case 4: return mxfp4_lds_go<4, RW>(s, grid, p, lds);
        default: return mxfp4_lds_go<8, RW>(s, grid, p, lds);
        }
    }
    dim3 grid((unsigned)ceil_div(p.N, 4), grouped ? (unsigned)p.n_experts : 1u), block(256);
    set_plan(ctx, grouped ? "mxfp4_moe_gemv_bf16" : "mxfp4_gemv_bf16", grid, block, 1, 1, 0);
    if (ctx->plan_only) return OXQ_OK;
    if (((uintptr_t)p.blocks & 15) || ((uintptr_t)p.x & 15) || (p.K % 8))
        return fail(OXQ_ERR_UNSUPPORTED, "mxfp4 gemv: blocks and x must be 16-byte aligned");
    const int M = (int)p.M, K = (int)p.K, N = (int)p.N;
    const int64_t rows_hint2 = grouped ? 8 : p.M;
#define OXQ_GO(MBv)                                                                                   \
    hipLaunchKernelGGL((mxfp4_gemv_kernel<MBv>), grid, block, 0, s, (const uint16_t *)p.x, p.blocks,  \
                       p.scales, (const uint16_t *)p.bias, (uint16_t *)p.y, p.expert_offsets,        \
                       p.token_ids, M, K, N)
    if (rows_hint2 <= 1) OXQ_GO(1);
    else if (rows_hint2 <= 2) OXQ_GO(2);
    else if (rows_hint2 <= 4) OXQ_GO(4);
    else OXQ_GO(8);
#undef OXQ_GO
    OXQ_HIP_CHECK(hipGetLastError());
    return OXQ_OK;
}

int launch_mxfp4_dequant(oxq_ctx *ctx, hipStream_t s, const Mxfp4Problem &p, float *out_nk) {
    const size_t nblocks = (size_t)p.N * (p.K >> 5);
    dim3 grid((unsigned)ceil_div((int64_t)nblocks, 256)), block(256);
    set_plan(ctx, "mxfp4_dequant", grid, block, 1, 1, 0);
    if (ctx->plan_only) return OXQ_OK;
    if ((uintptr_t)p.blocks & 15)
        return fail(OXQ_ERR_UNSUPPORTED, "mxfp4 dequant: blocks must be 16-byte aligned");
    hipLaunchKernelGGL(mxfp4_dequant_kernel, grid, block, 0, s, p.blocks, p.scales, out_nk, nblocks);
    OXQ_HIP_CHECK(hipGetLastError());
    return OXQ_OK;
}

}  // namespace oxq
