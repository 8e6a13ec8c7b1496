// Pieces of the resident-layer kernels that more than one source file uses: the bit-exact tile
// dequant of a pair of weights, the block geometry of the 64-column layout (described in pk4.hip)
// and the epilogue in which a workgroup's waves add their partial tiles in wave order.
#pragma once

#include "oxq_device.hpp"
#include "oxq_internal.hpp"
#include "oxq_mfma.hpp"

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

// ---- shared by the prefill kernels (rows x eight waves of 64 columns a workgroup, x through LDS) ----
typedef __attribute__((address_space(3))) void *pk4g_lds_ptr_t;
// 16 bytes a lane from global memory into LDS at lds + 16 lane.  Kept out of the kernel template: the host pass
// rejects the 16-byte form where it instantiates a template, and then drops the kernel's stub without a word.
__device__ __forceinline__ void pk4g_load_lds16(__amdgpu_buffer_rsrc_t rs, unsigned char *lds, int voff, int soff) {
    __builtin_amdgcn_raw_ptr_buffer_load_lds(rs, (pk4g_lds_ptr_t)lds, 16, voff, soff, 0, 0);
}
template <int N> __device__ __forceinline__ void pk4g_wait_vmcnt() {
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}

// Workgroup -> (row tile, strip group).  Bands of 8 row tiles are cut into squares of 8 row tiles x 8 strip groups,
// 64 neighbouring workgroups each (neighbour i runs on XCD i % 8: a row tile stays on one XCD); the last RT % 8
// row tiles are numbered row tile first, so that no XCD is handed only idle workgroups.
__device__ __forceinline__ void pk4g_tile_of(int id, int RT, int NG, int &rt, int &g) {
    const int full = (RT >> 3) * ((NG + 7) >> 3) * 64, tail = RT & 7;
    if (id < full) {
        const int sq = id >> 6, within = id & 63, bands = RT >> 3;
        rt = (sq % bands) * 8 + (within & 7), g = (sq / bands) * 8 + (within >> 3);
    } else {
        rt = (RT & ~7) + (id - full) % tail, g = (id - full) / tail;
    }
}

// bf16 has no packed 16-bit arithmetic: a weight goes nibble -> f32 -> fma -> (a pair at a time) bf16.  Masked in
// place, a byte of the word holds q (low nibbles) or 16 q (high nibbles), which v_cvt_f32_ubyteN widens in one
// instruction; the high nibbles' fma takes s / 16.  (q - z) s is exact in f32 either way: the same bits as
// Pk4T<BF16Traits>::deq, with a sixth fewer instructions.
struct Pk4gBf16 {
    float s, s16, c;  // scale, scale / 16, -z * scale
    __device__ __forceinline__ void set(float scale, float minus_z) { s = scale, s16 = scale * 0.0625f, c = minus_z * scale; }
    // the pair in bytes B and B + 2 of v; HIGH: v holds high nibbles
    template <int B, bool HIGH> __device__ __forceinline__ uint32_t pair(uint32_t v) const {
        const float lo = (float)((v >> (8 * B)) & 0xFFu), hi = (float)((v >> (8 * B + 16)) & 0xFFu);
        const float m = HIGH ? s16 : s;
        return __builtin_bit_cast(uint32_t, __builtin_convertvector(float2_t{__builtin_fmaf(lo, m, c), __builtin_fmaf(hi, m, c)}, bf16x2_t));
    }
};
__device__ __forceinline__ void pk4g_nibbles(uint32_t w, uint32_t &lo, uint32_t &hi) {
    lo = w & 0x0F0F0F0Fu, hi = w & 0xF0F0F0F0u;
    asm volatile("" : "+v"(lo), "+v"(hi));  // keep the masks here: folded into the byte extracts they cost one each
}

constexpr int PK4N_BW = 272;  // 16-column strips: words of one block, 256 of weights and 16 of pairs

// The constants of one column and block from its pair word {-z, s}; deq() = T((q - z) * s) of a row pair.
template <typename TT> struct Pk4N;
template <> struct Pk4N<F16Traits> {
    uint32_t ce, co, sp;  // -(1024 + z), -(64 + z), s, each in both halves
    __device__ __forceinline__ void prep(uint32_t zw) {
        const uint32_t nz = perm_b32(zw, zw, 0x01000100u);
        typedef _Float16 h2 __attribute__((ext_vector_type(2)));
        ce = __builtin_bit_cast(uint32_t, __builtin_bit_cast(h2, nz) + __builtin_bit_cast(h2, 0xE400E400u));
        co = __builtin_bit_cast(uint32_t, __builtin_bit_cast(h2, nz) + __builtin_bit_cast(h2, 0xD400D400u));
        sp = perm_b32(zw, zw, 0x03020302u);
    }
    // the odd pairs' constant from the even pairs': -(1024 + z) + 960 (exact); for kernels short of registers
    __device__ __forceinline__ void odd_from_even() {
        typedef _Float16 h2 __attribute__((ext_vector_type(2)));
        uint32_t e = ce;
        asm volatile("" : "+v"(e));
        co = __builtin_bit_cast(uint32_t, __builtin_bit_cast(h2, e) + __builtin_bit_cast(h2, 0x63806380u));
    }
    __device__ __forceinline__ uint32_t deq(uint32_t p, int pp) const {
        return MfmaOps<F16Traits>::dequant_pair(p, (pp & 1) ? co : ce, sp);
    }
    // (bias + q) - (bias + z): the exact integers q - z as a pair of f16
    __device__ __forceinline__ uint32_t minus_zero(uint32_t p, int pp) const {
        typedef _Float16 h2 __attribute__((ext_vector_type(2)));
        return __builtin_bit_cast(uint32_t, __builtin_bit_cast(h2, p) + __builtin_bit_cast(h2, (pp & 1) ? co : ce));
    }
};
template <> struct Pk4N<BF16Traits> {
    uint32_t c0, c1;
    __device__ __forceinline__ void prep(uint32_t zw) {
        const float sf = __builtin_bit_cast(float, zw & 0xFFFF0000u);
        const float nz = __builtin_bit_cast(float, zw << 16);
        c0 = __builtin_bit_cast(uint32_t, sf);
        c1 = __builtin_bit_cast(uint32_t, (nz - 128.0f) * sf);
    }
    __device__ __forceinline__ uint32_t deq(uint32_t p, int) const { return Pk4T<BF16Traits>::deq(p, c0, c1); }
    __device__ __forceinline__ uint32_t minus_zero(uint32_t p, int) const { return p; }  // f16 only
    __device__ __forceinline__ void odd_from_even() {}
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

// words of one block: weights, then the 64 words of zero/scale pairs
__host__ __device__ constexpr int pk4_block_words(int bits) { return 1024 * (bits / 4) + 64; }

// The 8 waves' partial 16*MT x 64 tiles meet in LDS and are added in wave order; then either the
// fused gate|up activation, the K slice's f32 partial, or the result in the layer dtype.
template <typename TT, int MT, int NW = 8>
__device__ __forceinline__ void pk4_epilogue(const float4_t (&acc)[MT][4], const uint16_t *__restrict__ bias,
                                             uint16_t *__restrict__ y, float *__restrict__ ws, int M, int N, int j,
                                             int m0, int act, int wave, int lane) {
    constexpr int NT = NW * 64, ROWS = 16 * MT;
    extern __shared__ __attribute__((aligned(16))) unsigned char pk4_lds[];
    // each wave into its own slot, float4 = the lane's four columns of one row
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

// The same sum for a plain layer (no fused activation, one K slice), in the accumulator's own lane
// layout: wave w' adds the 16 * MT / NW (row tile, row-in-quad) planes it owns over the NW slots in
// wave order (the same order and so the same bits as pk4_epilogue), every LDS access a lane-linear
// 16-byte one (no bank conflicts; in pk4_epilogue's row-major read two rows of a 16-lane group share
// their banks).  Lane (ni, kb) ends up with row 16 mt + 4 kb + e, columns 4 ni .. 4 ni + 3: 8 bytes of y.
// ws != nullptr: this workgroup is one K slice of several; its f32 partial tile goes to ws[M][N] (the slice's
// plane) and a second kernel adds the planes in slice order and applies the bias.
template <typename TT, int MT, int NW = 8>
__device__ __forceinline__ void pk4_epilogue_lanes(const float4_t (&acc)[MT][4], const uint16_t *__restrict__ bias,
                                                   uint16_t *__restrict__ y, int M, int N, int j, int m0, int wave,
                                                   int lane, float *__restrict__ ws = nullptr) {
    static_assert((4 * MT) % NW == 0 || NW % (4 * MT) == 0, "planes divide over the waves");
    extern __shared__ __attribute__((aligned(16))) unsigned char pk4_lds[];
    float4_t *red = (float4_t *)pk4_lds;  // [NW][MT][4 e][64 lanes]
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int e = 0; e < 4; ++e)
            red[((wave * MT + mt) * 4 + e) * 64 + lane] = float4_t{acc[mt][0][e], acc[mt][1][e], acc[mt][2][e], acc[mt][3][e]};
    __syncthreads();
    constexpr int PLANES = 4 * MT;
    constexpr int PER = PLANES >= NW ? PLANES / NW : 1;
    if (PLANES < NW && wave >= PLANES) return;
    const int ni = lane & 15, kb = lane >> 4;
    float4_t bv = float4_t{0.f, 0.f, 0.f, 0.f};
    if (bias) {
        const uint2 b = *(const uint2 *)(bias + 64 * j + 4 * ni);
        bv = float4_t{TT::to_f32((uint16_t)(b.x & 0xFFFFu)), TT::to_f32((uint16_t)(b.x >> 16)),
                      TT::to_f32((uint16_t)(b.y & 0xFFFFu)), TT::to_f32((uint16_t)(b.y >> 16))};
    }
#pragma unroll
    for (int i = 0; i < PER; ++i) {
        const int c = wave * PER + i, mt = c >> 2, e = c & 3;
        float4_t v = float4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int s = 0; s < NW; ++s) v += red[((s * MT + mt) * 4 + e) * 64 + lane];
        const int row = m0 + 16 * mt + 4 * kb + e;
        if (row < M && ws) {
            *(float4_t *)(ws + (size_t)row * N + 64 * j + 4 * ni) = v;
        } else if (row < M) {
            if (bias) v += bv;
            const uint2 o = uint2{(uint32_t)TT::from_f32(v[0]) | ((uint32_t)TT::from_f32(v[1]) << 16),
                                  (uint32_t)TT::from_f32(v[2]) | ((uint32_t)TT::from_f32(v[3]) << 16)};
            *(uint2 *)(y + (size_t)row * N + 64 * j + 4 * ni) = o;
        }
    }
}

// Strips of 16 columns (the narrow form of pk4.hip, the GGUF matrix-core kernels): the waves' partial tiles meet
// in LDS as in the wide form; a thread then owns (row, column ni of every strip of the workgroup) and adds the
// waves in order.
template <typename TT, int MT, int NS, int NW>
__device__ __forceinline__ void pk4n_epilogue(const float4_t (&acc)[MT][NS], const uint16_t *__restrict__ bias,
                                              uint16_t *__restrict__ y, float *__restrict__ ws, int M, int N, int j,
                                              int m0, int wave, int lane) {
    constexpr int NT = NW * 64, ROWS = 16 * MT;
    extern __shared__ __attribute__((aligned(16))) unsigned char pk4_lds[];
    // every wave into its own activation slot (other waves may still be reading theirs): [MT][4 e][64 lanes][NS]
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            float *dst = (float *)(pk4_lds + (size_t)wave * MT * 4096) + ((mt * 4 + e) * 64 + lane) * NS;
            if constexpr (NS == 4) *(float4_t *)dst = float4_t{acc[mt][0][e], acc[mt][1][e], acc[mt][2][e], acc[mt][3][e]};
            else dst[0] = acc[mt][0][e];
        }
    __syncthreads();
    for (int t = threadIdx.x; t < ROWS * 16; t += NT) {
        const int ml = t >> 4, ni = t & 15;
        if (m0 + ml >= M) continue;
        const int mt = ml >> 4, r = ml & 15, kb = r >> 2, e = r & 3;
        float v[NS];
#pragma unroll
        for (int f = 0; f < NS; ++f) v[f] = 0.f;
#pragma unroll
        for (int s = 0; s < NW; ++s) {
            const float *src = (const float *)(pk4_lds + (size_t)s * MT * 4096) + ((mt * 4 + e) * 64 + kb * 16 + ni) * NS;
            if constexpr (NS == 4) {
                const float4_t q = *(const float4_t *)src;
                v[0] += q[0], v[1] += q[1], v[2] += q[2], v[3] += q[3];
            } else {
                v[0] += src[0];
            }
        }
#pragma unroll
        for (int f = 0; f < NS; ++f) {
            const int n = 16 * (NS * j + f) + ni;
            if (gridDim.y > 1) {  // this K slice's f32 partial; a second kernel adds the slices in order
                ws[((size_t)blockIdx.y * M + (m0 + ml)) * N + n] = v[f];
            } else {
                float o = v[f];
                if (bias) o += TT::to_f32(bias[n]);
                y[(size_t)(m0 + ml) * N + n] = TT::from_f32(o);
            }
        }
    }
}

}  // namespace oxq
