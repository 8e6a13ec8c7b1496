// Batched W4A16 tile GEMM on the matrix cores (M >= 9 rows).
//
//   y[M, N] = x[M, K] . dequant(W)[K, N],  f32 accumulation, result in x's dtype.
//
// Reference semantics: mpp_gemm.metal:84-266 (staged quant GEMM: the B tile is
// dequantized to the 16-bit activation type, T((q - z) * s), before the matrix
// unit; f32 accumulate).  The B operand built here is bit-identical to the
// dense dequant op's output for the same elements.
//
// AWQ 4-bit mapping onto v_mfma_f32_16x16x32_{f16,bf16}: lane (c = lane % 16,
// kb = lane / 16) reads the packed word of column group c for the 8 rows
// k0 + 8*kb .. +7.  Those 8 words hold, per nibble slot s, the 8 consecutive-k
// values of output column 8*j + order(s): exactly one B fragment per slot, so
// 8 MFMAs per K-step of 32 cover 128 output columns with no cross-lane
// movement; the AWQ interleave is absorbed by the column index of each
// MFMA's result.  Rows are paired with v_perm so one AND-OR produces two
// exact 16-bit integers, then (q - z) * s is a packed add + packed multiply.
//
// A workgroup of 4 waves covers 16*MT rows x 512 columns; K is split across
// workgroups; the slices are summed in index order by a second launch.

#include "oxq_device.hpp"
#include "oxq_internal.hpp"
#include "oxq_mfma.hpp"

#include <cstdlib>

namespace oxq {

template <typename TT, int MT>
__global__ __launch_bounds__(256) void awq4_mfma_kernel(
    const uint16_t *__restrict__ x, const uint32_t *__restrict__ qw,
    const uint32_t *__restrict__ qz, const uint16_t *__restrict__ sc,
    const uint16_t *__restrict__ bias, uint16_t *__restrict__ y, float *__restrict__ ws,
    int M, int K, int N, int gshift, int kslice, int S) {
    typedef MfmaOps<TT> Ops;
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int c = lane & 15, kb = lane >> 4;
    const int PW = N >> 3;
    const int rowbytes = PW * 4;
    const int jw = blockIdx.x * 64 + wave * 16 + c;  // packed word column of this lane
    const bool col_ok = jw < PW;
    const int jws = col_ok ? jw : PW - 1;            // clamp loads, discard results
    const int slice = blockIdx.y;
    const int m0 = blockIdx.z * (16 * MT);
    const int k_begin = slice * kslice;
    const int k_end = min(K, k_begin + kslice);
    const int gsize = 1 << gshift;

    // Raw buffer addressing: lane part in a VGPR offset, row part in a scalar offset.
    const __amdgpu_buffer_rsrc_t rs_w = make_rsrc(qw, (uint32_t)K * (uint32_t)rowbytes);
    const __amdgpu_buffer_rsrc_t rs_x = make_rsrc(x, (uint32_t)M * (uint32_t)K * 2u);
    const __amdgpu_buffer_rsrc_t rs_z = make_rsrc(qz, (uint32_t)(K >> gshift) * (uint32_t)rowbytes);
    const __amdgpu_buffer_rsrc_t rs_s = make_rsrc(sc, (uint32_t)(K >> gshift) * (uint32_t)N * 2u);
    const int voff_w = (kb * 8 * PW + jws) * 4;
    const int voff_z = jws * 4;
    const int voff_s = jws * 16;
    int voff_a[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
        int r = m0 + mt * 16 + c;
        r = r < M ? r : M - 1;  // extra rows are computed and discarded
        voff_a[mt] = (r * K + kb * 8) * 2;
    }
    const NibbleMasks nm = nibble_masks();

    float4_t acc[MT][8];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int s = 0; s < 8; ++s) acc[mt][s] = float4_t{0.f, 0.f, 0.f, 0.f};

    struct Step {
        uint32_t w[8];
        u32x4_t a[MT];
    };
    auto load_step = [&](int k0, Step &st) {
#pragma unroll
        for (int i = 0; i < 8; ++i)
            st.w[i] = __builtin_amdgcn_raw_buffer_load_b32(rs_w, voff_w, (k0 + i) * rowbytes, 0);
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
            st.a[mt] = __builtin_amdgcn_raw_buffer_load_b128(rs_x, voff_a[mt], k0 * 2, 0);
    };

    // group parameters, fetched one group ahead of use
    uint32_t zw_next;
    u32x4_t sv_next;
    auto load_group = [&](int g) {
        zw_next = __builtin_amdgcn_raw_buffer_load_b32(rs_z, voff_z, g * rowbytes, 0);
        sv_next = __builtin_amdgcn_raw_buffer_load_b128(rs_s, voff_s, g * N * 2, 0);
    };
    uint32_t negzb[8], sp[8];
    auto use_group = [&]() {
#pragma unroll
        for (int s = 0; s < 8; ++s) {
            const int col = awq_slot_col(s);
            const uint32_t pr = sv_next[col >> 1];
            const uint32_t sb = (col & 1) ? (pr >> 16) : (pr & 0xFFFFu);
            sp[s] = sb | (sb << 16);
            negzb[s] = Ops::splat(-((float)((zw_next >> (4 * s)) & 0xFu) + TT::bias(s)));
        }
    };
    auto compute = [&](const Step &st) {
        // one fragment (8 consecutive k of one column set) at a time keeps few registers live
        uint32_t tl[4], th[4];
#pragma unroll
        for (int pp = 0; pp < 4; ++pp) {
            tl[pp] = pack_lo16(st.w[2 * pp], st.w[2 * pp + 1]);
            th[pp] = pack_hi16(st.w[2 * pp], st.w[2 * pp + 1]);
        }
#pragma unroll
        for (int s = 0; s < 8; ++s) {
            uint32_t b[4];
#pragma unroll
            for (int pp = 0; pp < 4; ++pp) {
                const uint32_t pr = TT::unpack1(s < 4 ? tl[pp] : th[pp], s & 3, nm);
                b[pp] = Ops::dequant_pair(pr, negzb[s], sp[s]);
            }
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) {
                const uint32_t a[4] = {st.a[mt][0], st.a[mt][1], st.a[mt][2], st.a[mt][3]};
                acc[mt][s] = Ops::mfma(a, b, acc[mt][s]);
            }
        }
    };
    // A K-step of 32 rows never straddles a group (group size is a multiple of 32).
    auto step_group = [&](int k0) {
        if ((k0 & (gsize - 1)) == 0 || k0 == k_begin) {  // wave-uniform
            use_group();
            const int gn = (k0 >> gshift) + 1;
            if ((gn << gshift) < k_end) load_group(gn);
        }
    };

    Step sa, sb;
    if (k_begin < k_end) {
        load_group(k_begin >> gshift);
        load_step(k_begin, sa);
    }
    for (int k0 = k_begin; k0 < k_end; k0 += 64) {
        const bool has_b = k0 + 32 < k_end;
        if (has_b) load_step(k0 + 32, sb);
        step_group(k0);
        compute(sa);
        if (has_b) {
            if (k0 + 64 < k_end) load_step(k0 + 64, sa);
            step_group(k0 + 32);
            compute(sb);
        }
    }

    // D layout: lane (c, rb = lane / 16) holds rows 4*rb + i, column c of each tile.
    const int rb = kb;
    const int nbase = jw * 8;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int m = m0 + mt * 16 + rb * 4 + i;
            if (m < M && col_ok) {
                float v[8];
#pragma unroll
                for (int s = 0; s < 8; ++s) v[awq_slot_col(s)] = acc[mt][s][i];
                if (S == 1) {
                    uint32_t o[4];
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        float lo = v[2 * q], hi = v[2 * q + 1];
                        if (bias) {
                            lo += TT::to_f32(bias[nbase + 2 * q]);
                            hi += TT::to_f32(bias[nbase + 2 * q + 1]);
                        }
                        o[q] = (uint32_t)TT::from_f32(lo) | ((uint32_t)TT::from_f32(hi) << 16);
                    }
                    *(u32x4_t *)(y + (size_t)m * N + nbase) = u32x4_t{o[0], o[1], o[2], o[3]};
                } else {
                    float *dst = ws + ((size_t)slice * M + m) * N + nbase;
                    *(float4_t *)dst = float4_t{v[0], v[1], v[2], v[3]};
                    *(float4_t *)(dst + 4) = float4_t{v[4], v[5], v[6], v[7]};
                }
            }
        }
    }
}

// ---------------------------------------------------------------------------
// Pipelined variant for group sizes >= 128.
//
// One workgroup iteration = a K block of 128 rows (4 MFMA steps).  The
// activation tile of the block is staged in LDS (double buffered, padded rows
// so the 16 lanes of a fragment read hit distinct banks) and shared by the 4
// waves; packed weights are prefetched 4 steps ahead into a register ring, so
// a wave has ~8 KB of weight loads in flight.  With one wave per SIMD (the
// 64-row tile needs 128 accumulator registers) that ring is what hides HBM
// latency.
// ---------------------------------------------------------------------------
template <typename TT, int MT>
__global__ __launch_bounds__(256) void awq4_mfma_pipe_kernel(
    const uint16_t *__restrict__ x, const uint32_t *__restrict__ qw,
    const uint32_t *__restrict__ qz, const uint16_t *__restrict__ sc,
    const uint16_t *__restrict__ bias, uint16_t *__restrict__ y, float *__restrict__ ws,
    int M, int K, int N, int gshift, int kslice, int S) {
    typedef MfmaOps<TT> Ops;
    constexpr int KB = 128;                 // K rows per block
    constexpr int D = KB / 32;              // MFMA steps per block = prefetch depth
    constexpr int ROWS = 16 * MT;
    constexpr int RS = KB * 2 + 16;         // padded LDS row stride in bytes
    constexpr int CHUNKS = ROWS * (KB / 8); // 16-byte chunks per activation block
    constexpr int CPT = (CHUNKS + 255) / 256;
    __shared__ __attribute__((aligned(16))) unsigned char lds_a[2][ROWS * RS];

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int c = lane & 15, kb = lane >> 4;
    const int PW = N >> 3;
    const int rowbytes = PW * 4;
    const int jw = blockIdx.x * 64 + wave * 16 + c;
    const bool col_ok = jw < PW;
    const int jws = col_ok ? jw : PW - 1;
    const int slice = blockIdx.y;
    const int m0 = blockIdx.z * ROWS;
    const int k_begin = slice * kslice;
    const int k_end = min(K, k_begin + kslice);
    const int nblk = (k_end - k_begin) / KB;
    const int gsize = 1 << gshift;

    const __amdgpu_buffer_rsrc_t rs_w = make_rsrc(qw, (uint32_t)K * (uint32_t)rowbytes);
    const __amdgpu_buffer_rsrc_t rs_x = make_rsrc(x, (uint32_t)M * (uint32_t)K * 2u);
    const __amdgpu_buffer_rsrc_t rs_z = make_rsrc(qz, (uint32_t)(K >> gshift) * (uint32_t)rowbytes);
    const __amdgpu_buffer_rsrc_t rs_s = make_rsrc(sc, (uint32_t)(K >> gshift) * (uint32_t)N * 2u);
    const int voff_w = (kb * 8 * PW + jws) * 4;
    const int voff_z = jws * 4;
    const int voff_s = jws * 16;
    const NibbleMasks nm = nibble_masks();

    // staging map: chunk q of this thread -> (row, 8-k chunk) of the activation block
    int a_goff[CPT], a_loff[CPT];
#pragma unroll
    for (int q = 0; q < CPT; ++q) {
        const int idx = threadIdx.x + q * 256;
        const int row = idx / (KB / 8), kc = idx % (KB / 8);
        int r = m0 + row;
        r = r < M ? r : M - 1;
        a_goff[q] = (r * K + kc * 8) * 2;
        a_loff[q] = (idx < CHUNKS) ? row * RS + kc * 16 : -1;
    }
    int a_roff[MT];  // LDS offset of this lane's fragment inside a block, step 0
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) a_roff[mt] = (mt * 16 + c) * RS + kb * 16;

    float4_t acc[MT][8];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int s = 0; s < 8; ++s) acc[mt][s] = float4_t{0.f, 0.f, 0.f, 0.f};

    uint32_t ring[D][8];
    auto load_w = [&](int k0, uint32_t (&w)[8]) {
#pragma unroll
        for (int i = 0; i < 8; ++i)
            w[i] = __builtin_amdgcn_raw_buffer_load_b32(rs_w, voff_w, (k0 + i) * rowbytes, 0);
    };
    u32x4_t areg[CPT];
    auto load_a = [&](int k0) {
#pragma unroll
        for (int q = 0; q < CPT; ++q)
            areg[q] = __builtin_amdgcn_raw_buffer_load_b128(rs_x, a_goff[q], k0 * 2, 0);
    };
    auto store_a = [&](int buf) {
#pragma unroll
        for (int q = 0; q < CPT; ++q)
            if (a_loff[q] >= 0) *(u32x4_t *)(&lds_a[buf][a_loff[q]]) = areg[q];
    };

    uint32_t zw_next;
    u32x4_t sv_next;
    auto load_group = [&](int g) {
        zw_next = __builtin_amdgcn_raw_buffer_load_b32(rs_z, voff_z, g * rowbytes, 0);
        sv_next = __builtin_amdgcn_raw_buffer_load_b128(rs_s, voff_s, g * N * 2, 0);
    };
    uint32_t negzb[8], sp[8];
    auto use_group = [&]() {
#pragma unroll
        for (int s = 0; s < 8; ++s) {
            const int col = awq_slot_col(s);
            const uint32_t pr = sv_next[col >> 1];
            const uint32_t sb = (col & 1) ? (pr >> 16) : (pr & 0xFFFFu);
            sp[s] = sb | (sb << 16);
            negzb[s] = Ops::splat(-((float)((zw_next >> (4 * s)) & 0xFu) + TT::bias(s)));
        }
    };

    if (nblk > 0) {
        load_group(k_begin >> gshift);
        load_a(k_begin);
#pragma unroll
        for (int d = 0; d < D; ++d) load_w(k_begin + d * 32, ring[d]);
        store_a(0);
    }
    __syncthreads();

    for (int blk = 0; blk < nblk; ++blk) {
        const int kblk = k_begin + blk * KB;
        const bool more = blk + 1 < nblk;
        if (more) load_a(kblk + KB);
        if ((kblk & (gsize - 1)) == 0 || blk == 0) {  // wave-uniform: entering a new group
            use_group();
            const int gn = (kblk >> gshift) + 1;
            if ((gn << gshift) < k_end) load_group(gn);
        }
        const unsigned char *abuf = lds_a[blk & 1];
#pragma unroll
        for (int d = 0; d < D; ++d) {
            u32x4_t af[MT];
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) af[mt] = *(const u32x4_t *)(abuf + a_roff[mt] + d * 64);
            uint32_t tl[4], th[4];
#pragma unroll
            for (int pp = 0; pp < 4; ++pp) {
                tl[pp] = pack_lo16(ring[d][2 * pp], ring[d][2 * pp + 1]);
                th[pp] = pack_hi16(ring[d][2 * pp], ring[d][2 * pp + 1]);
            }
            if (more) load_w(kblk + KB + d * 32, ring[d]);  // refill this ring slot
#pragma unroll
            for (int s = 0; s < 8; ++s) {
                uint32_t b[4];
#pragma unroll
                for (int pp = 0; pp < 4; ++pp) {
                    const uint32_t pr = TT::unpack1(s < 4 ? tl[pp] : th[pp], s & 3, nm);
                    b[pp] = Ops::dequant_pair(pr, negzb[s], sp[s]);
                }
#pragma unroll
                for (int mt = 0; mt < MT; ++mt) {
                    const uint32_t a[4] = {af[mt][0], af[mt][1], af[mt][2], af[mt][3]};
                    acc[mt][s] = Ops::mfma(a, b, acc[mt][s]);
                }
            }
        }
        if (more) store_a((blk + 1) & 1);
        __syncthreads();
    }

    const int rb = kb;
    const int nbase = jw * 8;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int m = m0 + mt * 16 + rb * 4 + i;
            if (m < M && col_ok) {
                float v[8];
#pragma unroll
                for (int s = 0; s < 8; ++s) v[awq_slot_col(s)] = acc[mt][s][i];
                if (S == 1) {
                    uint32_t o[4];
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        float lo = v[2 * q], hi = v[2 * q + 1];
                        if (bias) {
                            lo += TT::to_f32(bias[nbase + 2 * q]);
                            hi += TT::to_f32(bias[nbase + 2 * q + 1]);
                        }
                        o[q] = (uint32_t)TT::from_f32(lo) | ((uint32_t)TT::from_f32(hi) << 16);
                    }
                    *(u32x4_t *)(y + (size_t)m * N + nbase) = u32x4_t{o[0], o[1], o[2], o[3]};
                } else {
                    float *dst = ws + ((size_t)slice * M + m) * N + nbase;
                    *(float4_t *)dst = float4_t{v[0], v[1], v[2], v[3]};
                    *(float4_t *)(dst + 4) = float4_t{v[4], v[5], v[6], v[7]};
                }
            }
        }
    }
}

// ---------------------------------------------------------------------------
// K-split-in-workgroup variant: the 4 waves of a workgroup share one
// 16*MT x 128 output tile and each takes a quarter of the workgroup's K range;
// their accumulators are combined through LDS.  Compared with four waves side
// by side this quarters the number of f32 partial tiles that cross workgroups
// (the dominant cost of the 64-row tile), at the price of 64-byte row segments
// per wave.  Workgroup ids are remapped so that the two tiles sharing a
// 128-byte line of every weight row run on the same XCD (shared L2).
// Activations come straight from L2 into a register double buffer; packed
// weights are prefetched 4 steps ahead.
// ---------------------------------------------------------------------------
template <typename TT, int MT>
__global__ __launch_bounds__(256) void awq4_mfma_ksplit_kernel(
    const uint16_t *__restrict__ x, const uint32_t *__restrict__ qw,
    const uint32_t *__restrict__ qz, const uint16_t *__restrict__ sc,
    const uint16_t *__restrict__ bias, uint16_t *__restrict__ y, float *__restrict__ ws,
    int M, int K, int N, int gshift, int kslice, int S, int ctiles) {
    typedef MfmaOps<TT> Ops;
    constexpr int D = 4;  // weight prefetch depth in 32-row steps
    __shared__ __attribute__((aligned(16))) float red[MT * 8 * 64 * 4];

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int c = lane & 15, kb = lane >> 4;
    const int PW = N >> 3;
    const int rowbytes = PW * 4;

    // XCD-aware id remap: ids b and b+8 (same XCD, dispatched together) get adjacent tiles
    const int total = ctiles * S;
    int u = blockIdx.x;
    if (u < (total / 16) * 16) {
        const int xcd = u & 7, q = u >> 3;
        u = (q >> 1) * 16 + xcd * 2 + (q & 1);
    }
    const int tile = u % ctiles, slice = u / ctiles;

    const int jw = tile * 16 + c;
    const bool col_ok = jw < PW;
    const int jws = col_ok ? jw : PW - 1;
    const int m0 = blockIdx.z * (16 * MT);
    const int kq = kslice >> 2;                       // this wave's share of the slice
    const int k_begin = slice * kslice + wave * kq;
    const int k_end = min(K, k_begin + kq);
    const int nsteps = k_end > k_begin ? (k_end - k_begin) >> 5 : 0;
    const int gsize = 1 << gshift;

    const __amdgpu_buffer_rsrc_t rs_w = make_rsrc(qw, (uint32_t)K * (uint32_t)rowbytes);
    const __amdgpu_buffer_rsrc_t rs_x = make_rsrc(x, (uint32_t)M * (uint32_t)K * 2u);
    const __amdgpu_buffer_rsrc_t rs_z = make_rsrc(qz, (uint32_t)(K >> gshift) * (uint32_t)rowbytes);
    const __amdgpu_buffer_rsrc_t rs_s = make_rsrc(sc, (uint32_t)(K >> gshift) * (uint32_t)N * 2u);
    const int voff_w = (kb * 8 * PW + jws) * 4;
    const int voff_z = jws * 4;
    const int voff_s = jws * 16;
    int voff_a[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
        int r = m0 + mt * 16 + c;
        r = r < M ? r : M - 1;
        voff_a[mt] = (r * K + kb * 8) * 2;
    }
    const NibbleMasks nm = nibble_masks();

    float4_t acc[MT][8];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int s = 0; s < 8; ++s) acc[mt][s] = float4_t{0.f, 0.f, 0.f, 0.f};

    uint32_t ring[D][8];
    auto load_w = [&](int k0, uint32_t (&w)[8]) {
#pragma unroll
        for (int i = 0; i < 8; ++i)
            w[i] = __builtin_amdgcn_raw_buffer_load_b32(rs_w, voff_w, (k0 + i) * rowbytes, 0);
    };
    u32x4_t abuf[2][MT];
    auto load_a = [&](int k0, u32x4_t (&a)[MT]) {
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
            a[mt] = __builtin_amdgcn_raw_buffer_load_b128(rs_x, voff_a[mt], k0 * 2, 0);
    };
    uint32_t zw_next;
    u32x4_t sv_next;
    auto load_group = [&](int g) {
        zw_next = __builtin_amdgcn_raw_buffer_load_b32(rs_z, voff_z, g * rowbytes, 0);
        sv_next = __builtin_amdgcn_raw_buffer_load_b128(rs_s, voff_s, g * N * 2, 0);
    };
    uint32_t negzb[8], sp[8];
    auto use_group = [&]() {
#pragma unroll
        for (int s = 0; s < 8; ++s) {
            const int col = awq_slot_col(s);
            const uint32_t pr = sv_next[col >> 1];
            const uint32_t sb = (col & 1) ? (pr >> 16) : (pr & 0xFFFFu);
            sp[s] = sb | (sb << 16);
            negzb[s] = Ops::splat(-((float)((zw_next >> (4 * s)) & 0xFu) + TT::bias(s)));
        }
    };
    auto compute = [&](const uint32_t (&w)[8], const u32x4_t (&a)[MT], uint32_t (&tl)[4], uint32_t (&th)[4]) {
#pragma unroll
        for (int s = 0; s < 8; ++s) {
            uint32_t b[4];
#pragma unroll
            for (int pp = 0; pp < 4; ++pp) {
                const uint32_t pr = TT::unpack1(s < 4 ? tl[pp] : th[pp], s & 3, nm);
                b[pp] = Ops::dequant_pair(pr, negzb[s], sp[s]);
            }
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) {
                const uint32_t av[4] = {a[mt][0], a[mt][1], a[mt][2], a[mt][3]};
                acc[mt][s] = Ops::mfma(av, b, acc[mt][s]);
            }
        }
        (void)w;
    };

    if (nsteps > 0) {
        load_group(k_begin >> gshift);
        load_a(k_begin, abuf[0]);
#pragma unroll
        for (int d = 0; d < D; ++d)
            if (d < nsteps) load_w(k_begin + d * 32, ring[d]);
    }
    // steps are processed in rounds of D so ring slots are compile-time indices
    for (int base = 0; base < nsteps; base += D) {
#pragma unroll
        for (int d = 0; d < D; ++d) {
            const int si = base + d;
            if (si < nsteps) {  // wave-uniform
                const int k0 = k_begin + si * 32;
                if (si + 1 < nsteps) load_a(k0 + 32, abuf[(d + 1) & 1]);
                if ((k0 & (gsize - 1)) == 0 || si == 0) {
                    use_group();
                    const int gn = (k0 >> gshift) + 1;
                    if ((gn << gshift) < k_end) load_group(gn);
                }
                uint32_t tl[4], th[4];
#pragma unroll
                for (int pp = 0; pp < 4; ++pp) {
                    tl[pp] = pack_lo16(ring[d][2 * pp], ring[d][2 * pp + 1]);
                    th[pp] = pack_hi16(ring[d][2 * pp], ring[d][2 * pp + 1]);
                }
                if (si + D < nsteps) load_w(k0 + D * 32, ring[d]);
                compute(ring[d], abuf[d & 1], tl, th);
            }
        }
    }

    // combine the four K quarters: waves 1..3 hand their accumulators to wave 0
    for (int r = 1; r < 4; ++r) {
        if (wave == r) {
#pragma unroll
            for (int mt = 0; mt < MT; ++mt)
#pragma unroll
                for (int s = 0; s < 8; ++s)
                    *(float4_t *)(&red[((mt * 8 + s) * 64 + lane) * 4]) = acc[mt][s];
        }
        __syncthreads();
        if (wave == 0) {
#pragma unroll
            for (int mt = 0; mt < MT; ++mt)
#pragma unroll
                for (int s = 0; s < 8; ++s)
                    acc[mt][s] += *(const float4_t *)(&red[((mt * 8 + s) * 64 + lane) * 4]);
        }
        __syncthreads();
    }
    if (wave != 0) return;

    const int rb = kb;
    const int nbase = jw * 8;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int m = m0 + mt * 16 + rb * 4 + i;
            if (m < M && col_ok) {
                float v[8];
#pragma unroll
                for (int s = 0; s < 8; ++s) v[awq_slot_col(s)] = acc[mt][s][i];
                if (S == 1) {
                    uint32_t o[4];
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        float lo = v[2 * q], hi = v[2 * q + 1];
                        if (bias) {
                            lo += TT::to_f32(bias[nbase + 2 * q]);
                            hi += TT::to_f32(bias[nbase + 2 * q + 1]);
                        }
                        o[q] = (uint32_t)TT::from_f32(lo) | ((uint32_t)TT::from_f32(hi) << 16);
                    }
                    *(u32x4_t *)(y + (size_t)m * N + nbase) = u32x4_t{o[0], o[1], o[2], o[3]};
                } else {
                    float *dst = ws + ((size_t)slice * M + m) * N + nbase;
                    *(float4_t *)dst = float4_t{v[0], v[1], v[2], v[3]};
                    *(float4_t *)(dst + 4) = float4_t{v[4], v[5], v[6], v[7]};
                }
            }
        }
    }
}

template <typename TT>
static int launch_awq4_mfma(oxq_ctx *ctx, hipStream_t s, const Wna16Problem &p) {
    const int M = (int)p.M, K = (int)p.K, N = (int)p.N;
    int mt = M <= 16 ? 1 : (M <= 32 ? 2 : (M <= 48 ? 3 : 4));
    {
        const int mt_env = tune(ctx, OXQ_TUNE_MFMA_MT, 0);
        if (mt_env >= 1 && mt_env <= 4 && mt_env < mt) mt = mt_env;
    }
    const int mtiles = (int)ceil_div(M, 16 * mt);
    const char *dt = TT::DTYPE == 1 ? "f16" : "bf16";
    char name[64];

    // --- K split inside the workgroup: 128-column tiles, slices of whole 512-row units
    const int variant = tune(ctx, OXQ_TUNE_MFMA_VARIANT, 0);  // 0 auto (pipe), 1 ksplit, 2 pipe, 3 simple
    if (variant == 1 && p.group_size >= 32 && K % 512 == 0 &&
        (512 % p.group_size == 0 || p.group_size % 512 == 0)) {
        const int ctiles = (int)ceil_div(N, 128);
        const int units = K / 512;
        int S = tune(ctx, OXQ_TUNE_MFMA_SPLITK, (int)ceil_div(ctx->num_cus, (int64_t)ctiles * mtiles));
        if (S < 1) S = 1;
        if (S > units) S = units;
        int kslice = (int)ceil_div(units, S) * 512;
        S = (int)ceil_div(K, kslice);
        while (S > 1 && (uint64_t)S * M * N * 4 > ctx->workspace_bytes) {
            --S;
            kslice = (int)ceil_div(units, S) * 512;
            S = (int)ceil_div(K, kslice);
        }
        dim3 grid((unsigned)(ctiles * S), 1, (unsigned)mtiles), block(256);
        const uint64_t ws_bytes = S > 1 ? (uint64_t)S * M * N * 4 : 0;
        snprintf(name, sizeof name, "awq4_mfma_ksplit_%s_mt%d", dt, mt);
        set_plan(ctx, name, grid, block, S, 1, ws_bytes);
        if (ctx->plan_only) {
            if (S > 1) add_launch(ctx);
            return OXQ_OK;
        }
#define OXQ_GO(MTv)                                                                                \
    hipLaunchKernelGGL((awq4_mfma_ksplit_kernel<TT, MTv>), grid, block, 0, s, (const uint16_t *)p.x, \
                       p.qweight, p.qzeros, (const uint16_t *)p.scales, (const uint16_t *)p.bias,  \
                       (uint16_t *)p.y, (float *)ctx->workspace, M, K, N, p.group_shift, kslice, S, \
                       ctiles)
        switch (mt) {
        case 1: OXQ_GO(1); break;
        case 2: OXQ_GO(2); break;
        case 3: OXQ_GO(3); break;
        default: OXQ_GO(4); break;
        }
#undef OXQ_GO
        OXQ_HIP_CHECK(hipGetLastError());
        if (S > 1)
            return launch_splitk_reduce(ctx, s, (const float *)ctx->workspace, p.bias, p.y, M, N, S,
                                        p.dtype);
        return OXQ_OK;
    }

    // --- four waves side by side: 512-column tiles
    const int ctiles = (int)ceil_div(N, 512);
    // K slices: whole groups (and whole 32-row MFMA steps), about one workgroup per CU
    const int step = (int)(p.group_size > 32 ? p.group_size : 32);
    const int units = K / step;
    int S = tune(ctx, OXQ_TUNE_MFMA_SPLITK, ctx->num_cus / (mtiles * ctiles));
    if (S < 1) S = 1;
    if (S > units) S = units;
    const int kslice = (int)ceil_div(units, S) * step;
    S = (int)ceil_div(K, kslice);
    // keep the partials inside the workspace
    while (S > 1 && (uint64_t)S * M * N * 4 > ctx->workspace_bytes) --S;
    const int kslice2 = (int)ceil_div(units, S) * step;
    S = (int)ceil_div(K, kslice2);
    dim3 grid((unsigned)ctiles, (unsigned)S, (unsigned)mtiles), block(256);
    const uint64_t ws_bytes = S > 1 ? (uint64_t)S * M * N * 4 : 0;
    const bool pipe = variant != 3 && p.group_size >= 128 && kslice2 % 128 == 0 && K % 128 == 0;
    snprintf(name, sizeof name, "awq4_mfma%s_%s_mt%d", pipe ? "_pipe" : "", dt, mt);
    set_plan(ctx, name, grid, block, S, 1, ws_bytes);
    if (ctx->plan_only) {
        if (S > 1) add_launch(ctx);
        return OXQ_OK;
    }
    if (ws_bytes > ctx->workspace_bytes)
        return fail(OXQ_ERR_WORKSPACE, "w4a16 tile gemm: needs %llu workspace bytes, ctx holds %zu",
                    (unsigned long long)ws_bytes, ctx->workspace_bytes);
#define OXQ_GO(MTv)                                                                              \
    if (pipe)                                                                                    \
        hipLaunchKernelGGL((awq4_mfma_pipe_kernel<TT, MTv>), grid, block, 0, s,                  \
                           (const uint16_t *)p.x, p.qweight, p.qzeros, (const uint16_t *)p.scales, \
                           (const uint16_t *)p.bias, (uint16_t *)p.y, (float *)ctx->workspace, M, K, \
                           N, p.group_shift, kslice2, S);                                        \
    else                                                                                         \
        hipLaunchKernelGGL((awq4_mfma_kernel<TT, MTv>), grid, block, 0, s, (const uint16_t *)p.x, \
                           p.qweight, p.qzeros, (const uint16_t *)p.scales,                      \
                           (const uint16_t *)p.bias, (uint16_t *)p.y, (float *)ctx->workspace, M, K, \
                           N, p.group_shift, kslice2, S)
    switch (mt) {
    case 1: OXQ_GO(1); break;
    case 2: OXQ_GO(2); break;
    case 3: OXQ_GO(3); break;
    default: OXQ_GO(4); break;
    }
#undef OXQ_GO
    OXQ_HIP_CHECK(hipGetLastError());
    if (S > 1)
        return launch_splitk_reduce(ctx, s, (const float *)ctx->workspace, p.bias, p.y, M, N, S, p.dtype);
    return OXQ_OK;
}

bool awq4_mfma_ok(const Wna16Problem &p) {
    if (p.bits != 4 || p.pack_dim != OXQ_PACK_OUT) return false;
    if ((uint64_t)p.K * (uint64_t)(p.N / 2) >= (1ull << 31)) return false;  // 32-bit buffer offsets
    if ((uint64_t)p.M * (uint64_t)p.K * 2 >= (1ull << 31)) return false;
    if ((uint64_t)(p.K / p.group_size) * (uint64_t)p.N * 2 >= (1ull << 31)) return false;
    if (p.K % 32 != 0 || p.N % 8 != 0) return false;
    if (p.group_size % 32 != 0) return false;  // a 32-row MFMA step stays inside one group
    if (((uintptr_t)p.x | (uintptr_t)p.scales | (uintptr_t)p.y) & 15) return false;
    return true;
}

// The tile-major copy built in the ctx workspace, then the resident-layer kernels on it: two launches (the repack
// is one pass over the weights: about 45 us at 5120 x 13824, 4-bit).  A caller that holds the layer should hold a
// PackedQuantLinear, which repacks once.
static bool transient_repack_fits(const oxq_ctx *ctx, const Wna16Problem &p) {
    return p.M > 8 && pk4_eligible(p) && !ctx->plan_only && tune(ctx, OXQ_TUNE_TRANSIENT_REPACK, 1) &&
           !tune(ctx, OXQ_TUNE_FORCE_GENERIC, 0) &&
           ((pk4_weight_bytes(p.K, p.N, p.bits) + 255) & ~(size_t)255) <= ctx->workspace_bytes;
}
static int launch_transient_repack(oxq_ctx *ctx, hipStream_t s, const Wna16Problem &p) {
    Pk4Weights w{(uint32_t *)ctx->workspace, nullptr, p.K, p.N, p.group_shift, p.dtype, p.bits, 0,
                   p.pack_dim == OXQ_PACK_IN ? 32 : 16, 64};
    int rc = launch_pk4_prepack(ctx, s, p, w);
    if (rc != OXQ_OK) return rc;
    Pk4Problem q;
    q.x = p.x;
    q.bias = p.bias;
    q.y = p.y;
    q.M = p.M;
    q.act = 0;
    q.no_split = 1;  // the workspace holds the copy: no room for K slices' partials
    q.w = w;
    rc = launch_pk4_forward(ctx, s, q);
    ctx->plan.launches = 2;
    return rc;
}

int launch_wna16_mfma(oxq_ctx *ctx, hipStream_t s, const Wna16Problem &p) {
    // Prefill sizes: the resident layout's kernels (x shared in LDS by eight strips, or two with K split inside
    // the workgroup) run at two to six times the rate of the kernels on the checkpoint layout - 4096 x 14336 at
    // 2048 rows: 197 (f16) / 216 (bf16) us against 377 / 1313 - which pays for the repack (36 us on that layer) from
    // a few hundred rows on in f16 (the checkpoint-layout kernel does 0.19 us a row there) and from under a
    // hundred in bf16 (0.64 us a row): 2048 rows 377 -> 232 and 1313 -> 252 us with the repack included.
    // The GPTQ kernel on the checkpoint layout holds 0.6 PFLOP/s in both types: the repack pays from 640 rows too
    // (5120 x 13824 at 2048 rows: 430 / 478 -> 269 / 289 us).
    const bool awq = awq4_mfma_ok(p), gptq = !awq && gptq_tile_ok(p) && tune(ctx, OXQ_TUNE_GPTQ_TILE, 1) != 2;
    const int64_t repack_from = awq && p.dtype != OXQ_F16 ? 80 : 640;
    if (p.M >= repack_from && (awq || gptq) && transient_repack_fits(ctx, p)) return launch_transient_repack(ctx, s, p);
    if (awq4_mfma_ok(p) && !tune(ctx, OXQ_TUNE_FORCE_GENERIC, 0))
        return p.dtype == OXQ_F16 ? launch_awq4_mfma<F16Traits>(ctx, s, p)
                                  : launch_awq4_mfma<BF16Traits>(ctx, s, p);
    if (gptq_tile_ok(p) && tune(ctx, OXQ_TUNE_GPTQ_TILE, 1) && !tune(ctx, OXQ_TUNE_FORCE_GENERIC, 0))
        return launch_gptq_tile(ctx, s, p);
    // Layouts without a tile kernel of their own on the checkpoint layout (8-bit AWQ, unaligned GPTQ): when the
    // tile-major copy fits the ctx workspace, build it there and run the resident-layer kernel on it: one launch
    // more instead of one GEMV pass over the weights per 8 rows (35 - 45 us each): ahead from m = 9.
    if (transient_repack_fits(ctx, p)) return launch_transient_repack(ctx, s, p);
    // Otherwise (unaligned shapes, copies larger than the workspace): the GEMV kernel over chunks of 8
    // rows, as the reference does below its tile-GEMM threshold (linear.rs:457-480).
    uint32_t launches = 0;
    const size_t eb = 2;
    for (int64_t m0 = 0; m0 < p.M; m0 += 8) {
        Wna16Problem c = p;
        c.M = (p.M - m0) < 8 ? (p.M - m0) : 8;
        c.x = (const uint8_t *)p.x + (size_t)m0 * p.K * eb;
        c.y = (uint8_t *)p.y + (size_t)m0 * p.N * eb;
        int rc = launch_wna16_gemv(ctx, s, c);
        if (rc != OXQ_OK) return rc;
        ++launches;
    }
    ctx->plan.launches = launches;
    return OXQ_OK;
}

}  // namespace oxq
