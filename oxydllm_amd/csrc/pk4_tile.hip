// Resident 4-bit layers in 64-column strips (layout: pk4.hip), 49 - 64 rows of x: the tile GEMM of
// the reference's staged quant GEMM range (mpp_gemm.metal:84-266, metal_ops.rs:2599-2797) as one
// straight-line kernel per K length.
//
// Same decomposition as pk4_mfma_kernel - one workgroup of 8 waves per strip, the waves split K in
// contiguous runs of NBLK blocks and add their 64 x 64 partial tiles in LDS in wave order - and the same
// arithmetic (B = T((q - z) * s), bit-identical to the dense dequant, f32 accumulation), so results
// are bit-identical to that kernel's.  What differs is how the operands travel:
//
//  * Weights: a wave requests its whole share (NBLK blocks of 4 KB and their zero/scale pairs) before
//    it waits for anything.  With a ring one block deep the launch lasted as long as a wave's chain of
//    request -> arrive -> multiply rounds; requested up front the HBM latency is paid once.
//  * Activations go from global memory straight into LDS (buffer loads with the LDS bit: no trip through
//    vector registers, no ds_write), half a block (64 rows x 64 elements of K = 8 KB) per stage, two
//    stages per wave.  A lane's 16 bytes land at LDS position stage + 16 * lane whatever it fetched,
//    so the bank swizzle sits on the global side: lane (row r = l / 8, position p = l % 8) of load q
//    fetches chunk p ^ ((r' >> 1) & 7) of row r' = 8 q + r, and the fragment read of (row, chunk c)
//    goes to position c ^ ((row >> 1) & 7).  Loads are whole 128-byte lines, reads conflict-free.
//  * The registers this frees (64 for a block of x, 16 of ring) hold the up-front weights.
//
// The compiler does not order LDS reads against these loads (it emits neither the vmcnt wait in front of a
// fragment read nor the lgkmcnt wait in front of a load that overwrites a stage), so every such wait
// is written out below; the counts are exact because the code has no loop and no conditional request.

#include "pk4_common.hpp"

namespace oxq {

template <int N> __device__ __forceinline__ void wait_vmcnt() {
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}
__device__ __forceinline__ void wait_lds_reads() { asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); }

typedef __attribute__((address_space(3))) void *lds_ptr_t;

template <typename TT, int NBLK>
__global__ __launch_bounds__(512) void pk4_tile64_kernel(const uint16_t *__restrict__ x,
                                                         const uint32_t *__restrict__ pw,
                                                         const uint16_t *__restrict__ bias,
                                                         uint16_t *__restrict__ y, float *__restrict__ ws, int M,
                                                         int K, int N, int act) {
    typedef MfmaOps<TT> Ops;
    constexpr int MT = 4, NSTG = 2 * NBLK;
    constexpr int BB = pk4_block_words(4) * 4;  // 4352 bytes a block
    constexpr int STAGE = 8192, SLOT = 2 * STAGE;
    extern __shared__ __attribute__((aligned(16))) unsigned char pk4_lds[];

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int ni = lane & 15, kb = lane >> 4;
    const int j = blockIdx.x;
    const int NB = K >> 7;           // == 8 * NBLK (launcher)
    const int cb0 = wave * NBLK;
    unsigned char *slot = pk4_lds + wave * SLOT;

    const __amdgpu_buffer_rsrc_t rs_w = make_rsrc(pw + (size_t)j * NB * (BB / 4), (uint32_t)NB * (uint32_t)BB);
    const __amdgpu_buffer_rsrc_t rs_x = make_rsrc(x, (uint32_t)M * (uint32_t)K * 2u);
    const int voff_w = lane * 16;
    const int voff_z = 4096 + (ni * 4 + kb) * 4;
    // x load q of a stage: rows 8q .. 8q+7; the lane's row carries the range check (a row past M lies
    // beyond the descriptor: zeros, and zeros are what the LDS receives)
    int xo[8];
#pragma unroll
    for (int q = 0; q < 8; ++q) {
        const int row = 8 * q + (lane >> 3);
        const int chunk = (lane & 7) ^ ((row >> 1) & 7);
        xo[q] = row * K * 2 + chunk * 16;
    }
    // fragment read (row tile mt, step t = 2h + u): row 16 mt + ni, chunk 2 kb + u of the stage
    int a_rd[2];
#pragma unroll
    for (int u = 0; u < 2; ++u) a_rd[u] = ni * 128 + ((((2 * kb + u) ^ (ni >> 1)) & 7) << 4);
    const NibbleMasks nm = nibble_masks();

    auto dma = [&](int s) {  // stage s = half (s & 1) of block cb0 + s / 2 -> LDS stage s & 1
        const int so = (cb0 + (s >> 1)) * 256 + (s & 1) * 128;
#pragma unroll
        for (int q = 0; q < 8; ++q)
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rs_x, (lds_ptr_t)(slot + (s & 1) * STAGE + q * 1024), 16, xo[q], so, 0, 0);
    };
    u32x4_t wv[NBLK][4];
    uint32_t zv[NBLK];
    auto load_w = [&](int b) {
#pragma unroll
        for (int st = 0; st < 4; ++st)
            wv[b][st] = __builtin_amdgcn_raw_buffer_load_b128(rs_w, voff_w, (cb0 + b) * BB + st * 1024, 2);
        zv[b] = __builtin_amdgcn_raw_buffer_load_b32(rs_w, voff_z, (cb0 + b) * BB, 2);
    };
    auto frags = [&](int s, int u, uint32_t (&a)[MT][4]) {
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            const u32x4_t av = *(const u32x4_t *)(slot + (s & 1) * STAGE + mt * 2048 + a_rd[u]);
            a[mt][0] = av[0], a[mt][1] = av[1], a[mt][2] = av[2], a[mt][3] = av[3];
        }
    };

    // requests, in the order of use; 5 loads a block of weights, 8 a stage of x
    dma(0);
    load_w(0);
    __builtin_amdgcn_sched_barrier(0);  // the requests stay in this order (the wait counts below rely on it)
    dma(1);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int b = 1; b < NBLK; ++b) {
        load_w(b);
        __builtin_amdgcn_sched_barrier(0);
    }

    float4_t acc[MT][4];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int f = 0; f < 4; ++f) acc[mt][f] = float4_t{0.f, 0.f, 0.f, 0.f};
    uint32_t negzb[4], sp[4];

    auto multiply = [&](int b, int t, const uint32_t (&a)[MT][4]) {
        const u32x4_t w = wv[b][t];
        const uint32_t wp[4] = {w[0], w[1], w[2], w[3]};
#pragma unroll
        for (int f = 0; f < 4; ++f) {
            uint32_t bq[4];
#pragma unroll
            for (int pp = 0; pp < 4; ++pp) bq[pp] = Pk4T<TT>::deq(TT::unpack1(wp[pp], f, nm), negzb[f], sp[f]);
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) acc[mt][f] = Ops::mfma(a[mt], bq, acc[mt][f]);
        }
    };
    auto pairs = [&](int b) {
        const auto p16 = __builtin_amdgcn_permlane16_swap(zv[b], zv[b], false, false);
        const uint32_t even = p16[0], odd = p16[1];
        const auto pe = __builtin_amdgcn_permlane32_swap(even, even, false, false);
        const auto po = __builtin_amdgcn_permlane32_swap(odd, odd, false, false);
        const uint32_t zq[4] = {pe[0], po[0], pe[1], po[1]};
#pragma unroll
        for (int f = 0; f < 4; ++f) Pk4T<TT>::prep(zq[f], negzb[f], sp[f]);
    };

    // Two fragment sets: the next step's fragments are read while this step multiplies.
    // Loads younger than stage 0's: 5 + 8 + 5 (NBLK - 1).
    uint32_t a0[MT][4], a1[MT][4];
    wait_vmcnt<5 + 8 + 5 * (NBLK - 1)>();
    frags(0, 0, a0);
#pragma unroll
    for (int s = 0; s < NSTG; ++s) {
        const int b = s >> 1, h = s & 1;
        if (h == 0) pairs(b);
        frags(s, 1, a1);
        multiply(b, 2 * h, a0);
        // stage s is read: its slot takes stage s + 2
        wait_lds_reads();
        if (s + 2 < NSTG) dma(s + 2);
        if (s + 1 < NSTG) {
            // loads younger than stage s + 1's: the 8 just issued (if any); for s = 0 also the later blocks' weights
            if (s == 0) wait_vmcnt<5 * (NBLK - 1) + 8>();
            else if (s + 2 < NSTG) wait_vmcnt<8>();
            else wait_vmcnt<0>();
            frags(s + 1, 0, a0);
        }
        multiply(b, 2 * h + 1, a1);
    }
    // every x load has been waited for: the slots are free for the partial tiles
    if (!act) pk4_epilogue_lanes<TT, MT>(acc, bias, y, M, N, j, 0, wave, lane);
    else pk4_epilogue<TT, MT>(acc, bias, y, ws, M, N, j, 0, act, wave, lane);
}

template <typename TT, int NBLK>
static int pk4_tile64_go(hipStream_t s, dim3 grid, const Pk4Problem &p) {
    const size_t lds = (size_t)8 * 16384;
    static LdsGrant lds_grant;
    OXQ_HIP_CHECK(lds_grant.ensure((const void *)pk4_tile64_kernel<TT, NBLK>, lds));
    hipLaunchKernelGGL((pk4_tile64_kernel<TT, NBLK>), grid, dim3(512), lds, s, (const uint16_t *)p.x, p.w.pw,
                       (const uint16_t *)p.bias, (uint16_t *)p.y, (float *)p.ws, (int)p.M, (int)p.w.K, (int)p.w.N,
                       p.act);
    OXQ_HIP_CHECK(hipGetLastError());
    return OXQ_OK;
}

// Shapes this file has a kernel for: 4-bit, 64-column strips, one K slice of 8 * NBLK blocks, 49 - 64 rows.
bool pk4_tile64_takes(const Pk4Problem &p, int ks) {
    if (p.w.bits != 4 || p.w.strip == 16 || ks != 1 || p.M <= 48 || p.M > 64) return false;
    const int64_t NB = p.w.K / 128;
    return NB == 32 || NB == 40;
}

int launch_pk4_tile64(oxq_ctx *ctx, hipStream_t s, const Pk4Problem &p) {
    (void)ctx;
    const int NB = (int)(p.w.K / 128);
    dim3 grid((unsigned)(p.w.N / 64));
    const bool f16 = p.w.dtype == OXQ_F16;
    if (NB == 32) return f16 ? pk4_tile64_go<F16Traits, 4>(s, grid, p) : pk4_tile64_go<BF16Traits, 4>(s, grid, p);
    if (NB == 40) return f16 ? pk4_tile64_go<F16Traits, 5>(s, grid, p) : pk4_tile64_go<BF16Traits, 5>(s, grid, p);
    return fail(OXQ_ERR_UNSUPPORTED, "pk4_tile64: no kernel for K = %lld", (long long)p.w.K);
}

}  // namespace oxq
