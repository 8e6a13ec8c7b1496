// A measurement aid, not part of the reference's interface: a plain streaming read of a device
// buffer with the launch shape of the resident-layer kernel (512-thread workgroups, each reading one
// contiguous span with 16-byte loads, eight in flight per lane).  What this kernel takes for a given
// byte count, launch included, is what the memory system gives a read-once kernel with no arithmetic
// at all; the GEMV kernels' times are set beside it.
#include "oxq_device.hpp"
#include "oxq_internal.hpp"

namespace oxq {

template <int POLICY>
__global__ __launch_bounds__(512) void calib_read_kernel(const uint8_t *__restrict__ src, uint32_t *__restrict__ out,
                                                         uint32_t span) {
    // span: bytes per workgroup, a multiple of 8 KiB (512 lanes x 16 bytes); up to 8 loads a lane in flight
    // (loads past the span get an offset beyond the descriptor: no memory access)
    const __amdgpu_buffer_rsrc_t rs = make_rsrc(src + (size_t)blockIdx.x * span, span);
    const int voff = threadIdx.x * 16;
    u32x4_t acc = {0u, 0u, 0u, 0u};
    for (uint32_t base = 0; base < span; base += 65536u) {
        u32x4_t v[8];
#pragma unroll
        for (int q = 0; q < 8; ++q)
            v[q] = __builtin_amdgcn_raw_buffer_load_b128(rs, base + q * 8192u < span ? voff : 0x7FFFFF00, (int)(base + q * 8192u), POLICY);
#pragma unroll
        for (int q = 0; q < 8; ++q) acc ^= v[q];
    }
    const uint32_t r = acc[0] ^ acc[1] ^ acc[2] ^ acc[3];
    // one word per workgroup keeps the loads alive; the value itself is an xor checksum of the span
    uint32_t w = wave_all_reduce(r, [](uint32_t a, uint32_t b) { return a ^ b; });
    __shared__ uint32_t part[8];
    if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = w;
    __syncthreads();
    if (threadIdx.x == 0) {
        uint32_t t = 0;
#pragma unroll
        for (int q = 0; q < 8; ++q) t ^= part[q];
        out[blockIdx.x] = t;
    }
}

// Every lane requests its whole share (NL loads of 16 bytes, a wave load apart) before it waits: the
// order in which the straight-line matmul kernels request their weights.
template <int POLICY, int NL, int NW>
__global__ __launch_bounds__(NW * 64) void calib_upfront_kernel(const uint8_t *__restrict__ src, uint32_t *__restrict__ out,
                                                              uint32_t span) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const __amdgpu_buffer_rsrc_t rs = make_rsrc(src + (size_t)blockIdx.x * span, span);
    u32x4_t v[NL];
#pragma unroll
    for (int q = 0; q < NL; ++q)
        v[q] = __builtin_amdgcn_raw_buffer_load_b128(rs, lane * 16, (wave * NL + q) * 1024, POLICY);
    u32x4_t acc = {0u, 0u, 0u, 0u};
#pragma unroll
    for (int q = 0; q < NL; ++q) acc ^= v[q];
    const uint32_t r = acc[0] ^ acc[1] ^ acc[2] ^ acc[3];
    uint32_t w = wave_all_reduce(r, [](uint32_t a, uint32_t b) { return a ^ b; });
    __shared__ uint32_t part[NW];
    if (lane == 0) part[wave] = w;
    __syncthreads();
    if (threadIdx.x == 0) {
        uint32_t t = 0;
#pragma unroll
        for (int q = 0; q < NW; ++q) t ^= part[q];
        out[blockIdx.x] = t;
    }
}

template <int NW>
__global__ __launch_bounds__(NW * 64) void empty_kernel(uint32_t *out) {
    if (out != nullptr && threadIdx.x == 0xFFFFu) out[0] = 1u;  // never true: nothing is read or written
}

int launch_empty(oxq_ctx *ctx, hipStream_t s, int workgroups, int threads, int lds_bytes) {
    dim3 grid((unsigned)workgroups), block((unsigned)threads);
    set_plan(ctx, "empty", grid, block, 1, 1, 0);
    if (ctx->plan_only) return OXQ_OK;
    static LdsGrant g8, g16;
    if (threads <= 512) {
        OXQ_HIP_CHECK(g8.ensure((const void *)empty_kernel<8>, (size_t)lds_bytes));
        hipLaunchKernelGGL(empty_kernel<8>, grid, block, (size_t)lds_bytes, s, (uint32_t *)nullptr);
    } else {
        OXQ_HIP_CHECK(g16.ensure((const void *)empty_kernel<16>, (size_t)lds_bytes));
        hipLaunchKernelGGL(empty_kernel<16>, grid, block, (size_t)lds_bytes, s, (uint32_t *)nullptr);
    }
    OXQ_HIP_CHECK(hipGetLastError());
    return OXQ_OK;
}

// A launch whose workgroups meet at one grid barrier: thread 0 of every workgroup takes a ticket from a
// device-scope counter and waits until the counter has reached the end of its ticket's round (the counter
// is never reset: round r ends at (r + 1) * workgroups, so replays need no clearing).  The wait is bounded:
// after `spin_limit` polls a workgroup gives up, raises the error word and leaves, so every wave exits
// whatever happens.  The caller must launch no more workgroups than are resident at once.
template <int NW>
__global__ __launch_bounds__(NW * 64) void grid_barrier_kernel(unsigned *counter, unsigned *err, unsigned workgroups,
                                                               unsigned spin_limit) {
    if (threadIdx.x == 0) {
        const unsigned t = __hip_atomic_fetch_add(counter, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        const unsigned target = (t / workgroups + 1u) * workgroups;
        unsigned polls = 0;
        while ((int)(__hip_atomic_load(counter, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) - target) < 0) {
            if (++polls > spin_limit) {
                __hip_atomic_store(err, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                break;
            }
            __builtin_amdgcn_s_sleep(1);
        }
    }
    __syncthreads();
}

int launch_grid_barrier(oxq_ctx *ctx, hipStream_t s, int workgroups, int threads, unsigned *counter, unsigned *err,
                        unsigned spin_limit) {
    dim3 grid((unsigned)workgroups), block((unsigned)threads);
    set_plan(ctx, "grid_barrier", grid, block, 1, 1, 0);
    if (ctx->plan_only) return OXQ_OK;
    if (threads <= 512)
        hipLaunchKernelGGL(grid_barrier_kernel<8>, grid, block, 0, s, counter, err, (unsigned)workgroups, spin_limit);
    else
        hipLaunchKernelGGL(grid_barrier_kernel<16>, grid, block, 0, s, counter, err, (unsigned)workgroups, spin_limit);
    OXQ_HIP_CHECK(hipGetLastError());
    return OXQ_OK;
}

int launch_calib_upfront(oxq_ctx *ctx, hipStream_t s, const uint8_t *src, uint64_t bytes, int workgroups, int waves,
                         int nontemporal, uint32_t *out) {
    const uint64_t span = bytes / (uint64_t)workgroups;
    const int nl = (int)(span / ((uint64_t)waves * 1024));
    dim3 grid((unsigned)workgroups), block((unsigned)waves * 64);
    char name[48];
    snprintf(name, sizeof name, "calib_upfront_%dw_%dl%s", waves, nl, nontemporal ? "_nt" : "");
    set_plan(ctx, name, grid, block, 1, 1, 0);
    if (ctx->plan_only) return OXQ_OK;
#define OXQ_UF(NLv)                                                                                              \
    case NLv:                                                                                                    \
        if (waves == 8) {                                                                                        \
            if (nontemporal) hipLaunchKernelGGL((calib_upfront_kernel<2, NLv, 8>), grid, block, 0, s, src, out, (uint32_t)span); \
            else hipLaunchKernelGGL((calib_upfront_kernel<0, NLv, 8>), grid, block, 0, s, src, out, (uint32_t)span);             \
        } else {                                                                                                 \
            if (nontemporal) hipLaunchKernelGGL((calib_upfront_kernel<2, NLv, 16>), grid, block, 0, s, src, out, (uint32_t)span); \
            else hipLaunchKernelGGL((calib_upfront_kernel<0, NLv, 16>), grid, block, 0, s, src, out, (uint32_t)span);            \
        }                                                                                                        \
        break;
    switch (nl) {
        OXQ_UF(1) OXQ_UF(2) OXQ_UF(4) OXQ_UF(6) OXQ_UF(8) OXQ_UF(9) OXQ_UF(10) OXQ_UF(12) OXQ_UF(16) OXQ_UF(17) OXQ_UF(20)
        OXQ_UF(24) OXQ_UF(32)
    default: return fail(OXQ_ERR_UNSUPPORTED, "read_upfront: no kernel for %d loads a lane (1, 2, 4, 6, 8, 9, 10, 12, 16, 17, 20, 24, 32)", nl);
    }
#undef OXQ_UF
    OXQ_HIP_CHECK(hipGetLastError());
    return OXQ_OK;
}

// Two request streams on one compute unit.  Waves 0 .. 7 of a workgroup read the workgroup's span of `w`
// (cold: HBM) with every load requested up front; waves 8 .. 11 read all of `x` (the same bytes in every
// workgroup: L2 hits) straight into LDS, two 8 KB stages in flight each.  which: 1 = only the first
// stream, 2 = only the second, 3 = both.  A compute unit serves its requests in issue order at a rate set
// by what they wait for, so "both" takes about the sum of the two, not the larger: the measurement that
// prices the rows of x a tile kernel re-reads per strip.
typedef __attribute__((address_space(3))) void *calib_lds_ptr_t;
template <int NL>
__global__ __launch_bounds__(768) void calib_two_streams_kernel(const uint8_t *__restrict__ w, const uint8_t *__restrict__ x,
                                                               uint32_t *__restrict__ out, uint32_t span, uint32_t x_bytes,
                                                               int which) {
    extern __shared__ __attribute__((aligned(16))) unsigned char calib_lds[];
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    u32x4_t acc = {0u, 0u, 0u, 0u};
    if (wave < 8) {
        if (which & 1) {
            const __amdgpu_buffer_rsrc_t rs = make_rsrc(w + (size_t)blockIdx.x * span, span);
            u32x4_t v[NL];
#pragma unroll
            for (int q = 0; q < NL; ++q) v[q] = __builtin_amdgcn_raw_buffer_load_b128(rs, lane * 16, (wave * NL + q) * 1024, 2);
#pragma unroll
            for (int q = 0; q < NL; ++q) acc ^= v[q];
        }
    } else if (which & 2) {
        const __amdgpu_buffer_rsrc_t rs = make_rsrc(x, x_bytes);
        const int lw = wave - 8;
        const uint32_t share = x_bytes / 4;            // bytes this wave moves, in stages of 8 KB
        const int nst = (int)(share / 8192);
        unsigned char *slot = calib_lds + lw * 16384;
        auto stage = [&](int s) {
#pragma unroll
            for (int q = 0; q < 8; ++q)
                __builtin_amdgcn_raw_ptr_buffer_load_lds(rs, (calib_lds_ptr_t)(slot + (s & 1) * 8192 + q * 1024), 16, lane * 16,
                                                         (int)(lw * share) + s * 8192 + q * 1024, 0, 0);
        };
        stage(0);
        if (nst > 1) stage(1);
        for (int s = 0; s < nst; ++s) {
            if (s + 2 <= nst) asm volatile("s_waitcnt vmcnt(8)" ::: "memory");
            else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            if (s + 2 < nst) stage(s + 2);
        }
    }
    const uint32_t r = acc[0] ^ acc[1] ^ acc[2] ^ acc[3];
    if (r == 0x9E3779B9u && out) out[blockIdx.x] = r;  // keeps the loads alive; the word is not a checksum
}

int launch_calib_two_streams(oxq_ctx *ctx, hipStream_t s, const uint8_t *w, uint64_t w_bytes, const uint8_t *x,
                             uint64_t x_bytes, int workgroups, int which, uint32_t *out) {
    const uint64_t span = w_bytes / (uint64_t)workgroups;
    const int nl = (int)(span / 8192);
    dim3 grid((unsigned)workgroups), block(768);
    char name[48];
    snprintf(name, sizeof name, "calib_two_streams_%d", which);
    set_plan(ctx, name, grid, block, 1, 1, 0);
    if (ctx->plan_only) return OXQ_OK;
    const size_t lds = 4 * 16384;
    switch (nl) {
    case 8: hipLaunchKernelGGL((calib_two_streams_kernel<8>), grid, block, lds, s, w, x, out, (uint32_t)span, (uint32_t)x_bytes, which); break;
    case 16: hipLaunchKernelGGL((calib_two_streams_kernel<16>), grid, block, lds, s, w, x, out, (uint32_t)span, (uint32_t)x_bytes, which); break;
    case 17: hipLaunchKernelGGL((calib_two_streams_kernel<17>), grid, block, lds, s, w, x, out, (uint32_t)span, (uint32_t)x_bytes, which); break;
    default: return fail(OXQ_ERR_UNSUPPORTED, "two_streams: %d KiB a wave (64, 128 or 136 KiB a workgroup)", nl);
    }
    OXQ_HIP_CHECK(hipGetLastError());
    return OXQ_OK;
}

int launch_calib_read(oxq_ctx *ctx, hipStream_t s, const uint8_t *src, uint64_t bytes, int workgroups, int nontemporal,
                      uint32_t *out) {
    const uint64_t span = bytes / (uint64_t)workgroups;
    dim3 grid((unsigned)workgroups), block(512);
    set_plan(ctx, nontemporal ? "calib_read_nt" : "calib_read", grid, block, 1, 1, 0);
    if (ctx->plan_only) return OXQ_OK;
    if (nontemporal)
        hipLaunchKernelGGL(calib_read_kernel<2>, grid, block, 0, s, src, out, (uint32_t)span);
    else
        hipLaunchKernelGGL(calib_read_kernel<0>, grid, block, 0, s, src, out, (uint32_t)span);
    OXQ_HIP_CHECK(hipGetLastError());
    return OXQ_OK;
}

}  // namespace oxq
