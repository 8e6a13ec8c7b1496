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
