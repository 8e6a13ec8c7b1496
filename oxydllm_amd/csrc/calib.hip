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
