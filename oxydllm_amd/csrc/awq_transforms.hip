// Load-time transforms on the device.  Three produce AWQ-layout tensors:
//   compressed-tensors int4 (pack-quantized) -> AWQ layout   (awq.rs:187-254 compressed_to_awq)
//   concatenation of AWQ parts along the output dimension    (awq.rs:256-323 concat_awq_along_out)
//   round-to-nearest 4-bit group quantization of a dense      (awq.rs:637-742 rtn_quantize_awq)
//   weight into AWQ tensors
// and one on GGUF block bytes: the q/k row de-interleave       (gguf_weights.rs:255-291 depermute_qk_rows)
// The reference runs them on the CPU when a checkpoint is loaded; here the checkpoint tensors
// are already in HBM, so they are a handful of small kernels.  Integer outputs are bit-exact by
// construction; the quantizer uses the same f32 operations in the same order as the
// reference (IEEE division, round half away from zero).

#include "oxq_device.hpp"
#include "oxq_internal.hpp"

namespace oxq {

// ---- compressed-tensors -> AWQ --------------------------------------------------------
// ct[o][c] holds columns 8c..8c+7 of output row o, nibble i % 8 = q + 8, LSB first.
// AWQ word (i, jw) nibble k holds row jw * 8 + order[k] at input i (awq.rs:214-236).
// Thread (jw, c) reads the 8 words of rows 8 jw .. 8 jw + 7 at column block c and writes the
// 8 AWQ words of inputs 8 c .. 8 c + 7; consecutive threads are consecutive jw, so the writes
// coalesce.
__global__ __launch_bounds__(256) void ct_to_awq_kernel(const uint32_t *__restrict__ ct,
                                                        uint32_t *__restrict__ qweight, int out_f,
                                                        int packed_in) {
    const int packed_out = out_f >> 3;
    const size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= (size_t)packed_out * packed_in) return;
    const int jw = (int)(idx % packed_out), c = (int)(idx / packed_out);
    uint32_t row[8];
#pragma unroll
    for (int k = 0; k < 8; ++k) row[k] = ct[(size_t)(jw * 8 + awq_slot_col(k)) * packed_in + c];
#pragma unroll
    for (int r = 0; r < 8; ++r) {
        uint32_t w = 0;
#pragma unroll
        for (int k = 0; k < 8; ++k) w |= ((row[k] >> (4 * r)) & 0xFu) << (4 * k);
        qweight[(size_t)(c * 8 + r) * packed_out + jw] = w;
    }
}

__global__ __launch_bounds__(256) void fill_u32_kernel(uint32_t *__restrict__ p, size_t n, uint32_t v) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i < n) p[i] = v;
}

// [rows, cols] -> [cols, rows], element size ES bytes (scales [out, groups] -> [groups, out])
template <typename T>
__global__ __launch_bounds__(256) void transpose_kernel(const T *__restrict__ src, T *__restrict__ dst,
                                                        int rows, int cols) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= (size_t)rows * cols) return;
    const int r = (int)(i % rows), c = (int)(i / rows);  // consecutive threads write consecutive dst
    dst[i] = src[(size_t)r * cols + c];
}

int launch_compressed_to_awq(oxq_ctx *ctx, hipStream_t s, const uint32_t *ct, const void *scale_ct,
                             int scale_elem_bytes, uint32_t *qweight, uint32_t *qzeros, void *scales,
                             int64_t out_f, int64_t in_f, int64_t groups) {
    const int64_t packed_out = out_f / 8, packed_in = in_f / 8;
    dim3 grid((unsigned)ceil_div(packed_out * packed_in, 256)), block(256);
    set_plan(ctx, "compressed_to_awq", grid, block, 1, 3, 0);
    if (ctx->plan_only) return OXQ_OK;
    hipLaunchKernelGGL(ct_to_awq_kernel, grid, block, 0, s, ct, qweight, (int)out_f, (int)packed_in);
    const size_t nz = (size_t)groups * packed_out;
    hipLaunchKernelGGL(fill_u32_kernel, dim3((unsigned)ceil_div((int64_t)nz, 256)), block, 0, s, qzeros, nz,
                       0x88888888u);
    dim3 tgrid((unsigned)ceil_div(out_f * groups, 256));
    if (scale_elem_bytes == 2)
        hipLaunchKernelGGL((transpose_kernel<uint16_t>), tgrid, block, 0, s, (const uint16_t *)scale_ct,
                           (uint16_t *)scales, (int)out_f, (int)groups);
    else
        hipLaunchKernelGGL((transpose_kernel<uint32_t>), tgrid, block, 0, s, (const uint32_t *)scale_ct,
                           (uint32_t *)scales, (int)out_f, (int)groups);
    OXQ_HIP_CHECK(hipGetLastError());
    return OXQ_OK;
}

// ---- concatenation along the output dimension ---------------------------------------
// Copies a [rows, width] block of 32-bit words into a wider row-major destination.
__global__ __launch_bounds__(256) void copy2d_u32_kernel(const uint32_t *__restrict__ src,
                                                         uint32_t *__restrict__ dst, int rows, int width,
                                                         int dst_pitch, int dst_col) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= (size_t)rows * width) return;
    const int r = (int)(i / width), c = (int)(i % width);
    dst[(size_t)r * dst_pitch + dst_col + c] = src[i];
}

int launch_copy2d_u32(oxq_ctx *ctx, hipStream_t s, const void *src, void *dst, int64_t rows, int64_t width,
                      int64_t dst_pitch, int64_t dst_col) {
    if (ctx->plan_only || rows * width == 0) return OXQ_OK;
    hipLaunchKernelGGL(copy2d_u32_kernel, dim3((unsigned)ceil_div(rows * width, 256)), dim3(256), 0, s,
                       (const uint32_t *)src, (uint32_t *)dst, (int)rows, (int)width, (int)dst_pitch,
                       (int)dst_col);
    OXQ_HIP_CHECK(hipGetLastError());
    return OXQ_OK;
}

// ---- GGUF q/k row de-interleave --------------------------------------------------------
// gguf_weights.rs:255-291: HF row r of a head sits at interleaved row 2 (r % half) + r / half.
// Rows are independent runs of blocks, so this is a byte shuffle of whole rows (row lengths
// are even; copied as 16-bit words).
__global__ __launch_bounds__(256) void gguf_depermute_rows_kernel(const uint16_t *__restrict__ src,
                                                                  uint16_t *__restrict__ dst, int head_dim,
                                                                  int row_words, size_t total_words) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= total_words) return;
    const size_t row = i / row_words, w = i - row * row_words;
    const int h = (int)(row / head_dim), r = (int)(row % head_dim), half = head_dim >> 1;
    const size_t srow = (size_t)h * head_dim + 2 * (r % half) + r / half;
    dst[i] = src[srow * row_words + w];
}

int launch_gguf_depermute_rows(oxq_ctx *ctx, hipStream_t s, const uint8_t *src, uint8_t *dst, int64_t rows,
                               int64_t row_bytes, int64_t head_dim) {
    const size_t words = (size_t)rows * row_bytes / 2;
    dim3 grid((unsigned)ceil_div((int64_t)words, 256)), block(256);
    set_plan(ctx, "gguf_depermute_qk_rows", grid, block, 1, 1, 0);
    if (ctx->plan_only || words == 0) return OXQ_OK;
    hipLaunchKernelGGL(gguf_depermute_rows_kernel, grid, block, 0, s, (const uint16_t *)src, (uint16_t *)dst,
                       (int)head_dim, (int)(row_bytes / 2), words);
    OXQ_HIP_CHECK(hipGetLastError());
    return OXQ_OK;
}

// ---- round-to-nearest AWQ quantizer ---------------------------------------------------
// One workgroup of 8 waves per packed output word column j: wave w owns output row
// o = 8 j + w and walks its groups.  Per group (awq.rs:676-709): range extended to include
// 0, scale = (max - min) / 15, zero = round(-min / scale) clamped to [0, 15],
// q = round(v / scale + zero) clamped; a (nearly) constant-zero group stores scale = min,
// zero = 0, q = 1.  The eight rows' nibbles of one input meet in LDS and leave as one AWQ
// word (slot k <- row order[k], awq.rs:716-731).
template <typename T> __device__ __forceinline__ float rtn_to_f32(T v);
template <> __device__ __forceinline__ float rtn_to_f32<float>(float v) { return v; }
template <> __device__ __forceinline__ float rtn_to_f32<_Float16>(_Float16 v) { return (float)v; }
template <> __device__ __forceinline__ float rtn_to_f32<__bf16>(__bf16 v) {
    return __builtin_bit_cast(float, (uint32_t)__builtin_bit_cast(uint16_t, v) << 16);
}

__device__ __forceinline__ float wave_min(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v = fminf(v, __shfl_xor(v, off, WAVE));
    return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, WAVE));
    return v;
}

constexpr int RTN_CHUNK = 256;  // inputs of a group handled per pass through LDS

template <typename T>
__global__ __launch_bounds__(512) void rtn_quantize_awq_kernel(const T *__restrict__ weight,
                                                               uint32_t *__restrict__ qweight,
                                                               uint32_t *__restrict__ qzeros,
                                                               float *__restrict__ scales, int out_f, int in_f,
                                                               int group_size) {
    __shared__ uint8_t nib[8][RTN_CHUNK];
    __shared__ uint8_t znib[8];
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    const int j = blockIdx.x, o = j * 8 + w;
    const int packed_out = out_f >> 3, groups = in_f / group_size;
    const T *row = weight + (size_t)o * in_f;
    for (int g = 0; g < groups; ++g) {
        const T *grp = row + (size_t)g * group_size;
        float mn = rtn_to_f32(grp[0]), mx = mn;
        for (int i = lane; i < group_size; i += 64) {
            const float v = rtn_to_f32(grp[i]);
            mn = fminf(mn, v), mx = fmaxf(mx, v);
        }
        mn = fminf(wave_min(mn), 0.0f);
        mx = fmaxf(wave_max(mx), 0.0f);
        const bool flat = mx - mn < 1e-12f;
        const float scale = flat ? mn : (mx - mn) / 15.0f;
        const float zero = flat ? 0.0f : fminf(fmaxf(roundf(-mn / scale), 0.0f), 15.0f);
        if (lane == 0) {
            scales[(size_t)g * out_f + o] = scale;
            znib[w] = (uint8_t)zero;
        }
        for (int c0 = 0; c0 < group_size; c0 += RTN_CHUNK) {
            const int cn = min(RTN_CHUNK, group_size - c0);
            for (int i = lane; i < cn; i += 64) {
                const float v = rtn_to_f32(grp[c0 + i]);
                nib[w][i] = flat ? (uint8_t)1 : (uint8_t)fminf(fmaxf(roundf(v / scale + zero), 0.0f), 15.0f);
            }
            __syncthreads();
            for (int i = threadIdx.x; i < cn; i += 512) {
                uint32_t word = 0;
#pragma unroll
                for (int k = 0; k < 8; ++k) word |= (uint32_t)nib[awq_slot_col(k)][i] << (4 * k);
                qweight[(size_t)(g * group_size + c0 + i) * packed_out + j] = word;
            }
            if (c0 == 0 && threadIdx.x == 0) {
                uint32_t zw = 0;
#pragma unroll
                for (int k = 0; k < 8; ++k) zw |= (uint32_t)znib[awq_slot_col(k)] << (4 * k);
                qzeros[(size_t)g * packed_out + j] = zw;
            }
            __syncthreads();
        }
    }
}

int launch_rtn_quantize_awq(oxq_ctx *ctx, hipStream_t s, const void *weight, int dtype, uint32_t *qweight,
                            uint32_t *qzeros, float *scales, int64_t out_f, int64_t in_f, int64_t group_size) {
    dim3 grid((unsigned)(out_f / 8)), block(512);
    set_plan(ctx, "rtn_quantize_awq", grid, block, 1, 1, 0);
    if (ctx->plan_only) return OXQ_OK;
    switch (dtype) {
    case OXQ_F32:
        hipLaunchKernelGGL((rtn_quantize_awq_kernel<float>), grid, block, 0, s, (const float *)weight, qweight,
                           qzeros, scales, (int)out_f, (int)in_f, (int)group_size);
        break;
    case OXQ_F16:
        hipLaunchKernelGGL((rtn_quantize_awq_kernel<_Float16>), grid, block, 0, s, (const _Float16 *)weight,
                           qweight, qzeros, scales, (int)out_f, (int)in_f, (int)group_size);
        break;
    default:
        hipLaunchKernelGGL((rtn_quantize_awq_kernel<__bf16>), grid, block, 0, s, (const __bf16 *)weight, qweight,
                           qzeros, scales, (int)out_f, (int)in_f, (int)group_size);
        break;
    }
    OXQ_HIP_CHECK(hipGetLastError());
    return OXQ_OK;
}

}  // namespace oxq
