// Internal declarations shared by the host API and the kernel launchers.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdarg>
#include <algorithm>
#include <atomic>
#include <mutex>
#include <cstdint>
#include <cstdio>
#include <cstring>

#include "oxq.h"

// Tuning switches.  Each is read from the environment variable OXQ_<name> once, when a ctx is created,
// and can be set per ctx with oxq_ctx_set_tuning; the launchers only ever look at the ctx, so a forward
// call costs no getenv and two engine threads cannot race on the process environment.
#define OXQ_TUNE_LIST(X)                                                                                      \
    X(ACT_VEC) X(F8_MM_KS) X(F8_MM_MIN_M) X(F8_MM_MT) X(FORCE_GENERIC) X(GEMV_CFG) X(GEMV_GPW) X(GEMV_TILE)   \
    X(GGR_GRID) X(GGR_WAVES) X(GGUF_BIG_LDS) X(GGUF_GEMM_KS) X(GGUF_GEMM_MIN_M) X(GGUF_MFMA)                  \
    X(GGUF_MFMA_MAX_M) X(GGUF_MFMA_NS) X(GGUF_MM_KS) X(GGUF_MM_MIN_M) X(GGUF_MM_MT) X(GGUF_PW) X(GGUF_RPWG)   \
    X(GPTQ_TILE) X(GPTQ_TILE_KS) X(MFMA_MT) X(MFMA_SPLITK) X(MFMA_VARIANT) X(MXFP4_FR) X(MXFP4_GEMM_MIN_PAIRS) \
    X(MXFP4_GEMM_ROWS) X(MXFP4_MM)      \
    X(MXFP4_MM_KS) X(MXFP4_MM_MT) X(MXFP4_VARIANT) X(PK4N_NS1_ROWS) X(PK4N_W16) X(PK4_CONTIGUOUS)             \
    X(PK4_FOLD) X(PK4_FRONT) X(PK4_GEMM_KS) X(PK4_GEMM_MIN_M) X(PK4_GEMM_ROWS) X(PK4_KS) X(PK4_PLACE64)       \
    X(PK4_STRIP16) X(PK4_T64) X(PK4_XQ) X(PREPACK) X(SPLITK_MODE) X(TRANSIENT_REPACK)
enum oxq_tune_key {
#define OXQ_TUNE_ENUM(n) OXQ_TUNE_##n,
    OXQ_TUNE_LIST(OXQ_TUNE_ENUM)
#undef OXQ_TUNE_ENUM
    OXQ_TUNE_COUNT
};
constexpr int OXQ_TUNE_UNSET = -2147483647 - 1;

struct oxq_ctx {
    int device;             // HIP ordinal, or OXQ_DEVICE_PLAN_ONLY
    bool plan_only;
    void *workspace;        // split-K partial sums (f32)
    size_t workspace_bytes;
    unsigned *counters;     // arrival counters, zero between calls
    size_t n_counters;
    int num_cus;
    int splitk_mode;        // 0 auto, 1 fused last-arriver, 2 separate reduce kernel
    oxq_plan plan;
    struct oxq_weight_cache *wcache;  // tile-major copies the stateless ops made (opt-in), or null
    size_t wcache_limit;              // bytes the cache may hold; 0 = off
    int tuning[OXQ_TUNE_COUNT];       // tuning switches (OXQ_TUNE_UNSET = the launcher's own default)
};

namespace oxq {

int fail(int status, const char *fmt, ...) __attribute__((format(printf, 2, 3)));
const char *dtype_name(int dtype);

inline size_t dtype_size(int dtype) {
    switch (dtype) {
    case OXQ_F32: case OXQ_I32: case OXQ_U32: return 4;
    case OXQ_F16: case OXQ_BF16: return 2;
    case OXQ_U8: return 1;
    case OXQ_I64: return 8;
    default: return 0;
    }
}

inline int64_t numel(const oxq_tensor *t) {
    int64_t n = 1;
    for (int i = 0; i < t->rank; ++i) n *= t->dims[i];
    return n;
}

inline bool is_pow2(int64_t v) { return v > 0 && (v & (v - 1)) == 0; }
inline int ilog2(int64_t v) {
    int s = 0;
    while ((int64_t(1) << s) < v) ++s;
    return s;
}
inline int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }

// a tuning switch of this ctx, or `dflt` where neither the environment nor the caller set it
inline int tune(const oxq_ctx *ctx, oxq_tune_key key, int dflt) {
    const int v = ctx->tuning[key];
    return v == OXQ_TUNE_UNSET ? dflt : v;
}
inline bool tune_given(const oxq_ctx *ctx, oxq_tune_key key) { return ctx->tuning[key] != OXQ_TUNE_UNSET; }

void set_plan(oxq_ctx *ctx, const char *kernel, dim3 grid, dim3 block, uint32_t split_k,
              uint32_t launches, uint64_t ws_bytes);
void add_launch(oxq_ctx *ctx);

#define OXQ_HIP_CHECK(expr)                                                                   \
    do {                                                                                      \
        hipError_t _e = (expr);                                                               \
        if (_e != hipSuccess)                                                                 \
            return ::oxq::fail(OXQ_ERR_RUNTIME, "%s failed: %s", #expr, hipGetErrorString(_e)); \
    } while (0)

// A kernel's dynamic-LDS limit (hipFuncAttributeMaxDynamicSharedMemorySize) belongs to the pair
// (function, device).  One LdsGrant per kernel instantiation remembers what each device has been
// granted; the usual path is one atomic load, the raise happens under a lock so that a smaller
// request from another engine thread cannot overwrite a larger one.
struct LdsGrant {
    static constexpr int MAX_DEVICES = 64;
    std::atomic<size_t> granted[MAX_DEVICES] = {};
    hipError_t ensure(const void *fn, size_t lds) {
        int dev = 0;
        hipError_t e = hipGetDevice(&dev);
        if (e != hipSuccess) return e;
        if (dev < 0 || dev >= MAX_DEVICES)  // not remembered: ask every time
            return hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (lds <= granted[dev].load(std::memory_order_acquire)) return hipSuccess;
        static std::mutex mu;
        std::lock_guard<std::mutex> lock(mu);
        if (lds <= granted[dev].load(std::memory_order_relaxed)) return hipSuccess;
        e = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e == hipSuccess) granted[dev].store(lds, std::memory_order_release);
        return e;
    }
};

// ---- problem descriptors handed to the launchers (all validated) ----------

struct Wna16Problem {
    const void *x;          // [M, K] T
    const uint32_t *qweight;
    const uint32_t *qzeros;
    const void *scales;     // [G, N] T
    const void *bias;       // [N] T or nullptr
    void *y;                // [M, N] T
    int64_t M, K, N;
    int64_t group_size;
    int group_shift;
    int bits;               // 4 or 8
    int pack_dim;           // OXQ_PACK_OUT (AWQ) / OXQ_PACK_IN (GPTQ)
    int dtype;              // OXQ_F16 / OXQ_BF16
};

struct GgufProblem {
    const void *x;          // [M, K] act dtype
    const uint8_t *w;       // raw blocks
    const void *bias;       // [N] or nullptr (act dtype)
    void *y;                // [M, N]
    int64_t M, K, N;
    int quant;
    int act_dtype;          // OXQ_BF16 or OXQ_F32
    int act = 0;            // matrix-core copy of a fused gate|up layer: 1 + the gated activation (y is [M, N / 2])
};

struct Mxfp4Problem {
    const void *x;          // bf16
    const uint8_t *blocks;
    const uint8_t *scales;
    const void *bias;       // bf16 [E, N] / [N] or nullptr
    void *y;                // bf16
    int64_t M, K, N;
    // grouped form (n_experts > 0)
    int64_t n_experts;
    const int32_t *expert_offsets;
    const int32_t *token_ids;   // nullptr => identity
    int64_t n_pairs;
    // fused GPT-OSS SwiGLU over interleaved (gate, up) rows: y is [n_pairs, N / 2]
    int swiglu = 0;
    float swiglu_limit = 0.0f;
};
// launch_mxfp4_gemv returns this (positive) when p.swiglu is set and the kernel the problem size
// selects has no fused epilogue; nothing was enqueued
constexpr int OXQ_DECLINED = 1;

// Block-scaled F8E4M3 weight [N, K] bytes with an F32 scale grid [s_rows, s_cols] tiling it.
struct F8Problem {
    const void *x;          // [M, K] bf16 (nullptr for the dequant)
    const uint8_t *w;       // [N, K]
    const float *scales;    // [N / block_r, K / block_c]
    void *y;                // [M, N] bf16
    int64_t M, K, N;
    int64_t block_r, block_c, s_cols;
};

// A resident 4- or 8-bit layer repacked tile-major at load (layout: pk4.hip).
struct Pk4Weights {
    uint32_t *pw;           // [N/64][K/128]{[4][bits/4][64][4] weights, [16][4] {-(bias + z), s} pairs}
    uint32_t *pzs;          // unused (the pairs live inside the blocks of pw); kept null
    int64_t K, N;
    int group_shift;
    int dtype;              // OXQ_F16 / OXQ_BF16
    int bits;               // 4 or 8
    int64_t gate_half;      // 0, or N/2 for a fused gate|up layer: strip j holds gate columns
                            // [32j, 32j+32) then up columns [N/2 + 32j, N/2 + 32j + 32)
    int gemv_rows;          // rows up to which the reference runs its fused GEMV, which never rounds the
                            // dequantized weight (linear.rs:450-480: 16 AWQ, 32 GPTQ); 0 = 16
    int strip;              // columns of a strip of pw: 64 (or 0), or 16 (narrow 4-bit layers, see pk4.hip)
};

struct Pk4Problem {
    const void *x;          // [M, K] T
    const void *bias;       // [N] T or nullptr
    void *y;                // [M, N] T, or [M, N/2] with `act`
    int64_t M;
    int act;                // 0, or 1 + oxq_gated_act (gate|up layers only): y = act(gate) * up
    int no_split;           // the ctx workspace is taken (it holds the weights): one K slice only
    Pk4Weights w;
    void *ws = nullptr;     // filled in by the launcher: the ctx workspace for K-slice partials
};

// ---- launchers (defined in the .hip files) ---------------------------------
bool pk4_eligible(const Wna16Problem &p);
// resident 4-bit layers at prefill sizes: 64 rows x eight strips a workgroup (pk4_gemm.hip)
bool pk4_gemm_takes(const oxq_ctx *ctx, const Pk4Problem &p);
int launch_pk4_gemm(oxq_ctx *ctx, hipStream_t s, const Pk4Problem &p);
size_t pk4_weight_bytes(int64_t K, int64_t N, int bits);
int pk4_choose_strip(const oxq_ctx *ctx, int64_t K, int64_t N, int bits, int64_t gate_half);
size_t pk4_zs_bytes(int64_t K, int64_t N, int group_shift);
int launch_pk4_prepack(oxq_ctx *ctx, hipStream_t s, const Wna16Problem &src, const Pk4Weights &dst);
int launch_pk4_forward(oxq_ctx *ctx, hipStream_t s, const Pk4Problem &p);
int launch_pk4_dequant(oxq_ctx *ctx, hipStream_t s, const Pk4Weights &w, void *out_kn);
// 49 - 64 rows on a 4-bit layer in 64-column strips (pk4_tile.hip)
bool pk4_tile64_takes(const Pk4Problem &p, int ks);
int launch_pk4_tile64(oxq_ctx *ctx, hipStream_t s, const Pk4Problem &p);
int launch_wna16_gemv(oxq_ctx *ctx, hipStream_t s, const Wna16Problem &p);
bool awq4_mfma_ok(const Wna16Problem &p);
bool gptq_tile_ok(const Wna16Problem &p);
int launch_gptq_tile(oxq_ctx *ctx, hipStream_t s, const Wna16Problem &p);
int launch_wna16_mfma(oxq_ctx *ctx, hipStream_t s, const Wna16Problem &p);
int launch_wna16_dequant(oxq_ctx *ctx, hipStream_t s, const Wna16Problem &p, void *out_kn);
int launch_gguf_gemv(oxq_ctx *ctx, hipStream_t s, const GgufProblem &p);
int launch_gguf_dequant(oxq_ctx *ctx, hipStream_t s, const GgufProblem &p, float *out_nk);
// m > 8, bf16: tile matmul on the matrix cores (weights rounded to bf16 as the reference's mul_mm does)
// resident (strip-major) copy of a GGUF weight and its decode GEMV (gguf_res.hip)
bool gguf_res_eligible(int quant, int64_t K, int64_t N);
size_t gguf_res_bytes(int quant, int64_t K, int64_t N);
bool gguf_res_takes(int64_t K, int64_t M, int act_dtype);
int launch_gguf_res_repack(oxq_ctx *ctx, hipStream_t s, int quant, const uint8_t *w, void *pw, int64_t K, int64_t N);
int launch_gguf_res_dequant(oxq_ctx *ctx, hipStream_t s, int quant, const void *pw, int64_t K, int64_t N, float *out_nk);
int launch_gguf_res_gemv(oxq_ctx *ctx, hipStream_t s, const GgufProblem &p);  // p.w = the copy
// matrix-core copy of a GGUF weight for 16-bit activations and its matmul (gguf_mfma.hip)
bool gguf_mfma_eligible(const oxq_ctx *ctx, int quant, int64_t K, int64_t N);
bool gguf_mfma_takes(const oxq_ctx *ctx, int64_t M, int64_t N, int act_dtype);
int launch_gguf_mfma_repack(oxq_ctx *ctx, hipStream_t s, int quant, const uint8_t *w, void *pw, int64_t K, int64_t N,
                            int64_t gate_half = 0);
int launch_gguf_mfma_dequant(oxq_ctx *ctx, hipStream_t s, int quant, const void *pw, int64_t K, int64_t N, float *out_nk,
                             int64_t gate_half = 0);
int launch_gguf_mfma(oxq_ctx *ctx, hipStream_t s, const GgufProblem &p);  // p.w = the copy
// the prefill kernel on the same copy (csrc/gguf_mfma.hip: ggm_gemm_kernel)
bool gguf_gemm_takes(const oxq_ctx *ctx, int quant, int64_t M, int64_t K, int64_t N, int act_dtype);
int launch_gguf_gemm(oxq_ctx *ctx, hipStream_t s, const GgufProblem &p);  // p.w = the copy
bool gguf_mm_eligible(const oxq_ctx *ctx, const GgufProblem &p);
int launch_gguf_mm(oxq_ctx *ctx, hipStream_t s, const GgufProblem &p);
// load-time transforms into the AWQ layout (awq_transforms.hip)
int launch_compressed_to_awq(oxq_ctx *ctx, hipStream_t s, const uint32_t *ct, const void *scale_ct,
                             int scale_elem_bytes, uint32_t *qweight, uint32_t *qzeros, void *scales,
                             int64_t out_f, int64_t in_f, int64_t groups);
int launch_copy2d_u32(oxq_ctx *ctx, hipStream_t s, const void *src, void *dst, int64_t rows, int64_t width,
                      int64_t dst_pitch, int64_t dst_col);
int launch_gguf_depermute_rows(oxq_ctx *ctx, hipStream_t s, const uint8_t *src, uint8_t *dst, int64_t rows,
                               int64_t row_bytes, int64_t head_dim);
int launch_rtn_quantize_awq(oxq_ctx *ctx, hipStream_t s, const void *weight, int dtype, uint32_t *qweight,
                            uint32_t *qzeros, float *scales, int64_t out_f, int64_t in_f, int64_t group_size);
// block-scaled F8E4M3 (f8_block.hip; the tile matmul for m > 8 lives in blockq_mm.hip)
int launch_cast_f8e4m3_f32(oxq_ctx *ctx, hipStream_t s, const uint8_t *in, float *out, size_t n);
int launch_f8_block_dequant(oxq_ctx *ctx, hipStream_t s, const F8Problem &p, uint16_t *out);
int launch_f8_gemv(oxq_ctx *ctx, hipStream_t s, const F8Problem &p);
bool f8_mm_eligible(const oxq_ctx *ctx, const F8Problem &p);
int launch_f8_mm(oxq_ctx *ctx, hipStream_t s, const F8Problem &p);
// MXFP4 prefill (plain m > 16, or grouped with many pairs per expert): same tile matmul
int launch_mxfp4_mm(oxq_ctx *ctx, hipStream_t s, const Mxfp4Problem &p);
int launch_mxfp4_gemv(oxq_ctx *ctx, hipStream_t s, const Mxfp4Problem &p);
int launch_mxfp4_dequant(oxq_ctx *ctx, hipStream_t s, const Mxfp4Problem &p, float *out_nk);
// resident experts: tile-major copy (layout: mxfp4_gemv.hip) and the decode GEMV on it
bool mxfp4_res_eligible(int64_t K, int64_t N);
size_t mxfp4_res_weight_bytes(int64_t E, int64_t K, int64_t N);
size_t mxfp4_res_scale_bytes(int64_t E, int64_t K, int64_t N);
int launch_mxfp4_repack(oxq_ctx *ctx, hipStream_t s, const uint8_t *blocks, const uint8_t *scales, void *pw, void *ps,
                        int64_t E, int64_t K, int64_t N);
int launch_mxfp4_res_dequant(oxq_ctx *ctx, hipStream_t s, const void *pw, const void *ps, int64_t expert, int64_t K,
                             int64_t N, float *out_nk);
int launch_mxfp4_res_gemv(oxq_ctx *ctx, hipStream_t s, const Mxfp4Problem &p);
// prefill on the resident copy: 0 = not taken, else the rows of a tile; p.M = rows of x
int mxfp4_gemm_form(const oxq_ctx *ctx, int64_t n_pairs, int64_t E, int64_t K, int64_t N);
int launch_mxfp4_res_gemm(oxq_ctx *ctx, hipStream_t s, const Mxfp4Problem &p);
// mixture-of-experts glue (moe_glue.hip)
int launch_moe_route(oxq_ctx *ctx, hipStream_t s, const void *logits, int dtype, int64_t T, int64_t E, int64_t top_k,
                     int norm_topk, int32_t *top_idx, float *top_vals);
int launch_moe_route_group(oxq_ctx *ctx, hipStream_t s, const void *logits, int dtype, int64_t T, int64_t E,
                           int64_t top_k, int norm_topk, int32_t *top_idx, float *top_vals, int32_t *offsets,
                           int32_t *tokens, float *weights, int32_t *pair_pos);
int launch_moe_group(oxq_ctx *ctx, hipStream_t s, const int32_t *top_idx, const float *top_vals, int64_t P, int64_t E,
                     int64_t top_k, int32_t *offsets, int32_t *tokens, float *weights, int32_t *pair_pos);
int launch_activation_mul(oxq_ctx *ctx, hipStream_t s, const void *gate, const void *up, void *out, int dtype,
                          int64_t n, int kind);
int launch_gated_activation(oxq_ctx *ctx, hipStream_t s, const void *gu, void *out, int dtype, int64_t rows,
                            int64_t half_n, int kind, float limit);
int launch_moe_combine(oxq_ctx *ctx, hipStream_t s, const void *eo, const int32_t *pair_pos, const float *top_vals,
                       void *out, int dtype, int64_t T, int64_t H, int64_t top_k);
// plain streaming read (calib.hip): bytes = workgroups * span, span a multiple of 64 KiB
int launch_calib_read(oxq_ctx *ctx, hipStream_t s, const uint8_t *src, uint64_t bytes, int workgroups, int nontemporal,
                      uint32_t *out);
// the same read with every lane's share requested up front; an empty launch (calib.hip)
int launch_calib_upfront(oxq_ctx *ctx, hipStream_t s, const uint8_t *src, uint64_t bytes, int workgroups, int waves,
                         int nontemporal, uint32_t *out);
int launch_empty(oxq_ctx *ctx, hipStream_t s, int workgroups, int threads, int lds_bytes);
int launch_grid_barrier(oxq_ctx *ctx, hipStream_t s, int workgroups, int threads, unsigned *counter, unsigned *err,
                        unsigned spin_limit);
int launch_calib_two_streams(oxq_ctx *ctx, hipStream_t s, const uint8_t *w, uint64_t w_bytes, const uint8_t *x,
                             uint64_t x_bytes, int workgroups, int which, uint32_t *out);
// y[M,N] = sum over S slices of ws[s][M][N] (+ bias), slices added in index order.
int launch_splitk_reduce(oxq_ctx *ctx, hipStream_t s, const float *ws, const void *bias, void *y,
                         int64_t M, int64_t N, int S, int dtype);

}  // namespace oxq
