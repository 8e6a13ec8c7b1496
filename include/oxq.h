/*
 * oxq.h - C ABI of the MI355X (gfx950) quantized-weight matmul library.
 *
 * The library replaces, one for one, the op functions oxydLLM's linear layers
 * call for packed-quantized weights (reference: src/common/metal_ops.rs) and
 * the three layer types that route to them (src/common/linear.rs,
 * src/common/mxfp4.rs).  Each declaration cites the reference interface it
 * stands in for.
 *
 * Conventions
 *  - Every tensor argument is an `oxq_tensor` descriptor: a device pointer to
 *    element 0 (any storage offset already applied), element type, rank and
 *    dims.  The library never owns, frees or reallocates caller memory.
 *  - Outputs are caller-allocated (the reference ops allocate their result;
 *    a C ABI cannot return a framework tensor).  Shapes are checked.
 *  - All validation runs on the host before anything is enqueued and mirrors
 *    the reference's `bail!` conditions; a failed call enqueues nothing.
 *  - Calls return 0 on success or a negative `oxq_status`; the message of the
 *    last failure on the calling thread is available from oxq_last_error().
 *  - Work is enqueued asynchronously on `stream` (a hipStream_t, NULL = the
 *    default stream).  No call synchronizes the device.
 *  - One `oxq_ctx` per engine thread / stream: the ctx owns a split-K
 *    workspace that concurrent calls on the same ctx would race on.
 *  - A ctx created with device = OXQ_DEVICE_PLAN_ONLY validates arguments and
 *    computes the launch plan but launches nothing; it needs no GPU.
 */
#ifndef OXQ_H
#define OXQ_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define OXQ_VERSION_MAJOR 0
#define OXQ_VERSION_MINOR 1

#define OXQ_DEVICE_HOST (-1)      /* oxq_tensor.device: host memory (always rejected by ops) */
#define OXQ_DEVICE_PLAN_ONLY (-1) /* oxq_ctx_create: validate + plan, never launch */

typedef enum oxq_status {
    OXQ_OK = 0,
    OXQ_ERR_ARG = -1,        /* NULL pointer / bad enum */
    OXQ_ERR_DTYPE = -2,      /* element type not accepted by the op */
    OXQ_ERR_SHAPE = -3,      /* rank / dims / byte-count mismatch */
    OXQ_ERR_CONTIGUOUS = -4, /* x (or qweight) must be contiguous */
    OXQ_ERR_M_RANGE = -5,    /* m outside the op's decode range [1, 8] */
    OXQ_ERR_GROUP = -6,      /* group size not a power of two / not dividing K */
    OXQ_ERR_DEVICE = -7,     /* tensor not resident on the ctx device */
    OXQ_ERR_BITS = -8,       /* bits not in {4, 8} */
    OXQ_ERR_RUNTIME = -9,    /* HIP runtime failure */
    OXQ_ERR_WORKSPACE = -10, /* problem needs more split-K workspace than the ctx holds */
    OXQ_ERR_UNSUPPORTED = -11,
    OXQ_ERR_IO = -12,    /* a checkpoint file could not be opened or mapped */
    OXQ_ERR_FORMAT = -13 /* a checkpoint file or JSON text is malformed */
} oxq_status;

typedef enum oxq_dtype {
    OXQ_F32 = 0,
    OXQ_F16 = 1,
    OXQ_BF16 = 2,
    OXQ_U8 = 3,
    OXQ_I32 = 4,
    OXQ_U32 = 5,
    OXQ_I64 = 6
} oxq_dtype;

/* reference: awq.rs:27-31 (PackDim).  OUT = AWQ layout, IN = GPTQ layout. */
typedef enum oxq_pack_dim { OXQ_PACK_OUT = 0, OXQ_PACK_IN = 1 } oxq_pack_dim;

/* reference: metal_ops.rs:5211-5223 (GgufFastQuant); the four formats built here. */
typedef enum oxq_gguf_quant {
    OXQ_GGUF_Q4_0 = 0,
    OXQ_GGUF_Q8_0 = 1,
    OXQ_GGUF_Q4_K = 2,
    OXQ_GGUF_Q6_K = 3,
    OXQ_GGUF_Q4_1 = 4,
    OXQ_GGUF_Q5_0 = 5,
    OXQ_GGUF_Q5_1 = 6,
    OXQ_GGUF_Q2_K = 7,
    OXQ_GGUF_Q3_K = 8,
    OXQ_GGUF_Q5_K = 9
} oxq_gguf_quant;

#define OXQ_MAX_RANK 4

typedef struct oxq_tensor {
    void *data;                 /* device pointer to element 0 */
    int32_t dtype;              /* oxq_dtype */
    int32_t rank;               /* 1..OXQ_MAX_RANK */
    int64_t dims[OXQ_MAX_RANK]; /* row-major */
    int32_t contiguous;         /* non-zero when densely packed row-major */
    int32_t device;             /* HIP device ordinal, OXQ_DEVICE_HOST for host memory */
} oxq_tensor;

/* What the last successful call on a ctx launched (or would launch). */
typedef struct oxq_plan {
    char kernel[64];
    uint32_t grid[3];
    uint32_t block[3];
    uint32_t split_k;         /* number of K slices combined in fixed order */
    uint32_t launches;        /* kernel launches the call enqueued */
    uint64_t workspace_bytes; /* split-K partials used */
} oxq_plan;

typedef struct oxq_ctx oxq_ctx;

/* ---- context -------------------------------------------------------------
 * No counterpart in the reference (candle owns its Metal device/encoder,
 * metal_ops.rs:1367-1403); holds the device ordinal and split-K workspace. */
int oxq_ctx_create(int device, oxq_ctx **out);
int oxq_ctx_destroy(oxq_ctx *ctx);
int oxq_ctx_device(const oxq_ctx *ctx);
int oxq_ctx_last_plan(const oxq_ctx *ctx, oxq_plan *out);
const char *oxq_last_error(void);
const char *oxq_status_name(int status);
void oxq_version(int *major, int *minor);

/* ---- tuning switches -----------------------------------------------------------
 * No counterpart in the reference.  Every switch that selects between kernels or launch shapes
 * (OXQ_PK4_FRONT, OXQ_PK4_KS, OXQ_FORCE_GENERIC, ...: the list is OXQ_TUNE_LIST in the library's
 * sources) lives in the ctx.  oxq_ctx_create reads each once from the environment variable of the
 * same name; oxq_ctx_set_tuning overrides one for this ctx, oxq_ctx_reset_tuning(ctx, name) returns it
 * to the environment's value (name = NULL: all of them).  The op functions never read the
 * environment.  An unknown name is OXQ_ERR_ARG.  Meant for tests and for tuning runs. */
int oxq_ctx_set_tuning(oxq_ctx *ctx, const char *name, int value);
int oxq_ctx_reset_tuning(oxq_ctx *ctx, const char *name);

/* ---- opt-in weight cache behind the stateless ops -----------------------------
 * The reference's layers call the op functions with the same resident tensors on every forward
 * (linear.rs:482-533).  With this cache on, oxq_w4a16_matmul / oxq_w8a16_matmul / oxq_gptq_matmul /
 * oxq_mpp_quant_matmul remember a (qweight, qzeros, scales) triple by its device addresses: the first
 * call builds the tile-major copy that oxq_packed_quant_linear_new builds (one extra launch and a
 * hipMalloc; skipped while the stream is being captured, where the call takes its usual path) and
 * later calls run the resident-layer kernel on it, with that layer's arithmetic (few rows: unrounded
 * weights, f32 fold; above: tile GEMM on weights rounded to the activation type).  Shapes the
 * resident layout does not cover take the usual path.  The copy costs the packed tensors' size
 * again; least recently used copies go when max_bytes is reached.  oxq_gguf_quant_matmul does the
 * same for the GGUF formats that have a strip-major form (see oxq_qlinear_new) at the rows that form takes
 * (f32: 1 - 8; bf16: 1 - 32 on the matrix-core copy, there also for oxq_gguf_quant_mul_mm), keyed by the
 * address of the block bytes and the layout, with the copy that oxq_qlinear_new builds; and
 * oxq_mxfp4_moe_matmul / oxq_mxfp4_moe_gate_up_swiglu for stacked expert tensors with n a multiple of 16,
 * keyed by the addresses of blocks and scales, with the copy and the kernels of oxq_mxfp4_experts_new (the
 * SwiGLU then fused at every size).
 *
 * A copy that served a call while the stream was being captured is part of that graph: it stays, and
 * counts against max_bytes, until oxq_ctx_forget_weights or oxq_ctx_destroy frees it - either of which
 * invalidates every graph captured with it.  Dropping a copy (eviction, a smaller max_bytes, forget)
 * calls hipFree, which waits for the device: the one place where these op functions can synchronise.
 * When the weights in use need more room than max_bytes, the copies that were used within the last
 * (copies + 1) calls stay and the others run on the checkpoint layout, rather than every call rebuilding
 * a copy.
 *
 * Contract: while a triple is cached its tensors must neither change nor be freed and reused - the
 * ctx cannot see that.  Call oxq_ctx_forget_weights(ctx, qweight->data) (for a GGUF or MXFP4 weight: the
 * address of its block bytes) before doing so (NULL drops every copy).  Off by default (max_bytes = 0, or OXQ_WEIGHT_CACHE_MB in the environment).
 * No counterpart in the reference, whose ops read the checkpoint layout directly. */
int oxq_ctx_set_weight_cache(oxq_ctx *ctx, int64_t max_bytes);
int oxq_ctx_forget_weights(oxq_ctx *ctx, const void *qweight_data);
int oxq_ctx_weight_cache_bytes(const oxq_ctx *ctx, int64_t *bytes, int64_t *entries);

/* Block layout of a GGUF format: metal_ops.rs:5228-5241 (block_layout). */
int oxq_gguf_block_layout(int quant, int64_t *block_elems, int64_t *block_bytes);

/* ---- decode GEMV ops (1 <= m <= 8) ---------------------------------------
 * y[m,N] = x[m,K] . dequant(W), f32 accumulate, result in x's dtype.
 * x, scales: F16 or BF16 (same type); qweight/qzeros: I32 or U32. */

/* metal_ops.rs:1821 w4a16_matmul(x, qweight, qzeros, scales)
 * qweight [K, N/8] AWQ-interleaved, qzeros [K/g, N/8], scales [K/g, N]. */
int oxq_w4a16_matmul(oxq_ctx *ctx, void *stream, const oxq_tensor *x, const oxq_tensor *qweight,
                     const oxq_tensor *qzeros, const oxq_tensor *scales, const oxq_tensor *out);

/* No counterpart in the reference.  oxq_w4a16_matmul for callers that cannot allocate device
 * memory (code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc):
 * same arguments, checks, kernels and result bits, but the split-K partial sums go to a static
 * device array inside the library (16 MiB on every GPU the library runs on, held until the process
 * ends) instead of the ctx workspace, the K slices are always added by a second launch, and the
 * call makes no allocation of any kind.  A call whose partial sums (slices * m * N * 4 bytes) exceed
 * 16 MiB fails with OXQ_ERR_WORKSPACE and enqueues nothing; a shape whose K slices the generic kernel
 * can only add with arrival counters (N not a multiple of 4 and more than one slice) fails with
 * OXQ_ERR_UNSUPPORTED, likewise before anything is enqueued.  Every call on a GPU shares that GPU's
 * array: calls that overlap on one GPU (two streams, two threads) race; serialise them. */
int oxq_w4a16_matmul_static(oxq_ctx *ctx, void *stream, const oxq_tensor *x, const oxq_tensor *qweight,
                            const oxq_tensor *qzeros, const oxq_tensor *scales, const oxq_tensor *out);

/* metal_ops.rs:1835 w8a16_matmul: qweight [K, N/4] identity slot order. */
int oxq_w8a16_matmul(oxq_ctx *ctx, void *stream, const oxq_tensor *x, const oxq_tensor *qweight,
                     const oxq_tensor *qzeros, const oxq_tensor *scales, const oxq_tensor *out);

/* metal_ops.rs:2281 gptq_matmul(x, qweight, qzeros, scales, bits)
 * qweight [K/pf, N] sequential along K, qzeros [K/g, N/pf] (stored zero-1). */
int oxq_gptq_matmul(oxq_ctx *ctx, void *stream, const oxq_tensor *x, const oxq_tensor *qweight,
                    const oxq_tensor *qzeros, const oxq_tensor *scales, uint32_t bits,
                    const oxq_tensor *out);

/* ---- dense dequant ops: out [K, N] in the scales' dtype ------------------ */

/* metal_ops.rs:1873 dequantize_w4 */
int oxq_dequantize_w4(oxq_ctx *ctx, void *stream, const oxq_tensor *qweight,
                      const oxq_tensor *qzeros, const oxq_tensor *scales, const oxq_tensor *out);
/* metal_ops.rs:1886 dequantize_w8 */
int oxq_dequantize_w8(oxq_ctx *ctx, void *stream, const oxq_tensor *qweight,
                      const oxq_tensor *qzeros, const oxq_tensor *scales, const oxq_tensor *out);
/* metal_ops.rs:2305 dequantize_gptq_packed(qweight, qzeros, scales, bits) */
int oxq_dequantize_gptq_packed(oxq_ctx *ctx, void *stream, const oxq_tensor *qweight,
                               const oxq_tensor *qzeros, const oxq_tensor *scales, uint32_t bits,
                               const oxq_tensor *out);

/* ---- batched tile GEMM (matrix cores) ------------------------------------
 * metal_ops.rs:2748 mpp_quant_matmul / 2771 maybe_mpp_quant_matmul
 * y[m,N] = x[m,K] . dequant(W) on MFMA tiles, any m >= 1, F16 or BF16.
 * The `maybe_` form declines (returns OXQ_OK with *taken = 0, nothing
 * enqueued) when m < OXQ_MFMA_MIN_M or x is not contiguous, as the reference
 * declines below MPP_GEMM_MIN_M (metal_ops.rs:2326). */
#define OXQ_MFMA_MIN_M 9
int oxq_mpp_quant_matmul(oxq_ctx *ctx, void *stream, const oxq_tensor *x,
                         const oxq_tensor *qweight, const oxq_tensor *qzeros,
                         const oxq_tensor *scales, uint32_t bits, int pack_dim,
                         const oxq_tensor *out);
int oxq_maybe_mpp_quant_matmul(oxq_ctx *ctx, void *stream, const oxq_tensor *x,
                               const oxq_tensor *qweight, const oxq_tensor *qzeros,
                               const oxq_tensor *scales, uint32_t bits, int pack_dim,
                               const oxq_tensor *out, int *taken);

/* ---- load-time transforms into the AWQ layout ----------------------------
 * The reference runs these on the CPU while a checkpoint loads; here the
 * checkpoint tensors are already device-resident.  All outputs are caller
 * allocated.
 */

/* awq.rs:187-254 compressed_to_awq: compressed-tensors pack-quantized int4
 * (weight_packed [out, in/8] I32/U32, nibble i%8 of word (o, i/8) = q + 8;
 * weight_scale [out, groups]) -> AWQ qweight [in, out/8], qzeros
 * [groups, out/8] (all 0x88888888), scales [groups, out] of weight_scale's dtype. */
int oxq_compressed_to_awq(oxq_ctx *ctx, void *stream, const oxq_tensor *weight_packed,
                          const oxq_tensor *weight_scale, const oxq_tensor *qweight_out,
                          const oxq_tensor *qzeros_out, const oxq_tensor *scales_out);

/* awq.rs:256-323 concat_awq_along_out: fuses n_parts AWQ weights that share
 * in_features, group size and bits (QKV, gate|up) into one along the output
 * dimension.  qweights / qzeros / scales are arrays of n_parts descriptors. */
int oxq_concat_awq_along_out(oxq_ctx *ctx, void *stream, int bits, int n_parts, const oxq_tensor *qweights,
                             const oxq_tensor *qzeros, const oxq_tensor *scales, const oxq_tensor *qweight_out,
                             const oxq_tensor *qzeros_out, const oxq_tensor *scales_out);

/* awq.rs:637-742 rtn_quantize_awq: round-to-nearest 4-bit group quantization of
 * a dense [out, in] weight (F32, F16 or BF16; tied lm_head, loader.rs:1060-1076)
 * into AWQ qweight [in, out/8], qzeros [in/g, out/8] and F32 scales [in/g, out]. */
int oxq_rtn_quantize_awq(oxq_ctx *ctx, void *stream, const oxq_tensor *weight, int64_t group_size,
                         const oxq_tensor *qweight_out, const oxq_tensor *qzeros_out,
                         const oxq_tensor *scales_out);

/* gguf_weights.rs:255-291 depermute_qk_rows: undoes the per-head row interleave
 * llama.cpp's converter applies to the q/k projections of Llama-family models
 * (HF row r of a head is stored at row 2 (r % (head_dim/2)) + r / (head_dim/2));
 * a row-wise byte shuffle valid for every block format.  `out` must not alias
 * `weight_bytes`. */
int oxq_gguf_depermute_qk_rows(oxq_ctx *ctx, void *stream, const oxq_tensor *weight_bytes, int64_t in_features,
                               int64_t out_features, int quant, int64_t n_heads, int64_t head_dim,
                               const oxq_tensor *out);

/* ---- block-scaled F8E4M3 (fn variant) ------------------------------------
 * Weight: U8 [out, in] holding E4M3 encodings (1 sign, 4 exponent bits with
 * bias 7, 3 mantissa bits; S.1111.111 is NaN, no infinity); scales: F32
 * [s_rows, s_cols] grid tiling it evenly.  A weight value is
 * bf16(f32(bf16(f8)) * scale) (quant_kernels.metal:3877-3911).
 */

/* metal_ops.rs:5562 cast_f8e4m3_to_f32: elementwise widening, any shape. */
int oxq_cast_f8e4m3_to_f32(oxq_ctx *ctx, void *stream, const oxq_tensor *t, const oxq_tensor *out);

/* metal_ops.rs:5809 f8_block_dequant_bf16: dense BF16 [out, in]. */
int oxq_f8_block_dequant_bf16(oxq_ctx *ctx, void *stream, const oxq_tensor *bytes,
                              const oxq_tensor *scales, const oxq_tensor *out);

/* metal_ops.rs:5788 f8_gemv: x BF16 [m, in], 1 <= m <= 8 -> BF16 [m, out]. */
int oxq_f8_gemv(oxq_ctx *ctx, void *stream, const oxq_tensor *x, const oxq_tensor *bytes,
                const oxq_tensor *scales, const oxq_tensor *out);

/* moe.rs:106-113 Fp8Cached::forward: any m (GEMV up to 8 rows, tile matmul beyond). */
int oxq_f8_matmul(oxq_ctx *ctx, void *stream, const oxq_tensor *x, const oxq_tensor *bytes,
                  const oxq_tensor *scales, const oxq_tensor *out);

/* ---- GGUF block-quant ops -------------------------------------------------
 * weight_bytes: U8 [N * K/block_elems * block_bytes], row n = consecutive
 * ggml blocks.  x and out: BF16 (the reference's contract) or F32 (the
 * benchmark's f32-activation configuration); x and out share a dtype. */

/* metal_ops.rs:5819 gguf_quant_matmul: 1 <= m <= 8 */
int oxq_gguf_quant_matmul(oxq_ctx *ctx, void *stream, const oxq_tensor *x,
                          const oxq_tensor *weight_bytes, int64_t in_features,
                          int64_t out_features, int quant, const oxq_tensor *out);
/* metal_ops.rs:5973 gguf_quant_mul_mm: any m */
int oxq_gguf_quant_mul_mm(oxq_ctx *ctx, void *stream, const oxq_tensor *x,
                          const oxq_tensor *weight_bytes, int64_t in_features,
                          int64_t out_features, int quant, const oxq_tensor *out);
/* Dense dequant [N, K] f32 of a GGUF weight (no reference op: the reference
 * tests compare against candle's QTensor::dequantize, metal_ops.rs:6405-6417;
 * this exposes the kernels' own decode so it can be checked bit for bit). */
int oxq_gguf_dequantize(oxq_ctx *ctx, void *stream, const oxq_tensor *weight_bytes,
                        int64_t in_features, int64_t out_features, int quant,
                        const oxq_tensor *out);

/* ---- MXFP4 ----------------------------------------------------------------
 * metal_ops.rs:6197 mxfp4_matmul(x, blocks, scales, k, n): x/out BF16,
 * blocks U8 [n*k/32*16], scales U8 [n*k/32], any m >= 1 (gemv kernel for
 * m <= 8, tiled beyond, metal_ops.rs:6204-6222). */
int oxq_mxfp4_matmul(oxq_ctx *ctx, void *stream, const oxq_tensor *x, const oxq_tensor *blocks,
                     const oxq_tensor *scales, int64_t k, int64_t n, const oxq_tensor *out);
/* Dense dequant [n, k] f32 (device twin of mxfp4.rs:35 dequantize_mxfp4_f32). */
int oxq_mxfp4_dequantize(oxq_ctx *ctx, void *stream, const oxq_tensor *blocks,
                         const oxq_tensor *scales, int64_t k, int64_t n, const oxq_tensor *out);

/* Grouped expert GEMV: every active expert of one MoE projection in a single
 * launch.  Stands in for the per-expert loop of moe.rs:593-605 over
 * Mxfp4Linear::forward (mxfp4.rs:119-154).
 *  x           BF16 [n_tokens, k]           (gather_rows != 0) or
 *              BF16 [n_pairs, k]            (gather_rows == 0: row i is pair i)
 *  blocks      U8 [n_experts, n, k/32, 16]; scales U8 [n_experts, n, k/32]
 *  bias        BF16 [n_experts, n] or NULL
 *  expert_offsets I32 [n_experts + 1]: pairs of expert e are
 *              [offsets[e], offsets[e+1]) in token_ids / out rows
 *  token_ids   I32 [n_pairs]: source row of x for each pair (gather_rows != 0)
 *  out         BF16 [n_pairs, n]: out[p] = x[row(p)] . W_e^T + bias_e */
int oxq_mxfp4_moe_matmul(oxq_ctx *ctx, void *stream, const oxq_tensor *x,
                         const oxq_tensor *blocks, const oxq_tensor *scales,
                         const oxq_tensor *bias, const oxq_tensor *expert_offsets,
                         const oxq_tensor *token_ids, int gather_rows, int64_t k, int64_t n,
                         const oxq_tensor *out);

/* The gate_up projection of every active GPT-OSS expert followed by the clamped SwiGLU over its
 * interleaved (gate, up) output rows (moe.rs:152-173: rows 2c and 2c + 1 give output c), in one launch:
 * arguments as oxq_mxfp4_moe_matmul, out BF16 [n_pairs, n / 2].  Both factors are rounded to BF16 before
 * the activation, so the result equals oxq_mxfp4_moe_matmul + oxq_gated_activation(OXQ_ACT_GPT_OSS_SWIGLU)
 * bit for bit.  *fused = 1 when the launch was enqueued; *fused = 0 with OXQ_OK and nothing enqueued when
 * this problem size runs on a kernel without the fused epilogue (many pairs per expert go to the tile
 * matmul): make the two calls instead. */
int oxq_mxfp4_moe_gate_up_swiglu(oxq_ctx *ctx, void *stream, const oxq_tensor *x, const oxq_tensor *blocks,
                                 const oxq_tensor *scales, const oxq_tensor *bias,
                                 const oxq_tensor *expert_offsets, const oxq_tensor *token_ids, int gather_rows,
                                 int64_t k, int64_t n, float limit, const oxq_tensor *out, int *fused);

/* ---- resident MXFP4 experts ---------------------------------------------------
 * moe.rs:366-417 (load_gpt_oss keeps the stacked tensors of a projection, [E, n, k/32, 16] blocks and
 * [E, n, k/32] scales, for the life of the model) and moe.rs:563-607 (dispatch_sparse runs them).
 * `new` is the load-time step: when n is a multiple of 16 it builds a tile-major copy in device memory
 * owned by the handle (matrix-core operand order, one contiguous run per 16 rows; the checkpoint tensors'
 * size plus at most one block in four per row) and synchronises the null stream once; every call then
 * runs on that copy: the decode GEMV below three pairs an expert on average, tiles of 16 - 128 of an expert's
 * pairs above, both with the fused SwiGLU.  The caller's tensors are borrowed and must outlive the handle:
 * shapes that do not qualify (and an x of 2 GiB or more) run on them, with the stateless ops' kernels.
 * OXQ_PREPACK=0 in the environment disables the copy. */
typedef struct oxq_mxfp4_experts oxq_mxfp4_experts;
int oxq_mxfp4_experts_new(oxq_ctx *ctx, const oxq_tensor *blocks, const oxq_tensor *scales,
                          const oxq_tensor *bias_or_null, int64_t n_experts, int64_t k, int64_t n,
                          oxq_mxfp4_experts **out);
/* Arguments and result of oxq_mxfp4_moe_matmul without the weight tensors. */
int oxq_mxfp4_experts_matmul(oxq_mxfp4_experts *experts, void *stream, const oxq_tensor *x,
                             const oxq_tensor *expert_offsets, const oxq_tensor *token_ids, int gather_rows,
                             const oxq_tensor *out);
/* Arguments and result of oxq_mxfp4_moe_gate_up_swiglu without the weight tensors. */
int oxq_mxfp4_experts_gate_up_swiglu(oxq_mxfp4_experts *experts, void *stream, const oxq_tensor *x,
                                     const oxq_tensor *expert_offsets, const oxq_tensor *token_ids,
                                     int gather_rows, float limit, const oxq_tensor *out, int *fused);
/* *resident = 1 if decode sizes run on the handle's own tile-major copy. */
int oxq_mxfp4_experts_is_resident(const oxq_mxfp4_experts *experts, int *resident);
/* Dense dequant [n, k] F32 of one expert, read back from what the GEMV streams (the copy, if there is one). */
int oxq_mxfp4_experts_dequantize(oxq_mxfp4_experts *experts, void *stream, int64_t expert, const oxq_tensor *out);
void oxq_mxfp4_experts_free(oxq_mxfp4_experts *experts);

/* ---- mixture-of-experts glue: the steps either side of the expert GEMVs -----
 * The reference does these on the host / with one launch per expert
 * (moe.rs:466-607); here they run on the device and feed oxq_mxfp4_moe_matmul. */

/* moe.rs:466-486 + linear.rs:160-171: softmax over experts in f32, stable
 * descending top-k, optional renormalisation by the sum of the chosen.
 *  logits    F32 | F16 | BF16 [n_tokens, n_experts]
 *  top_idx   I32 [n_tokens, top_k] (out)    top_vals  F32 [n_tokens, top_k] (out);  top_k <= 64 */
int oxq_moe_route(oxq_ctx *ctx, void *stream, const oxq_tensor *logits, int64_t top_k, int norm_topk,
                  const oxq_tensor *top_idx, const oxq_tensor *top_vals);

/* moe.rs:563-590 dispatch_sparse: (token, slot) pairs grouped by expert, tokens
 * ascending inside an expert.  P = n_tokens * top_k; n_experts <= 256.
 *  expert_offsets I32 [n_experts + 1]   token_ids I32 [P]   pair_weights F32 [P]
 *  pair_pos       I32 [n_tokens, top_k]: where pair (token, slot) went (for the combine) */
int oxq_moe_group(oxq_ctx *ctx, void *stream, const oxq_tensor *top_idx, const oxq_tensor *top_vals,
                  int64_t n_experts, const oxq_tensor *expert_offsets, const oxq_tensor *token_ids,
                  const oxq_tensor *pair_weights, const oxq_tensor *pair_pos);

/* oxq_moe_route followed by oxq_moe_group (n_experts = logits' second dim) as one call, same arguments and
 * outputs; up to 64 (token, slot) pairs and 256 experts, i.e. decode, it is one launch instead of two. */
int oxq_moe_route_group(oxq_ctx *ctx, void *stream, const oxq_tensor *logits, int64_t top_k, int norm_topk,
                        const oxq_tensor *top_idx, const oxq_tensor *top_vals, const oxq_tensor *expert_offsets,
                        const oxq_tensor *token_ids, const oxq_tensor *pair_weights, const oxq_tensor *pair_pos);

typedef enum oxq_gated_act {
    OXQ_ACT_GATED_SILU = 0,      /* [.., gate | up]: silu(gate) * up, ffn_kernels.metal:19-68 */
    OXQ_ACT_GATED_GELU_TANH = 1, /* [.., gate | up]: gelu_tanh(gate) * up, ffn_kernels.metal:115-160 */
    OXQ_ACT_GPT_OSS_SWIGLU = 2   /* interleaved (gate, up), clamped, alpha 1.702: moe.rs:152-173 */
} oxq_gated_act;

/* gate_up [rows, 2*I] -> out [rows, I], same dtype (F32 | F16 | BF16); f32 math, one
 * rounding.  `limit` is only read by OXQ_ACT_GPT_OSS_SWIGLU. */
int oxq_gated_activation(oxq_ctx *ctx, void *stream, const oxq_tensor *gate_up, int kind, float limit,
                         const oxq_tensor *out);

/* metal_ops.rs:1252 silu_mul_fused and :1271 gelu_tanh_mul_fused (kernels ffn_kernels.metal:72-110 and
 * 164-200), the GateUpProjection::Separate arm of ffn.rs:386-413: out = act(gate) * up elementwise over
 * two tensors of one dtype (F32 | F16 | BF16) and one element count; f32 math, one rounding.  `kind` is
 * OXQ_ACT_GATED_SILU or OXQ_ACT_GATED_GELU_TANH.  Gives the bits of oxq_gated_activation on [gate | up]. */
int oxq_activation_mul(oxq_ctx *ctx, void *stream, const oxq_tensor *gate, const oxq_tensor *up, int kind,
                       const oxq_tensor *out);

/* moe.rs:592-605: out[token] = sum over slots of top_vals[token, slot] *
 * expert_out[pair_pos[token, slot]]  (f32 accumulation in slot order, one rounding).
 *  expert_out T [P, hidden]   out T [n_tokens, hidden] */
int oxq_moe_combine(oxq_ctx *ctx, void *stream, const oxq_tensor *expert_out, const oxq_tensor *pair_pos,
                    const oxq_tensor *top_vals, const oxq_tensor *out);

/* ---- layers ----------------------------------------------------------------
 * Host-side mirrors of the reference layer types; they hold descriptors of
 * caller-owned resident weights and route by m exactly where the reference
 * routes.  `x` may have any leading dims; m is their product. */

/* linear.rs:403-534 PackedQuantLinear::{new, forward}.  scales must already be
 * in the runtime dtype (`dtype`), as after the cast at linear.rs:437.
 *
 * Like the reference's constructor, `new` is the load-time step: for layers
 * with in_features and group size multiples of 128, out_features a multiple
 * of 64 and at most 128 groups it builds a tile-major copy of qweight/qzeros/scales in device memory owned by
 * the layer (same size as the checkpoint tensors, plus 1.5 bytes per column
 * and 128 rows; strips of 64 output columns, or of 16 for 4-bit layers of at
 * most 8192 columns and 4096 - 14336 rows, such as attention and down projections) and forward never reads the caller's tensors again; it
 * synchronises the null stream once.  Other layers keep descriptors of the
 * caller-owned tensors.  OXQ_PREPACK=0 in the environment disables the copy. */
typedef struct oxq_packed_quant_linear oxq_packed_quant_linear;
int oxq_packed_quant_linear_new(oxq_ctx *ctx, uint32_t bits, int pack_dim,
                                const oxq_tensor *qweight, const oxq_tensor *qzeros,
                                const oxq_tensor *scales, const oxq_tensor *bias_or_null,
                                int dtype, oxq_packed_quant_linear **out);
/* ffn.rs:386-400 FeedForward::forward, GateUpProjection::Fused arm: the fused gate|up projection
 * (qweight etc. of out_features = 2 * intermediate, gate columns first, as concat_awq_along_out builds
 * it) followed by gated_silu_fused / gated_gelu_tanh_fused (metal_ops.rs, ffn_kernels.metal:19-160),
 * in one launch.  forward writes act(gate(x)) * up(x), [.., intermediate], and out_features reports
 * intermediate; both factors are rounded to `dtype` before the activation, so the result equals
 * oxq_packed_quant_linear_forward followed by oxq_gated_activation bit for bit.  `act` is
 * OXQ_ACT_GATED_SILU or OXQ_ACT_GATED_GELU_TANH.  Only layers that qualify for the resident copy
 * (see above) can be built this way; others return OXQ_ERR_UNSUPPORTED and take the two calls. */
int oxq_packed_quant_linear_new_gate_up(oxq_ctx *ctx, uint32_t bits, int pack_dim, const oxq_tensor *qweight,
                                        const oxq_tensor *qzeros, const oxq_tensor *scales,
                                        const oxq_tensor *bias_or_null, int act, int dtype,
                                        oxq_packed_quant_linear **out);
int oxq_packed_quant_linear_forward(oxq_packed_quant_linear *layer, void *stream,
                                    const oxq_tensor *x, const oxq_tensor *out);
int oxq_packed_quant_linear_in_features(const oxq_packed_quant_linear *layer, int64_t *k);
int oxq_packed_quant_linear_out_features(const oxq_packed_quant_linear *layer, int64_t *n);
/* *prepacked = 1 if forward runs on the layer-owned tile-major copy. */
int oxq_packed_quant_linear_is_prepacked(const oxq_packed_quant_linear *layer, int *prepacked);
/* linear.rs:510-523: dense dequant of the layer's weights, out = [in, out]
 * in the layer dtype; element-for-element what forward feeds the matrix cores. */
int oxq_packed_quant_linear_dequantize(oxq_packed_quant_linear *layer, void *stream,
                                       const oxq_tensor *out);
void oxq_packed_quant_linear_free(oxq_packed_quant_linear *layer);

/* linear.rs:179-393 QLinear / GgufFastPath::{build, forward_decode, forward_prefill}. */
typedef struct oxq_qlinear oxq_qlinear;
int oxq_qlinear_new(oxq_ctx *ctx, int quant, const oxq_tensor *weight_bytes, int64_t in_features,
                    int64_t out_features, const oxq_tensor *bias_or_null, int out_dtype,
                    oxq_qlinear **out);
/* ffn.rs:307-373, 386-413: the fused gate|up projection of a block-quantized FFN (GateUpProjection::Packed: rows
 * 0 .. I - 1 of weight_bytes are gate_proj, I .. 2I - 1 up_proj; a loader fuses separate ffn_gate / ffn_up tensors
 * by concatenating their bytes) with gated_silu_fused / gated_gelu_tanh_fused (ffn_kernels.metal:19-160) run in the
 * matmul's epilogue: out_features = 2I, forward writes [.., I] = act(gate(x)) * up(x), bit for bit what
 * oxq_gated_activation gives on the plain layer's output.  Needs a BF16 layer that takes the matrix-core copy (see
 * oxq_qlinear_is_resident below), else OXQ_ERR_UNSUPPORTED.  Every row count runs in one launch: up to 32 rows
 * the integer kernel of the copy; above that, where enough workgroups of 64 rows fill the chip, the copy's prefill
 * kernel (the plain layer takes the same kernel at the same sizes: the same bits); otherwise row tiles of 32 that
 * each read the weights again (with the unrounded weights that the plain layer's tile matmul rounds to bf16) -
 * oxq_mlp_forward sends those row counts (more than OXQ_GGUF_FUSED_ACT_ROWS where the prefill kernel does not take
 * the call) through the plain layer's path and the activation by itself, so that a FeedForward over this layer
 * gives the plain layers' bits at every row count. */
#define OXQ_GGUF_FUSED_ACT_ROWS 32
int oxq_qlinear_new_gate_up(oxq_ctx *ctx, int quant, const oxq_tensor *weight_bytes, int64_t in_features,
                            int64_t out_features, const oxq_tensor *bias_or_null, int act, int out_dtype,
                            oxq_qlinear **out);
int oxq_qlinear_forward(oxq_qlinear *layer, void *stream, const oxq_tensor *x,
                        const oxq_tensor *out);
/* linear.rs:225-240 (the fast path's own copy of the block bytes).  For layers of any of the ten formats
 * with out_features % 16 == 0 and in_features a multiple of 128 (256 for the K-quants) oxq_qlinear_new
 * builds a layer-owned copy of the blocks in strips of 16 rows (the file's bytes per weight; Q3_K: 112 for
 * 110 bytes a super-block; so twice the
 * layer's bytes while the caller keeps weight_bytes); forward then runs 1 - 4 rows of x on that copy (f32
 * rows up to 8, in two passes of four) and everything else on weight_bytes as before.  A BF16 layer of Q4_0,
 * Q4_1, Q5_0, Q5_1, Q8_0, Q4_K, Q5_K or Q6_K holds the copy in the matrix-core layout instead (the same size), on
 * which one launch takes 1 - 32 rows with the GEMV's arithmetic at every
 * row count: integer sums, one f32 scale per sub-block, the weights never rounded to bf16 (the reference's
 * prefill tiles round them above 8 rows).  The tuning switch OXQ_PREPACK=0 turns the copy off, OXQ_GGUF_MFMA=0
 * keeps the first layout for BF16 layers too.
 * *resident = 1 if the layer holds the copy. */
int oxq_qlinear_is_resident(const oxq_qlinear *layer, int *resident);
/* Dense f32 [out_features, in_features] of the layer's weights, read from the copy when there is one:
 * bit for bit what oxq_gguf_dequantize returns for weight_bytes. */
int oxq_qlinear_dequantize(oxq_qlinear *layer, void *stream, const oxq_tensor *out);
void oxq_qlinear_free(oxq_qlinear *layer);

/* mxfp4.rs:67-169 Mxfp4Linear::{new, forward}. */
typedef struct oxq_mxfp4_linear oxq_mxfp4_linear;
int oxq_mxfp4_linear_new(oxq_ctx *ctx, const oxq_tensor *blocks, const oxq_tensor *scales,
                         const oxq_tensor *bias_or_null, int64_t in_features,
                         int64_t out_features, oxq_mxfp4_linear **out);
int oxq_mxfp4_linear_forward(oxq_mxfp4_linear *layer, void *stream, const oxq_tensor *x,
                             const oxq_tensor *out);
void oxq_mxfp4_linear_free(oxq_mxfp4_linear *layer);

/* ffn.rs:22-474 FeedForward (the gated MLP) over the quantized arms of AnyLinear (linear.rs:536-542):
 * down(act(gate(x)) * up(x)).  The MLP borrows its projections: they must outlive it. */
typedef enum oxq_linear_kind {
    OXQ_LINEAR_PACKED_QUANT = 0, /* oxq_packed_quant_linear* */
    OXQ_LINEAR_GGUF = 1,         /* oxq_qlinear* */
    OXQ_LINEAR_MXFP4 = 2         /* oxq_mxfp4_linear* */
} oxq_linear_kind;
typedef struct oxq_any_linear {
    int kind; /* oxq_linear_kind */
    void *layer;
} oxq_any_linear;
typedef enum oxq_gate_up_kind {
    OXQ_GATE_UP_FUSED = 0,    /* ffn.rs GateUpProjection::Fused and ::Packed: one projection, [gate | up] columns;
                               * a layer from oxq_packed_quant_linear_new_gate_up runs the activation in its matmul */
    OXQ_GATE_UP_SEPARATE = 1, /* ::Separate: gate_proj and up_proj, then silu_mul / gelu_tanh_mul */
    OXQ_GATE_UP_SIMPLE = 2    /* ::Simple: ungated, act(up(x)) */
} oxq_gate_up_kind;
typedef struct oxq_mlp oxq_mlp;
/* `a` is gate_up_proj (FUSED), gate_proj (SEPARATE) or up_proj (SIMPLE); `b` is up_proj for SEPARATE and NULL
 * otherwise.  Shape checks as ffn.rs:227-233, 255-261, 270-276, 323-346.  `activation` is
 * OXQ_ACT_GATED_SILU or OXQ_ACT_GATED_GELU_TANH. */
int oxq_mlp_new(oxq_ctx *ctx, int gate_up_kind, const oxq_any_linear *a, const oxq_any_linear *b_or_null,
                const oxq_any_linear *down, int64_t intermediate, int activation, oxq_mlp **out);
/* Elements (of the projections' output dtype) that forward needs in `scratch` for `rows` rows of x. */
int oxq_mlp_scratch_elems(const oxq_mlp *mlp, int64_t rows, int64_t *elems);
/* ffn.rs:386-474 FeedForward::forward.  x [.., in_features] -> out [.., out_features]; the
 * intermediates live in the caller's `scratch`, nothing is allocated. */
int oxq_mlp_forward(oxq_mlp *mlp, void *stream, const oxq_tensor *x, const oxq_tensor *scratch,
                    const oxq_tensor *out);
int oxq_mlp_in_features(const oxq_mlp *mlp, int64_t *k);
int oxq_mlp_out_features(const oxq_mlp *mlp, int64_t *n);
void oxq_mlp_free(oxq_mlp *mlp);

#ifdef __cplusplus
}
#endif
#endif /* OXQ_H */
