// Host side of the C ABI: context, argument validation (device-free, mirrors
// the reference's checks in src/common/metal_ops.rs before every dispatch) and
// routing to the kernel launchers.

#include "oxq_internal.hpp"
#include "oxq_bench.h"

#include <cstdlib>
#include <new>
#include <vector>

namespace oxq {

static thread_local char g_last_error[512] = "";

int fail(int status, const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_last_error, sizeof g_last_error, fmt, ap);
    va_end(ap);
    return status;
}

const char *dtype_name(int dtype) {
    switch (dtype) {
    case OXQ_F32: return "F32";
    case OXQ_F16: return "F16";
    case OXQ_BF16: return "BF16";
    case OXQ_U8: return "U8";
    case OXQ_I32: return "I32";
    case OXQ_U32: return "U32";
    case OXQ_I64: return "I64";
    default: return "?";
    }
}

void set_plan(oxq_ctx *ctx, const char *kernel, dim3 grid, dim3 block, uint32_t split_k,
              uint32_t launches, uint64_t ws_bytes) {
    oxq_plan &pl = ctx->plan;
    memset(&pl, 0, sizeof pl);
    snprintf(pl.kernel, sizeof pl.kernel, "%s", kernel);
    pl.grid[0] = grid.x; pl.grid[1] = grid.y; pl.grid[2] = grid.z;
    pl.block[0] = block.x; pl.block[1] = block.y; pl.block[2] = block.z;
    pl.split_k = split_k;
    pl.launches = launches;
    pl.workspace_bytes = ws_bytes;
}

void add_launch(oxq_ctx *ctx) { ctx->plan.launches++; }

static void dims_str(const oxq_tensor *t, char *buf, size_t n) {
    size_t off = 0;
    off += snprintf(buf + off, n - off, "[");
    for (int i = 0; i < t->rank && off < n; ++i)
        off += snprintf(buf + off, n - off, "%s%lld", i ? ", " : "", (long long)t->dims[i]);
    if (off < n) snprintf(buf + off, n - off, "]");
}

// Basic descriptor sanity + residency.  `op` prefixes the message.
static int check_tensor(const oxq_ctx *ctx, const char *op, const char *what, const oxq_tensor *t) {
    if (!t) return fail(OXQ_ERR_ARG, "%s: %s is NULL", op, what);
    if (t->rank < 1 || t->rank > OXQ_MAX_RANK)
        return fail(OXQ_ERR_SHAPE, "%s: %s rank %d out of [1, %d]", op, what, t->rank, OXQ_MAX_RANK);
    for (int i = 0; i < t->rank; ++i)
        if (t->dims[i] < 0) return fail(OXQ_ERR_SHAPE, "%s: %s has a negative dim", op, what);
    if (dtype_size(t->dtype) == 0) return fail(OXQ_ERR_DTYPE, "%s: %s has an unknown dtype", op, what);
    if (t->device == OXQ_DEVICE_HOST)
        return fail(OXQ_ERR_DEVICE,
                    "%s: %s must be GPU-resident (HIP-only path; host tensors go through the CPU "
                    "dequantize path)", op, what);
    if (!ctx->plan_only) {
        if (t->device != ctx->device)
            return fail(OXQ_ERR_DEVICE, "%s: %s is on device %d, ctx is on device %d", op, what,
                        t->device, ctx->device);
        if (!t->data && numel(t) > 0) return fail(OXQ_ERR_ARG, "%s: %s has a NULL data pointer", op, what);
    }
    return OXQ_OK;
}

#define OXQ_TRY(expr)              \
    do {                           \
        int _rc = (expr);          \
        if (_rc != OXQ_OK) return _rc; \
    } while (0)

static bool is_packed_dtype(int dt) { return dt == OXQ_I32 || dt == OXQ_U32; }
static bool is_float_dtype(int d) { return d == OXQ_F32 || d == OXQ_F16 || d == OXQ_BF16; }

// Validation shared by the AWQ/GPTQ GEMV, dequant and tile-GEMM ops.
// Order follows W4A16Matmul::metal_fwd (metal_ops.rs:1506-1566),
// GptqMatmul::metal_fwd (1975-2044), DequantizeW4 (1736-1754),
// DequantizeGptqPacked (2187-2214) and MppQuantMatmul (2631-2684).
enum Wna16Kind { KIND_GEMV, KIND_DEQUANT, KIND_TILE };

static int check_wna16(oxq_ctx *ctx, const char *op, Wna16Kind kind, const oxq_tensor *x,
                       const oxq_tensor *qweight, const oxq_tensor *qzeros,
                       const oxq_tensor *scales, uint32_t bits, int pack_dim,
                       const oxq_tensor *out, Wna16Problem *p) {
    if (!ctx) return fail(OXQ_ERR_ARG, "%s: ctx is NULL", op);
    if (bits != 4 && bits != 8)
        return fail(OXQ_ERR_BITS, "%s: bits must be 4 or 8, got %u", op, bits);
    if (pack_dim != OXQ_PACK_OUT && pack_dim != OXQ_PACK_IN)
        return fail(OXQ_ERR_ARG, "%s: bad pack_dim %d", op, pack_dim);
    if (kind != KIND_DEQUANT) OXQ_TRY(check_tensor(ctx, op, "x", x));
    OXQ_TRY(check_tensor(ctx, op, "qweight", qweight));
    OXQ_TRY(check_tensor(ctx, op, "qzeros", qzeros));
    OXQ_TRY(check_tensor(ctx, op, "scales", scales));
    OXQ_TRY(check_tensor(ctx, op, "out", out));
    char b0[96], b1[96];

    int64_t m = 1, in_features = 0;
    if (kind != KIND_DEQUANT) {
        if (!x->contiguous) return fail(OXQ_ERR_CONTIGUOUS, "%s: x must be contiguous", op);
        dims_str(x, b0, sizeof b0);
        if (x->rank != 2) return fail(OXQ_ERR_SHAPE, "%s: x must be 2-D [m, in], got %s", op, b0);
        if (kind == KIND_GEMV && !(x->dims[0] >= 1 && x->dims[0] <= 8))
            return fail(OXQ_ERR_M_RANGE,
                        "%s: x must be [m, in] with m in 1..=8 (decode GEMV path), got %s", op, b0);
        if (x->dims[0] < 1) return fail(OXQ_ERR_SHAPE, "%s: x has no rows, got %s", op, b0);
        m = x->dims[0];
        in_features = x->dims[1];
    } else if (!qweight->contiguous) {
        return fail(OXQ_ERR_CONTIGUOUS, "%s: qweight must be contiguous", op);
    }
    if (qweight->rank != 2)
        return fail(OXQ_ERR_SHAPE, "%s: qweight must be 2-D", op);
    if (scales->rank != 2) return fail(OXQ_ERR_SHAPE, "%s: scales must be 2-D [groups, out]", op);
    if (!is_packed_dtype(qweight->dtype) || !is_packed_dtype(qzeros->dtype))
        return fail(OXQ_ERR_DTYPE, "%s: qweight/qzeros must be I32 or U32, got %s/%s", op,
                    dtype_name(qweight->dtype), dtype_name(qzeros->dtype));
    if (!qweight->contiguous || !qzeros->contiguous || !scales->contiguous)
        return fail(OXQ_ERR_CONTIGUOUS, "%s: qweight, qzeros and scales must be contiguous", op);

    const int64_t pf = 32 / bits;
    const int64_t groups = scales->dims[0], out_features = scales->dims[1];
    int64_t K;
    if (pack_dim == OXQ_PACK_OUT) {
        const int64_t qw_in = qweight->dims[0], packed_out = qweight->dims[1];
        if (qzeros->rank != 2 || qzeros->dims[0] != groups || qzeros->dims[1] != packed_out) {
            dims_str(qzeros, b0, sizeof b0);
            return fail(OXQ_ERR_SHAPE, "%s: qzeros shape %s != [%lld, %lld]", op, b0,
                        (long long)groups, (long long)packed_out);
        }
        // AwqShape::new_bits (metal_ops.rs:1434-1458)
        if (packed_out * pf != out_features)
            return fail(OXQ_ERR_SHAPE, "W%uA16: qweight packed_out %lld (x%lld) != scales out %lld",
                        bits, (long long)packed_out, (long long)pf, (long long)out_features);
        if (groups == 0 || qw_in % groups != 0)
            return fail(OXQ_ERR_GROUP, "W%uA16: in_features %lld not divisible by groups %lld", bits,
                        (long long)qw_in, (long long)groups);
        K = qw_in;
    } else {
        const int64_t packed_in = qweight->dims[0], qw_out = qweight->dims[1];
        if (qw_out != out_features)
            return fail(OXQ_ERR_SHAPE, "%s: qweight dim1 %lld != scales out_features %lld", op,
                        (long long)qw_out, (long long)out_features);
        if (qzeros->rank != 2 || qzeros->dims[0] != groups || qzeros->dims[1] * pf != out_features) {
            dims_str(qzeros, b0, sizeof b0);
            return fail(OXQ_ERR_SHAPE, "%s: qzeros shape %s != [%lld, %lld]", op, b0,
                        (long long)groups, (long long)(out_features / pf));
        }
        // GptqShape::new_bits (metal_ops.rs:1923-1943)
        K = packed_in * pf;
        if (groups == 0 || K % groups != 0)
            return fail(OXQ_ERR_GROUP, "GPTQ-W%uA16: in_features %lld not divisible by groups %lld",
                        bits, (long long)K, (long long)groups);
        if (out_features % pf != 0)
            return fail(OXQ_ERR_SHAPE,
                        "GPTQ-W%uA16: out_features %lld not divisible by pack_factor %lld", bits,
                        (long long)out_features, (long long)pf);
    }
    const int64_t group_size = K / groups;
    if (kind != KIND_DEQUANT && in_features != K)
        return fail(OXQ_ERR_SHAPE, "%s: x in_features %lld != weight in_features %lld", op,
                    (long long)in_features, (long long)K);
    dims_str(out, b1, sizeof b1);
    if (kind == KIND_DEQUANT) {
        if (out->rank != 2 || out->dims[0] != K || out->dims[1] != out_features)
            return fail(OXQ_ERR_SHAPE, "%s: output shape %s != [%lld, %lld]", op, b1, (long long)K,
                        (long long)out_features);
    } else if (out->rank != 2 || out->dims[0] != m || out->dims[1] != out_features) {
        return fail(OXQ_ERR_SHAPE, "%s: output shape %s != [%lld, %lld]", op, b1, (long long)m,
                    (long long)out_features);
    }
    if (!out->contiguous) return fail(OXQ_ERR_CONTIGUOUS, "%s: out must be contiguous", op);
    const int act = kind == KIND_DEQUANT ? scales->dtype : x->dtype;
    if (kind != KIND_DEQUANT && scales->dtype != x->dtype)
        return fail(OXQ_ERR_DTYPE, "%s: scales dtype %s must match x dtype %s", op,
                    dtype_name(scales->dtype), dtype_name(x->dtype));
    if (act != OXQ_F16 && act != OXQ_BF16)
        return fail(OXQ_ERR_DTYPE, "%s: unsupported (bits, dtype) combo (%u, %s)", op, bits,
                    dtype_name(act));
    if (out->dtype != act)
        return fail(OXQ_ERR_DTYPE, "%s: out dtype %s must be %s", op, dtype_name(out->dtype),
                    dtype_name(act));
    if (!is_pow2(group_size))
        return fail(OXQ_ERR_GROUP, "%s: group_size %lld must be a power of two", op,
                    (long long)group_size);
    if (pack_dim == OXQ_PACK_IN && group_size % pf != 0)
        return fail(OXQ_ERR_GROUP, "%s: group_size %lld must be a multiple of pack_factor %lld", op,
                    (long long)group_size, (long long)pf);
    if (K > INT32_MAX || out_features > INT32_MAX || m > INT32_MAX)
        return fail(OXQ_ERR_SHAPE, "%s: dimension exceeds 2^31-1", op);

    p->x = x ? x->data : nullptr;
    p->qweight = (const uint32_t *)qweight->data;
    p->qzeros = (const uint32_t *)qzeros->data;
    p->scales = scales->data;
    p->bias = nullptr;
    p->y = out->data;
    p->M = m;
    p->K = K;
    p->N = out_features;
    p->group_size = group_size;
    p->group_shift = ilog2(group_size);
    p->bits = (int)bits;
    p->pack_dim = pack_dim;
    p->dtype = act;
    return OXQ_OK;
}

static int check_bias(const oxq_ctx *ctx, const char *op, const oxq_tensor *bias, int64_t n, int dtype) {
    if (!bias) return OXQ_OK;
    OXQ_TRY(check_tensor(ctx, op, "bias", bias));
    if (numel(bias) != n || !bias->contiguous)
        return fail(OXQ_ERR_SHAPE, "%s: bias must be a contiguous [%lld] tensor", op, (long long)n);
    if (bias->dtype != dtype)
        return fail(OXQ_ERR_DTYPE, "%s: bias dtype %s must be %s", op, dtype_name(bias->dtype),
                    dtype_name(dtype));
    return OXQ_OK;
}

// ---- GGUF -------------------------------------------------------------------
static const char *gguf_name(int q) {
    switch (q) {
    case OXQ_GGUF_Q4_0: return "Q4_0";
    case OXQ_GGUF_Q8_0: return "Q8_0";
    case OXQ_GGUF_Q4_K: return "Q4K";
    case OXQ_GGUF_Q6_K: return "Q6K";
    case OXQ_GGUF_Q4_1: return "Q4_1";
    case OXQ_GGUF_Q5_0: return "Q5_0";
    case OXQ_GGUF_Q5_1: return "Q5_1";
    case OXQ_GGUF_Q2_K: return "Q2K";
    case OXQ_GGUF_Q3_K: return "Q3K";
    case OXQ_GGUF_Q5_K: return "Q5K";
    default: return "?";
    }
}

// GgufQuantMatmul::metal_fwd (metal_ops.rs:5357-5431) / GgufQuantMulMM (5872-5919).
static int check_gguf(oxq_ctx *ctx, const char *op, bool decode, bool dequant, const oxq_tensor *x,
                      const oxq_tensor *w, int64_t in_features, int64_t out_features, int quant,
                      const oxq_tensor *out, GgufProblem *p) {
    if (!ctx) return fail(OXQ_ERR_ARG, "%s: ctx is NULL", op);
    int64_t be, bb;
    if (oxq_gguf_block_layout(quant, &be, &bb) != OXQ_OK)
        return fail(OXQ_ERR_ARG, "%s: unknown GGUF quant %d", op, quant);
    const char *qn = gguf_name(quant);
    if (!dequant) OXQ_TRY(check_tensor(ctx, op, "x", x));
    OXQ_TRY(check_tensor(ctx, op, "weight_bytes", w));
    OXQ_TRY(check_tensor(ctx, op, "out", out));
    char b0[96];
    int act = OXQ_F32;
    int64_t m = 1;
    if (!dequant) {
        act = x->dtype;
        if (out->dtype != OXQ_BF16 && out->dtype != OXQ_F32)
            return fail(OXQ_ERR_DTYPE, "%s (%s): out must be BF16 or F32, got %s", op, qn,
                        dtype_name(out->dtype));
        if (act != OXQ_BF16 && act != OXQ_F32)
            return fail(OXQ_ERR_DTYPE, "%s (%s): x must be BF16 or F32, got %s", op, qn, dtype_name(act));
        if (out->dtype != act)
            return fail(OXQ_ERR_DTYPE, "%s (%s): out dtype %s must match x dtype %s", op, qn,
                        dtype_name(out->dtype), dtype_name(act));
    } else if (out->dtype != OXQ_F32) {
        return fail(OXQ_ERR_DTYPE, "%s (%s): out must be F32, got %s", op, qn, dtype_name(out->dtype));
    }
    if (w->dtype != OXQ_U8)
        return fail(OXQ_ERR_DTYPE, "%s (%s): weight_bytes must be U8, got %s", op, qn,
                    dtype_name(w->dtype));
    if (in_features <= 0 || out_features <= 0 || in_features % be != 0)
        return fail(OXQ_ERR_SHAPE, "%s (%s): in_features %lld must be a multiple of %lld", op, qn,
                    (long long)in_features, (long long)be);
    if (!dequant) {
        m = x->rank >= 1 ? x->dims[0] : 0;
        if (decode && !(m >= 1 && m <= 8))
            return fail(OXQ_ERR_M_RANGE, "%s (%s): m %lld out of [1, 8]", op, qn, (long long)m);
        if (!x->contiguous) return fail(OXQ_ERR_CONTIGUOUS, "%s (%s): x must be contiguous", op, qn);
        dims_str(x, b0, sizeof b0);
        if (x->rank != 2 || x->dims[1] != in_features || m < 1)
            return fail(OXQ_ERR_SHAPE, "%s (%s): x shape %s != [%s, %lld]", op, qn, b0,
                        decode ? "m" : "M", (long long)in_features);
    }
    dims_str(out, b0, sizeof b0);
    const int64_t o0 = dequant ? out_features : m, o1 = dequant ? in_features : out_features;
    if (out->rank != 2 || out->dims[0] != o0 || out->dims[1] != o1 || !out->contiguous)
        return fail(OXQ_ERR_SHAPE, "%s (%s): output shape %s != [%lld, %lld]", op, qn, b0,
                    (long long)o0, (long long)o1);
    const int64_t expected = out_features * (in_features / be) * bb;
    if (numel(w) != expected || !w->contiguous)
        return fail(OXQ_ERR_SHAPE,
                    "%s (%s): weight_bytes has %lld bytes, expected %lld (out=%lld x "
                    "blocks_per_row=%lld x %lld)", op, qn, (long long)numel(w), (long long)expected,
                    (long long)out_features, (long long)(in_features / be), (long long)bb);
    if (in_features > INT32_MAX || out_features > INT32_MAX)
        return fail(OXQ_ERR_SHAPE, "%s: dimension exceeds 2^31-1", op);
    p->x = x ? x->data : nullptr;
    p->w = (const uint8_t *)w->data;
    p->bias = nullptr;
    p->y = out->data;
    p->M = m;
    p->K = in_features;
    p->N = out_features;
    p->quant = quant;
    p->act_dtype = act;
    return OXQ_OK;
}

// Mxfp4Matmul::metal_fwd (metal_ops.rs:6009-6058)
static int check_mxfp4(oxq_ctx *ctx, const char *op, bool dequant, const oxq_tensor *x,
                       const oxq_tensor *blocks, const oxq_tensor *scales, int64_t k, int64_t n,
                       int64_t n_experts, const oxq_tensor *out, Mxfp4Problem *p) {
    if (!ctx) return fail(OXQ_ERR_ARG, "%s: ctx is NULL", op);
    if (!dequant) OXQ_TRY(check_tensor(ctx, op, "x", x));
    OXQ_TRY(check_tensor(ctx, op, "blocks", blocks));
    OXQ_TRY(check_tensor(ctx, op, "scales", scales));
    OXQ_TRY(check_tensor(ctx, op, "out", out));
    char b0[96];
    if (!dequant && (out->dtype != OXQ_BF16 || x->dtype != OXQ_BF16))
        return fail(OXQ_ERR_DTYPE, "%s: x/out must be BF16, got %s/%s", op, dtype_name(x->dtype),
                    dtype_name(out->dtype));
    if (dequant && out->dtype != OXQ_F32)
        return fail(OXQ_ERR_DTYPE, "%s: out must be F32, got %s", op, dtype_name(out->dtype));
    if (blocks->dtype != OXQ_U8 || scales->dtype != OXQ_U8)
        return fail(OXQ_ERR_DTYPE, "%s: blocks/scales must be U8", op);
    if (k <= 0 || n <= 0 || k % 32 != 0)
        return fail(OXQ_ERR_SHAPE, "%s: K %lld must be a multiple of 32", op, (long long)k);
    const int64_t nb = k / 32;
    const int64_t e = n_experts > 0 ? n_experts : 1;
    if (numel(blocks) != e * n * nb * 16 || numel(scales) != e * n * nb || !blocks->contiguous ||
        !scales->contiguous)
        return fail(OXQ_ERR_SHAPE, "%s: blocks %lld / scales %lld elements don't match [%lld, %lld]",
                    op, (long long)numel(blocks), (long long)numel(scales), (long long)n, (long long)k);
    int64_t m = 1;
    if (!dequant) {
        if (!x->contiguous) return fail(OXQ_ERR_CONTIGUOUS, "%s: x must be contiguous", op);
        dims_str(x, b0, sizeof b0);
        if (x->rank != 2 || x->dims[1] != k || x->dims[0] < 1)
            return fail(OXQ_ERR_SHAPE, "%s: x shape %s != [m, %lld]", op, b0, (long long)k);
        m = x->dims[0];
    }
    if (k > INT32_MAX || n > INT32_MAX) return fail(OXQ_ERR_SHAPE, "%s: dimension exceeds 2^31-1", op);
    p->x = x ? x->data : nullptr;
    p->blocks = (const uint8_t *)blocks->data;
    p->scales = (const uint8_t *)scales->data;
    p->bias = nullptr;
    p->y = out->data;
    p->M = m;
    p->K = k;
    p->N = n;
    p->n_experts = 0;
    p->expert_offsets = nullptr;
    p->token_ids = nullptr;
    p->n_pairs = 0;
    return OXQ_OK;
}

}  // namespace oxq

using namespace oxq;

// -----------------------------------------------------------------------------
// Split-K partial sums for the allocation-free entry point (oxq_w4a16_matmul_static): a device
// array that exists from the moment the code object is loaded, one copy per GPU, each at its own
// address.  In host code the name `scratch` is only a handle for hipGetSymbolAddress; the address
// it returns (per device, taken once with that device current) is what kernels and copies use.
// -----------------------------------------------------------------------------
#define OXQ_STATIC_SCRATCH_BYTES (16u << 20)
static __device__ __align__(256) unsigned char scratch[OXQ_STATIC_SCRATCH_BYTES];

namespace oxq {
static constexpr int SCRATCH_MAX_DEVICES = 64;
static std::atomic<void *> g_scratch_ptr[SCRATCH_MAX_DEVICES] = {};
static std::mutex g_scratch_mu;

// The calling thread must have `device` current.
static int scratch_lookup(int device, void **out) {
    if (device < 0 || device >= SCRATCH_MAX_DEVICES)
        return fail(OXQ_ERR_DEVICE, "static scratch: device ordinal %d outside 0..%d", device, SCRATCH_MAX_DEVICES - 1);
    void *ptr = g_scratch_ptr[device].load(std::memory_order_acquire);
    if (!ptr) {
        std::lock_guard<std::mutex> lock(g_scratch_mu);
        ptr = g_scratch_ptr[device].load(std::memory_order_relaxed);
        if (!ptr) {
            hipError_t e = hipGetSymbolAddress((void **)&ptr, HIP_SYMBOL(scratch));
            if (e != hipSuccess || !ptr)
                return fail(OXQ_ERR_RUNTIME, "static scratch: hipGetSymbolAddress on device %d failed: %s", device,
                            hipGetErrorString(e));
            g_scratch_ptr[device].store(ptr, std::memory_order_release);
        }
    }
    *out = ptr;
    return OXQ_OK;
}
}  // namespace oxq

struct oxq_mxfp4_experts {
    oxq_ctx *ctx;
    oxq_tensor blocks, scales, bias;  // the caller's tensors (prefill sizes and ineligible shapes run on them)
    bool has_bias;
    int64_t n_experts, k, n;
    void *pw, *ps;                    // resident tile-major copy; null when the shape does not qualify
    bool owns;                        // pw / ps are device allocations of this handle (not a plan-only ctx's stand-ins)
};

// =============================================================================
// C ABI
// =============================================================================
extern "C" {

void oxq_version(int *major, int *minor) {
    if (major) *major = OXQ_VERSION_MAJOR;
    if (minor) *minor = OXQ_VERSION_MINOR;
}

const char *oxq_last_error(void) { return g_last_error; }

const char *oxq_status_name(int status) {
    switch (status) {
    case OXQ_OK: return "OXQ_OK";
    case OXQ_ERR_ARG: return "OXQ_ERR_ARG";
    case OXQ_ERR_DTYPE: return "OXQ_ERR_DTYPE";
    case OXQ_ERR_SHAPE: return "OXQ_ERR_SHAPE";
    case OXQ_ERR_CONTIGUOUS: return "OXQ_ERR_CONTIGUOUS";
    case OXQ_ERR_M_RANGE: return "OXQ_ERR_M_RANGE";
    case OXQ_ERR_GROUP: return "OXQ_ERR_GROUP";
    case OXQ_ERR_DEVICE: return "OXQ_ERR_DEVICE";
    case OXQ_ERR_BITS: return "OXQ_ERR_BITS";
    case OXQ_ERR_RUNTIME: return "OXQ_ERR_RUNTIME";
    case OXQ_ERR_WORKSPACE: return "OXQ_ERR_WORKSPACE";
    case OXQ_ERR_UNSUPPORTED: return "OXQ_ERR_UNSUPPORTED";
    case OXQ_ERR_IO: return "OXQ_ERR_IO";
    case OXQ_ERR_FORMAT: return "OXQ_ERR_FORMAT";
    default: return "OXQ_ERR_?";
    }
}

int oxq_gguf_block_layout(int quant, int64_t *block_elems, int64_t *block_bytes) {
    int64_t e, b;
    switch (quant) {
    case OXQ_GGUF_Q4_0: e = 32; b = 18; break;
    case OXQ_GGUF_Q8_0: e = 32; b = 34; break;
    case OXQ_GGUF_Q4_K: e = 256; b = 144; break;
    case OXQ_GGUF_Q6_K: e = 256; b = 210; break;
    case OXQ_GGUF_Q4_1: e = 32; b = 20; break;
    case OXQ_GGUF_Q5_0: e = 32; b = 22; break;
    case OXQ_GGUF_Q5_1: e = 32; b = 24; break;
    case OXQ_GGUF_Q2_K: e = 256; b = 84; break;
    case OXQ_GGUF_Q3_K: e = 256; b = 110; break;
    case OXQ_GGUF_Q5_K: e = 256; b = 176; break;
    default: return fail(OXQ_ERR_ARG, "unknown GGUF quant %d", quant);
    }
    if (block_elems) *block_elems = e;
    if (block_bytes) *block_bytes = b;
    return OXQ_OK;
}

// Names of the tuning switches: OXQ_<name> as an environment variable and as the key of oxq_ctx_set_tuning.
static const char *const kTuneNames[OXQ_TUNE_COUNT] = {
#define OXQ_TUNE_NAME(n) "OXQ_" #n,
    OXQ_TUNE_LIST(OXQ_TUNE_NAME)
#undef OXQ_TUNE_NAME
};

static int tune_from_env(int key) {
    const char *v = getenv(kTuneNames[key]);
    return (v && *v) ? atoi(v) : OXQ_TUNE_UNSET;
}

static int tune_key_of(const char *name) {
    if (!name) return -1;
    for (int k = 0; k < OXQ_TUNE_COUNT; ++k)
        if (strcmp(name, kTuneNames[k]) == 0) return k;
    return -1;
}

int oxq_ctx_set_tuning(oxq_ctx *ctx, const char *name, int value) {
    if (!ctx) return fail(OXQ_ERR_ARG, "oxq_ctx_set_tuning: ctx is NULL");
    const int k = tune_key_of(name);
    if (k < 0) return fail(OXQ_ERR_ARG, "oxq_ctx_set_tuning: unknown switch '%s'", name ? name : "(null)");
    ctx->tuning[k] = value;
    if (k == OXQ_TUNE_SPLITK_MODE) ctx->splitk_mode = value;
    return OXQ_OK;
}

int oxq_ctx_reset_tuning(oxq_ctx *ctx, const char *name) {
    if (!ctx) return fail(OXQ_ERR_ARG, "oxq_ctx_reset_tuning: ctx is NULL");
    if (name) {
        const int k = tune_key_of(name);
        if (k < 0) return fail(OXQ_ERR_ARG, "oxq_ctx_reset_tuning: unknown switch '%s'", name);
        ctx->tuning[k] = tune_from_env(k);
    } else {
        for (int k = 0; k < OXQ_TUNE_COUNT; ++k) ctx->tuning[k] = tune_from_env(k);
    }
    ctx->splitk_mode = tune(ctx, OXQ_TUNE_SPLITK_MODE, 0);
    return OXQ_OK;
}

int oxq_ctx_create(int device, oxq_ctx **out) {
    if (!out) return fail(OXQ_ERR_ARG, "oxq_ctx_create: out is NULL");
    *out = nullptr;
    oxq_ctx *ctx = new (std::nothrow) oxq_ctx();
    if (!ctx) return fail(OXQ_ERR_RUNTIME, "oxq_ctx_create: out of host memory");
    memset(ctx, 0, sizeof *ctx);
    ctx->device = device;
    ctx->plan_only = device == OXQ_DEVICE_PLAN_ONLY;
    ctx->num_cus = 256;
    const char *ws_env = getenv("OXQ_WORKSPACE_MB");
    const size_t ws_mb = (ws_env && atoi(ws_env) > 0) ? (size_t)atoi(ws_env) : 64;
    ctx->workspace_bytes = ws_mb << 20;
    ctx->n_counters = 16384;
    for (int k = 0; k < OXQ_TUNE_COUNT; ++k) ctx->tuning[k] = tune_from_env(k);
    ctx->splitk_mode = tune(ctx, OXQ_TUNE_SPLITK_MODE, 0);
    {
        const char *m = getenv("OXQ_WEIGHT_CACHE_MB");
        ctx->wcache_limit = (m && atoi(m) > 0) ? (size_t)atoi(m) << 20 : 0;
    }
    if (ctx->plan_only) {
        *out = ctx;
        return OXQ_OK;
    }
    int count = 0;
    hipError_t e = hipGetDeviceCount(&count);
    if (e != hipSuccess || device < 0 || device >= count) {
        delete ctx;
        return fail(OXQ_ERR_DEVICE, "oxq_ctx_create: no HIP device %d (%d visible%s%s)", device,
                    count, e != hipSuccess ? ": " : "", e != hipSuccess ? hipGetErrorString(e) : "");
    }
    int prev = 0;
    (void)hipGetDevice(&prev);
    int rc = OXQ_OK;
    do {
        if ((e = hipSetDevice(device)) != hipSuccess) break;
        int cus = 0;
        if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, device) == hipSuccess &&
            cus > 0)
            ctx->num_cus = cus;
        if ((e = hipMalloc(&ctx->workspace, ctx->workspace_bytes)) != hipSuccess) break;
        if ((e = hipMalloc((void **)&ctx->counters, ctx->n_counters * sizeof(unsigned))) != hipSuccess)
            break;
        if ((e = hipMemset(ctx->counters, 0, ctx->n_counters * sizeof(unsigned))) != hipSuccess) break;
        e = hipDeviceSynchronize();
        // this device's address of the static scratch array, looked up once while it is current
        void *sp = nullptr;
        if (e == hipSuccess && scratch_lookup(device, &sp) != OXQ_OK) rc = OXQ_ERR_RUNTIME;
    } while (0);
    (void)hipSetDevice(prev);
    if (e == hipSuccess && rc != OXQ_OK) {  // scratch_lookup has set the message
        (void)hipFree(ctx->workspace);
        (void)hipFree(ctx->counters);
        delete ctx;
        return rc;
    }
    if (e != hipSuccess) {
        rc = fail(OXQ_ERR_RUNTIME, "oxq_ctx_create: %s", hipGetErrorString(e));
        if (ctx->workspace) (void)hipFree(ctx->workspace);
        if (ctx->counters) (void)hipFree(ctx->counters);
        delete ctx;
        return rc;
    }
    *out = ctx;
    return OXQ_OK;
}

static void wcache_destroy(oxq_ctx *ctx);  // frees every cached weight copy and the cache itself

int oxq_ctx_destroy(oxq_ctx *ctx) {
    if (!ctx) return OXQ_OK;
    if (!ctx->plan_only) {
        wcache_destroy(ctx);
        if (ctx->workspace) (void)hipFree(ctx->workspace);
        if (ctx->counters) (void)hipFree(ctx->counters);
    }
    delete ctx;
    return OXQ_OK;
}

int oxq_ctx_device(const oxq_ctx *ctx) { return ctx ? ctx->device : OXQ_DEVICE_PLAN_ONLY; }

int oxq_ctx_last_plan(const oxq_ctx *ctx, oxq_plan *out) {
    if (!ctx || !out) return fail(OXQ_ERR_ARG, "oxq_ctx_last_plan: NULL argument");
    *out = ctx->plan;
    return OXQ_OK;
}

// ---- measurement aid ----------------------------------------------------------
int oxq_calib_read(oxq_ctx *ctx, void *stream, const oxq_tensor *src, int workgroups, int nontemporal,
                   const oxq_tensor *checksums) {
    if (!ctx || !src || !checksums) return fail(OXQ_ERR_ARG, "CalibRead: NULL argument");
    OXQ_TRY(check_tensor(ctx, "CalibRead", "src", src));
    OXQ_TRY(check_tensor(ctx, "CalibRead", "checksums", checksums));
    if (src->dtype != OXQ_U8 || !src->contiguous)
        return fail(OXQ_ERR_DTYPE, "CalibRead: src must be a contiguous U8 tensor, got %s", dtype_name(src->dtype));
    if ((checksums->dtype != OXQ_U32 && checksums->dtype != OXQ_I32) || !checksums->contiguous)
        return fail(OXQ_ERR_DTYPE, "CalibRead: checksums must be a contiguous U32/I32 tensor, got %s",
                    dtype_name(checksums->dtype));
    const int64_t bytes = numel(src);
    if (workgroups < 1 || workgroups > 65535 || numel(checksums) < workgroups)
        return fail(OXQ_ERR_SHAPE, "CalibRead: %d workgroups need 1..65535 and one checksum word each (got %lld)",
                    workgroups, (long long)numel(checksums));
    if (bytes <= 0 || bytes % ((int64_t)workgroups * 8192) != 0 || bytes / workgroups >= (int64_t(1) << 31))
        return fail(OXQ_ERR_SHAPE,
                    "CalibRead: %lld bytes over %d workgroups: every workgroup reads a span that is a multiple "
                    "of 8 KiB and below 2 GiB", (long long)bytes, workgroups);
    if (!ctx->plan_only && ((uintptr_t)src->data & 15))
        return fail(OXQ_ERR_UNSUPPORTED, "CalibRead: src must be 16-byte aligned");
    return launch_calib_read(ctx, (hipStream_t)stream, (const uint8_t *)src->data, (uint64_t)bytes, workgroups,
                             nontemporal, (uint32_t *)checksums->data);
}

int oxq_bench_read_upfront(oxq_ctx *ctx, void *stream, const oxq_tensor *src, int workgroups, int waves,
                           int nontemporal, const oxq_tensor *checksums) {
    if (!ctx || !src || !checksums) return fail(OXQ_ERR_ARG, "ReadUpfront: NULL argument");
    OXQ_TRY(check_tensor(ctx, "ReadUpfront", "src", src));
    OXQ_TRY(check_tensor(ctx, "ReadUpfront", "checksums", checksums));
    if (src->dtype != OXQ_U8 || !src->contiguous)
        return fail(OXQ_ERR_DTYPE, "ReadUpfront: src must be a contiguous U8 tensor, got %s", dtype_name(src->dtype));
    if ((checksums->dtype != OXQ_U32 && checksums->dtype != OXQ_I32) || !checksums->contiguous)
        return fail(OXQ_ERR_DTYPE, "ReadUpfront: checksums must be a contiguous U32/I32 tensor, got %s",
                    dtype_name(checksums->dtype));
    const int64_t bytes = numel(src);
    if (waves != 8 && waves != 16) return fail(OXQ_ERR_ARG, "ReadUpfront: %d waves a workgroup (8 or 16)", waves);
    if (workgroups < 1 || workgroups > 65535 || numel(checksums) < workgroups)
        return fail(OXQ_ERR_SHAPE, "ReadUpfront: %d workgroups need 1..65535 and one checksum word each (got %lld)",
                    workgroups, (long long)numel(checksums));
    const int64_t per_wave = (int64_t)workgroups * waves * 1024;
    if (bytes <= 0 || bytes % per_wave != 0 || bytes / per_wave > 32)
        return fail(OXQ_ERR_SHAPE, "ReadUpfront: %lld bytes over %d workgroups of %d waves: every wave reads 1 .. 32 KiB "
                    "in whole KiB", (long long)bytes, workgroups, waves);
    if (!ctx->plan_only && ((uintptr_t)src->data & 15))
        return fail(OXQ_ERR_UNSUPPORTED, "ReadUpfront: src must be 16-byte aligned");
    return launch_calib_upfront(ctx, (hipStream_t)stream, (const uint8_t *)src->data, (uint64_t)bytes, workgroups, waves,
                                nontemporal, (uint32_t *)checksums->data);
}

int oxq_bench_two_streams(oxq_ctx *ctx, void *stream, const oxq_tensor *w, const oxq_tensor *x, int workgroups,
                          int which, const oxq_tensor *checksums) {
    if (!ctx || !w || !x || !checksums) return fail(OXQ_ERR_ARG, "TwoStreams: NULL argument");
    OXQ_TRY(check_tensor(ctx, "TwoStreams", "w", w));
    OXQ_TRY(check_tensor(ctx, "TwoStreams", "x", x));
    OXQ_TRY(check_tensor(ctx, "TwoStreams", "checksums", checksums));
    if (w->dtype != OXQ_U8 || !w->contiguous || x->dtype != OXQ_U8 || !x->contiguous)
        return fail(OXQ_ERR_DTYPE, "TwoStreams: w and x must be contiguous U8 tensors");
    if ((checksums->dtype != OXQ_U32 && checksums->dtype != OXQ_I32) || !checksums->contiguous)
        return fail(OXQ_ERR_DTYPE, "TwoStreams: checksums must be a contiguous U32/I32 tensor");
    if (which < 1 || which > 3) return fail(OXQ_ERR_ARG, "TwoStreams: which = %d (1 w, 2 x, 3 both)", which);
    const int64_t wb = numel(w), xb = numel(x);
    if (workgroups < 1 || workgroups > 65535 || numel(checksums) < workgroups)
        return fail(OXQ_ERR_SHAPE, "TwoStreams: %d workgroups need 1..65535 and one checksum word each", workgroups);
    const int64_t span = wb / workgroups;
    if (wb <= 0 || wb % workgroups != 0 || (span != 8 * 8192 && span != 16 * 8192 && span != 17 * 8192))
        return fail(OXQ_ERR_SHAPE, "TwoStreams: w must be workgroups x 64, 128 or 136 KiB (got %lld bytes)", (long long)wb);
    if (xb <= 0 || xb % (4 * 8192) != 0 || xb >= (int64_t(1) << 31))
        return fail(OXQ_ERR_SHAPE, "TwoStreams: x must be a multiple of 32 KiB below 2 GiB (got %lld bytes)", (long long)xb);
    if (!ctx->plan_only && (((uintptr_t)w->data | (uintptr_t)x->data) & 15))
        return fail(OXQ_ERR_UNSUPPORTED, "TwoStreams: w and x must be 16-byte aligned");
    return launch_calib_two_streams(ctx, (hipStream_t)stream, (const uint8_t *)w->data, (uint64_t)wb, (const uint8_t *)x->data,
                                    (uint64_t)xb, workgroups, which, (uint32_t *)checksums->data);
}

int oxq_bench_empty_launch(oxq_ctx *ctx, void *stream, int workgroups, int threads, int lds_bytes) {
    if (!ctx) return fail(OXQ_ERR_ARG, "EmptyLaunch: ctx is NULL");
    if (workgroups < 1 || workgroups > 65535 || threads < 64 || threads > 1024 || threads % 64 != 0 || lds_bytes < 0 ||
        lds_bytes > 160 * 1024)
        return fail(OXQ_ERR_ARG, "EmptyLaunch: %d workgroups of %d threads with %d bytes of LDS", workgroups, threads,
                    lds_bytes);
    return launch_empty(ctx, (hipStream_t)stream, workgroups, threads, lds_bytes);
}

int oxq_bench_grid_barrier(oxq_ctx *ctx, void *stream, int workgroups, int threads, const oxq_tensor *state,
                           uint32_t spin_limit) {
    if (!ctx || !state) return fail(OXQ_ERR_ARG, "GridBarrier: NULL argument");
    if (workgroups < 1 || threads < 64 || threads > 1024 || threads % 64 != 0)
        return fail(OXQ_ERR_ARG, "GridBarrier: %d workgroups of %d threads", workgroups, threads);
    // every workgroup must be resident at once, or the ones that are would wait for ones that cannot start
    const int resident = (ctx->num_cus > 0 ? ctx->num_cus : 256) * (threads <= 512 ? 2 : 1);
    if (workgroups > resident)
        return fail(OXQ_ERR_ARG, "GridBarrier: %d workgroups of %d threads are not resident at once on %d compute units",
                    workgroups, threads, ctx->num_cus);
    if ((state->dtype != OXQ_I32 && state->dtype != OXQ_U32) || state->rank != 1 || state->dims[0] < 2 || !state->contiguous)
        return fail(OXQ_ERR_SHAPE, "GridBarrier: state must be two contiguous 32-bit words {counter, error}");
    if (!ctx->plan_only && (state->device == OXQ_DEVICE_HOST || !state->data))
        return fail(OXQ_ERR_DEVICE, "GridBarrier: state must be a device tensor");
    if (spin_limit == 0 || spin_limit > (1u << 22)) return fail(OXQ_ERR_ARG, "GridBarrier: spin limit %u", spin_limit);
    return launch_grid_barrier(ctx, (hipStream_t)stream, workgroups, threads, (unsigned *)state->data,
                               (unsigned *)state->data + 1, spin_limit);
}

// ---- opt-in cache of tile-major weight copies behind the stateless ops ---------------------------
// The reference's ops are called with the same resident tensors on every forward (linear.rs:482-533
// passes the layer's own qweight / qzeros / scales).  A caller that swaps in only the op functions,
// not the layer types, can let the ctx remember those tensors by address: the first call on a
// (qweight, qzeros, scales) triple builds the resident layers' tile-major copy, later calls run the
// resident-layer kernel on it.  Off unless oxq_ctx_set_weight_cache (or OXQ_WEIGHT_CACHE_MB) gives
// it room: the ctx cannot see a caller overwrite or free those tensors, so the caller has to say
// so (oxq_ctx_forget_weights).
struct oxq_weight_cache {
    struct Entry {
        const void *qw, *qz, *sc;
        int64_t K, N;
        int group_shift, dtype, bits, pack_dim;
        Pk4Weights w;
        size_t bytes;
        uint64_t last_use;
        bool pinned;  // a captured graph holds this copy's address: only forget / destroy may free it
    };
    std::vector<Entry> entries;
    size_t bytes = 0;
    uint64_t tick = 0;
};

static void wcache_drop(oxq_ctx *ctx, size_t i) {
    oxq_weight_cache *c = ctx->wcache;
    (void)hipFree(c->entries[i].w.pw);  // waits for the device: no kernel still reads the copy
    c->bytes -= c->entries[i].bytes;
    c->entries.erase(c->entries.begin() + (long)i);
}

static void wcache_clear(oxq_ctx *ctx) {
    if (!ctx->wcache) return;
    while (!ctx->wcache->entries.empty()) wcache_drop(ctx, ctx->wcache->entries.size() - 1);
}

static void wcache_destroy(oxq_ctx *ctx) {
    if (!ctx->wcache) return;
    int prev = 0;
    (void)hipGetDevice(&prev);
    (void)hipSetDevice(ctx->device);
    wcache_clear(ctx);
    (void)hipSetDevice(prev);
    delete ctx->wcache;
    ctx->wcache = nullptr;
}

// Makes room for `bytes` more.  Least recently used copies go first, except those a captured graph may hold
// (pinned) and those used within the last entries + 1 calls: when the working set is larger than the limit,
// evicting what the next calls will ask for again would rebuild a copy on every call - far slower than the
// checkpoint-layout kernel the copy replaces - so the newcomer takes that kernel instead and the copies stay.
// False: no room.  (hipFree, which a dropped copy costs, waits for the device.)
static bool wcache_make_room(oxq_ctx *ctx, size_t bytes) {
    oxq_weight_cache *c = ctx->wcache;
    if (bytes > ctx->wcache_limit) return false;
    while (c->bytes + bytes > ctx->wcache_limit) {
        size_t lru = c->entries.size();
        for (size_t i = 0; i < c->entries.size(); ++i)
            if (!c->entries[i].pinned && (lru == c->entries.size() || c->entries[i].last_use < c->entries[lru].last_use)) lru = i;
        if (lru == c->entries.size()) return false;
        if (c->tick - c->entries[lru].last_use <= c->entries.size() + 1) return false;
        wcache_drop(ctx, lru);
    }
    return true;
}

// A hit while the stream is being captured puts the copy's address into the graph: from then on the copy stays
// until the caller forgets the weight or destroys the ctx (either of which invalidates that graph).
static void wcache_pin_if_capturing(hipStream_t s, oxq_weight_cache::Entry *e) {
    hipStreamCaptureStatus cs = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(s, &cs) != hipSuccess) {
        (void)hipGetLastError();
        return;
    }
    if (cs != hipStreamCaptureStatusNone) e->pinned = true;
}

// true: the call was served (rc holds its status).  false: take the checkpoint-layout path.
static bool wcache_forward(oxq_ctx *ctx, hipStream_t s, const Wna16Problem &p, int *rc) {
    if (!ctx->wcache_limit || ctx->plan_only || !pk4_eligible(p)) return false;
    if (((uintptr_t)p.x | (uintptr_t)p.y) & 15) return false;
    if (!ctx->wcache) {
        ctx->wcache = new (std::nothrow) oxq_weight_cache();
        if (!ctx->wcache) return false;
    }
    oxq_weight_cache *c = ctx->wcache;
    ++c->tick;  // one tick a call, hit or not: an entry's age is counted in calls
    oxq_weight_cache::Entry *hit = nullptr;
    for (auto &e : c->entries)
        if (e.qw == p.qweight && e.qz == p.qzeros && e.sc == p.scales && e.K == p.K && e.N == p.N &&
            e.group_shift == p.group_shift && e.dtype == p.dtype && e.bits == p.bits && e.pack_dim == p.pack_dim) {
            hit = &e;
            break;
        }
    if (!hit) {
        // building a copy allocates: not while the stream is being captured into a graph
        hipStreamCaptureStatus cs = hipStreamCaptureStatusNone;
        if (hipStreamIsCapturing(s, &cs) != hipSuccess || cs != hipStreamCaptureStatusNone) {
            (void)hipGetLastError();
            return false;
        }
        const size_t bytes = (pk4_weight_bytes(p.K, p.N, p.bits) + 255) & ~(size_t)255;
        if (!wcache_make_room(ctx, bytes)) return false;
        void *mem = nullptr;
        if (hipMalloc(&mem, bytes) != hipSuccess) {
            (void)hipGetLastError();
            return false;
        }
        oxq_weight_cache::Entry e{p.qweight, p.qzeros, p.scales, p.K, p.N, p.group_shift, p.dtype, p.bits, p.pack_dim,
                                  Pk4Weights{(uint32_t *)mem, nullptr, p.K, p.N, p.group_shift, p.dtype, p.bits, 0,
                                             p.pack_dim == OXQ_PACK_IN ? 32 : 16, pk4_choose_strip(ctx, p.K, p.N, p.bits, 0)},
                                  bytes, 0, false};
        const int prc = launch_pk4_prepack(ctx, s, p, e.w);  // on the caller's stream, ahead of the matmul
        if (prc != OXQ_OK) {
            (void)hipFree(mem);
            *rc = prc;
            return true;
        }
        try {
            c->entries.push_back(e);
        } catch (...) {
            (void)hipFree(mem);
            return false;
        }
        c->bytes += bytes;
        hit = &c->entries.back();
    }
    hit->last_use = c->tick;
    wcache_pin_if_capturing(s, hit);
    Pk4Problem q;
    q.x = p.x;
    q.bias = p.bias;
    q.y = p.y;
    q.M = p.M;
    q.act = 0;
    q.no_split = 0;
    q.w = hit->w;
    *rc = launch_pk4_forward(ctx, s, q);
    return true;
}

// The same for a GGUF weight: the copy is the strip-major one of the QLinear layers - the matrix-core layout
// for bf16 activations (the rows its kernels take: up to 32, and prefill sizes), the rotated one of the vector
// GEMV for f32 (1 - 8 rows).  Entry fields: qw = the block bytes, bits = the ggml format, pack_dim = -1 (rotated) or -2
// (matrix-core), w.pw = the copy.
static bool wcache_forward_gguf(oxq_ctx *ctx, hipStream_t s, const GgufProblem &p, int *rc) {
    if (!ctx->wcache_limit || ctx->plan_only || !gguf_res_eligible(p.quant, p.K, p.N)) return false;
    const bool mfma = p.act_dtype == OXQ_BF16 && gguf_mfma_eligible(ctx, p.quant, p.K, p.N);
    const bool gemm = mfma && gguf_gemm_takes(ctx, p.quant, p.M, p.K, p.N, p.act_dtype);  // prefill sizes, same copy
    if (!gemm && !(mfma ? gguf_mfma_takes(ctx, p.M, p.N, p.act_dtype) : gguf_res_takes(p.K, p.M, p.act_dtype))) return false;
    const int kind = mfma ? -2 : -1;
    if (((uintptr_t)p.x & 15) || ((uintptr_t)p.w & 1)) return false;
    if (!ctx->wcache) {
        ctx->wcache = new (std::nothrow) oxq_weight_cache();
        if (!ctx->wcache) return false;
    }
    oxq_weight_cache *c = ctx->wcache;
    ++c->tick;
    oxq_weight_cache::Entry *hit = nullptr;
    for (auto &e : c->entries)
        if (e.qw == p.w && e.qz == nullptr && e.sc == nullptr && e.K == p.K && e.N == p.N && e.bits == p.quant &&
            e.pack_dim == kind) {
            hit = &e;
            break;
        }
    if (!hit) {
        hipStreamCaptureStatus cs = hipStreamCaptureStatusNone;
        if (hipStreamIsCapturing(s, &cs) != hipSuccess || cs != hipStreamCaptureStatusNone) {
            (void)hipGetLastError();
            return false;
        }
        const size_t bytes = (gguf_res_bytes(p.quant, p.K, p.N) + 255) & ~(size_t)255;
        if (!wcache_make_room(ctx, bytes)) return false;
        void *mem = nullptr;
        if (hipMalloc(&mem, bytes) != hipSuccess) {
            (void)hipGetLastError();
            return false;
        }
        oxq_weight_cache::Entry e{p.w, nullptr, nullptr, p.K, p.N, 0, 0, p.quant, kind,
                                  Pk4Weights{(uint32_t *)mem, nullptr, p.K, p.N, 0, 0, 0, 0, 0, 0}, bytes, 0, false};
        const int prc = mfma ? launch_gguf_mfma_repack(ctx, s, p.quant, p.w, mem, p.K, p.N) : launch_gguf_res_repack(ctx, s, p.quant, p.w, mem, p.K, p.N);
        if (prc != OXQ_OK) {
            (void)hipFree(mem);
            *rc = prc;
            return true;
        }
        try {
            c->entries.push_back(e);
        } catch (...) {
            (void)hipFree(mem);
            return false;
        }
        c->bytes += bytes;
        hit = &c->entries.back();
    }
    hit->last_use = c->tick;
    wcache_pin_if_capturing(s, hit);
    GgufProblem q = p;
    q.w = (const uint8_t *)hit->w.pw;
    *rc = gemm ? launch_gguf_gemm(ctx, s, q) : mfma ? launch_gguf_mfma(ctx, s, q) : launch_gguf_res_gemv(ctx, s, q);
    return true;
}

int oxq_ctx_set_weight_cache(oxq_ctx *ctx, int64_t max_bytes) {
    if (!ctx) return fail(OXQ_ERR_ARG, "oxq_ctx_set_weight_cache: ctx is NULL");
    if (max_bytes < 0) return fail(OXQ_ERR_ARG, "oxq_ctx_set_weight_cache: max_bytes %lld is negative", (long long)max_bytes);
    ctx->wcache_limit = (size_t)max_bytes;
    if (ctx->wcache) {
        int prev = 0;
        (void)hipGetDevice(&prev);
        (void)hipSetDevice(ctx->device);
        // copies a captured graph may hold stay (and count against the limit) until they are forgotten
        while (ctx->wcache->bytes > ctx->wcache_limit) {
            const size_t n = ctx->wcache->entries.size();
            size_t lru = n;
            for (size_t i = 0; i < n; ++i)
                if (!ctx->wcache->entries[i].pinned &&
                    (lru == n || ctx->wcache->entries[i].last_use < ctx->wcache->entries[lru].last_use)) lru = i;
            if (lru == n) break;
            wcache_drop(ctx, lru);
        }
        (void)hipSetDevice(prev);
    }
    return OXQ_OK;
}

int oxq_ctx_forget_weights(oxq_ctx *ctx, const void *qweight_data) {
    if (!ctx) return fail(OXQ_ERR_ARG, "oxq_ctx_forget_weights: ctx is NULL");
    if (!ctx->wcache) return OXQ_OK;
    int prev = 0;
    (void)hipGetDevice(&prev);
    (void)hipSetDevice(ctx->device);
    if (!qweight_data) wcache_clear(ctx);
    else
        for (size_t i = ctx->wcache->entries.size(); i-- > 0;)
            if (ctx->wcache->entries[i].qw == qweight_data) wcache_drop(ctx, i);
    (void)hipSetDevice(prev);
    return OXQ_OK;
}

int oxq_ctx_weight_cache_bytes(const oxq_ctx *ctx, int64_t *bytes, int64_t *entries) {
    if (!ctx) return fail(OXQ_ERR_ARG, "oxq_ctx_weight_cache_bytes: ctx is NULL");
    if (bytes) *bytes = ctx->wcache ? (int64_t)ctx->wcache->bytes : 0;
    if (entries) *entries = ctx->wcache ? (int64_t)ctx->wcache->entries.size() : 0;
    return OXQ_OK;
}

// ---- AWQ / GPTQ -------------------------------------------------------------
int oxq_w4a16_matmul(oxq_ctx *ctx, void *stream, const oxq_tensor *x, const oxq_tensor *qweight,
                     const oxq_tensor *qzeros, const oxq_tensor *scales, const oxq_tensor *out) {
    Wna16Problem p;
    OXQ_TRY(check_wna16(ctx, "W4A16Matmul", KIND_GEMV, x, qweight, qzeros, scales, 4, OXQ_PACK_OUT,
                        out, &p));
    int crc;
    if (wcache_forward(ctx, (hipStream_t)stream, p, &crc)) return crc;
    return launch_wna16_gemv(ctx, (hipStream_t)stream, p);
}

// oxq_w4a16_matmul for callers that cannot allocate: same validation, same kernels, same bits, but
// the split-K partial sums live in this device's copy of the static `scratch` array instead of the
// ctx workspace, and the slices are always added by the second launch (plain stores, no arrival
// counters: nothing in the array has to start at zero).  Calls no allocator.
int oxq_w4a16_matmul_static(oxq_ctx *ctx, void *stream, const oxq_tensor *x, const oxq_tensor *qweight,
                            const oxq_tensor *qzeros, const oxq_tensor *scales, const oxq_tensor *out) {
    Wna16Problem p;
    OXQ_TRY(check_wna16(ctx, "W4A16MatmulStatic", KIND_GEMV, x, qweight, qzeros, scales, 4, OXQ_PACK_OUT,
                        out, &p));
    oxq_ctx shadow = *ctx;  // the launchers read workspace, its size and the reduction mode from a ctx
    shadow.workspace = nullptr;
    shadow.workspace_bytes = ~(size_t)0;
    shadow.counters = nullptr;
    shadow.n_counters = 0xFFFFFFFFu;
    shadow.splitk_mode = 2;
    shadow.wcache = nullptr;
    shadow.wcache_limit = 0;
    shadow.plan_only = true;  // first pass: what would this call need?
    OXQ_TRY(launch_wna16_gemv(&shadow, (hipStream_t)stream, p));
    if (shadow.plan.workspace_bytes > OXQ_STATIC_SCRATCH_BYTES)
        return fail(OXQ_ERR_WORKSPACE,
                    "W4A16MatmulStatic: the call needs %llu bytes of split-K partial sums, the static scratch "
                    "array holds %u (m = %lld, n = %lld, %u slices): use oxq_w4a16_matmul",
                    (unsigned long long)shadow.plan.workspace_bytes, OXQ_STATIC_SCRATCH_BYTES, (long long)p.M,
                    (long long)p.N, shadow.plan.split_k);
    if (shadow.plan.split_k > 1 && shadow.plan.launches < 2)
        return fail(OXQ_ERR_UNSUPPORTED, "W4A16MatmulStatic: this shape sums its K slices with arrival counters");
    if (ctx->plan_only) {
        ctx->plan = shadow.plan;
        return OXQ_OK;
    }
    void *sp = g_scratch_ptr[ctx->device >= 0 && ctx->device < SCRATCH_MAX_DEVICES ? ctx->device : 0].load(
        std::memory_order_acquire);
    if (!sp) return fail(OXQ_ERR_RUNTIME, "W4A16MatmulStatic: no static scratch address for device %d", ctx->device);
    shadow.plan_only = false;
    shadow.workspace = sp;
    shadow.workspace_bytes = OXQ_STATIC_SCRATCH_BYTES;
    const int rc = launch_wna16_gemv(&shadow, (hipStream_t)stream, p);
    if (rc == OXQ_OK) ctx->plan = shadow.plan;
    return rc;
}

int oxq_w8a16_matmul(oxq_ctx *ctx, void *stream, const oxq_tensor *x, const oxq_tensor *qweight,
                     const oxq_tensor *qzeros, const oxq_tensor *scales, const oxq_tensor *out) {
    Wna16Problem p;
    OXQ_TRY(check_wna16(ctx, "W8A16Matmul", KIND_GEMV, x, qweight, qzeros, scales, 8, OXQ_PACK_OUT,
                        out, &p));
    int crc;
    if (wcache_forward(ctx, (hipStream_t)stream, p, &crc)) return crc;
    return launch_wna16_gemv(ctx, (hipStream_t)stream, p);
}

int oxq_gptq_matmul(oxq_ctx *ctx, void *stream, const oxq_tensor *x, const oxq_tensor *qweight,
                    const oxq_tensor *qzeros, const oxq_tensor *scales, uint32_t bits,
                    const oxq_tensor *out) {
    Wna16Problem p;
    OXQ_TRY(check_wna16(ctx, "GptqMatmul", KIND_GEMV, x, qweight, qzeros, scales, bits, OXQ_PACK_IN,
                        out, &p));
    int crc;
    if (wcache_forward(ctx, (hipStream_t)stream, p, &crc)) return crc;
    return launch_wna16_gemv(ctx, (hipStream_t)stream, p);
}

int oxq_dequantize_w4(oxq_ctx *ctx, void *stream, const oxq_tensor *qweight,
                      const oxq_tensor *qzeros, const oxq_tensor *scales, const oxq_tensor *out) {
    Wna16Problem p;
    OXQ_TRY(check_wna16(ctx, "DequantizeW4", KIND_DEQUANT, nullptr, qweight, qzeros, scales, 4,
                        OXQ_PACK_OUT, out, &p));
    return launch_wna16_dequant(ctx, (hipStream_t)stream, p, out->data);
}

int oxq_dequantize_w8(oxq_ctx *ctx, void *stream, const oxq_tensor *qweight,
                      const oxq_tensor *qzeros, const oxq_tensor *scales, const oxq_tensor *out) {
    Wna16Problem p;
    OXQ_TRY(check_wna16(ctx, "DequantizeW8", KIND_DEQUANT, nullptr, qweight, qzeros, scales, 8,
                        OXQ_PACK_OUT, out, &p));
    return launch_wna16_dequant(ctx, (hipStream_t)stream, p, out->data);
}

int oxq_dequantize_gptq_packed(oxq_ctx *ctx, void *stream, const oxq_tensor *qweight,
                               const oxq_tensor *qzeros, const oxq_tensor *scales, uint32_t bits,
                               const oxq_tensor *out) {
    Wna16Problem p;
    OXQ_TRY(check_wna16(ctx, "DequantizeGptq", KIND_DEQUANT, nullptr, qweight, qzeros, scales, bits,
                        OXQ_PACK_IN, out, &p));
    return launch_wna16_dequant(ctx, (hipStream_t)stream, p, out->data);
}

int oxq_mpp_quant_matmul(oxq_ctx *ctx, void *stream, const oxq_tensor *x,
                         const oxq_tensor *qweight, const oxq_tensor *qzeros,
                         const oxq_tensor *scales, uint32_t bits, int pack_dim,
                         const oxq_tensor *out) {
    Wna16Problem p;
    OXQ_TRY(check_wna16(ctx, "MppQuantMatmul", KIND_TILE, x, qweight, qzeros, scales, bits, pack_dim,
                        out, &p));
    int crc;
    if (wcache_forward(ctx, (hipStream_t)stream, p, &crc)) return crc;
    return launch_wna16_mfma(ctx, (hipStream_t)stream, p);
}

int oxq_maybe_mpp_quant_matmul(oxq_ctx *ctx, void *stream, const oxq_tensor *x,
                               const oxq_tensor *qweight, const oxq_tensor *qzeros,
                               const oxq_tensor *scales, uint32_t bits, int pack_dim,
                               const oxq_tensor *out, int *taken) {
    if (!taken) return fail(OXQ_ERR_ARG, "maybe_mpp_quant_matmul: taken is NULL");
    *taken = 0;
    // decline rules: metal_ops.rs:2779-2791
    if (!x || !scales) return fail(OXQ_ERR_ARG, "maybe_mpp_quant_matmul: NULL tensor");
    if ((x->dtype != OXQ_BF16 && x->dtype != OXQ_F16) || scales->dtype != x->dtype) return OXQ_OK;
    if (x->device == OXQ_DEVICE_HOST) return OXQ_OK;
    if (x->rank != 2 || x->dims[0] < OXQ_MFMA_MIN_M || !x->contiguous) return OXQ_OK;
    int rc = oxq_mpp_quant_matmul(ctx, stream, x, qweight, qzeros, scales, bits, pack_dim, out);
    if (rc == OXQ_OK) *taken = 1;
    return rc;
}

// ---- GGUF ---------------------------------------------------------------------
int oxq_gguf_quant_matmul(oxq_ctx *ctx, void *stream, const oxq_tensor *x,
                          const oxq_tensor *weight_bytes, int64_t in_features,
                          int64_t out_features, int quant, const oxq_tensor *out) {
    GgufProblem p;
    OXQ_TRY(check_gguf(ctx, "GgufQuantMatmul", true, false, x, weight_bytes, in_features,
                       out_features, quant, out, &p));
    int rc = OXQ_OK;
    if (wcache_forward_gguf(ctx, (hipStream_t)stream, p, &rc)) return rc;
    // Prefill sizes without a cached copy: the matrix-core copy built in the ctx workspace (one pass over the
    // blocks: 10 us for 4096 x 4096 Q4_K), then its prefill kernel, which runs at 1.5 - 1.8 x the tile matmul on the
    // file layout - ahead from about a thousand rows.  Two launches.
    if (!ctx->plan_only && p.act_dtype == OXQ_BF16 && p.M >= 1024 && tune(ctx, OXQ_TUNE_TRANSIENT_REPACK, 1) &&
        gguf_mfma_eligible(ctx, quant, p.K, p.N) && gguf_gemm_takes(ctx, quant, p.M, p.K, p.N, p.act_dtype) &&
        ((uintptr_t)p.x & 15) == 0 && ((uintptr_t)p.w & 1) == 0 &&
        ((gguf_res_bytes(quant, p.K, p.N) + 255) & ~(size_t)255) <= ctx->workspace_bytes) {
        rc = launch_gguf_mfma_repack(ctx, (hipStream_t)stream, quant, p.w, ctx->workspace, p.K, p.N);
        if (rc != OXQ_OK) return rc;
        GgufProblem q = p;
        q.w = (const uint8_t *)ctx->workspace;
        rc = launch_gguf_gemm(ctx, (hipStream_t)stream, q);
        ctx->plan.launches = 2;
        return rc;
    }
    if (gguf_mm_eligible(ctx, p)) return launch_gguf_mm(ctx, (hipStream_t)stream, p);
    return launch_gguf_gemv(ctx, (hipStream_t)stream, p);
}

int oxq_gguf_quant_mul_mm(oxq_ctx *ctx, void *stream, const oxq_tensor *x,
                          const oxq_tensor *weight_bytes, int64_t in_features,
                          int64_t out_features, int quant, const oxq_tensor *out) {
    GgufProblem p;
    OXQ_TRY(check_gguf(ctx, "GgufQuantMulMM", false, false, x, weight_bytes, in_features,
                       out_features, quant, out, &p));
    int rc = OXQ_OK;
    if (wcache_forward_gguf(ctx, (hipStream_t)stream, p, &rc)) return rc;
    // Prefill sizes without a cached copy: the matrix-core copy built in the ctx workspace (one pass over the
    // blocks: 10 us for 4096 x 4096 Q4_K), then its prefill kernel, which runs at 1.5 - 1.8 x the tile matmul on the
    // file layout - ahead from about a thousand rows.  Two launches.
    if (!ctx->plan_only && p.act_dtype == OXQ_BF16 && p.M >= 1024 && tune(ctx, OXQ_TUNE_TRANSIENT_REPACK, 1) &&
        gguf_mfma_eligible(ctx, quant, p.K, p.N) && gguf_gemm_takes(ctx, quant, p.M, p.K, p.N, p.act_dtype) &&
        ((uintptr_t)p.x & 15) == 0 && ((uintptr_t)p.w & 1) == 0 &&
        ((gguf_res_bytes(quant, p.K, p.N) + 255) & ~(size_t)255) <= ctx->workspace_bytes) {
        rc = launch_gguf_mfma_repack(ctx, (hipStream_t)stream, quant, p.w, ctx->workspace, p.K, p.N);
        if (rc != OXQ_OK) return rc;
        GgufProblem q = p;
        q.w = (const uint8_t *)ctx->workspace;
        rc = launch_gguf_gemm(ctx, (hipStream_t)stream, q);
        ctx->plan.launches = 2;
        return rc;
    }
    if (gguf_mm_eligible(ctx, p)) return launch_gguf_mm(ctx, (hipStream_t)stream, p);
    return launch_gguf_gemv(ctx, (hipStream_t)stream, p);
}

int oxq_gguf_dequantize(oxq_ctx *ctx, void *stream, const oxq_tensor *weight_bytes,
                        int64_t in_features, int64_t out_features, int quant,
                        const oxq_tensor *out) {
    GgufProblem p;
    OXQ_TRY(check_gguf(ctx, "GgufDequantize", false, true, nullptr, weight_bytes, in_features,
                       out_features, quant, out, &p));
    return launch_gguf_dequant(ctx, (hipStream_t)stream, p, (float *)out->data);
}

// ---- load-time transforms into the AWQ layout --------------------------------------
static int check_2d(const char *op, const char *what, const oxq_tensor *t, int64_t d0, int64_t d1) {
    if (t->rank != 2 || t->dims[0] != d0 || t->dims[1] != d1 || !t->contiguous)
        return fail(OXQ_ERR_SHAPE, "%s: %s must be a contiguous [%lld, %lld]", op, what, (long long)d0,
                    (long long)d1);
    return OXQ_OK;
}

// awq.rs:187-254
int oxq_compressed_to_awq(oxq_ctx *ctx, void *stream, const oxq_tensor *weight_packed,
                          const oxq_tensor *weight_scale, const oxq_tensor *qweight_out,
                          const oxq_tensor *qzeros_out, const oxq_tensor *scales_out) {
    const char *op = "compressed_to_awq";
    if (!ctx) return fail(OXQ_ERR_ARG, "%s: ctx is NULL", op);
    OXQ_TRY(check_tensor(ctx, op, "weight_packed", weight_packed));
    OXQ_TRY(check_tensor(ctx, op, "weight_scale", weight_scale));
    OXQ_TRY(check_tensor(ctx, op, "qweight_out", qweight_out));
    OXQ_TRY(check_tensor(ctx, op, "qzeros_out", qzeros_out));
    OXQ_TRY(check_tensor(ctx, op, "scales_out", scales_out));
    if (weight_packed->rank != 2) return fail(OXQ_ERR_SHAPE, "%s: weight_packed must be 2-D [out, in/8]", op);
    if (weight_scale->rank != 2) return fail(OXQ_ERR_SHAPE, "%s: weight_scale must be 2-D [out, groups]", op);
    if (!weight_packed->contiguous || !weight_scale->contiguous)
        return fail(OXQ_ERR_CONTIGUOUS, "%s: inputs must be contiguous", op);
    if (!is_packed_dtype(weight_packed->dtype))
        return fail(OXQ_ERR_DTYPE, "%s: weight_packed must be I32 or U32, got %s", op,
                    dtype_name(weight_packed->dtype));
    if (!is_float_dtype(weight_scale->dtype))
        return fail(OXQ_ERR_DTYPE, "%s: weight_scale must be F32, F16 or BF16", op);
    const int64_t out_f = weight_packed->dims[0], packed_in = weight_packed->dims[1], in_f = packed_in * 8;
    const int64_t groups = weight_scale->dims[1];
    if (weight_scale->dims[0] != out_f)
        return fail(OXQ_ERR_SHAPE, "%s: weight_scale dim0 %lld != weight_packed out_features %lld", op,
                    (long long)weight_scale->dims[0], (long long)out_f);
    if (groups == 0 || in_f % groups != 0)
        return fail(OXQ_ERR_SHAPE, "%s: in_features %lld not divisible by scale groups %lld", op, (long long)in_f,
                    (long long)groups);
    if (out_f % 8 != 0)
        return fail(OXQ_ERR_SHAPE, "%s: out_features %lld not divisible by pack factor 8", op, (long long)out_f);
    if (!is_packed_dtype(qweight_out->dtype) || !is_packed_dtype(qzeros_out->dtype) ||
        scales_out->dtype != weight_scale->dtype)
        return fail(OXQ_ERR_DTYPE, "%s: outputs must be packed I32/U32 and scales of the checkpoint's dtype", op);
    OXQ_TRY(check_2d(op, "qweight_out", qweight_out, in_f, out_f / 8));
    OXQ_TRY(check_2d(op, "qzeros_out", qzeros_out, groups, out_f / 8));
    OXQ_TRY(check_2d(op, "scales_out", scales_out, groups, out_f));
    if (out_f > INT32_MAX || in_f > INT32_MAX) return fail(OXQ_ERR_SHAPE, "%s: dimension exceeds 2^31-1", op);
    return launch_compressed_to_awq(ctx, (hipStream_t)stream, (const uint32_t *)weight_packed->data,
                                    weight_scale->data, (int)dtype_size(weight_scale->dtype),
                                    (uint32_t *)qweight_out->data, (uint32_t *)qzeros_out->data, scales_out->data,
                                    out_f, in_f, groups);
}

// awq.rs:256-323
int oxq_concat_awq_along_out(oxq_ctx *ctx, void *stream, int bits, int n_parts, const oxq_tensor *qweights,
                             const oxq_tensor *qzeros, const oxq_tensor *scales, const oxq_tensor *qweight_out,
                             const oxq_tensor *qzeros_out, const oxq_tensor *scales_out) {
    const char *op = "AWQ fuse";
    if (!ctx) return fail(OXQ_ERR_ARG, "%s: ctx is NULL", op);
    if (n_parts <= 0 || !qweights || !scales) return fail(OXQ_ERR_ARG, "concat_awq_along_out: no parts");
    if (!qzeros) return fail(OXQ_ERR_ARG, "%s: qzeros missing on a part, not an AWQ tensor", op);
    if (bits != 4 && bits != 8) return fail(OXQ_ERR_BITS, "%s: bits must be 4 or 8, got %d", op, bits);
    const int64_t pf = 32 / bits;
    int64_t in_f = 0, groups = 0, total_out = 0;
    for (int i = 0; i < n_parts; ++i) {
        char what[32];
        snprintf(what, sizeof what, "part %d qweight", i);
        OXQ_TRY(check_tensor(ctx, op, what, &qweights[i]));
        snprintf(what, sizeof what, "part %d qzeros", i);
        OXQ_TRY(check_tensor(ctx, op, what, &qzeros[i]));
        snprintf(what, sizeof what, "part %d scales", i);
        OXQ_TRY(check_tensor(ctx, op, what, &scales[i]));
        const oxq_tensor &qw = qweights[i], &qz = qzeros[i], &sc = scales[i];
        if (qw.rank != 2 || qz.rank != 2 || sc.rank != 2 || !qw.contiguous || !qz.contiguous || !sc.contiguous)
            return fail(OXQ_ERR_SHAPE, "%s: part %d tensors must be contiguous and 2-D", op, i);
        if (!is_packed_dtype(qw.dtype) || !is_packed_dtype(qz.dtype))
            return fail(OXQ_ERR_DTYPE, "%s: part %d qweight/qzeros must be I32 or U32", op, i);
        if (sc.dtype != scales[0].dtype || (sc.dtype != OXQ_F16 && sc.dtype != OXQ_BF16 && sc.dtype != OXQ_F32))
            return fail(OXQ_ERR_DTYPE, "%s: part %d scales dtype differs from part 0 or is not a float type", op, i);
        const int64_t out_i = sc.dims[1];
        if (out_i % pf != 0)
            return fail(OXQ_ERR_SHAPE, "%s: part %d out_features %lld not divisible by pack_factor %lld", op, i,
                        (long long)out_i, (long long)pf);
        if (qw.dims[1] * pf != out_i || qz.dims[1] * pf != out_i || qz.dims[0] != sc.dims[0] || sc.dims[0] == 0 ||
            qw.dims[0] % sc.dims[0] != 0)
            return fail(OXQ_ERR_SHAPE, "%s: part %d tensors do not describe one AWQ weight", op, i);
        if (i == 0) {
            in_f = qw.dims[0];
            groups = sc.dims[0];
        } else {
            if (qw.dims[0] != in_f)
                return fail(OXQ_ERR_SHAPE, "%s: in_features mismatch at part %d: expected %lld, got %lld", op, i,
                            (long long)in_f, (long long)qw.dims[0]);
            if (sc.dims[0] != groups)
                return fail(OXQ_ERR_SHAPE, "%s: group_size mismatch at part %d: expected %lld, got %lld", op, i,
                            (long long)(in_f / groups), (long long)(qw.dims[0] / sc.dims[0]));
        }
        total_out += out_i;
    }
    OXQ_TRY(check_tensor(ctx, op, "qweight_out", qweight_out));
    OXQ_TRY(check_tensor(ctx, op, "qzeros_out", qzeros_out));
    OXQ_TRY(check_tensor(ctx, op, "scales_out", scales_out));
    if (!is_packed_dtype(qweight_out->dtype) || !is_packed_dtype(qzeros_out->dtype) ||
        scales_out->dtype != scales[0].dtype)
        return fail(OXQ_ERR_DTYPE, "%s: outputs must be packed I32/U32 and scales of the parts' dtype", op);
    OXQ_TRY(check_2d(op, "qweight_out", qweight_out, in_f, total_out / pf));
    OXQ_TRY(check_2d(op, "qzeros_out", qzeros_out, groups, total_out / pf));
    OXQ_TRY(check_2d(op, "scales_out", scales_out, groups, total_out));
    if (total_out > INT32_MAX || in_f > INT32_MAX) return fail(OXQ_ERR_SHAPE, "%s: dimension exceeds 2^31-1", op);
    const int64_t sb = (int64_t)dtype_size(scales[0].dtype);
    if ((total_out * sb) % 4 != 0) return fail(OXQ_ERR_SHAPE, "%s: scales rows must be a multiple of 4 bytes", op);
    set_plan(ctx, "concat_awq_along_out", dim3(1), dim3(256), 1, (uint32_t)(3 * n_parts), 0);
    int64_t col = 0;
    for (int i = 0; i < n_parts; ++i) {
        const int64_t out_i = scales[i].dims[1];
        // widths in 32-bit words; out_i is a multiple of the pack factor, so 16-bit scale rows are whole words
        OXQ_TRY(launch_copy2d_u32(ctx, (hipStream_t)stream, qweights[i].data, qweight_out->data, in_f, out_i / pf,
                                  total_out / pf, col / pf));
        OXQ_TRY(launch_copy2d_u32(ctx, (hipStream_t)stream, qzeros[i].data, qzeros_out->data, groups, out_i / pf,
                                  total_out / pf, col / pf));
        OXQ_TRY(launch_copy2d_u32(ctx, (hipStream_t)stream, scales[i].data, scales_out->data, groups, out_i * sb / 4,
                                  total_out * sb / 4, col * sb / 4));
        col += out_i;
    }
    return OXQ_OK;
}

// awq.rs:637-742
int oxq_rtn_quantize_awq(oxq_ctx *ctx, void *stream, const oxq_tensor *weight, int64_t group_size,
                         const oxq_tensor *qweight_out, const oxq_tensor *qzeros_out,
                         const oxq_tensor *scales_out) {
    const char *op = "rtn_quantize_awq";
    if (!ctx) return fail(OXQ_ERR_ARG, "%s: ctx is NULL", op);
    OXQ_TRY(check_tensor(ctx, op, "weight", weight));
    OXQ_TRY(check_tensor(ctx, op, "qweight_out", qweight_out));
    OXQ_TRY(check_tensor(ctx, op, "qzeros_out", qzeros_out));
    OXQ_TRY(check_tensor(ctx, op, "scales_out", scales_out));
    if (weight->rank != 2) return fail(OXQ_ERR_SHAPE, "%s: weight must be 2-D [out, in]", op);
    if (!weight->contiguous) return fail(OXQ_ERR_CONTIGUOUS, "%s: weight must be contiguous", op);
    if (!is_float_dtype(weight->dtype)) return fail(OXQ_ERR_DTYPE, "%s: weight must be F32, F16 or BF16", op);
    const int64_t out_f = weight->dims[0], in_f = weight->dims[1];
    if (out_f % 8 != 0)
        return fail(OXQ_ERR_SHAPE, "%s: out_features (%lld) must be a multiple of 8", op, (long long)out_f);
    if (group_size <= 0 || in_f % group_size != 0)
        return fail(OXQ_ERR_GROUP, "%s: in_features (%lld) not divisible by group_size (%lld)", op, (long long)in_f,
                    (long long)group_size);
    const int64_t groups = in_f / group_size;
    if (!is_packed_dtype(qweight_out->dtype) || !is_packed_dtype(qzeros_out->dtype) || scales_out->dtype != OXQ_F32)
        return fail(OXQ_ERR_DTYPE, "%s: outputs must be packed I32/U32 and F32 scales", op);
    OXQ_TRY(check_2d(op, "qweight_out", qweight_out, in_f, out_f / 8));
    OXQ_TRY(check_2d(op, "qzeros_out", qzeros_out, groups, out_f / 8));
    OXQ_TRY(check_2d(op, "scales_out", scales_out, groups, out_f));
    if (out_f > INT32_MAX || in_f > INT32_MAX) return fail(OXQ_ERR_SHAPE, "%s: dimension exceeds 2^31-1", op);
    return launch_rtn_quantize_awq(ctx, (hipStream_t)stream, weight->data, weight->dtype,
                                   (uint32_t *)qweight_out->data, (uint32_t *)qzeros_out->data,
                                   (float *)scales_out->data, out_f, in_f, group_size);
}

// gguf_weights.rs:255-291
int oxq_gguf_depermute_qk_rows(oxq_ctx *ctx, void *stream, const oxq_tensor *weight_bytes, int64_t in_features,
                               int64_t out_features, int quant, int64_t n_heads, int64_t head_dim,
                               const oxq_tensor *out) {
    const char *op = "depermute_qk_rows";
    if (!ctx) return fail(OXQ_ERR_ARG, "%s: ctx is NULL", op);
    int64_t be, bb;
    if (oxq_gguf_block_layout(quant, &be, &bb) != OXQ_OK) return fail(OXQ_ERR_ARG, "%s: unknown GGUF quant %d", op, quant);
    OXQ_TRY(check_tensor(ctx, op, "weight_bytes", weight_bytes));
    OXQ_TRY(check_tensor(ctx, op, "out", out));
    if (n_heads <= 0 || head_dim <= 0 || out_features != n_heads * head_dim || head_dim % 2 != 0)
        return fail(OXQ_ERR_SHAPE, "%s: shape [%lld, %lld] incompatible with %lld heads x %lld dims", op,
                    (long long)out_features, (long long)in_features, (long long)n_heads, (long long)head_dim);
    if (in_features <= 0 || in_features % be != 0)
        return fail(OXQ_ERR_SHAPE, "%s: row length %lld not divisible by %s block size %lld", op, (long long)in_features,
                    gguf_name(quant), (long long)be);
    const int64_t row_bytes = in_features / be * bb, total = out_features * row_bytes;
    if (weight_bytes->dtype != OXQ_U8 || out->dtype != OXQ_U8)
        return fail(OXQ_ERR_DTYPE, "%s: weight_bytes and out must be U8", op);
    if (!weight_bytes->contiguous || !out->contiguous || numel(weight_bytes) != total || numel(out) != total)
        return fail(OXQ_ERR_SHAPE, "%s: weight_bytes and out must be contiguous tensors of %lld bytes", op,
                    (long long)total);
    if (weight_bytes->data == out->data && total > 0 && !ctx->plan_only)
        return fail(OXQ_ERR_ARG, "%s: out must not alias weight_bytes", op);
    if (row_bytes / 2 > INT32_MAX || head_dim > INT32_MAX) return fail(OXQ_ERR_SHAPE, "%s: dimension exceeds 2^31-1", op);
    return launch_gguf_depermute_rows(ctx, (hipStream_t)stream, (const uint8_t *)weight_bytes->data,
                                      (uint8_t *)out->data, out_features, row_bytes, head_dim);
}

// ---- block-scaled F8E4M3 -----------------------------------------------------------
// metal_ops.rs:5562
int oxq_cast_f8e4m3_to_f32(oxq_ctx *ctx, void *stream, const oxq_tensor *t, const oxq_tensor *out) {
    const char *op = "cast-f8e4m3-f32";
    if (!ctx) return fail(OXQ_ERR_ARG, "%s: ctx is NULL", op);
    OXQ_TRY(check_tensor(ctx, op, "input", t));
    OXQ_TRY(check_tensor(ctx, op, "out", out));
    if (t->dtype != OXQ_U8) return fail(OXQ_ERR_DTYPE, "%s: expected F8E4M3 bytes (U8) input, got %s", op, dtype_name(t->dtype));
    if (!t->contiguous) return fail(OXQ_ERR_CONTIGUOUS, "%s: input must be contiguous", op);
    if (out->dtype != OXQ_F32 || !out->contiguous || numel(out) != numel(t))
        return fail(OXQ_ERR_SHAPE, "%s: out must be a contiguous F32 tensor of the input's size", op);
    return launch_cast_f8e4m3_f32(ctx, (hipStream_t)stream, (const uint8_t *)t->data, (float *)out->data,
                                  (size_t)numel(t));
}

// shared checks of F8BlockDequantBf16 (metal_ops.rs:5589-5613) and F8Gemv (5703-5731)
static int check_f8(oxq_ctx *ctx, const char *op, const oxq_tensor *x, const oxq_tensor *bytes,
                    const oxq_tensor *scales, const oxq_tensor *out, bool decode, F8Problem *p) {
    if (!ctx) return fail(OXQ_ERR_ARG, "%s: ctx is NULL", op);
    if (x) OXQ_TRY(check_tensor(ctx, op, "x", x));
    OXQ_TRY(check_tensor(ctx, op, "bytes", bytes));
    OXQ_TRY(check_tensor(ctx, op, "scales", scales));
    OXQ_TRY(check_tensor(ctx, op, "out", out));
    if (bytes->dtype != OXQ_U8 || scales->dtype != OXQ_F32)
        return fail(OXQ_ERR_DTYPE, "%s: expected U8 bytes and F32 scales, got %s/%s", op, dtype_name(bytes->dtype),
                    dtype_name(scales->dtype));
    if (!bytes->contiguous || !scales->contiguous) return fail(OXQ_ERR_CONTIGUOUS, "%s: inputs must be contiguous", op);
    if (bytes->rank != 2 || scales->rank != 2) return fail(OXQ_ERR_SHAPE, "%s: bytes and scales must be 2-D", op);
    const int64_t rows = bytes->dims[0], cols = bytes->dims[1], s_rows = scales->dims[0], s_cols = scales->dims[1];
    if (s_rows == 0 || s_cols == 0 || rows % s_rows != 0 || cols % s_cols != 0)
        return fail(OXQ_ERR_SHAPE, "%s: scale grid [%lld, %lld] does not tile weight [%lld, %lld]", op,
                    (long long)s_rows, (long long)s_cols, (long long)rows, (long long)cols);
    if (rows > INT32_MAX || cols > INT32_MAX) return fail(OXQ_ERR_SHAPE, "%s: dimension exceeds 2^31-1", op);
    int64_t m = 0;
    if (x) {
        if (x->dtype != OXQ_BF16) return fail(OXQ_ERR_DTYPE, "%s: x must be BF16, got %s", op, dtype_name(x->dtype));
        if (!x->contiguous) return fail(OXQ_ERR_CONTIGUOUS, "%s: x must be contiguous", op);
        if (x->rank != 2 || x->dims[1] != cols || x->dims[0] == 0 || (decode && x->dims[0] > 8)) {
            char b0[96];
            dims_str(x, b0, sizeof b0);
            return fail(decode && x->rank == 2 && x->dims[1] == cols ? OXQ_ERR_M_RANGE : OXQ_ERR_SHAPE,
                        "%s: x shape %s incompatible with in_features %lld%s", op, b0, (long long)cols,
                        decode ? " (m must be 1..=8)" : "");
        }
        m = x->dims[0];
        if (out->dtype != OXQ_BF16 || out->rank != 2 || out->dims[0] != m || out->dims[1] != rows || !out->contiguous)
            return fail(OXQ_ERR_SHAPE, "%s: out must be a contiguous BF16 [%lld, %lld]", op, (long long)m,
                        (long long)rows);
        if (m > INT32_MAX) return fail(OXQ_ERR_SHAPE, "%s: dimension exceeds 2^31-1", op);
    } else if (out->dtype != OXQ_BF16 || out->rank != 2 || out->dims[0] != rows || out->dims[1] != cols ||
               !out->contiguous) {
        return fail(OXQ_ERR_SHAPE, "%s: out must be a contiguous BF16 [%lld, %lld]", op, (long long)rows,
                    (long long)cols);
    }
    p->x = x ? x->data : nullptr;
    p->w = (const uint8_t *)bytes->data;
    p->scales = (const float *)scales->data;
    p->y = out->data;
    p->M = m, p->K = cols, p->N = rows;
    p->block_r = rows / s_rows, p->block_c = cols / s_cols, p->s_cols = s_cols;
    return OXQ_OK;
}

// metal_ops.rs:5809
int oxq_f8_block_dequant_bf16(oxq_ctx *ctx, void *stream, const oxq_tensor *bytes, const oxq_tensor *scales,
                              const oxq_tensor *out) {
    F8Problem p;
    OXQ_TRY(check_f8(ctx, "f8-block-dequant-bf16", nullptr, bytes, scales, out, false, &p));
    return launch_f8_block_dequant(ctx, (hipStream_t)stream, p, (uint16_t *)out->data);
}

// metal_ops.rs:5788 (1 <= m <= 8)
int oxq_f8_gemv(oxq_ctx *ctx, void *stream, const oxq_tensor *x, const oxq_tensor *bytes,
                const oxq_tensor *scales, const oxq_tensor *out) {
    F8Problem p;
    OXQ_TRY(check_f8(ctx, "f8-gemv", x, bytes, scales, out, true, &p));
    if (f8_mm_eligible(ctx, p)) return launch_f8_mm(ctx, (hipStream_t)stream, p);
    return launch_f8_gemv(ctx, (hipStream_t)stream, p);
}

// moe.rs:106-113 Fp8Cached::forward: the GEMV for decode-sized batches, beyond it the
// dequantized weight times x - here without materializing the dense weight
int oxq_f8_matmul(oxq_ctx *ctx, void *stream, const oxq_tensor *x, const oxq_tensor *bytes,
                  const oxq_tensor *scales, const oxq_tensor *out) {
    F8Problem p;
    OXQ_TRY(check_f8(ctx, "f8-matmul", x, bytes, scales, out, false, &p));
    if (f8_mm_eligible(ctx, p)) return launch_f8_mm(ctx, (hipStream_t)stream, p);
    return launch_f8_gemv(ctx, (hipStream_t)stream, p);
}

// ---- MXFP4 ---------------------------------------------------------------------
int oxq_mxfp4_matmul(oxq_ctx *ctx, void *stream, const oxq_tensor *x, const oxq_tensor *blocks,
                     const oxq_tensor *scales, int64_t k, int64_t n, const oxq_tensor *out) {
    Mxfp4Problem p;
    OXQ_TRY(check_mxfp4(ctx, "Mxfp4Matmul", false, x, blocks, scales, k, n, 0, out, &p));
    char b0[96];
    dims_str(out, b0, sizeof b0);
    if (out->rank != 2 || out->dims[0] != p.M || out->dims[1] != n || !out->contiguous)
        return fail(OXQ_ERR_SHAPE, "Mxfp4Matmul: output shape %s != [%lld, %lld]", b0,
                    (long long)p.M, (long long)n);
    return launch_mxfp4_gemv(ctx, (hipStream_t)stream, p);
}

int oxq_mxfp4_dequantize(oxq_ctx *ctx, void *stream, const oxq_tensor *blocks,
                         const oxq_tensor *scales, int64_t k, int64_t n, const oxq_tensor *out) {
    Mxfp4Problem p;
    OXQ_TRY(check_mxfp4(ctx, "Mxfp4Dequantize", true, nullptr, blocks, scales, k, n, 0, out, &p));
    if (out->rank != 2 || out->dims[0] != n || out->dims[1] != k || !out->contiguous)
        return fail(OXQ_ERR_SHAPE, "Mxfp4Dequantize: output must be a contiguous [%lld, %lld]",
                    (long long)n, (long long)k);
    return launch_mxfp4_dequant(ctx, (hipStream_t)stream, p, (float *)out->data);
}

// The grouped MXFP4 op behind the weight cache: the stacked expert tensors of a projection (keyed by the addresses
// of blocks and scales) get the resident experts' tile-major copy on their first call; later calls run the decode
// GEMV or the tiles of an expert's pairs on it, as an oxq_mxfp4_experts handle would.
static bool wcache_forward_mxfp4(oxq_ctx *ctx, hipStream_t s, const Mxfp4Problem &p, int *rc) {
    if (!ctx->wcache_limit || ctx->plan_only || p.n_experts <= 0 || !mxfp4_res_eligible(p.K, p.N)) return false;
    if (((uintptr_t)p.x & 15) || ((uintptr_t)p.blocks & 15)) return false;
    const bool prefill = (uint64_t)p.M * (uint64_t)p.K * 2u < (1ull << 31) && ((uintptr_t)p.y & 3) == 0 &&
                         mxfp4_gemm_form(ctx, p.n_pairs, p.n_experts, p.K, p.N) != 0;
    if (!prefill && p.n_pairs >= 8 * p.n_experts) return false;  // the tile matmul on the caller's tensors
    const int kind = -3;
    if (!ctx->wcache) {
        ctx->wcache = new (std::nothrow) oxq_weight_cache();
        if (!ctx->wcache) return false;
    }
    oxq_weight_cache *c = ctx->wcache;
    ++c->tick;
    oxq_weight_cache::Entry *hit = nullptr;
    for (auto &e : c->entries)
        if (e.qw == p.blocks && e.qz == nullptr && e.sc == p.scales && e.K == p.K && e.N == p.N && e.bits == (int)p.n_experts &&
            e.pack_dim == kind) {
            hit = &e;
            break;
        }
    const size_t w_bytes = (mxfp4_res_weight_bytes(p.n_experts, p.K, p.N) + 255) & ~(size_t)255;
    if (!hit) {
        hipStreamCaptureStatus cs = hipStreamCaptureStatusNone;
        if (hipStreamIsCapturing(s, &cs) != hipSuccess || cs != hipStreamCaptureStatusNone) {
            (void)hipGetLastError();
            return false;
        }
        const size_t bytes = w_bytes + ((mxfp4_res_scale_bytes(p.n_experts, p.K, p.N) + 255) & ~(size_t)255);
        if (!wcache_make_room(ctx, bytes)) return false;
        void *mem = nullptr;
        if (hipMalloc(&mem, bytes) != hipSuccess) {
            (void)hipGetLastError();
            return false;
        }
        oxq_weight_cache::Entry e{p.blocks, nullptr, p.scales, p.K, p.N, 0, 0, (int)p.n_experts, kind,
                                  Pk4Weights{(uint32_t *)mem, nullptr, p.K, p.N, 0, 0, 0, 0, 0, 0}, bytes, 0, false};
        const int prc = launch_mxfp4_repack(ctx, s, p.blocks, p.scales, mem, (unsigned char *)mem + w_bytes, p.n_experts, p.K, p.N);
        if (prc != OXQ_OK) {
            (void)hipFree(mem);
            *rc = prc;
            return true;
        }
        try {
            c->entries.push_back(e);
        } catch (...) {
            (void)hipFree(mem);
            return false;
        }
        c->bytes += bytes;
        hit = &c->entries.back();
    }
    hit->last_use = c->tick;
    wcache_pin_if_capturing(s, hit);
    Mxfp4Problem q = p;
    q.blocks = (const uint8_t *)hit->w.pw;
    q.scales = (const uint8_t *)hit->w.pw + w_bytes;
    *rc = prefill ? launch_mxfp4_res_gemm(ctx, s, q) : launch_mxfp4_res_gemv(ctx, s, q);
    return true;
}

static int moe_matmul_impl(const char *op, oxq_ctx *ctx, void *stream, const oxq_tensor *x, const oxq_tensor *blocks,
                           const oxq_tensor *scales, const oxq_tensor *bias, const oxq_tensor *expert_offsets,
                           const oxq_tensor *token_ids, int gather_rows, int64_t k, int64_t n, bool swiglu, float limit,
                           const oxq_tensor *out, int *fused) {
    if (!ctx) return fail(OXQ_ERR_ARG, "%s: ctx is NULL", op);
    if (fused) *fused = 0;
    OXQ_TRY(check_tensor(ctx, op, "expert_offsets", expert_offsets));
    if (expert_offsets->dtype != OXQ_I32 || expert_offsets->rank != 1 || expert_offsets->dims[0] < 2 ||
        !expert_offsets->contiguous)
        return fail(OXQ_ERR_SHAPE, "%s: expert_offsets must be a contiguous I32 [n_experts + 1]", op);
    const int64_t n_experts = expert_offsets->dims[0] - 1;
    Mxfp4Problem p;
    OXQ_TRY(check_mxfp4(ctx, op, false, x, blocks, scales, k, n, n_experts, out, &p));
    if (swiglu && (n & 1)) return fail(OXQ_ERR_SHAPE, "%s: interleaved gate / up rows need an even n, got %lld", op, (long long)n);
    const int64_t out_cols = swiglu ? n / 2 : n;
    if (out->rank != 2 || out->dims[1] != out_cols || !out->contiguous)
        return fail(OXQ_ERR_SHAPE, "%s: out must be a contiguous [n_pairs, %lld]", op, (long long)out_cols);
    const int64_t n_pairs = out->dims[0];
    if (gather_rows) {
        OXQ_TRY(check_tensor(ctx, op, "token_ids", token_ids));
        if (token_ids->dtype != OXQ_I32 || numel(token_ids) != n_pairs || !token_ids->contiguous)
            return fail(OXQ_ERR_SHAPE, "%s: token_ids must be a contiguous I32 [%lld]", op,
                        (long long)n_pairs);
    } else if (x->dims[0] != n_pairs) {
        return fail(OXQ_ERR_SHAPE, "%s: x has %lld rows, out has %lld", op, (long long)x->dims[0],
                    (long long)n_pairs);
    }
    if (bias) {
        OXQ_TRY(check_tensor(ctx, op, "bias", bias));
        if (bias->dtype != OXQ_BF16 || numel(bias) != n_experts * n || !bias->contiguous)
            return fail(OXQ_ERR_SHAPE, "%s: bias must be a contiguous BF16 [%lld, %lld]", op,
                        (long long)n_experts, (long long)n);
        p.bias = bias->data;
    }
    p.n_experts = n_experts;
    p.expert_offsets = (const int32_t *)expert_offsets->data;
    p.token_ids = gather_rows ? (const int32_t *)token_ids->data : nullptr;
    p.n_pairs = n_pairs;
    p.swiglu = swiglu ? 1 : 0;
    p.swiglu_limit = limit;
    int crc = OXQ_OK;
    if (wcache_forward_mxfp4(ctx, (hipStream_t)stream, p, &crc)) {
        if (crc == OXQ_OK && fused) *fused = 1;
        return crc;
    }
    const int rc = launch_mxfp4_gemv(ctx, (hipStream_t)stream, p);
    if (rc == OXQ_DECLINED) return OXQ_OK;  // *fused stays 0, nothing was enqueued
    if (rc == OXQ_OK && fused) *fused = 1;
    return rc;
}

int oxq_mxfp4_moe_matmul(oxq_ctx *ctx, void *stream, const oxq_tensor *x,
                         const oxq_tensor *blocks, const oxq_tensor *scales,
                         const oxq_tensor *bias, const oxq_tensor *expert_offsets,
                         const oxq_tensor *token_ids, int gather_rows, int64_t k, int64_t n,
                         const oxq_tensor *out) {
    return moe_matmul_impl("Mxfp4MoeMatmul", ctx, stream, x, blocks, scales, bias, expert_offsets, token_ids,
                           gather_rows, k, n, false, 0.0f, out, nullptr);
}

int oxq_mxfp4_moe_gate_up_swiglu(oxq_ctx *ctx, void *stream, const oxq_tensor *x, const oxq_tensor *blocks,
                                 const oxq_tensor *scales, const oxq_tensor *bias,
                                 const oxq_tensor *expert_offsets, const oxq_tensor *token_ids, int gather_rows,
                                 int64_t k, int64_t n, float limit, const oxq_tensor *out, int *fused) {
    if (!fused) return fail(OXQ_ERR_ARG, "Mxfp4MoeGateUpSwiglu: fused is NULL");
    return moe_matmul_impl("Mxfp4MoeGateUpSwiglu", ctx, stream, x, blocks, scales, bias, expert_offsets, token_ids,
                           gather_rows, k, n, true, limit, out, fused);
}

// ---- resident MXFP4 experts (moe.rs:366-417 load_gpt_oss keeps the stacked tensors for the model's life) ----
int oxq_mxfp4_experts_new(oxq_ctx *ctx, const oxq_tensor *blocks, const oxq_tensor *scales, const oxq_tensor *bias,
                          int64_t n_experts, int64_t k, int64_t n, oxq_mxfp4_experts **out) {
    const char *op = "Mxfp4Experts";
    if (!ctx || !out) return fail(OXQ_ERR_ARG, "%s: NULL argument", op);
    *out = nullptr;
    OXQ_TRY(check_tensor(ctx, op, "blocks", blocks));
    OXQ_TRY(check_tensor(ctx, op, "scales", scales));
    if (blocks->dtype != OXQ_U8 || scales->dtype != OXQ_U8)
        return fail(OXQ_ERR_DTYPE, "%s: blocks/scales must be U8, got %s/%s", op, dtype_name(blocks->dtype),
                    dtype_name(scales->dtype));
    if (n_experts <= 0 || k <= 0 || n <= 0 || k % 32 != 0)
        return fail(OXQ_ERR_SHAPE, "%s: %lld experts of [%lld, %lld]: K must be a positive multiple of 32", op,
                    (long long)n_experts, (long long)n, (long long)k);
    if (k > INT32_MAX || n > INT32_MAX || n_experts > 65535)
        return fail(OXQ_ERR_SHAPE, "%s: dimension out of range", op);
    const int64_t nb = k / 32;
    if (numel(blocks) != n_experts * n * nb * 16 || numel(scales) != n_experts * n * nb || !blocks->contiguous ||
        !scales->contiguous)
        return fail(OXQ_ERR_SHAPE, "%s: blocks %lld / scales %lld elements don't match %lld x [%lld, %lld]", op,
                    (long long)numel(blocks), (long long)numel(scales), (long long)n_experts, (long long)n,
                    (long long)k);
    if (bias) {
        OXQ_TRY(check_tensor(ctx, op, "bias", bias));
        if (bias->dtype != OXQ_BF16 || numel(bias) != n_experts * n || !bias->contiguous)
            return fail(OXQ_ERR_SHAPE, "%s: bias must be a contiguous BF16 [%lld, %lld]", op, (long long)n_experts,
                        (long long)n);
    }
    oxq_mxfp4_experts *h = new (std::nothrow) oxq_mxfp4_experts();
    if (!h) return fail(OXQ_ERR_RUNTIME, "%s: out of host memory", op);
    h->ctx = ctx;
    h->blocks = *blocks;
    h->scales = *scales;
    h->has_bias = bias != nullptr;
    if (bias) h->bias = *bias;
    h->n_experts = n_experts;
    h->k = k;
    h->n = n;
    h->pw = h->ps = nullptr;
    h->owns = false;
    const bool want = tune(ctx, OXQ_TUNE_PREPACK, 1) != 0 && mxfp4_res_eligible(k, n) && !((uintptr_t)blocks->data & 15);
    if (want && !ctx->plan_only) {
        int prev = 0;
        (void)hipGetDevice(&prev);
        hipError_t e = hipSetDevice(ctx->device);
        int rc = OXQ_OK;
        if (e == hipSuccess) e = hipMalloc(&h->pw, mxfp4_res_weight_bytes(n_experts, k, n));
        if (e == hipSuccess) e = hipMalloc(&h->ps, mxfp4_res_scale_bytes(n_experts, k, n));
        if (e != hipSuccess) {
            rc = fail(OXQ_ERR_RUNTIME, "%s: repack allocation failed: %s", op, hipGetErrorString(e));
        } else {
            rc = launch_mxfp4_repack(ctx, nullptr, (const uint8_t *)blocks->data, (const uint8_t *)scales->data, h->pw,
                                     h->ps, n_experts, k, n);
            if (rc == OXQ_OK && (e = hipStreamSynchronize(nullptr)) != hipSuccess)
                rc = fail(OXQ_ERR_RUNTIME, "%s: repack failed: %s", op, hipGetErrorString(e));
        }
        (void)hipSetDevice(prev);
        if (rc != OXQ_OK) {
            if (h->pw) (void)hipFree(h->pw);
            if (h->ps) (void)hipFree(h->ps);
            delete h;
            return rc;
        }
        h->owns = true;
    } else if (want) {
        h->pw = h->ps = (void *)16;  // plan-only: routes as a resident copy would, nothing is dereferenced
    }
    *out = h;
    return OXQ_OK;
}

static int experts_forward(oxq_mxfp4_experts *h, void *stream, const oxq_tensor *x, const oxq_tensor *expert_offsets,
                           const oxq_tensor *token_ids, int gather_rows, bool swiglu, float limit, const oxq_tensor *out,
                           int *fused) {
    const char *op = swiglu ? "Mxfp4ExpertsGateUpSwiglu" : "Mxfp4ExpertsMatmul";
    if (!h) return fail(OXQ_ERR_ARG, "%s: handle is NULL", op);
    // same checks and, for the sizes the resident kernel does not take, the same kernels as the stateless op
    oxq_ctx *ctx = h->ctx;
    if (fused) *fused = 0;
    OXQ_TRY(check_tensor(ctx, op, "expert_offsets", expert_offsets));
    if (expert_offsets->dtype != OXQ_I32 || expert_offsets->rank != 1 || expert_offsets->dims[0] != h->n_experts + 1 ||
        !expert_offsets->contiguous)
        return fail(OXQ_ERR_SHAPE, "%s: expert_offsets must be a contiguous I32 [%lld]", op, (long long)h->n_experts + 1);
    const bool resident = h->pw != nullptr;
    const int64_t n_pairs = (out && out->rank == 2) ? out->dims[0] : 0;
    // many pairs per expert (prefill) convert a weight once per 64 tokens: the prefill kernel on the copy, or
    // (sizes it does not take) the tile matmul, which reads the checkpoint layout
    // (its 32-bit offsets into x hold up to 2 GiB; more than that takes the tile matmul as before)
    const bool prefill = resident && x && x->rank == 2 && (uint64_t)x->dims[0] * (uint64_t)h->k * 2u < (1ull << 31) &&
                         ((uintptr_t)x->data & 15) == 0 && out && ((uintptr_t)out->data & 3) == 0 &&  // (two outputs a store)
                         mxfp4_gemm_form(ctx, n_pairs, h->n_experts, h->k, h->n) != 0;
    if (!resident || (!prefill && n_pairs >= 8 * h->n_experts))
        return moe_matmul_impl(op, ctx, stream, x, &h->blocks, &h->scales, h->has_bias ? &h->bias : nullptr, expert_offsets,
                               token_ids, gather_rows, h->k, h->n, swiglu, limit, out, fused);
    Mxfp4Problem p;
    OXQ_TRY(check_mxfp4(ctx, op, false, x, &h->blocks, &h->scales, h->k, h->n, h->n_experts, out, &p));
    if (swiglu && (h->n & 1)) return fail(OXQ_ERR_SHAPE, "%s: interleaved gate / up rows need an even n", op);
    const int64_t out_cols = swiglu ? h->n / 2 : h->n;
    if (out->rank != 2 || out->dims[1] != out_cols || !out->contiguous)
        return fail(OXQ_ERR_SHAPE, "%s: out must be a contiguous [n_pairs, %lld]", op, (long long)out_cols);
    if (gather_rows) {
        OXQ_TRY(check_tensor(ctx, op, "token_ids", token_ids));
        if (token_ids->dtype != OXQ_I32 || numel(token_ids) != n_pairs || !token_ids->contiguous)
            return fail(OXQ_ERR_SHAPE, "%s: token_ids must be a contiguous I32 [%lld]", op, (long long)n_pairs);
    } else if (x->dims[0] != n_pairs) {
        return fail(OXQ_ERR_SHAPE, "%s: x has %lld rows, out has %lld", op, (long long)x->dims[0], (long long)n_pairs);
    }
    p.blocks = (const uint8_t *)h->pw;
    p.scales = (const uint8_t *)h->ps;
    p.bias = h->has_bias ? h->bias.data : nullptr;
    p.n_experts = h->n_experts;
    p.expert_offsets = (const int32_t *)expert_offsets->data;
    p.token_ids = gather_rows ? (const int32_t *)token_ids->data : nullptr;
    p.n_pairs = n_pairs;
    p.swiglu = swiglu ? 1 : 0;
    p.swiglu_limit = limit;
    p.M = x->dims[0];
    // many pairs an expert (prefill): 64-row tiles on the same copy
    const int rc = prefill ? launch_mxfp4_res_gemm(ctx, (hipStream_t)stream, p) : launch_mxfp4_res_gemv(ctx, (hipStream_t)stream, p);
    if (rc == OXQ_OK && fused) *fused = 1;
    return rc;
}

int oxq_mxfp4_experts_matmul(oxq_mxfp4_experts *h, void *stream, const oxq_tensor *x, const oxq_tensor *expert_offsets,
                             const oxq_tensor *token_ids, int gather_rows, const oxq_tensor *out) {
    return experts_forward(h, stream, x, expert_offsets, token_ids, gather_rows, false, 0.0f, out, nullptr);
}

int oxq_mxfp4_experts_gate_up_swiglu(oxq_mxfp4_experts *h, void *stream, const oxq_tensor *x,
                                     const oxq_tensor *expert_offsets, const oxq_tensor *token_ids, int gather_rows,
                                     float limit, const oxq_tensor *out, int *fused) {
    if (!fused) return fail(OXQ_ERR_ARG, "Mxfp4ExpertsGateUpSwiglu: fused is NULL");
    return experts_forward(h, stream, x, expert_offsets, token_ids, gather_rows, true, limit, out, fused);
}

int oxq_mxfp4_experts_is_resident(const oxq_mxfp4_experts *h, int *resident) {
    if (!h || !resident) return fail(OXQ_ERR_ARG, "Mxfp4Experts: NULL argument");
    *resident = h->pw != nullptr;
    return OXQ_OK;
}

int oxq_mxfp4_experts_dequantize(oxq_mxfp4_experts *h, void *stream, int64_t expert, const oxq_tensor *out) {
    const char *op = "Mxfp4ExpertsDequantize";
    if (!h || !out) return fail(OXQ_ERR_ARG, "%s: NULL argument", op);
    if (expert < 0 || expert >= h->n_experts)
        return fail(OXQ_ERR_ARG, "%s: expert %lld outside 0..%lld", op, (long long)expert, (long long)h->n_experts - 1);
    OXQ_TRY(check_tensor(h->ctx, op, "out", out));
    if (out->dtype != OXQ_F32 || out->rank != 2 || out->dims[0] != h->n || out->dims[1] != h->k || !out->contiguous)
        return fail(OXQ_ERR_SHAPE, "%s: out must be a contiguous F32 [%lld, %lld]", op, (long long)h->n, (long long)h->k);
    if (h->pw)
        return launch_mxfp4_res_dequant(h->ctx, (hipStream_t)stream, h->pw, h->ps, expert, h->k, h->n, (float *)out->data);
    Mxfp4Problem p;
    memset(&p, 0, sizeof p);
    const int64_t nb = h->k / 32;
    p.blocks = (const uint8_t *)h->blocks.data + (size_t)expert * h->n * nb * 16;
    p.scales = (const uint8_t *)h->scales.data + (size_t)expert * h->n * nb;
    p.K = h->k;
    p.N = h->n;
    return launch_mxfp4_dequant(h->ctx, (hipStream_t)stream, p, (float *)out->data);
}

void oxq_mxfp4_experts_free(oxq_mxfp4_experts *h) {
    if (!h) return;
    if (h->owns) {  // by the handle's own flag: the experts may outlive their ctx
        if (h->pw) (void)hipFree(h->pw);
        if (h->ps) (void)hipFree(h->ps);
    }
    delete h;
}

// ---- mixture-of-experts glue (moe.rs:466-607, ffn_kernels.metal, moe.rs:152-173) --------


static int check_moe_route(oxq_ctx *ctx, const oxq_tensor *logits, int64_t top_k, const oxq_tensor *top_idx,
                           const oxq_tensor *top_vals) {
    const char *op = "MoeRoute";
    if (!ctx) return fail(OXQ_ERR_ARG, "%s: ctx is NULL", op);
    OXQ_TRY(check_tensor(ctx, op, "logits", logits));
    OXQ_TRY(check_tensor(ctx, op, "top_idx", top_idx));
    OXQ_TRY(check_tensor(ctx, op, "top_vals", top_vals));
    if (logits->rank != 2 || !logits->contiguous)
        return fail(OXQ_ERR_SHAPE, "%s: logits must be a contiguous [n_tokens, n_experts]", op);
    if (!is_float_dtype(logits->dtype))
        return fail(OXQ_ERR_DTYPE, "%s: logits must be F32, F16 or BF16, got %s", op, dtype_name(logits->dtype));
    const int64_t T = logits->dims[0], E = logits->dims[1];
    if (top_k < 1 || top_k > E || top_k > 64)
        return fail(OXQ_ERR_ARG, "%s: top_k %lld must be in 1..=min(n_experts %lld, 64)", op, (long long)top_k,
                    (long long)E);
    if (E > 4096) return fail(OXQ_ERR_UNSUPPORTED, "%s: at most 4096 experts", op);
    if (top_idx->dtype != OXQ_I32 || top_idx->rank != 2 || top_idx->dims[0] != T || top_idx->dims[1] != top_k ||
        !top_idx->contiguous)
        return fail(OXQ_ERR_SHAPE, "%s: top_idx must be a contiguous I32 [%lld, %lld]", op, (long long)T,
                    (long long)top_k);
    if (top_vals->dtype != OXQ_F32 || top_vals->rank != 2 || top_vals->dims[0] != T || top_vals->dims[1] != top_k ||
        !top_vals->contiguous)
        return fail(OXQ_ERR_SHAPE, "%s: top_vals must be a contiguous F32 [%lld, %lld]", op, (long long)T,
                    (long long)top_k);
    return OXQ_OK;
}

int oxq_moe_route(oxq_ctx *ctx, void *stream, const oxq_tensor *logits, int64_t top_k, int norm_topk,
                  const oxq_tensor *top_idx, const oxq_tensor *top_vals) {
    OXQ_TRY(check_moe_route(ctx, logits, top_k, top_idx, top_vals));
    return launch_moe_route(ctx, (hipStream_t)stream, logits->data, logits->dtype, logits->dims[0], logits->dims[1],
                            top_k, norm_topk ? 1 : 0, (int32_t *)top_idx->data, (float *)top_vals->data);
}

static int check_moe_group(oxq_ctx *ctx, const oxq_tensor *top_idx, const oxq_tensor *top_vals, int64_t n_experts,
                           const oxq_tensor *expert_offsets, const oxq_tensor *token_ids,
                           const oxq_tensor *pair_weights, const oxq_tensor *pair_pos) {
    const char *op = "MoeGroup";
    if (!ctx) return fail(OXQ_ERR_ARG, "%s: ctx is NULL", op);
    OXQ_TRY(check_tensor(ctx, op, "top_idx", top_idx));
    OXQ_TRY(check_tensor(ctx, op, "top_vals", top_vals));
    OXQ_TRY(check_tensor(ctx, op, "expert_offsets", expert_offsets));
    OXQ_TRY(check_tensor(ctx, op, "token_ids", token_ids));
    OXQ_TRY(check_tensor(ctx, op, "pair_weights", pair_weights));
    OXQ_TRY(check_tensor(ctx, op, "pair_pos", pair_pos));
    if (top_idx->dtype != OXQ_I32 || top_idx->rank != 2 || !top_idx->contiguous)
        return fail(OXQ_ERR_SHAPE, "%s: top_idx must be a contiguous I32 [n_tokens, top_k]", op);
    const int64_t T = top_idx->dims[0], top_k = top_idx->dims[1], P = T * top_k;
    if (top_vals->dtype != OXQ_F32 || numel(top_vals) != P || !top_vals->contiguous)
        return fail(OXQ_ERR_SHAPE, "%s: top_vals must be a contiguous F32 [%lld, %lld]", op, (long long)T,
                    (long long)top_k);
    if (n_experts < 1 || n_experts > 256)
        return fail(OXQ_ERR_ARG, "%s: n_experts %lld must be in 1..=256", op, (long long)n_experts);
    if (top_k < 1) return fail(OXQ_ERR_SHAPE, "%s: top_k must be positive", op);
    if (expert_offsets->dtype != OXQ_I32 || numel(expert_offsets) != n_experts + 1 || !expert_offsets->contiguous)
        return fail(OXQ_ERR_SHAPE, "%s: expert_offsets must be a contiguous I32 [%lld]", op,
                    (long long)(n_experts + 1));
    if (token_ids->dtype != OXQ_I32 || numel(token_ids) != P || !token_ids->contiguous)
        return fail(OXQ_ERR_SHAPE, "%s: token_ids must be a contiguous I32 [%lld]", op, (long long)P);
    if (pair_weights->dtype != OXQ_F32 || numel(pair_weights) != P || !pair_weights->contiguous)
        return fail(OXQ_ERR_SHAPE, "%s: pair_weights must be a contiguous F32 [%lld]", op, (long long)P);
    if (pair_pos->dtype != OXQ_I32 || numel(pair_pos) != P || !pair_pos->contiguous)
        return fail(OXQ_ERR_SHAPE, "%s: pair_pos must be a contiguous I32 [%lld, %lld]", op, (long long)T,
                    (long long)top_k);
    if (P > INT32_MAX) return fail(OXQ_ERR_SHAPE, "%s: too many pairs", op);
    return OXQ_OK;
}

int oxq_moe_group(oxq_ctx *ctx, void *stream, const oxq_tensor *top_idx, const oxq_tensor *top_vals,
                  int64_t n_experts, const oxq_tensor *expert_offsets, const oxq_tensor *token_ids,
                  const oxq_tensor *pair_weights, const oxq_tensor *pair_pos) {
    OXQ_TRY(check_moe_group(ctx, top_idx, top_vals, n_experts, expert_offsets, token_ids, pair_weights, pair_pos));
    return launch_moe_group(ctx, (hipStream_t)stream, (const int32_t *)top_idx->data, (const float *)top_vals->data,
                            numel(top_idx), n_experts, top_idx->dims[1], (int32_t *)expert_offsets->data,
                            (int32_t *)token_ids->data, (float *)pair_weights->data, (int32_t *)pair_pos->data);
}

// moe.rs:466-486 followed by 563-590, as one call
int oxq_moe_route_group(oxq_ctx *ctx, void *stream, const oxq_tensor *logits, int64_t top_k, int norm_topk,
                        const oxq_tensor *top_idx, const oxq_tensor *top_vals, const oxq_tensor *expert_offsets,
                        const oxq_tensor *token_ids, const oxq_tensor *pair_weights, const oxq_tensor *pair_pos) {
    OXQ_TRY(check_moe_route(ctx, logits, top_k, top_idx, top_vals));
    const int64_t T = logits->dims[0], E = logits->dims[1];
    OXQ_TRY(check_moe_group(ctx, top_idx, top_vals, E, expert_offsets, token_ids, pair_weights, pair_pos));
    if (T >= 1 && T * top_k <= 64)  // decode sizes: one launch
        return launch_moe_route_group(ctx, (hipStream_t)stream, logits->data, logits->dtype, T, E, top_k,
                                      norm_topk ? 1 : 0, (int32_t *)top_idx->data, (float *)top_vals->data,
                                      (int32_t *)expert_offsets->data, (int32_t *)token_ids->data,
                                      (float *)pair_weights->data, (int32_t *)pair_pos->data);
    OXQ_TRY(launch_moe_route(ctx, (hipStream_t)stream, logits->data, logits->dtype, T, E, top_k, norm_topk ? 1 : 0,
                             (int32_t *)top_idx->data, (float *)top_vals->data));
    return launch_moe_group(ctx, (hipStream_t)stream, (const int32_t *)top_idx->data, (const float *)top_vals->data,
                            T * top_k, E, top_k, (int32_t *)expert_offsets->data, (int32_t *)token_ids->data,
                            (float *)pair_weights->data, (int32_t *)pair_pos->data);
}

int oxq_gated_activation(oxq_ctx *ctx, void *stream, const oxq_tensor *gate_up, int kind, float limit,
                         const oxq_tensor *out) {
    const char *op = "GatedActivation";
    if (!ctx) return fail(OXQ_ERR_ARG, "%s: ctx is NULL", op);
    OXQ_TRY(check_tensor(ctx, op, "gate_up", gate_up));
    OXQ_TRY(check_tensor(ctx, op, "out", out));
    if (kind != OXQ_ACT_GATED_SILU && kind != OXQ_ACT_GATED_GELU_TANH && kind != OXQ_ACT_GPT_OSS_SWIGLU)
        return fail(OXQ_ERR_ARG, "%s: unknown activation kind %d", op, kind);
    if (!gate_up->contiguous || !out->contiguous)
        return fail(OXQ_ERR_CONTIGUOUS, "%s: gate_up and out must be contiguous", op);
    if (!is_float_dtype(gate_up->dtype) || out->dtype != gate_up->dtype)
        return fail(OXQ_ERR_DTYPE, "%s: gate_up and out must share a dtype of F32, F16 or BF16", op);
    const int64_t last = gate_up->dims[gate_up->rank - 1];
    if (last % 2 != 0)  // metal_ops.rs:1237-1245: last dim must be 2 * intermediate_size
        return fail(OXQ_ERR_SHAPE, "%s: last dim %lld is not 2 * intermediate_size", op, (long long)last);
    const int64_t half_n = last / 2;
    const int64_t rows = half_n > 0 ? numel(gate_up) / last : 0;
    if (out->rank != gate_up->rank || out->dims[out->rank - 1] != half_n || numel(out) != rows * half_n)
        return fail(OXQ_ERR_SHAPE, "%s: out must be [.., %lld]", op, (long long)half_n);
    if (half_n > INT32_MAX) return fail(OXQ_ERR_SHAPE, "%s: dimension exceeds 2^31-1", op);
    return launch_gated_activation(ctx, (hipStream_t)stream, gate_up->data, out->data, gate_up->dtype, rows, half_n,
                                   kind, limit);
}

int oxq_activation_mul(oxq_ctx *ctx, void *stream, const oxq_tensor *gate, const oxq_tensor *up, int kind,
                       const oxq_tensor *out) {
    const char *op = kind == OXQ_ACT_GATED_GELU_TANH ? "GeluTanhMulOp" : "SiluMulOp";
    if (!ctx) return fail(OXQ_ERR_ARG, "%s: ctx is NULL", op);
    OXQ_TRY(check_tensor(ctx, op, "gate", gate));
    OXQ_TRY(check_tensor(ctx, op, "up", up));
    OXQ_TRY(check_tensor(ctx, op, "out", out));
    if (kind != OXQ_ACT_GATED_SILU && kind != OXQ_ACT_GATED_GELU_TANH)
        return fail(OXQ_ERR_ARG, "%s: activation kind %d has no two-tensor form", op, kind);
    if (!gate->contiguous || !up->contiguous)  // metal_ops.rs:649-651
        return fail(OXQ_ERR_CONTIGUOUS, "%s: both inputs must be contiguous", op);
    if (!out->contiguous) return fail(OXQ_ERR_CONTIGUOUS, "%s: out must be contiguous", op);
    if (gate->dtype != up->dtype)  // metal_ops.rs:652-658
        return fail(OXQ_ERR_DTYPE, "%s: dtype mismatch %s vs %s", op, dtype_name(gate->dtype), dtype_name(up->dtype));
    if (!is_float_dtype(gate->dtype))
        return fail(OXQ_ERR_DTYPE, "%s: unsupported dtype %s", op, dtype_name(gate->dtype));
    if (out->dtype != gate->dtype) return fail(OXQ_ERR_DTYPE, "%s: out must have the inputs' dtype", op);
    const int64_t n = numel(gate);
    if (numel(up) != n) return fail(OXQ_ERR_SHAPE, "%s: shape mismatch", op);  // metal_ops.rs:659-662
    if (numel(out) != n) return fail(OXQ_ERR_SHAPE, "%s: out must have the inputs' shape", op);
    return launch_activation_mul(ctx, (hipStream_t)stream, gate->data, up->data, out->data, gate->dtype, n, kind);
}

int oxq_moe_combine(oxq_ctx *ctx, void *stream, const oxq_tensor *expert_out, const oxq_tensor *pair_pos,
                    const oxq_tensor *top_vals, const oxq_tensor *out) {
    const char *op = "MoeCombine";
    if (!ctx) return fail(OXQ_ERR_ARG, "%s: ctx is NULL", op);
    OXQ_TRY(check_tensor(ctx, op, "expert_out", expert_out));
    OXQ_TRY(check_tensor(ctx, op, "pair_pos", pair_pos));
    OXQ_TRY(check_tensor(ctx, op, "top_vals", top_vals));
    OXQ_TRY(check_tensor(ctx, op, "out", out));
    if (pair_pos->dtype != OXQ_I32 || pair_pos->rank != 2 || !pair_pos->contiguous)
        return fail(OXQ_ERR_SHAPE, "%s: pair_pos must be a contiguous I32 [n_tokens, top_k]", op);
    const int64_t T = pair_pos->dims[0], top_k = pair_pos->dims[1], P = T * top_k;
    if (top_vals->dtype != OXQ_F32 || numel(top_vals) != P || !top_vals->contiguous)
        return fail(OXQ_ERR_SHAPE, "%s: top_vals must be a contiguous F32 [%lld, %lld]", op, (long long)T,
                    (long long)top_k);
    if (expert_out->rank != 2 || expert_out->dims[0] != P || !expert_out->contiguous)
        return fail(OXQ_ERR_SHAPE, "%s: expert_out must be a contiguous [%lld, hidden]", op, (long long)P);
    const int64_t H = expert_out->dims[1];
    if (!is_float_dtype(expert_out->dtype) || out->dtype != expert_out->dtype)
        return fail(OXQ_ERR_DTYPE, "%s: expert_out and out must share a dtype of F32, F16 or BF16", op);
    if (out->rank != 2 || out->dims[0] != T || out->dims[1] != H || !out->contiguous)
        return fail(OXQ_ERR_SHAPE, "%s: out must be a contiguous [%lld, %lld]", op, (long long)T, (long long)H);
    if (H > INT32_MAX || T > INT32_MAX) return fail(OXQ_ERR_SHAPE, "%s: dimension exceeds 2^31-1", op);
    return launch_moe_combine(ctx, (hipStream_t)stream, expert_out->data, (const int32_t *)pair_pos->data,
                              (const float *)top_vals->data, out->data, out->dtype, T, H, top_k);
}

}  // extern "C"

// =============================================================================
// Layers: host mirrors of linear.rs / mxfp4.rs
// =============================================================================
namespace oxq {

static int flatten_rows(const char *op, const oxq_tensor *x, int64_t in_features, oxq_tensor *x2,
                        int64_t *m_out) {
    if (!x) return fail(OXQ_ERR_ARG, "%s: x is NULL", op);
    if (x->rank < 1 || x->rank > OXQ_MAX_RANK) return fail(OXQ_ERR_SHAPE, "%s: bad x rank", op);
    const int64_t last = x->dims[x->rank - 1];
    if (last != in_features)
        return fail(OXQ_ERR_SHAPE, "%s: input last dim %lld != in_features %lld", op, (long long)last,
                    (long long)in_features);
    if (!x->contiguous)
        return fail(OXQ_ERR_CONTIGUOUS, "%s: x must be contiguous (the caller owns the copy the "
                                        "reference makes with .contiguous())", op);
    int64_t m = 1;
    for (int i = 0; i < x->rank - 1; ++i) m *= x->dims[i];
    *x2 = *x;
    x2->rank = 2;
    x2->dims[0] = m;
    x2->dims[1] = in_features;
    *m_out = m;
    return OXQ_OK;
}

static int flatten_out(const char *op, const oxq_tensor *out, int64_t m, int64_t n, oxq_tensor *o2) {
    if (!out) return fail(OXQ_ERR_ARG, "%s: out is NULL", op);
    if (out->rank < 1 || out->rank > OXQ_MAX_RANK || out->dims[out->rank - 1] != n || numel(out) != m * n ||
        !out->contiguous)
        return fail(OXQ_ERR_SHAPE, "%s: out must be contiguous with %lld rows of %lld", op,
                    (long long)m, (long long)n);
    *o2 = *out;
    o2->rank = 2;
    o2->dims[0] = m;
    o2->dims[1] = n;
    return OXQ_OK;
}

}  // namespace oxq

struct oxq_packed_quant_linear {
    oxq_ctx *ctx;
    oxq_tensor qweight, qzeros, scales, bias;
    bool has_bias;
    int64_t in_features, out_features;
    uint32_t bits;
    int pack_dim;
    int dtype;
    // linear.rs:450-455 gemv_max_m: the reference keeps batches up to 16 (AWQ) /
    // 32 (GPTQ) on the GEMV kernel in chunks of 8 because its only alternative
    // below m = 64 is a full dense dequant.  Here every m > 8 runs the MFMA tile
    // kernel, which reads the packed weights once.
    int64_t gemv_max_m() const { return 8; }
    // 4- and 8-bit layers with tile-aligned shapes keep a tile-major copy of the
    // weights made at load (pk4.hip); forward then runs one kernel for every m
    // and no longer touches the caller's checkpoint tensors.
    bool prepacked;
    Pk4Weights pk;
    // 0, or 1 + oxq_gated_act for a fused gate|up layer whose forward applies the gated
    // activation in the matmul's epilogue: out = act(gate) * up, [.., out_features / 2]
    int act;
};

// Load-time repack of an eligible layer.  Shapes the repacked kernels do
// not cover simply keep the checkpoint layout; errors in the tensors themselves
// surface at forward, where the reference reports them.
static int prepack_layer(oxq_packed_quant_linear *l) {
    oxq_ctx *ctx = l->ctx;
    if (tune(ctx, OXQ_TUNE_PREPACK, 1) == 0) return OXQ_OK;
    oxq_tensor shape_only = l->scales;  // [K, N] descriptor for the shape checks, never written
    shape_only.rank = 2;
    shape_only.dims[0] = l->in_features;
    shape_only.dims[1] = l->out_features;
    shape_only.contiguous = 1;
    Wna16Problem src;
    if (check_wna16(ctx, "PackedQuantLinear", KIND_DEQUANT, nullptr, &l->qweight, &l->qzeros, &l->scales,
                    l->bits, l->pack_dim, &shape_only, &src) != OXQ_OK)
        return OXQ_OK;
    if (!pk4_eligible(src)) return OXQ_OK;
    l->pk.K = src.K;
    l->pk.N = src.N;
    l->pk.group_shift = src.group_shift;
    l->pk.dtype = l->dtype;
    l->pk.bits = src.bits;
    l->pk.gate_half = l->act ? src.N / 2 : 0;
    l->pk.gemv_rows = src.pack_dim == OXQ_PACK_IN ? 32 : 16;
    l->pk.strip = pk4_choose_strip(l->ctx, src.K, src.N, src.bits, l->pk.gate_half);
    if (ctx->plan_only) {
        l->prepacked = true;
        return OXQ_OK;
    }
    int prev = 0;
    (void)hipGetDevice(&prev);
    OXQ_HIP_CHECK(hipSetDevice(ctx->device));
    int rc = OXQ_OK;
    hipError_t e = hipMalloc((void **)&l->pk.pw, pk4_weight_bytes(src.K, src.N, src.bits));
    l->pk.pzs = nullptr;  // the zero/scale pairs live inside the blocks of pw
    if (e != hipSuccess) {
        rc = fail(OXQ_ERR_RUNTIME, "PackedQuantLinear: repack allocation failed: %s", hipGetErrorString(e));
    } else {
        rc = launch_pk4_prepack(ctx, nullptr, src, l->pk);
        if (rc == OXQ_OK && (e = hipStreamSynchronize(nullptr)) != hipSuccess)
            rc = fail(OXQ_ERR_RUNTIME, "PackedQuantLinear: repack failed: %s", hipGetErrorString(e));
    }
    (void)hipSetDevice(prev);
    if (rc == OXQ_OK) l->prepacked = true;
    return rc;
}

struct oxq_qlinear {
    oxq_ctx *ctx;
    oxq_tensor weight_bytes, bias;
    bool has_bias;
    int64_t in_features, out_features;
    int quant;
    int out_dtype;
    void *res = nullptr;    // layer-owned strip-major copy of the blocks
    bool resident = false;
    bool mfma = false;      // the copy is the matrix-core layout (bf16 layers), else the rotated one of the vector GEMV
    int act = 0;            // 0, or 1 + oxq_gated_act of a fused gate|up layer (matrix-core copy only)
};

// linear.rs:225-240: the fast path copies the block bytes at build; here the copy is strip-major
static int build_resident_gguf(oxq_qlinear *l) {
    if (tune(l->ctx, OXQ_TUNE_PREPACK, 1) == 0) return OXQ_OK;
    if (!gguf_res_eligible(l->quant, l->in_features, l->out_features)) return OXQ_OK;
    if (((uintptr_t)l->weight_bytes.data & 1) != 0) return OXQ_OK;
    oxq_ctx *ctx = l->ctx;
    // a bf16 layer (the reference's GPU path: bf16 x and y) of a format that has it takes the matrix-core layout
    l->mfma = l->out_dtype == OXQ_BF16 && gguf_mfma_eligible(ctx, l->quant, l->in_features, l->out_features);
    if (l->act && !l->mfma) return OXQ_OK;  // the caller reports it
    if (ctx->plan_only) {
        l->resident = true;
        return OXQ_OK;
    }
    int prev = 0;
    (void)hipGetDevice(&prev);
    OXQ_HIP_CHECK(hipSetDevice(ctx->device));
    int rc = OXQ_OK;
    hipError_t e = hipMalloc(&l->res, gguf_res_bytes(l->quant, l->in_features, l->out_features));
    if (e != hipSuccess) {
        l->res = nullptr;
        rc = fail(OXQ_ERR_RUNTIME, "QLinear: repack allocation failed: %s", hipGetErrorString(e));
    } else {
        const uint8_t *src = (const uint8_t *)l->weight_bytes.data;
        rc = l->mfma ? launch_gguf_mfma_repack(ctx, nullptr, l->quant, src, l->res, l->in_features, l->out_features,
                                               l->act ? l->out_features / 2 : 0)
                     : launch_gguf_res_repack(ctx, nullptr, l->quant, src, l->res, l->in_features, l->out_features);
        if (rc == OXQ_OK && (e = hipStreamSynchronize(nullptr)) != hipSuccess)
            rc = fail(OXQ_ERR_RUNTIME, "QLinear: repack failed: %s", hipGetErrorString(e));
    }
    (void)hipSetDevice(prev);
    if (rc == OXQ_OK) l->resident = true;
    return rc;
}

struct oxq_mxfp4_linear {
    oxq_ctx *ctx;
    oxq_tensor blocks, scales, bias;
    bool has_bias;
    int64_t in_features, out_features;
};

extern "C" {

static int new_packed_layer(const char *op, oxq_ctx *ctx, uint32_t bits, int pack_dim, const oxq_tensor *qweight,
                            const oxq_tensor *qzeros, const oxq_tensor *scales, const oxq_tensor *bias, int dtype,
                            int act, oxq_packed_quant_linear **out) {
    if (!ctx || !out) return fail(OXQ_ERR_ARG, "%s: NULL argument", op);
    *out = nullptr;
    if (bits != 4 && bits != 8)  // linear.rs:417-419
        return fail(OXQ_ERR_BITS, "%s: bits must be 4 or 8, got %u", op, bits);
    if (!qzeros) return fail(OXQ_ERR_ARG, "%s: qzeros missing", op);  // linear.rs:420-422
    if (pack_dim != OXQ_PACK_OUT && pack_dim != OXQ_PACK_IN)
        return fail(OXQ_ERR_ARG, "%s: bad pack_dim %d", op, pack_dim);
    OXQ_TRY(check_tensor(ctx, op, "qweight", qweight));
    OXQ_TRY(check_tensor(ctx, op, "qzeros", qzeros));
    OXQ_TRY(check_tensor(ctx, op, "scales", scales));
    if (qweight->rank != 2 || scales->rank != 2)
        return fail(OXQ_ERR_SHAPE, "%s: qweight and scales must be 2-D", op);
    const int64_t pf = 32 / bits;
    int64_t in_f, out_f;  // linear.rs:423-430
    if (pack_dim == OXQ_PACK_OUT) {
        in_f = qweight->dims[0];
        out_f = qweight->dims[1] * pf;
    } else {
        in_f = qweight->dims[0] * pf;
        out_f = qweight->dims[1];
    }
    if (scales->dims[1] != out_f)  // linear.rs:431-436
        return fail(OXQ_ERR_SHAPE, "%s: scales out_features %lld != derived %lld", op,
                    (long long)scales->dims[1], (long long)out_f);
    if (dtype != OXQ_F16 && dtype != OXQ_BF16)
        return fail(OXQ_ERR_DTYPE, "%s: runtime dtype must be F16 or BF16", op);
    if (scales->dtype != dtype)
        return fail(OXQ_ERR_DTYPE, "%s: scales must already be cast to %s (linear.rs:437), got %s",
                    op, dtype_name(dtype), dtype_name(scales->dtype));
    OXQ_TRY(check_bias(ctx, op, bias, out_f, dtype));
    oxq_packed_quant_linear *l = new (std::nothrow) oxq_packed_quant_linear();
    if (!l) return fail(OXQ_ERR_RUNTIME, "%s: out of host memory", op);
    l->ctx = ctx;
    l->qweight = *qweight;
    l->qzeros = *qzeros;
    l->scales = *scales;
    l->has_bias = bias != nullptr;
    if (bias) l->bias = *bias;
    l->in_features = in_f;
    l->out_features = out_f;
    l->bits = bits;
    l->pack_dim = pack_dim;
    l->dtype = dtype;
    l->prepacked = false;
    l->act = act;
    l->pk = Pk4Weights{nullptr, nullptr, 0, 0, 0, dtype, (int)bits, 0};
    int rc = prepack_layer(l);
    if (rc == OXQ_OK && act && !l->prepacked)
        rc = fail(OXQ_ERR_UNSUPPORTED,
                  "%s: the fused activation needs a resident layer (in_features and group size multiples of 128, "
                  "out_features a multiple of 64, at most 128 groups, OXQ_PREPACK not 0); build a plain layer and "
                  "call oxq_gated_activation on its output instead",
                  op);
    if (rc != OXQ_OK) {
        oxq_packed_quant_linear_free(l);
        return rc;
    }
    *out = l;
    return OXQ_OK;
}

int oxq_packed_quant_linear_new(oxq_ctx *ctx, uint32_t bits, int pack_dim,
                                const oxq_tensor *qweight, const oxq_tensor *qzeros,
                                const oxq_tensor *scales, const oxq_tensor *bias, int dtype,
                                oxq_packed_quant_linear **out) {
    return new_packed_layer("PackedQuantLinear", ctx, bits, pack_dim, qweight, qzeros, scales, bias, dtype, 0, out);
}

int oxq_packed_quant_linear_new_gate_up(oxq_ctx *ctx, uint32_t bits, int pack_dim, const oxq_tensor *qweight,
                                        const oxq_tensor *qzeros, const oxq_tensor *scales, const oxq_tensor *bias,
                                        int act, int dtype, oxq_packed_quant_linear **out) {
    const char *op = "PackedQuantLinear(gate|up)";
    if (act != OXQ_ACT_GATED_SILU && act != OXQ_ACT_GATED_GELU_TANH)
        return fail(OXQ_ERR_ARG, "%s: activation must be OXQ_ACT_GATED_SILU or OXQ_ACT_GATED_GELU_TANH, got %d", op, act);
    return new_packed_layer(op, ctx, bits, pack_dim, qweight, qzeros, scales, bias, dtype, act + 1, out);
}

// linear.rs:482-533 PackedQuantLinear::forward
int oxq_packed_quant_linear_forward(oxq_packed_quant_linear *l, void *stream, const oxq_tensor *x,
                                    const oxq_tensor *out) {
    const char *op = "PackedQuantLinear";
    if (!l) return fail(OXQ_ERR_ARG, "%s: layer is NULL", op);
    oxq_tensor x2, o2;
    int64_t m;
    OXQ_TRY(flatten_rows(op, x, l->in_features, &x2, &m));
    OXQ_TRY(flatten_out(op, out, m, l->act ? l->out_features / 2 : l->out_features, &o2));
    if (l->prepacked) {
        OXQ_TRY(check_tensor(l->ctx, op, "x", &x2));
        OXQ_TRY(check_tensor(l->ctx, op, "out", &o2));
        if (x2.dtype != l->dtype)
            return fail(OXQ_ERR_DTYPE, "%s: scales dtype %s must match x dtype %s", op,
                        dtype_name(l->dtype), dtype_name(x2.dtype));
        if (o2.dtype != l->dtype)
            return fail(OXQ_ERR_DTYPE, "%s: out dtype %s must be %s", op, dtype_name(o2.dtype),
                        dtype_name(l->dtype));
        if (m < 1) return fail(OXQ_ERR_SHAPE, "%s: x has no rows", op);
        Pk4Problem q;
        q.x = x2.data;
        q.bias = l->has_bias ? l->bias.data : nullptr;
        q.y = o2.data;
        q.M = m;
        q.act = l->act;
        q.no_split = 0;
        q.w = l->pk;
        return launch_pk4_forward(l->ctx, (hipStream_t)stream, q);
    }
    Wna16Problem p;
    const bool gemv = m <= l->gemv_max_m();
    OXQ_TRY(check_wna16(l->ctx, op, gemv ? KIND_GEMV : KIND_TILE, &x2, &l->qweight, &l->qzeros,
                        &l->scales, l->bits, l->pack_dim, &o2, &p));
    p.bias = l->has_bias ? l->bias.data : nullptr;
    return gemv ? launch_wna16_gemv(l->ctx, (hipStream_t)stream, p)
                : launch_wna16_mfma(l->ctx, (hipStream_t)stream, p);
}

int oxq_packed_quant_linear_in_features(const oxq_packed_quant_linear *l, int64_t *k) {
    if (!l || !k) return fail(OXQ_ERR_ARG, "PackedQuantLinear: NULL argument");
    *k = l->in_features;
    return OXQ_OK;
}
int oxq_packed_quant_linear_out_features(const oxq_packed_quant_linear *l, int64_t *n) {
    if (!l || !n) return fail(OXQ_ERR_ARG, "PackedQuantLinear: NULL argument");
    *n = l->act ? l->out_features / 2 : l->out_features;
    return OXQ_OK;
}
int oxq_packed_quant_linear_is_prepacked(const oxq_packed_quant_linear *l, int *prepacked) {
    if (!l || !prepacked) return fail(OXQ_ERR_ARG, "PackedQuantLinear: NULL argument");
    *prepacked = l->prepacked ? 1 : 0;
    return OXQ_OK;
}

// linear.rs:510-523: the layer's dense dequant (fallback of forward), [K, N]
int oxq_packed_quant_linear_dequantize(oxq_packed_quant_linear *l, void *stream, const oxq_tensor *out) {
    const char *op = "PackedQuantLinear::dequantize";
    if (!l) return fail(OXQ_ERR_ARG, "%s: layer is NULL", op);
    if (l->prepacked) {
        OXQ_TRY(check_tensor(l->ctx, op, "out", out));
        if (out->rank != 2 || out->dims[0] != l->in_features || out->dims[1] != l->out_features ||
            !out->contiguous)
            return fail(OXQ_ERR_SHAPE, "%s: output must be a contiguous [%lld, %lld] tensor", op,
                        (long long)l->in_features, (long long)l->out_features);
        if (out->dtype != l->dtype)
            return fail(OXQ_ERR_DTYPE, "%s: out dtype %s must be %s", op, dtype_name(out->dtype),
                        dtype_name(l->dtype));
        return launch_pk4_dequant(l->ctx, (hipStream_t)stream, l->pk, out->data);
    }
    Wna16Problem p;
    OXQ_TRY(check_wna16(l->ctx, op, KIND_DEQUANT, nullptr, &l->qweight, &l->qzeros, &l->scales, l->bits,
                        l->pack_dim, out, &p));
    return launch_wna16_dequant(l->ctx, (hipStream_t)stream, p, out->data);
}

void oxq_packed_quant_linear_free(oxq_packed_quant_linear *l) {
    if (!l) return;
    if (l->pk.pw) (void)hipFree(l->pk.pw);
    if (l->pk.pzs) (void)hipFree(l->pk.pzs);
    delete l;
}

// linear.rs:197-247 GgufFastPath::build
static int new_qlinear(const char *op, oxq_ctx *ctx, int quant, const oxq_tensor *weight_bytes, int64_t in_features,
                       int64_t out_features, const oxq_tensor *bias, int act, int out_dtype, oxq_qlinear **out) {
    if (!ctx || !out) return fail(OXQ_ERR_ARG, "%s: NULL argument", op);
    *out = nullptr;
    int64_t be, bb;
    OXQ_TRY(oxq_gguf_block_layout(quant, &be, &bb));
    OXQ_TRY(check_tensor(ctx, op, "weight_bytes", weight_bytes));
    if (weight_bytes->dtype != OXQ_U8) return fail(OXQ_ERR_DTYPE, "%s: weight_bytes must be U8", op);
    if (in_features <= 0 || out_features <= 0 || in_features % be != 0)
        return fail(OXQ_ERR_SHAPE, "%s: in_features %lld must be a multiple of %lld", op,
                    (long long)in_features, (long long)be);
    const int64_t expected = out_features * (in_features / be) * bb;  // linear.rs:227-237
    if (numel(weight_bytes) != expected)
        return fail(OXQ_ERR_SHAPE,
                    "GGUF fast path: weight has %lld bytes, expected %lld for shape [%lld, %lld]",
                    (long long)numel(weight_bytes), (long long)expected, (long long)out_features,
                    (long long)in_features);
    if (out_dtype != OXQ_BF16 && out_dtype != OXQ_F32)
        return fail(OXQ_ERR_DTYPE, "%s: out dtype must be BF16 or F32", op);
    OXQ_TRY(check_bias(ctx, op, bias, out_features, out_dtype));
    oxq_qlinear *l = new (std::nothrow) oxq_qlinear();
    if (!l) return fail(OXQ_ERR_RUNTIME, "%s: out of host memory", op);
    l->ctx = ctx;
    l->weight_bytes = *weight_bytes;
    l->has_bias = bias != nullptr;
    if (bias) l->bias = *bias;
    l->in_features = in_features;
    l->out_features = out_features;
    l->quant = quant;
    l->out_dtype = out_dtype;
    l->act = act;
    int rc = build_resident_gguf(l);
    if (rc == OXQ_OK && act && !(l->resident && l->mfma))
        rc = fail(OXQ_ERR_UNSUPPORTED,
                  "%s: the fused activation needs a BF16 layer on the matrix-core copy (Q4_0, Q4_1, Q5_0, Q5_1, Q8_0, "
                  "Q4_K, Q5_K or Q6_K, out_features a multiple of 16, in_features of 128 or 256, OXQ_PREPACK and "
                  "OXQ_GGUF_MFMA not 0); build a plain layer and call oxq_gated_activation on its output instead",
                  op);
    if (rc != OXQ_OK) {
        oxq_qlinear_free(l);
        return rc;
    }
    *out = l;
    return OXQ_OK;
}

int oxq_qlinear_new(oxq_ctx *ctx, int quant, const oxq_tensor *weight_bytes, int64_t in_features,
                    int64_t out_features, const oxq_tensor *bias, int out_dtype, oxq_qlinear **out) {
    return new_qlinear("QLinear", ctx, quant, weight_bytes, in_features, out_features, bias, 0, out_dtype, out);
}

int oxq_qlinear_new_gate_up(oxq_ctx *ctx, int quant, const oxq_tensor *weight_bytes, int64_t in_features,
                            int64_t out_features, const oxq_tensor *bias, int act, int out_dtype, oxq_qlinear **out) {
    const char *op = "QLinear(gate|up)";
    if (act != OXQ_ACT_GATED_SILU && act != OXQ_ACT_GATED_GELU_TANH)
        return fail(OXQ_ERR_ARG, "%s: activation must be OXQ_ACT_GATED_SILU or OXQ_ACT_GATED_GELU_TANH, got %d", op, act);
    if (out_features % 2 != 0) return fail(OXQ_ERR_SHAPE, "%s: out_features %lld is not gate and up halves", op, (long long)out_features);
    return new_qlinear(op, ctx, quant, weight_bytes, in_features, out_features, bias, act + 1, out_dtype, out);
}

// what forward does when the layer has no copy, or more rows than the copy's kernels take: the file layout
static int qlinear_forward_file_layout(oxq_qlinear *l, void *stream, const GgufProblem &p) {
    if (gguf_mm_eligible(l->ctx, p)) return launch_gguf_mm(l->ctx, (hipStream_t)stream, p);
    return launch_gguf_gemv(l->ctx, (hipStream_t)stream, p);
}

// linear.rs:324-351 QLinear::forward (fast-path arm), 250-284 forward_decode/prefill
int oxq_qlinear_forward(oxq_qlinear *l, void *stream, const oxq_tensor *x, const oxq_tensor *out) {
    const char *op = "QLinear";
    if (!l) return fail(OXQ_ERR_ARG, "%s: layer is NULL", op);
    oxq_tensor x2, o2;
    int64_t m;
    OXQ_TRY(flatten_rows(op, x, l->in_features, &x2, &m));
    OXQ_TRY(flatten_out(op, out, m, l->act ? l->out_features / 2 : l->out_features, &o2));
    if (out->dtype != l->out_dtype)
        return fail(OXQ_ERR_DTYPE, "%s: out dtype %s != layer out dtype %s", op,
                    dtype_name(out->dtype), dtype_name(l->out_dtype));
    GgufProblem p;
    const bool decode = m >= 1 && m <= 8;  // GGUF_BATCH_MAX, metal_ops.rs:5324
    if (l->act) {
        // the fused activation lives in the matrix-core kernel: every row count runs there, in row tiles of 32
        oxq_tensor full = o2;  // check_gguf sees the projection's own shape
        full.dims[full.rank - 1] = l->out_features;
        OXQ_TRY(check_gguf(l->ctx, "GgufQuantMulMM", false, false, &x2, &l->weight_bytes, l->in_features, l->out_features,
                           l->quant, &full, &p));
        if ((uintptr_t)p.x & 15) return fail(OXQ_ERR_UNSUPPORTED, "%s: x must be 16-byte aligned", op);
        p.bias = l->has_bias ? l->bias.data : nullptr;
        p.w = (const uint8_t *)l->res;
        p.act = l->act;
        if (gguf_gemm_takes(l->ctx, l->quant, p.M, p.K, p.N, p.act_dtype)) return launch_gguf_gemm(l->ctx, (hipStream_t)stream, p);
        return launch_gguf_mfma(l->ctx, (hipStream_t)stream, p);
    }
    OXQ_TRY(check_gguf(l->ctx, decode ? "GgufQuantMatmul" : "GgufQuantMulMM", decode, false, &x2,
                       &l->weight_bytes, l->in_features, l->out_features, l->quant, &o2, &p));
    p.bias = l->has_bias ? l->bias.data : nullptr;
    if (l->resident && l->mfma) {
        if (gguf_mfma_takes(l->ctx, p.M, p.N, p.act_dtype) && ((uintptr_t)p.x & 15) == 0) {
            p.w = (const uint8_t *)l->res;
            return launch_gguf_mfma(l->ctx, (hipStream_t)stream, p);
        }
        if (gguf_gemm_takes(l->ctx, l->quant, p.M, p.K, p.N, p.act_dtype) && ((uintptr_t)p.x & 15) == 0) {
            p.w = (const uint8_t *)l->res;
            return launch_gguf_gemm(l->ctx, (hipStream_t)stream, p);
        }
    } else if (l->resident && gguf_res_takes(p.K, p.M, p.act_dtype) && ((uintptr_t)p.x & 15) == 0) {
        p.w = (const uint8_t *)l->res;
        return launch_gguf_res_gemv(l->ctx, (hipStream_t)stream, p);
    }
    return qlinear_forward_file_layout(l, stream, p);
}

// The projection of a fused gate|up layer without its activation, [m, out_features], from the file layout: for
// callers that hold scratch for it (FeedForward at more rows than the fused kernel should take).
static int qlinear_forward_unfused(oxq_qlinear *l, void *stream, const oxq_tensor *x2, const oxq_tensor *gu) {
    GgufProblem p;
    const bool decode = x2->dims[0] >= 1 && x2->dims[0] <= 8;
    OXQ_TRY(check_gguf(l->ctx, decode ? "GgufQuantMatmul" : "GgufQuantMulMM", decode, false, x2, &l->weight_bytes,
                       l->in_features, l->out_features, l->quant, gu, &p));
    p.bias = l->has_bias ? l->bias.data : nullptr;
    return qlinear_forward_file_layout(l, stream, p);
}

// whether `rows` rows of a bf16 layer run the prefill kernel on its matrix-core copy (a fused gate|up layer then
// keeps its activation in that kernel's epilogue, and the plain layer takes the same kernel: the same bits)
static bool qlinear_prefill_on_copy(const oxq_qlinear *l, int64_t rows) {
    return l->resident && l->mfma && gguf_gemm_takes(l->ctx, l->quant, rows, l->in_features, l->out_features, l->out_dtype);
}

int oxq_qlinear_is_resident(const oxq_qlinear *l, int *resident) {
    if (!l || !resident) return fail(OXQ_ERR_ARG, "QLinear: NULL argument");
    *resident = l->resident ? 1 : 0;
    return OXQ_OK;
}

int oxq_qlinear_dequantize(oxq_qlinear *l, void *stream, const oxq_tensor *out) {
    const char *op = "QLinear dequantize";
    if (!l) return fail(OXQ_ERR_ARG, "%s: layer is NULL", op);
    OXQ_TRY(check_tensor(l->ctx, op, "out", out));
    if (out->dtype != OXQ_F32 || out->rank != 2 || out->dims[0] != l->out_features || out->dims[1] != l->in_features)
        return fail(OXQ_ERR_SHAPE, "%s: out must be F32 [%lld, %lld]", op, (long long)l->out_features,
                    (long long)l->in_features);
    if (!out->contiguous) return fail(OXQ_ERR_CONTIGUOUS, "%s: out must be contiguous", op);
    if (l->resident && l->mfma)
        return launch_gguf_mfma_dequant(l->ctx, (hipStream_t)stream, l->quant, l->res, l->in_features, l->out_features,
                                        (float *)out->data, l->act ? l->out_features / 2 : 0);
    if (l->resident)
        return launch_gguf_res_dequant(l->ctx, (hipStream_t)stream, l->quant, l->res, l->in_features, l->out_features,
                                       (float *)out->data);
    GgufProblem p{};
    p.w = (const uint8_t *)l->weight_bytes.data;
    p.K = l->in_features, p.N = l->out_features, p.quant = l->quant, p.act_dtype = OXQ_F32;
    return launch_gguf_dequant(l->ctx, (hipStream_t)stream, p, (float *)out->data);
}

void oxq_qlinear_free(oxq_qlinear *l) {
    if (!l) return;
    if (l->res) (void)hipFree(l->res);  // by address: the layer may outlive its ctx
    delete l;
}

// mxfp4.rs:78-116 Mxfp4Linear::new
int oxq_mxfp4_linear_new(oxq_ctx *ctx, const oxq_tensor *blocks, const oxq_tensor *scales,
                         const oxq_tensor *bias, int64_t in_features, int64_t out_features,
                         oxq_mxfp4_linear **out) {
    const char *op = "Mxfp4Linear";
    if (!ctx || !out) return fail(OXQ_ERR_ARG, "%s: NULL argument", op);
    *out = nullptr;
    OXQ_TRY(check_tensor(ctx, op, "blocks", blocks));
    OXQ_TRY(check_tensor(ctx, op, "scales", scales));
    if (blocks->dtype != OXQ_U8 || scales->dtype != OXQ_U8)
        return fail(OXQ_ERR_DTYPE, "%s: blocks/scales must be U8, got %s/%s", op,
                    dtype_name(blocks->dtype), dtype_name(scales->dtype));
    if (in_features <= 0 || in_features % 32 != 0)
        return fail(OXQ_ERR_SHAPE, "%s: in_features %lld must be a multiple of 32", op,
                    (long long)in_features);
    const int64_t nb = in_features / 32;
    if (numel(blocks) != out_features * nb * 16 || numel(scales) != out_features * nb)
        return fail(OXQ_ERR_SHAPE, "%s: blocks %lld / scales %lld elements don't match [%lld, %lld]",
                    op, (long long)numel(blocks), (long long)numel(scales), (long long)out_features,
                    (long long)in_features);
    OXQ_TRY(check_bias(ctx, op, bias, out_features, OXQ_BF16));
    oxq_mxfp4_linear *l = new (std::nothrow) oxq_mxfp4_linear();
    if (!l) return fail(OXQ_ERR_RUNTIME, "%s: out of host memory", op);
    l->ctx = ctx;
    l->blocks = *blocks;
    l->scales = *scales;
    l->has_bias = bias != nullptr;
    if (bias) l->bias = *bias;
    l->in_features = in_features;
    l->out_features = out_features;
    *out = l;
    return OXQ_OK;
}

// mxfp4.rs:119-154 Mxfp4Linear::forward
int oxq_mxfp4_linear_forward(oxq_mxfp4_linear *l, void *stream, const oxq_tensor *x,
                             const oxq_tensor *out) {
    const char *op = "Mxfp4Linear";
    if (!l) return fail(OXQ_ERR_ARG, "%s: layer is NULL", op);
    oxq_tensor x2, o2;
    int64_t m;
    if (x && x->rank >= 1 && x->dims[x->rank - 1] != l->in_features)
        return fail(OXQ_ERR_SHAPE, "%s: x last dim %lld != in_features %lld", op,
                    (long long)x->dims[x->rank - 1], (long long)l->in_features);
    OXQ_TRY(flatten_rows(op, x, l->in_features, &x2, &m));
    OXQ_TRY(flatten_out(op, out, m, l->out_features, &o2));
    Mxfp4Problem p;
    OXQ_TRY(check_mxfp4(l->ctx, "Mxfp4Matmul", false, &x2, &l->blocks, &l->scales, l->in_features,
                        l->out_features, 0, &o2, &p));
    p.bias = l->has_bias ? l->bias.data : nullptr;
    return launch_mxfp4_gemv(l->ctx, (hipStream_t)stream, p);
}

void oxq_mxfp4_linear_free(oxq_mxfp4_linear *l) { delete l; }

}  // extern "C"

// ---------------------------------------------------------------------------
// ffn.rs:22-474 FeedForward over the quantized arms of AnyLinear
// ---------------------------------------------------------------------------
struct oxq_mlp {
    oxq_ctx *ctx;
    int gate_up_kind;
    oxq_any_linear a, b, down;
    int64_t intermediate, in_features, out_features;
    int activation;
    int mid_dtype;   // dtype of the projections' outputs, which is what down_proj reads
    bool epilogue;   // `a` already applies the gated activation in its matmul
};

namespace oxq {

struct LinearInfo {
    oxq_ctx *ctx;
    int64_t in_features, out_features;  // out_features as forward writes them
    int out_dtype;
    int act;  // 0, or 1 + oxq_gated_act of a fused gate|up layer
};

static int linear_info(const char *op, const char *name, const oxq_any_linear *l, LinearInfo *info) {
    if (!l || !l->layer) return fail(OXQ_ERR_ARG, "%s: %s is NULL", op, name);
    switch (l->kind) {
    case OXQ_LINEAR_PACKED_QUANT: {
        const oxq_packed_quant_linear *q = (const oxq_packed_quant_linear *)l->layer;
        *info = LinearInfo{q->ctx, q->in_features, q->act ? q->out_features / 2 : q->out_features, q->dtype, q->act};
        return OXQ_OK;
    }
    case OXQ_LINEAR_GGUF: {
        const oxq_qlinear *q = (const oxq_qlinear *)l->layer;
        *info = LinearInfo{q->ctx, q->in_features, q->act ? q->out_features / 2 : q->out_features, q->out_dtype, q->act};
        return OXQ_OK;
    }
    case OXQ_LINEAR_MXFP4: {
        const oxq_mxfp4_linear *q = (const oxq_mxfp4_linear *)l->layer;
        *info = LinearInfo{q->ctx, q->in_features, q->out_features, OXQ_BF16, 0};
        return OXQ_OK;
    }
    default:
        return fail(OXQ_ERR_ARG, "%s: %s has unknown layer kind %d", op, name, l->kind);
    }
}

static int linear_forward(const oxq_any_linear &l, void *stream, const oxq_tensor *x, const oxq_tensor *out) {
    switch (l.kind) {
    case OXQ_LINEAR_PACKED_QUANT:
        return oxq_packed_quant_linear_forward((oxq_packed_quant_linear *)l.layer, stream, x, out);
    case OXQ_LINEAR_GGUF:
        return oxq_qlinear_forward((oxq_qlinear *)l.layer, stream, x, out);
    default:
        return oxq_mxfp4_linear_forward((oxq_mxfp4_linear *)l.layer, stream, x, out);
    }
}

// elements of `mid_dtype` that forward keeps between the projections, per row of x
static int64_t mlp_scratch_per_row(const oxq_mlp *m) {
    switch (m->gate_up_kind) {
    // (a GGUF layer with the fused activation runs many rows unfused, on the file layout)
    case OXQ_GATE_UP_FUSED: return (m->epilogue && m->a.kind != OXQ_LINEAR_GGUF) ? m->intermediate : 3 * m->intermediate;
    case OXQ_GATE_UP_SEPARATE: return 2 * m->intermediate;
    default: return m->intermediate;
    }
}

static oxq_tensor rows_view(const oxq_tensor *base, int64_t elem_offset, int64_t m, int64_t n) {
    oxq_tensor t = *base;
    t.data = (char *)base->data + elem_offset * dtype_size(base->dtype);
    t.rank = 2;
    t.dims[0] = m;
    t.dims[1] = n;
    t.contiguous = 1;
    return t;
}

}  // namespace oxq

extern "C" {

int oxq_mlp_new(oxq_ctx *ctx, int gate_up_kind, const oxq_any_linear *a, const oxq_any_linear *b,
                const oxq_any_linear *down, int64_t intermediate, int activation, oxq_mlp **out) {
    const char *op = "FeedForward";
    if (!ctx || !out) return fail(OXQ_ERR_ARG, "%s: NULL argument", op);
    *out = nullptr;
    if (gate_up_kind != OXQ_GATE_UP_FUSED && gate_up_kind != OXQ_GATE_UP_SEPARATE && gate_up_kind != OXQ_GATE_UP_SIMPLE)
        return fail(OXQ_ERR_ARG, "%s: unknown gate/up layout %d", op, gate_up_kind);
    if (activation != OXQ_ACT_GATED_SILU && activation != OXQ_ACT_GATED_GELU_TANH)
        return fail(OXQ_ERR_ARG, "%s: activation must be OXQ_ACT_GATED_SILU or OXQ_ACT_GATED_GELU_TANH, got %d", op,
                    activation);
    if (intermediate <= 0) return fail(OXQ_ERR_SHAPE, "%s: intermediate size %lld", op, (long long)intermediate);
    const bool separate = gate_up_kind == OXQ_GATE_UP_SEPARATE;
    if (separate != (b != nullptr))
        return fail(OXQ_ERR_ARG, "%s: the second projection belongs to the separate gate/up layout and to no other", op);
    LinearInfo ia, ib{}, id;
    OXQ_TRY(linear_info(op, separate ? "gate_proj" : gate_up_kind == OXQ_GATE_UP_FUSED ? "gate_up_proj" : "up_proj", a, &ia));
    if (separate) OXQ_TRY(linear_info(op, "up_proj", b, &ib));
    OXQ_TRY(linear_info(op, "down_proj", down, &id));
    if (ia.ctx != ctx || id.ctx != ctx || (separate && ib.ctx != ctx))
        return fail(OXQ_ERR_ARG, "%s: every projection must belong to this context", op);
    bool epilogue = false;
    if (gate_up_kind == OXQ_GATE_UP_FUSED) {
        epilogue = ia.act != 0;
        if (epilogue && ia.act != activation + 1)
            return fail(OXQ_ERR_ARG, "%s: gate_up_proj was built with another activation than the layer's", op);
        // ffn.rs:255-261: a fused projection carries 2 * intermediate columns
        if (ia.out_features != (epilogue ? intermediate : 2 * intermediate))
            return fail(OXQ_ERR_SHAPE, "%s: gate_up out_features %lld != 2*%lld", op,
                        (long long)(epilogue ? 2 * ia.out_features : ia.out_features), (long long)intermediate);
    } else {
        if (ia.act || (separate && ib.act))
            return fail(OXQ_ERR_ARG, "%s: a layer with a fused activation can only be the fused gate_up_proj", op);
        // ffn.rs:227-233, 270-276
        if (ia.out_features != intermediate || (separate && ib.out_features != intermediate))
            return fail(OXQ_ERR_SHAPE, "%s: gate/up out_features must both be %lld, got %lld and %lld", op,
                        (long long)intermediate, (long long)ia.out_features,
                        (long long)(separate ? ib.out_features : ia.out_features));
        if (separate && (ib.in_features != ia.in_features || ib.out_dtype != ia.out_dtype))
            return fail(OXQ_ERR_SHAPE, "%s: gate_proj and up_proj must share in_features and the output dtype", op);
    }
    if (id.act) return fail(OXQ_ERR_ARG, "%s: down_proj cannot carry a fused activation", op);
    if (id.in_features != intermediate)
        return fail(OXQ_ERR_SHAPE, "%s: down_proj in_features %lld != intermediate size %lld", op,
                    (long long)id.in_features, (long long)intermediate);
    if (!is_float_dtype(ia.out_dtype)) return fail(OXQ_ERR_DTYPE, "%s: projections must write F32, F16 or BF16", op);
    oxq_mlp *m = new (std::nothrow) oxq_mlp();
    if (!m) return fail(OXQ_ERR_RUNTIME, "%s: out of host memory", op);
    m->ctx = ctx;
    m->gate_up_kind = gate_up_kind;
    m->a = *a;
    if (separate) m->b = *b;
    m->down = *down;
    m->intermediate = intermediate;
    m->in_features = ia.in_features;
    m->out_features = id.out_features;
    m->activation = activation;
    m->mid_dtype = ia.out_dtype;
    m->epilogue = epilogue;
    *out = m;
    return OXQ_OK;
}

int oxq_mlp_scratch_elems(const oxq_mlp *m, int64_t rows, int64_t *elems) {
    if (!m || !elems || rows < 0) return fail(OXQ_ERR_ARG, "FeedForward: bad argument");
    *elems = rows * mlp_scratch_per_row(m);
    return OXQ_OK;
}

// ffn.rs:386-474 FeedForward::forward
int oxq_mlp_forward(oxq_mlp *m, void *stream, const oxq_tensor *x, const oxq_tensor *scratch, const oxq_tensor *out) {
    const char *op = "FeedForward";
    if (!m) return fail(OXQ_ERR_ARG, "%s: layer is NULL", op);
    oxq_tensor x2;
    int64_t rows;
    OXQ_TRY(flatten_rows(op, x, m->in_features, &x2, &rows));
    OXQ_TRY(check_tensor(m->ctx, op, "scratch", scratch));
    const int64_t I = m->intermediate, need = rows * mlp_scratch_per_row(m);
    if (scratch->dtype != m->mid_dtype || !scratch->contiguous || numel(scratch) < need)
        return fail(OXQ_ERR_SHAPE, "%s: scratch must be a contiguous %s tensor of at least %lld elements", op,
                    dtype_name(m->mid_dtype), (long long)need);
    oxq_tensor h;  // [rows, I]: act(gate) * up, the input of down_proj
    switch (m->gate_up_kind) {
    case OXQ_GATE_UP_FUSED:
        if (m->epilogue && m->a.kind == OXQ_LINEAR_GGUF && rows > OXQ_GGUF_FUSED_ACT_ROWS &&
            !qlinear_prefill_on_copy((const oxq_qlinear *)m->a.layer, rows)) {
            // every row tile of the fused kernel reads the weights again: the tile matmul and the activation by itself
            const oxq_tensor gu = rows_view(scratch, 0, rows, 2 * I);
            h = rows_view(scratch, rows * 2 * I, rows, I);
            OXQ_TRY(qlinear_forward_unfused((oxq_qlinear *)m->a.layer, stream, &x2, &gu));
            OXQ_TRY(oxq_gated_activation(m->ctx, stream, &gu, m->activation, 0.0f, &h));
        } else if (m->epilogue) {
            h = rows_view(scratch, 0, rows, I);
            OXQ_TRY(linear_forward(m->a, stream, &x2, &h));
        } else {
            const oxq_tensor gu = rows_view(scratch, 0, rows, 2 * I);
            h = rows_view(scratch, rows * 2 * I, rows, I);
            OXQ_TRY(linear_forward(m->a, stream, &x2, &gu));
            OXQ_TRY(oxq_gated_activation(m->ctx, stream, &gu, m->activation, 0.0f, &h));
        }
        break;
    case OXQ_GATE_UP_SEPARATE: {
        h = rows_view(scratch, 0, rows, I);
        const oxq_tensor u = rows_view(scratch, rows * I, rows, I);
        OXQ_TRY(linear_forward(m->a, stream, &x2, &h));
        OXQ_TRY(linear_forward(m->b, stream, &x2, &u));
        OXQ_TRY(oxq_activation_mul(m->ctx, stream, &h, &u, m->activation, &h));
        break;
    }
    default:
        h = rows_view(scratch, 0, rows, I);
        OXQ_TRY(linear_forward(m->a, stream, &x2, &h));
        if (rows > 0)
            OXQ_TRY(launch_activation_mul(m->ctx, (hipStream_t)stream, h.data, nullptr, h.data, h.dtype, rows * I,
                                          m->activation));
        break;
    }
    return linear_forward(m->down, stream, &h, out);
}

int oxq_mlp_in_features(const oxq_mlp *m, int64_t *k) {
    if (!m || !k) return fail(OXQ_ERR_ARG, "FeedForward: NULL argument");
    *k = m->in_features;
    return OXQ_OK;
}
int oxq_mlp_out_features(const oxq_mlp *m, int64_t *n) {
    if (!m || !n) return fail(OXQ_ERR_ARG, "FeedForward: NULL argument");
    *n = m->out_features;
    return OXQ_OK;
}

void oxq_mlp_free(oxq_mlp *m) { delete m; }

}  // extern "C"
