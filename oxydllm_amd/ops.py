"""Torch-facing binding of the C ABI, named after the reference's op functions
(``src/common/metal_ops.rs``) and layer types (``src/common/linear.rs``,
``src/common/mxfp4.rs``).

torch is plumbing only: it owns device memory and the current stream.  All
validation, routing and compute happen behind the C ABI; this module builds
descriptors, allocates the output the reference op would have allocated, and
raises :class:`OxqError` with the library's message on failure.
"""
from __future__ import annotations

import ctypes as C
from typing import Optional

import torch

from . import _lib
from ._lib import (BF16, F16, F32, GGUF_Q2_K, GGUF_Q3_K, GGUF_Q4_0, GGUF_Q4_1, GGUF_Q4_K, GGUF_Q5_0,
                   GGUF_Q5_1, GGUF_Q5_K, GGUF_Q6_K, GGUF_Q8_0, I32, I64, PACK_IN, PACK_OUT, U8, U32,
                   OxqError, OxqPlan, OxqTensor)

_DTYPES = {torch.float32: F32, torch.float16: F16, torch.bfloat16: BF16, torch.uint8: U8,
           torch.int32: I32, torch.int64: I64}
if hasattr(torch, "uint32"):
    _DTYPES[torch.uint32] = U32
_TORCH_OF = {F32: torch.float32, F16: torch.float16, BF16: torch.bfloat16}


def desc(t: Optional[torch.Tensor]):
    """Tensor -> pointer to an oxq_tensor descriptor (None -> NULL)."""
    if t is None:
        return None
    return C.byref(desc_struct(t))


def desc_struct(t) -> OxqTensor:
    """Tensor -> oxq_tensor descriptor by value (for arrays of descriptors)."""
    if isinstance(t, OxqTensor):
        return t
    if t.dtype not in _DTYPES:
        raise OxqError(-2, f"unsupported torch dtype {t.dtype}")
    if t.dim() < 1 or t.dim() > _lib.OXQ_MAX_RANK:
        raise OxqError(-3, f"rank {t.dim()} out of [1, {_lib.OXQ_MAX_RANK}]")
    d = OxqTensor()
    d.data = t.data_ptr()
    d.dtype = _DTYPES[t.dtype]
    d.rank = t.dim()
    for i, s in enumerate(t.shape):
        d.dims[i] = s
    d.contiguous = 1 if t.is_contiguous() else 0
    d.device = t.device.index if t.device.type == "cuda" else _lib.DEVICE_HOST
    if t.device.type == "cuda" and d.device is None:
        d.device = torch.cuda.current_device()
    return d


class Context:
    """One per engine thread / stream (owns the split-K workspace)."""

    def __init__(self, device: Optional[int] = None, plan_only: bool = False):
        self._lib = _lib.load()
        self.handle = C.c_void_p()
        if plan_only:
            dev = _lib.DEVICE_PLAN_ONLY
        else:
            dev = torch.cuda.current_device() if device is None else device
        _lib.check(self._lib.oxq_ctx_create(dev, C.byref(self.handle)))
        self.device = dev
        self.plan_only = plan_only

    def close(self):
        if self.handle:
            self._lib.oxq_ctx_destroy(self.handle)
            self.handle = C.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def last_plan(self) -> dict:
        p = OxqPlan()
        _lib.check(self._lib.oxq_ctx_last_plan(self.handle, C.byref(p)))
        return {"kernel": p.kernel.decode(), "grid": tuple(p.grid), "block": tuple(p.block),
                "split_k": p.split_k, "launches": p.launches, "workspace_bytes": p.workspace_bytes}

    def stream(self) -> int:
        if self.plan_only:
            return 0
        return torch.cuda.current_stream().cuda_stream

    def set_tuning(self, name: str, value: Optional[int]) -> None:
        """One tuning switch of this context (see include/oxq.h); ``None`` returns it to the
        environment's value, or to the launcher's default."""
        if value is None:
            _lib.check(self._lib.oxq_ctx_reset_tuning(self.handle, name.encode()))
        else:
            _lib.check(self._lib.oxq_ctx_set_tuning(self.handle, name.encode(), int(value)))

    def reset_tuning(self) -> None:
        _lib.check(self._lib.oxq_ctx_reset_tuning(self.handle, None))

    # opt-in cache of tile-major weight copies behind the stateless ops (see include/oxq.h)
    def set_weight_cache(self, max_bytes: int) -> None:
        _lib.check(self._lib.oxq_ctx_set_weight_cache(self.handle, int(max_bytes)))

    def forget_weights(self, qweight: Optional[torch.Tensor] = None) -> None:
        ptr = C.c_void_p(qweight.data_ptr()) if qweight is not None else C.c_void_p()
        _lib.check(self._lib.oxq_ctx_forget_weights(self.handle, ptr))

    def weight_cache_usage(self) -> tuple:
        b, n = C.c_int64(), C.c_int64()
        _lib.check(self._lib.oxq_ctx_weight_cache_bytes(self.handle, C.byref(b), C.byref(n)))
        return b.value, n.value


_default_ctx: dict = {}


def default_context() -> Context:
    dev = torch.cuda.current_device()
    if dev not in _default_ctx:
        _default_ctx[dev] = Context(dev)
    return _default_ctx[dev]


def _ctx(ctx: Optional[Context]) -> Context:
    return ctx if ctx is not None else default_context()


def _out_for(x: torch.Tensor, n: int, out, ctx):
    if out is not None:
        return out
    return torch.empty((x.shape[0], n), dtype=x.dtype, device=x.device)


# ---------------------------------------------------------------- AWQ / GPTQ ops
def calib_read(src, workgroups: int, nontemporal: bool, checksums, *, ctx: Optional[Context] = None):
    """Plain streaming read of ``src`` (uint8) by ``workgroups`` workgroups; ``checksums`` (int32/uint32,
    one word per workgroup) receives the xor of every span.  A measurement aid (see include/oxq_bench.h)."""
    ctx = _ctx(ctx)
    _lib.check(ctx._lib.oxq_calib_read(ctx.handle, ctx.stream(), desc(src), int(workgroups), int(bool(nontemporal)),
                                       desc(checksums)))
    return checksums


def read_upfront(src, workgroups: int, waves: int, nontemporal: bool, checksums, *, ctx: Optional[Context] = None):
    """The same read with every lane's share requested before the first wait (include/oxq_bench.h)."""
    ctx = _ctx(ctx)
    _lib.check(ctx._lib.oxq_bench_read_upfront(ctx.handle, ctx.stream(), desc(src), int(workgroups), int(waves),
                                               int(bool(nontemporal)), desc(checksums)))
    return checksums


def two_streams(w, x, workgroups: int, which: int, checksums, *, ctx: Optional[Context] = None):
    """Cold weight stream and L2-resident activation stream from every compute unit, alone (which = 1, 2) or
    together (3) (include/oxq_bench.h)."""
    ctx = _ctx(ctx)
    _lib.check(ctx._lib.oxq_bench_two_streams(ctx.handle, ctx.stream(), desc(w), desc(x), int(workgroups), int(which),
                                              desc(checksums)))


def empty_launch(workgroups: int, threads: int, lds_bytes: int = 0, *, ctx: Optional[Context] = None):
    """An empty kernel of the given launch shape (include/oxq_bench.h)."""
    ctx = _ctx(ctx)
    _lib.check(ctx._lib.oxq_bench_empty_launch(ctx.handle, ctx.stream(), int(workgroups), int(threads), int(lds_bytes)))


def grid_barrier(workgroups: int, threads: int, state, spin_limit: int = 1 << 18, *, ctx: Optional[Context] = None):
    """A launch that is one bounded grid barrier (include/oxq_bench.h); state: two zeroed int32 words
    {counter, error}, the error word is 1 afterwards if a workgroup gave up."""
    ctx = _ctx(ctx)
    _lib.check(ctx._lib.oxq_bench_grid_barrier(ctx.handle, ctx.stream(), int(workgroups), int(threads), desc(state),
                                               int(spin_limit)))


def w4a16_matmul(x, qweight, qzeros, scales, *, out=None, ctx: Optional[Context] = None):
    """metal_ops.rs:1821.  x [m,K] (m in 1..=8) -> [m,N] in x's dtype."""
    ctx = _ctx(ctx)
    out = _out_for(x, scales.shape[1], out, ctx)
    _lib.check(ctx._lib.oxq_w4a16_matmul(ctx.handle, ctx.stream(), desc(x), desc(qweight),
                                         desc(qzeros), desc(scales), desc(out)))
    return out


def w4a16_matmul_static(x, qweight, qzeros, scales, *, out, ctx: Optional[Context] = None):
    """``w4a16_matmul`` through the entry point that allocates nothing: the split-K partial sums go to
    the library's static device array (16 MiB per GPU) instead of the ctx workspace.  ``out`` is
    mandatory (this binding allocates nothing either); calls that overlap on one GPU race."""
    ctx = _ctx(ctx)
    _lib.check(ctx._lib.oxq_w4a16_matmul_static(ctx.handle, ctx.stream(), desc(x), desc(qweight),
                                                desc(qzeros), desc(scales), desc(out)))
    return out


def w8a16_matmul(x, qweight, qzeros, scales, *, out=None, ctx: Optional[Context] = None):
    """metal_ops.rs:1835."""
    ctx = _ctx(ctx)
    out = _out_for(x, scales.shape[1], out, ctx)
    _lib.check(ctx._lib.oxq_w8a16_matmul(ctx.handle, ctx.stream(), desc(x), desc(qweight),
                                         desc(qzeros), desc(scales), desc(out)))
    return out


def gptq_matmul(x, qweight, qzeros, scales, bits: int, *, out=None, ctx: Optional[Context] = None):
    """metal_ops.rs:2281."""
    ctx = _ctx(ctx)
    out = _out_for(x, scales.shape[1], out, ctx)
    _lib.check(ctx._lib.oxq_gptq_matmul(ctx.handle, ctx.stream(), desc(x), desc(qweight),
                                        desc(qzeros), desc(scales), bits, desc(out)))
    return out


def _dequant_out(qweight, scales, bits, pack_dim, out):
    if out is not None:
        return out
    pf = 32 // bits if bits in (4, 8) else 8
    k = qweight.shape[0] if pack_dim == PACK_OUT else qweight.shape[0] * pf
    return torch.empty((k, scales.shape[1]), dtype=scales.dtype, device=scales.device)


def dequantize_w4(qweight, qzeros, scales, *, out=None, ctx: Optional[Context] = None):
    """metal_ops.rs:1873 -> dense [K,N] in the scales' dtype."""
    ctx = _ctx(ctx)
    out = _dequant_out(qweight, scales, 4, PACK_OUT, out)
    _lib.check(ctx._lib.oxq_dequantize_w4(ctx.handle, ctx.stream(), desc(qweight), desc(qzeros),
                                          desc(scales), desc(out)))
    return out


def dequantize_w8(qweight, qzeros, scales, *, out=None, ctx: Optional[Context] = None):
    """metal_ops.rs:1886."""
    ctx = _ctx(ctx)
    out = _dequant_out(qweight, scales, 8, PACK_OUT, out)
    _lib.check(ctx._lib.oxq_dequantize_w8(ctx.handle, ctx.stream(), desc(qweight), desc(qzeros),
                                          desc(scales), desc(out)))
    return out


def dequantize_gptq_packed(qweight, qzeros, scales, bits: int, *, out=None,
                           ctx: Optional[Context] = None):
    """metal_ops.rs:2305."""
    ctx = _ctx(ctx)
    out = _dequant_out(qweight, scales, bits, PACK_IN, out)
    _lib.check(ctx._lib.oxq_dequantize_gptq_packed(ctx.handle, ctx.stream(), desc(qweight),
                                                   desc(qzeros), desc(scales), bits, desc(out)))
    return out


def mpp_quant_matmul(x, qweight, qzeros, scales, bits: int, pack_dim: int, *, out=None,
                     ctx: Optional[Context] = None):
    """metal_ops.rs:2748: tile GEMM on the matrix cores, any m."""
    ctx = _ctx(ctx)
    out = _out_for(x, scales.shape[1], out, ctx)
    _lib.check(ctx._lib.oxq_mpp_quant_matmul(ctx.handle, ctx.stream(), desc(x), desc(qweight),
                                             desc(qzeros), desc(scales), bits, pack_dim, desc(out)))
    return out


def maybe_mpp_quant_matmul(x, qweight, qzeros, scales, bits: int, pack_dim: int, *,
                           ctx: Optional[Context] = None):
    """metal_ops.rs:2771: returns None when the op declines (small m, wrong dtype...)."""
    ctx = _ctx(ctx)
    out = _out_for(x, scales.shape[1], None, ctx)
    taken = C.c_int(0)
    _lib.check(ctx._lib.oxq_maybe_mpp_quant_matmul(ctx.handle, ctx.stream(), desc(x), desc(qweight),
                                                   desc(qzeros), desc(scales), bits, pack_dim,
                                                   desc(out), C.byref(taken)))
    return out if taken.value else None


# ---------------------------------------------------------------- load-time transforms
def compressed_to_awq(weight_packed, weight_scale, *, ctx: Optional[Context] = None):
    """awq.rs:187-254: returns AWQ (qweight [in, out/8], qzeros [groups, out/8], scales [groups, out])."""
    ctx = _ctx(ctx)
    out_f, packed_in = weight_packed.shape
    groups = weight_scale.shape[1] if weight_scale.dim() == 2 else 0
    dev = weight_packed.device
    qweight = torch.empty((packed_in * 8, out_f // 8), dtype=torch.int32, device=dev)
    qzeros = torch.empty((groups, out_f // 8), dtype=torch.int32, device=dev)
    scales = torch.empty((groups, out_f), dtype=weight_scale.dtype, device=dev)
    _lib.check(ctx._lib.oxq_compressed_to_awq(ctx.handle, ctx.stream(), desc(weight_packed), desc(weight_scale),
                                              desc(qweight), desc(qzeros), desc(scales)))
    return qweight, qzeros, scales


def concat_awq_along_out(parts, bits: int = 4, *, ctx: Optional[Context] = None):
    """awq.rs:256-323: parts = [(qweight, qzeros, scales), ...] -> one fused AWQ triplet."""
    ctx = _ctx(ctx)
    n = len(parts)
    if n == 0:
        raise OxqError(-1, "concat_awq_along_out: no parts")
    arr = [(OxqTensor * n)(*[desc_struct(p[i]) for p in parts]) for i in range(3)]
    pf = 32 // bits if bits in (4, 8) else 8
    total = sum(int(p[2].shape[1]) for p in parts)
    dev = parts[0][0].device
    qweight = torch.empty((parts[0][0].shape[0], total // pf), dtype=torch.int32, device=dev)
    qzeros = torch.empty((parts[0][2].shape[0], total // pf), dtype=torch.int32, device=dev)
    scales = torch.empty((parts[0][2].shape[0], total), dtype=parts[0][2].dtype, device=dev)
    _lib.check(ctx._lib.oxq_concat_awq_along_out(ctx.handle, ctx.stream(), bits, n, arr[0], arr[1], arr[2],
                                                 desc(qweight), desc(qzeros), desc(scales)))
    return qweight, qzeros, scales


def rtn_quantize_awq(weight, group_size: int, *, ctx: Optional[Context] = None):
    """awq.rs:637-742: dense [out, in] -> AWQ 4-bit (qweight, qzeros, f32 scales)."""
    ctx = _ctx(ctx)
    out_f, in_f = weight.shape
    groups = in_f // group_size if group_size > 0 else 0
    dev = weight.device
    qweight = torch.empty((in_f, out_f // 8), dtype=torch.int32, device=dev)
    qzeros = torch.empty((groups, out_f // 8), dtype=torch.int32, device=dev)
    scales = torch.empty((groups, out_f), dtype=torch.float32, device=dev)
    _lib.check(ctx._lib.oxq_rtn_quantize_awq(ctx.handle, ctx.stream(), desc(weight), group_size, desc(qweight),
                                             desc(qzeros), desc(scales)))
    return qweight, qzeros, scales


def gguf_depermute_qk_rows(weight_bytes, in_features: int, out_features: int, quant: int, n_heads: int,
                           head_dim: int, *, ctx: Optional[Context] = None):
    """gguf_weights.rs:255-291: block bytes of a q/k projection back in the HF row order."""
    ctx = _ctx(ctx)
    out = torch.empty_like(weight_bytes)
    _lib.check(ctx._lib.oxq_gguf_depermute_qk_rows(ctx.handle, ctx.stream(), desc(weight_bytes), in_features,
                                                   out_features, quant, n_heads, head_dim, desc(out)))
    return out


# ---------------------------------------------------------------- block-scaled F8E4M3
def cast_f8e4m3_to_f32(t, *, ctx: Optional[Context] = None):
    """metal_ops.rs:5562: U8 tensor of E4M3 encodings -> F32 of the same shape."""
    ctx = _ctx(ctx)
    out = torch.empty(t.shape, dtype=torch.float32, device=t.device)
    _lib.check(ctx._lib.oxq_cast_f8e4m3_to_f32(ctx.handle, ctx.stream(), desc(t), desc(out)))
    return out


def f8_block_dequant_bf16(bytes_, scales, *, ctx: Optional[Context] = None):
    """metal_ops.rs:5809: U8 [out, in] + F32 scale grid -> BF16 [out, in]."""
    ctx = _ctx(ctx)
    out = torch.empty(tuple(bytes_.shape), dtype=torch.bfloat16, device=bytes_.device)
    _lib.check(ctx._lib.oxq_f8_block_dequant_bf16(ctx.handle, ctx.stream(), desc(bytes_), desc(scales), desc(out)))
    return out


def f8_gemv(x, bytes_, scales, *, out=None, ctx: Optional[Context] = None):
    """metal_ops.rs:5788: x BF16 [m <= 8, in] times the block-scaled F8 weight [out, in]."""
    ctx = _ctx(ctx)
    out = _out_for(x, bytes_.shape[0], out, ctx)
    _lib.check(ctx._lib.oxq_f8_gemv(ctx.handle, ctx.stream(), desc(x), desc(bytes_), desc(scales), desc(out)))
    return out


def f8_matmul(x, bytes_, scales, *, out=None, ctx: Optional[Context] = None):
    """moe.rs:106-113 (Fp8Cached::forward): any m."""
    ctx = _ctx(ctx)
    out = _out_for(x, bytes_.shape[0], out, ctx)
    _lib.check(ctx._lib.oxq_f8_matmul(ctx.handle, ctx.stream(), desc(x), desc(bytes_), desc(scales), desc(out)))
    return out


# ---------------------------------------------------------------- GGUF
def gguf_block_layout(quant: int):
    e, b = C.c_int64(), C.c_int64()
    _lib.check(_lib.load().oxq_gguf_block_layout(quant, C.byref(e), C.byref(b)))
    return e.value, b.value


def gguf_quant_matmul(x, weight_bytes, in_features: int, out_features: int, quant: int, *,
                      out=None, ctx: Optional[Context] = None):
    """metal_ops.rs:5819 (1 <= m <= 8)."""
    ctx = _ctx(ctx)
    out = _out_for(x, out_features, out, ctx)
    _lib.check(ctx._lib.oxq_gguf_quant_matmul(ctx.handle, ctx.stream(), desc(x), desc(weight_bytes),
                                              in_features, out_features, quant, desc(out)))
    return out


def gguf_quant_mul_mm(x, weight_bytes, in_features: int, out_features: int, quant: int, *,
                      out=None, ctx: Optional[Context] = None):
    """metal_ops.rs:5973 (any m)."""
    ctx = _ctx(ctx)
    out = _out_for(x, out_features, out, ctx)
    _lib.check(ctx._lib.oxq_gguf_quant_mul_mm(ctx.handle, ctx.stream(), desc(x), desc(weight_bytes),
                                              in_features, out_features, quant, desc(out)))
    return out


def gguf_dequantize(weight_bytes, in_features: int, out_features: int, quant: int, *,
                    ctx: Optional[Context] = None):
    ctx = _ctx(ctx)
    out = torch.empty((out_features, in_features), dtype=torch.float32, device=weight_bytes.device)
    _lib.check(ctx._lib.oxq_gguf_dequantize(ctx.handle, ctx.stream(), desc(weight_bytes),
                                            in_features, out_features, quant, desc(out)))
    return out


# ---------------------------------------------------------------- MXFP4
def mxfp4_matmul(x, blocks, scales, k: int, n: int, *, out=None, ctx: Optional[Context] = None):
    """metal_ops.rs:6197."""
    ctx = _ctx(ctx)
    out = _out_for(x, n, out, ctx)
    _lib.check(ctx._lib.oxq_mxfp4_matmul(ctx.handle, ctx.stream(), desc(x), desc(blocks),
                                         desc(scales), k, n, desc(out)))
    return out


def mxfp4_dequantize(blocks, scales, k: int, n: int, *, ctx: Optional[Context] = None):
    ctx = _ctx(ctx)
    out = torch.empty((n, k), dtype=torch.float32, device=blocks.device)
    _lib.check(ctx._lib.oxq_mxfp4_dequantize(ctx.handle, ctx.stream(), desc(blocks), desc(scales),
                                             k, n, desc(out)))
    return out


def mxfp4_moe_matmul(x, blocks, scales, bias, expert_offsets, token_ids, k: int, n: int, *,
                     out=None, ctx: Optional[Context] = None):
    """Grouped expert GEMV: out[p] = x[row(p)] . W_e^T + bias_e for every routed pair."""
    ctx = _ctx(ctx)
    gather = token_ids is not None
    n_pairs = token_ids.numel() if gather else x.shape[0]
    if out is None:
        out = torch.empty((n_pairs, n), dtype=x.dtype, device=x.device)
    _lib.check(ctx._lib.oxq_mxfp4_moe_matmul(ctx.handle, ctx.stream(), desc(x), desc(blocks),
                                             desc(scales), desc(bias), desc(expert_offsets),
                                             desc(token_ids), 1 if gather else 0, k, n, desc(out)))
    return out


# ---------------------------------------------------------------- mixture-of-experts glue
ACT_GATED_SILU, ACT_GATED_GELU_TANH, ACT_GPT_OSS_SWIGLU = 0, 1, 2


def mxfp4_moe_gate_up_swiglu(x, blocks, scales, bias, expert_offsets, token_ids, k: int, n: int, limit: float, *,
                             out=None, ctx: Optional[Context] = None):
    """gate_up projection of the routed pairs + GPT-OSS SwiGLU (moe.rs:152-173) -> [n_pairs, n / 2].  One
    launch where the decode kernel runs; otherwise the two calls it stands for (same bits either way)."""
    ctx = _ctx(ctx)
    gather = token_ids is not None
    n_pairs = token_ids.numel() if gather else x.shape[0]
    if out is None:
        out = torch.empty((n_pairs, n // 2), dtype=x.dtype, device=x.device)
    fused = C.c_int()
    _lib.check(ctx._lib.oxq_mxfp4_moe_gate_up_swiglu(ctx.handle, ctx.stream(), desc(x), desc(blocks), desc(scales),
                                                     desc(bias), desc(expert_offsets), desc(token_ids),
                                                     1 if gather else 0, k, n, float(limit), desc(out), C.byref(fused)))
    if not fused.value:
        gu = mxfp4_moe_matmul(x, blocks, scales, bias, expert_offsets, token_ids, k, n, ctx=ctx)
        gated_activation(gu, ACT_GPT_OSS_SWIGLU, limit, out=out, ctx=ctx)
    return out


class Mxfp4Experts:
    """The stacked MXFP4 expert tensors of one MoE projection, kept resident (moe.rs:366-417): ``blocks`` u8
    [E * n * k/32 * 16], ``scales`` u8 [E * n * k/32], ``bias`` bf16 [E, n] or None.  Construction builds the
    tile-major copy that decode sizes stream; the caller's tensors are borrowed (prefill sizes run on them)."""

    def __init__(self, blocks, scales, bias, n_experts: int, k: int, n: int, *, ctx: Optional[Context] = None):
        self.ctx = _ctx(ctx)
        self._keep = (blocks, scales, bias)
        self.n_experts, self.k, self.n = n_experts, k, n
        self.handle = C.c_void_p()
        _lib.check(self.ctx._lib.oxq_mxfp4_experts_new(self.ctx.handle, desc(blocks), desc(scales), desc(bias),
                                                       n_experts, k, n, C.byref(self.handle)))

    @property
    def resident(self) -> bool:
        r = C.c_int()
        _lib.check(self.ctx._lib.oxq_mxfp4_experts_is_resident(self.handle, C.byref(r)))
        return bool(r.value)

    def matmul(self, x, expert_offsets, token_ids, *, out=None):
        gather = token_ids is not None
        n_pairs = token_ids.numel() if gather else x.shape[0]
        if out is None:
            out = torch.empty((n_pairs, self.n), dtype=x.dtype, device=x.device)
        _lib.check(self.ctx._lib.oxq_mxfp4_experts_matmul(self.handle, self.ctx.stream(), desc(x), desc(expert_offsets),
                                                          desc(token_ids), 1 if gather else 0, desc(out)))
        return out

    def gate_up_swiglu(self, x, expert_offsets, token_ids, limit: float, *, out=None):
        gather = token_ids is not None
        n_pairs = token_ids.numel() if gather else x.shape[0]
        if out is None:
            out = torch.empty((n_pairs, self.n // 2), dtype=x.dtype, device=x.device)
        fused = C.c_int()
        _lib.check(self.ctx._lib.oxq_mxfp4_experts_gate_up_swiglu(self.handle, self.ctx.stream(), desc(x),
                                                                  desc(expert_offsets), desc(token_ids),
                                                                  1 if gather else 0, float(limit), desc(out),
                                                                  C.byref(fused)))
        if not fused.value:
            gu = self.matmul(x, expert_offsets, token_ids)
            gated_activation(gu, ACT_GPT_OSS_SWIGLU, limit, out=out, ctx=self.ctx)
        return out

    def dequantize(self, expert: int):
        out = torch.empty((self.n, self.k), dtype=torch.float32, device=self._keep[0].device)
        _lib.check(self.ctx._lib.oxq_mxfp4_experts_dequantize(self.handle, self.ctx.stream(), expert, desc(out)))
        return out

    def close(self):
        if self.handle:
            self.ctx._lib.oxq_mxfp4_experts_free(self.handle)
            self.handle = C.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


def moe_route(logits, top_k: int, norm_topk: bool = True, *, ctx: Optional[Context] = None):
    """moe.rs:466-486: softmax, stable descending top-k, optional renormalisation."""
    ctx = _ctx(ctx)
    T = logits.shape[0]
    idx = torch.empty((T, top_k), dtype=torch.int32, device=logits.device)
    vals = torch.empty((T, top_k), dtype=torch.float32, device=logits.device)
    _lib.check(ctx._lib.oxq_moe_route(ctx.handle, ctx.stream(), desc(logits), top_k, 1 if norm_topk else 0,
                                      desc(idx), desc(vals)))
    return idx, vals


def moe_group(top_idx, top_vals, n_experts: int, *, ctx: Optional[Context] = None):
    """moe.rs:563-590: (expert_offsets [E+1], token_ids [P], pair_weights [P], pair_pos [T,k])."""
    ctx = _ctx(ctx)
    T, k = top_idx.shape
    dev = top_idx.device
    offsets = torch.empty((n_experts + 1,), dtype=torch.int32, device=dev)
    tokens = torch.empty((T * k,), dtype=torch.int32, device=dev)
    weights = torch.empty((T * k,), dtype=torch.float32, device=dev)
    pos = torch.empty((T, k), dtype=torch.int32, device=dev)
    _lib.check(ctx._lib.oxq_moe_group(ctx.handle, ctx.stream(), desc(top_idx), desc(top_vals), n_experts,
                                      desc(offsets), desc(tokens), desc(weights), desc(pos)))
    return offsets, tokens, weights, pos


def moe_route_group(logits, top_k: int, norm_topk: bool = True, *, ctx: Optional[Context] = None):
    """moe_route + moe_group in one call (one launch for decode sizes): returns (top_idx, top_vals,
    expert_offsets, token_ids, pair_weights, pair_pos)."""
    ctx = _ctx(ctx)
    T, E = logits.shape
    dev = logits.device
    idx = torch.empty((T, top_k), dtype=torch.int32, device=dev)
    vals = torch.empty((T, top_k), dtype=torch.float32, device=dev)
    offsets = torch.empty((E + 1,), dtype=torch.int32, device=dev)
    tokens = torch.empty((T * top_k,), dtype=torch.int32, device=dev)
    weights = torch.empty((T * top_k,), dtype=torch.float32, device=dev)
    pos = torch.empty((T, top_k), dtype=torch.int32, device=dev)
    _lib.check(ctx._lib.oxq_moe_route_group(ctx.handle, ctx.stream(), desc(logits), top_k, 1 if norm_topk else 0,
                                            desc(idx), desc(vals), desc(offsets), desc(tokens), desc(weights),
                                            desc(pos)))
    return idx, vals, offsets, tokens, weights, pos


def gated_activation(gate_up, kind: int, limit: float = 0.0, *, out=None, ctx: Optional[Context] = None):
    """ffn_kernels.metal gated SiLU / GeLU-tanh over [.., gate | up]; moe.rs:152-173 GPT-OSS SwiGLU."""
    ctx = _ctx(ctx)
    if out is None:
        out = torch.empty(tuple(gate_up.shape[:-1]) + (gate_up.shape[-1] // 2,), dtype=gate_up.dtype,
                          device=gate_up.device)
    _lib.check(ctx._lib.oxq_gated_activation(ctx.handle, ctx.stream(), desc(gate_up), kind, float(limit),
                                             desc(out)))
    return out


def activation_mul(gate, up, kind: int, *, out=None, ctx: Optional[Context] = None):
    """metal_ops.rs:1252 silu_mul_fused / :1271 gelu_tanh_mul_fused: act(gate) * up over two tensors."""
    ctx = _ctx(ctx)
    if out is None:
        out = torch.empty_like(gate)
    _lib.check(ctx._lib.oxq_activation_mul(ctx.handle, ctx.stream(), desc(gate), desc(up), kind, desc(out)))
    return out


def silu_mul(gate, up, *, out=None, ctx: Optional[Context] = None):
    return activation_mul(gate, up, ACT_GATED_SILU, out=out, ctx=ctx)


def gelu_tanh_mul(gate, up, *, out=None, ctx: Optional[Context] = None):
    return activation_mul(gate, up, ACT_GATED_GELU_TANH, out=out, ctx=ctx)


def moe_combine(expert_out, pair_pos, top_vals, *, out=None, ctx: Optional[Context] = None):
    """moe.rs:592-605: out[t] = sum_s top_vals[t, s] * expert_out[pair_pos[t, s]]."""
    ctx = _ctx(ctx)
    if out is None:
        out = torch.empty((pair_pos.shape[0], expert_out.shape[1]), dtype=expert_out.dtype,
                          device=expert_out.device)
    _lib.check(ctx._lib.oxq_moe_combine(ctx.handle, ctx.stream(), desc(expert_out), desc(pair_pos),
                                        desc(top_vals), desc(out)))
    return out


# ---------------------------------------------------------------- layers
class PackedQuantLinear:
    """linear.rs:403-534.  Holds resident packed weights; routes by m."""

    def __init__(self, bits: int, pack_dim: int, qweight, qzeros, scales, bias=None,
                 dtype=torch.float16, ctx: Optional[Context] = None, gate_up_act: Optional[int] = None):
        """``gate_up_act`` (ACT_GATED_SILU / ACT_GATED_GELU_TANH) makes this the fused gate|up
        projection of a gated FFN (ffn.rs:386-400): forward returns act(gate) * up, [.., out/2]."""
        self.ctx = _ctx(ctx)
        self._keep = (qweight, qzeros, scales, bias)
        self.handle = C.c_void_p()
        if gate_up_act is None:
            _lib.check(self.ctx._lib.oxq_packed_quant_linear_new(
                self.ctx.handle, bits, pack_dim, desc(qweight), desc(qzeros), desc(scales), desc(bias),
                _DTYPES[dtype], C.byref(self.handle)))
        else:
            _lib.check(self.ctx._lib.oxq_packed_quant_linear_new_gate_up(
                self.ctx.handle, bits, pack_dim, desc(qweight), desc(qzeros), desc(scales), desc(bias),
                gate_up_act, _DTYPES[dtype], C.byref(self.handle)))
        k, n = C.c_int64(), C.c_int64()
        self.ctx._lib.oxq_packed_quant_linear_in_features(self.handle, C.byref(k))
        self.ctx._lib.oxq_packed_quant_linear_out_features(self.handle, C.byref(n))
        self.in_features, self.out_features = k.value, n.value
        self.weight_columns = n.value * (2 if gate_up_act is not None else 1)
        self.dtype = dtype
        flag = C.c_int()
        self.ctx._lib.oxq_packed_quant_linear_is_prepacked(self.handle, C.byref(flag))
        self.prepacked = bool(flag.value)
        if self.prepacked:          # the layer owns a tile-major copy; bias is still referenced
            self._keep = (bias,)

    def forward(self, x: torch.Tensor, out=None) -> torch.Tensor:
        if out is None:
            out = torch.empty(tuple(x.shape[:-1]) + (self.out_features,), dtype=x.dtype,
                              device=x.device)
        _lib.check(self.ctx._lib.oxq_packed_quant_linear_forward(self.handle, self.ctx.stream(),
                                                                 desc(x), desc(out)))
        return out

    def dequantize(self, out=None) -> torch.Tensor:
        """Dense [in, out] weights in the layer dtype (linear.rs:510-523)."""
        if out is None:
            dev = self._keep[0].device if self._keep[0] is not None else torch.device("cuda", self.ctx.device)
            out = torch.empty((self.in_features, self.weight_columns), dtype=self.dtype, device=dev)
        _lib.check(self.ctx._lib.oxq_packed_quant_linear_dequantize(self.handle, self.ctx.stream(),
                                                                    desc(out)))
        return out

    def __del__(self):
        try:
            if self.handle:
                self.ctx._lib.oxq_packed_quant_linear_free(self.handle)
                self.handle = C.c_void_p()
        except Exception:
            pass


class QLinear:
    """linear.rs:179-393 (GGUF fast path)."""

    def __init__(self, quant: int, weight_bytes, in_features: int, out_features: int, bias=None,
                 out_dtype=torch.bfloat16, ctx: Optional[Context] = None, gate_up_act: Optional[int] = None):
        """``gate_up_act`` (ACT_GATED_SILU / ACT_GATED_GELU_TANH) makes this the fused gate|up projection of a
        block-quantized FFN (ffn.rs:307-373 GateUpProjection::Packed): ``weight_bytes`` holds the gate rows followed
        by the up rows (``out_features`` = 2 I) and forward returns act(gate(x)) * up(x), [.., I]."""
        self.ctx = _ctx(ctx)
        self._keep = (weight_bytes, bias)
        self.handle = C.c_void_p()
        self.in_features = in_features
        self.weight_rows = out_features
        self.out_features = out_features if gate_up_act is None else out_features // 2
        if gate_up_act is None:
            _lib.check(self.ctx._lib.oxq_qlinear_new(
                self.ctx.handle, quant, desc(weight_bytes), in_features, out_features, desc(bias),
                _DTYPES[out_dtype], C.byref(self.handle)))
        else:
            _lib.check(self.ctx._lib.oxq_qlinear_new_gate_up(
                self.ctx.handle, quant, desc(weight_bytes), in_features, out_features, desc(bias), gate_up_act,
                _DTYPES[out_dtype], C.byref(self.handle)))

    def forward(self, x: torch.Tensor, out=None) -> torch.Tensor:
        if out is None:
            out = torch.empty(tuple(x.shape[:-1]) + (self.out_features,), dtype=x.dtype,
                              device=x.device)
        _lib.check(self.ctx._lib.oxq_qlinear_forward(self.handle, self.ctx.stream(), desc(x),
                                                     desc(out)))
        return out

    @property
    def resident(self) -> bool:
        """True if the layer holds the strip-major copy that 1 - 4 rows of x run on."""
        r = C.c_int(0)
        _lib.check(self.ctx._lib.oxq_qlinear_is_resident(self.handle, C.byref(r)))
        return bool(r.value)

    def dequantize(self) -> torch.Tensor:
        """Dense f32 [out_features, in_features], read from the layer's copy when it holds one."""
        out = torch.empty((self.weight_rows, self.in_features), dtype=torch.float32,
                          device=self._keep[0].device)
        _lib.check(self.ctx._lib.oxq_qlinear_dequantize(self.handle, self.ctx.stream(), desc(out)))
        return out

    def __del__(self):
        try:
            if self.handle:
                self.ctx._lib.oxq_qlinear_free(self.handle)
                self.handle = C.c_void_p()
        except Exception:
            pass


class Mxfp4Linear:
    """mxfp4.rs:67-169."""

    def __init__(self, blocks, scales, bias, in_features: int, out_features: int,
                 ctx: Optional[Context] = None):
        self.ctx = _ctx(ctx)
        self._keep = (blocks, scales, bias)
        self.handle = C.c_void_p()
        self.out_features = out_features
        _lib.check(self.ctx._lib.oxq_mxfp4_linear_new(
            self.ctx.handle, desc(blocks), desc(scales), desc(bias), in_features, out_features,
            C.byref(self.handle)))

    def forward(self, x: torch.Tensor, out=None) -> torch.Tensor:
        if out is None:
            out = torch.empty(tuple(x.shape[:-1]) + (self.out_features,), dtype=x.dtype,
                              device=x.device)
        _lib.check(self.ctx._lib.oxq_mxfp4_linear_forward(self.handle, self.ctx.stream(), desc(x),
                                                          desc(out)))
        return out

    def __del__(self):
        try:
            if self.handle:
                self.ctx._lib.oxq_mxfp4_linear_free(self.handle)
                self.handle = C.c_void_p()
        except Exception:
            pass


GATE_UP_FUSED, GATE_UP_SEPARATE, GATE_UP_SIMPLE = 0, 1, 2
_LINEAR_KINDS = {PackedQuantLinear: 0, QLinear: 1, Mxfp4Linear: 2}


class FeedForward:
    """ffn.rs:22-474 over the quantized projections: down(act(gate(x)) * up(x)).

    ``a`` is the fused gate|up projection (GATE_UP_FUSED; one built with ``gate_up_act=`` runs the
    activation in its matmul), gate_proj (GATE_UP_SEPARATE, ``b`` = up_proj) or the ungated up_proj
    (GATE_UP_SIMPLE)."""

    def __init__(self, gate_up_kind: int, a, b, down, intermediate_size: int, activation: int = ACT_GATED_SILU,
                 ctx: Optional[Context] = None):
        self.ctx = _ctx(ctx)
        self._keep = (a, b, down)
        self.handle = C.c_void_p()

        def any_linear(layer):
            if layer is None:
                return None
            kind = _LINEAR_KINDS.get(type(layer))
            if kind is None:
                raise OxqError(-1, f"FeedForward: {type(layer).__name__} is not a quantized projection")
            return C.byref(_lib.OxqAnyLinear(kind, layer.handle))

        _lib.check(self.ctx._lib.oxq_mlp_new(self.ctx.handle, gate_up_kind, any_linear(a), any_linear(b),
                                             any_linear(down), intermediate_size, activation, C.byref(self.handle)))
        k, n = C.c_int64(), C.c_int64()
        self.ctx._lib.oxq_mlp_in_features(self.handle, C.byref(k))
        self.ctx._lib.oxq_mlp_out_features(self.handle, C.byref(n))
        self.in_features, self.out_features = k.value, n.value
        self.gate_up_kind, self.intermediate_size, self.activation = gate_up_kind, intermediate_size, activation

    def scratch_elems(self, rows: int) -> int:
        e = C.c_int64()
        _lib.check(self.ctx._lib.oxq_mlp_scratch_elems(self.handle, rows, C.byref(e)))
        return e.value

    def forward(self, x: torch.Tensor, out=None, scratch=None) -> torch.Tensor:
        rows = x.numel() // max(x.shape[-1], 1)
        if scratch is None:
            scratch = torch.empty(max(self.scratch_elems(rows), 1), dtype=x.dtype, device=x.device)
        if out is None:
            out = torch.empty(tuple(x.shape[:-1]) + (self.out_features,), dtype=x.dtype, device=x.device)
        _lib.check(self.ctx._lib.oxq_mlp_forward(self.handle, self.ctx.stream(), desc(x), desc(scratch), desc(out)))
        return out

    def __del__(self):
        try:
            if self.handle:
                self.ctx._lib.oxq_mlp_free(self.handle)
                self.handle = C.c_void_p()
        except Exception:
            pass
