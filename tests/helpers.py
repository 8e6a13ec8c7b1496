"""Shared helpers for the parity tests."""
import numpy as np
import torch

import oracle
from oxydllm_amd import _lib

TORCH_DT = {oracle.F16: torch.float16, oracle.BF16: torch.bfloat16, oracle.F32: torch.float32}

# north-star tolerance: 2e-3 relative / 1e-2 absolute of the f32-accumulated reference
RTOL, ATOL = 2e-3, 1e-2


def fake(shape, dtype, device=0, contiguous=True):
    """Descriptor of a tensor that is never dereferenced (plan-only contexts)."""
    d = _lib.OxqTensor()
    d.data = 0
    d.dtype = dtype
    d.rank = len(shape)
    for i, s in enumerate(shape):
        d.dims[i] = s
    d.contiguous = 1 if contiguous else 0
    d.device = device
    return d


def to_dev(a: np.ndarray, dtype=None):
    t = torch.from_numpy(np.ascontiguousarray(a))
    if dtype is not None:
        t = t.to(dtype)
    return t.cuda()


def bits_of(t: torch.Tensor) -> np.ndarray:
    """Raw 16-bit patterns of an f16/bf16 tensor (uint16), or the f32 array."""
    t = t.detach().cpu().contiguous()
    if t.dtype in (torch.float16, torch.bfloat16):
        return t.view(torch.int16).numpy().view(np.uint16)
    return t.numpy()


def as_f32(t: torch.Tensor) -> np.ndarray:
    return t.detach().float().cpu().numpy()


# A bf16 result carries its own output rounding: half an ulp is 2^-8 relative, more
# than the 2e-3 the tolerance allows for the arithmetic.  The reference op ends with
# the same cast (`out.to_dtype(x.dtype())`, metal_ops.rs:1866), so for bf16 outputs
# the bound is widened by exactly that half ulp.  f16 (2^-11) needs no allowance.
BF16_HALF_ULP = 2.0 ** -8


def assert_close(got, ref: np.ndarray, what="", rtol=RTOL, atol=ATOL, bf16_out=None):
    if isinstance(got, torch.Tensor):
        if bf16_out is None:
            bf16_out = got.dtype == torch.bfloat16
        got = got.detach().float().cpu().numpy()
    if bf16_out:
        rtol = rtol + BF16_HALF_ULP
    got = np.asarray(got, dtype=np.float64)
    ref = np.asarray(ref, dtype=np.float64)
    assert got.shape == ref.shape, f"{what}: shape {got.shape} != {ref.shape}"
    assert np.all(np.isfinite(got)), f"{what}: non-finite output"
    err = np.abs(got - ref)
    bound = atol + rtol * np.abs(ref)
    bad = err > bound
    assert not bad.any(), (f"{what}: {bad.sum()} of {bad.size} outside {rtol} rel / {atol} abs; "
                           f"max err {err.max():.3e} at ref {ref.flat[err.argmax()]:.4f}")


def resident_rounds_weights(m: int, dt: int, gptq: bool) -> bool:
    """Whether a resident layer multiplies the dequantized weight rounded to the activation type at m
    rows (the reference's tile GEMM stages it so, mpp_gemm.metal:115-184) or unrounded (its fused GEMV,
    which serves up to 16 rows for AWQ and 32 for GPTQ, linear.rs:450-480).  f16 layers keep the
    unrounded form up to 48 rows: rounding to f16 moves a weight by 2^-12, inside the tolerance."""
    import oracle
    if m <= 16:
        return False
    if dt == oracle.F16:
        return m > 48
    return not (gptq and m <= 32)


GGUF_MATRIX_CORE_ROWS = 32


def gguf_on_matrix_cores(fmt: int, n: int, k: int, m: int, bf16: bool = True) -> bool:
    """Whether a resident bf16 QLinear of this format and shape runs m rows on its matrix-core copy: then the
    weights stay unrounded (the GEMV's arithmetic) also above 8 rows, where the reference's prefill tiles round
    them to bf16."""
    from oxydllm_amd import synth
    if not bf16 or fmt not in (synth.GGUF_Q4_0, synth.GGUF_Q8_0, synth.GGUF_Q4_K, synth.GGUF_Q6_K, synth.GGUF_Q4_1,
                               synth.GGUF_Q5_0, synth.GGUF_Q5_1, synth.GGUF_Q5_K):
        return False
    kq = fmt in (synth.GGUF_Q4_K, synth.GGUF_Q6_K, synth.GGUF_Q5_K)
    return n % 16 == 0 and k % (256 if kq else 128) == 0 and 1 <= m <= GGUF_MATRIX_CORE_ROWS


def round_x(x_f32: np.ndarray, dt: int) -> np.ndarray:
    """The activation values the kernel actually sees (x rounded to its 16-bit dtype)."""
    return oracle.round_through(x_f32, dt)


def tune(name, value, ctx=None):
    """Sets one tuning switch (``None``: back to its default) on ``ctx`` or the default context; conftest's
    autouse fixture returns the default context's switches to their defaults after every test."""
    from oxydllm_amd import ops
    (ctx if ctx is not None else ops.default_context()).set_tuning(name, value)
