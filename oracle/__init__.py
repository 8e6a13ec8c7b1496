"""ctypes binding of the CPU oracle (``oracle/oxq_oracle.c``).

TEST INFRASTRUCTURE ONLY: imported by ``tests/``, ``__graft_entry__.smoke()``
and the ``cpu_baseline`` leg of ``bench.py``.  The shipped package
(``oxydllm_amd``) never imports this module and has no CPU fallback.

All functions take and return numpy arrays; layouts follow the reference
(``src/common/awq.rs``, ``src/common/mxfp4.rs``, ggml block formats).
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboxq_oracle.so")

F32, F16, BF16 = 0, 1, 2
Q4_0, Q8_0, Q4_K, Q6_K, Q4_1, Q5_0, Q5_1, Q2_K, Q3_K, Q5_K = range(10)
GGUF_BLOCK_LAYOUT = {Q4_0: (32, 18), Q8_0: (32, 34), Q4_K: (256, 144), Q6_K: (256, 210),
                     Q4_1: (32, 20), Q5_0: (32, 22), Q5_1: (32, 24), Q2_K: (256, 84),
                     Q3_K: (256, 110), Q5_K: (256, 176)}


def build(force: bool = False) -> str:
    """Compile the oracle with gcc (``make -C oracle``)."""
    src = os.path.join(_HERE, "oxq_oracle.c")
    stale = (not os.path.exists(_LIB_PATH)
             or os.path.getmtime(_LIB_PATH) < os.path.getmtime(src))
    if force or stale:
        if force and os.path.exists(_LIB_PATH):
            os.remove(_LIB_PATH)
        subprocess.check_call(["make", "-C", _HERE, "-s"])
    return _LIB_PATH


_lib = None


def lib() -> C.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        _lib = C.CDLL(_LIB_PATH)
        _lib.orc_f32_to_f16.restype = C.c_uint16
        _lib.orc_f32_to_f16.argtypes = [C.c_float]
        _lib.orc_f32_to_bf16.restype = C.c_uint16
        _lib.orc_f32_to_bf16.argtypes = [C.c_float]
        _lib.orc_f16_to_f32.restype = C.c_float
        _lib.orc_f16_to_f32.argtypes = [C.c_uint16]
        _lib.orc_bf16_to_f32.restype = C.c_float
        _lib.orc_bf16_to_f32.argtypes = [C.c_uint16]
    return _lib


def _p(a: np.ndarray):
    return a.ctypes.data_as(C.c_void_p)


def _u32(a) -> np.ndarray:
    """Accept i32 / u32 / i64 packed tensors like read_packed_to_u32 (awq.rs:158-179)."""
    a = np.asarray(a)
    if a.dtype == np.int32:
        a = a.view(np.uint32)
    elif a.dtype == np.int64:
        a = a.astype(np.uint32)  # `as u32` truncation
    elif a.dtype != np.uint32:
        raise TypeError(f"Unsupported packed tensor dtype {a.dtype} (expected I32/U32/I64)")
    return np.ascontiguousarray(a)


def _f32(a) -> np.ndarray:
    return np.ascontiguousarray(np.asarray(a, dtype=np.float32))


def _check(rc: int, what: str):
    if rc != 0:
        raise ValueError(f"oracle {what}: error code {rc}")


# ---------------------------------------------------------------- conversions
def convert_f32(a, dtype: int) -> np.ndarray:
    """f32 -> raw bits in `dtype` (uint16 for F16/BF16, float32 for F32), RNE."""
    a = _f32(a)
    out = np.empty(a.shape, dtype=np.float32 if dtype == F32 else np.uint16)
    lib().orc_convert_f32(_p(a), _p(out), C.c_size_t(a.size), C.c_int(dtype))
    return out


def widen_to_f32(bits, dtype: int) -> np.ndarray:
    bits = np.ascontiguousarray(bits)
    out = np.empty(bits.shape, dtype=np.float32)
    lib().orc_widen_to_f32(_p(bits), _p(out), C.c_size_t(bits.size), C.c_int(dtype))
    return out


def round_through(a, dtype: int) -> np.ndarray:
    """f32 -> dtype -> f32 (what a 16-bit tensor holds, as f32)."""
    return widen_to_f32(convert_f32(a, dtype), dtype)


# ---------------------------------------------------------------- AWQ / GPTQ
def dequantize_awq(qweight, qzeros, scales) -> np.ndarray:
    """AWQ 4-bit -> [N, K] f32 (awq.rs:325-440)."""
    qweight, qzeros, scales = _u32(qweight), _u32(qzeros), _f32(scales)
    K, packed_out = qweight.shape
    groups, N = scales.shape
    if N % 8 or packed_out != N // 8:
        raise ValueError(f"AWQ qweight dim1 ({packed_out}) != out_features/8 ({N // 8})")
    if groups == 0 or K % groups:
        raise ValueError(f"quant in_features ({K}) not divisible by scales groups ({groups})")
    if qzeros.shape != (groups, packed_out):
        raise ValueError(f"AWQ qzeros shape {qzeros.shape} != [{groups}, {packed_out}]")
    out = np.empty((N, K), dtype=np.float32)
    _check(lib().orc_dequantize_awq(_p(qweight), _p(qzeros), _p(scales), C.c_int64(K),
                                    C.c_int64(N), C.c_int64(K // groups), _p(out)), "awq")
    return out


def gguf_depermute_qk_rows(data, row_bytes: int, n_heads: int, head_dim: int) -> np.ndarray:
    """gguf_weights.rs:255-291: HF row r of a head is read from interleaved row 2 (r % half) + r / half."""
    rows = np.ascontiguousarray(np.asarray(data, dtype=np.uint8)).reshape(n_heads * head_dim, row_bytes)
    if head_dim % 2:
        raise ValueError("depermute_qk_rows: odd head_dim")
    half = head_dim // 2
    r = np.arange(head_dim)
    src = (np.arange(n_heads)[:, None] * head_dim + 2 * (r % half) + r // half).reshape(-1)
    return rows[src].reshape(-1)


def cast_f8e4m3_to_f32(bytes_) -> np.ndarray:
    """metal_ops.rs:2942-2955: spec decode of E4M3fn bytes."""
    b = np.ascontiguousarray(np.asarray(bytes_, dtype=np.uint8))
    out = np.empty(b.shape, np.float32)
    lib().orc_cast_f8e4m3_to_f32(_p(b), _p(out), C.c_size_t(b.size))
    return out


def f8_block_dequant_bf16(bytes_, scales) -> np.ndarray:
    """quant_kernels.metal:3877-3911: bf16 bits [rows, cols] of bf16(f32(bf16(f8)) * scale)."""
    b = np.ascontiguousarray(np.asarray(bytes_, dtype=np.uint8))
    sc = _f32(scales)
    rows, cols = b.shape
    out = np.empty((rows, cols), np.uint16)
    _check(lib().orc_f8_block_dequant_bf16(_p(b), _p(sc), C.c_int64(rows), C.c_int64(cols),
                                           C.c_int64(sc.shape[0]), C.c_int64(sc.shape[1]), _p(out)), "f8_block_dequant")
    return out


def compressed_to_awq(weight_packed, weight_scale):
    """awq.rs:187-254: compressed-tensors int4 [out, in/8] + scales [out, groups] ->
    AWQ (qweight [in, out/8], qzeros [groups, out/8], scales f32 [groups, out])."""
    ct, sc = _u32(weight_packed), _f32(weight_scale)
    out_f, packed_in = ct.shape
    groups = sc.shape[1]
    if sc.shape[0] != out_f:
        raise ValueError("weight_scale dim0 != weight_packed out_features")
    in_f = packed_in * 8
    qweight = np.empty((in_f, out_f // 8), np.uint32)
    qzeros = np.empty((groups, out_f // 8), np.uint32)
    scales = np.empty((groups, out_f), np.float32)
    _check(lib().orc_compressed_to_awq(_p(ct), _p(sc), C.c_int64(out_f), C.c_int64(in_f), C.c_int64(groups),
                                       _p(qweight), _p(qzeros), _p(scales)), "compressed_to_awq")
    return qweight, qzeros, scales


def concat_awq_along_out(parts):
    """awq.rs:256-323: parts = [(qweight, qzeros, scales), ...] sharing in_features and groups."""
    if not parts:
        raise ValueError("concat_awq_along_out: no parts")
    k, g = parts[0][0].shape[0], parts[0][2].shape[0]
    for qw, qz, sc in parts[1:]:
        if qw.shape[0] != k:
            raise ValueError("AWQ fuse: in_features mismatch")
        if sc.shape[0] != g:
            raise ValueError("AWQ fuse: group_size mismatch")
    return tuple(np.concatenate([p[i] for p in parts], axis=1) for i in range(3))


def rtn_quantize_awq(weight, group_size: int):
    """awq.rs:637-742: dense [out, in] -> AWQ 4-bit (qweight, qzeros, scales f32)."""
    w = _f32(weight)
    out_f, in_f = w.shape
    if out_f % 8 or group_size <= 0 or in_f % group_size:
        raise ValueError("rtn_quantize_awq: shape not divisible")
    groups = in_f // group_size
    qweight = np.empty((in_f, out_f // 8), np.uint32)
    qzeros = np.empty((groups, out_f // 8), np.uint32)
    scales = np.empty((groups, out_f), np.float32)
    _check(lib().orc_rtn_quantize_awq(_p(w), C.c_int64(out_f), C.c_int64(in_f), C.c_int64(group_size),
                                      _p(qweight), _p(qzeros), _p(scales)), "rtn_quantize_awq")
    return qweight, qzeros, scales


def dequantize_awq8(qweight, qzeros, scales) -> np.ndarray:
    """AWQ-layout 8-bit (identity slot order) -> [N, K] f32."""
    qweight, qzeros, scales = _u32(qweight), _u32(qzeros), _f32(scales)
    K, packed_out = qweight.shape
    groups, N = scales.shape
    if N % 4 or packed_out != N // 4 or qzeros.shape != (groups, packed_out) or K % groups:
        raise ValueError("AWQ-8 shape mismatch")
    out = np.empty((N, K), dtype=np.float32)
    _check(lib().orc_dequantize_awq8(_p(qweight), _p(qzeros), _p(scales), C.c_int64(K),
                                     C.c_int64(N), C.c_int64(K // groups), _p(out)), "awq8")
    return out


def dequantize_gptq(qweight, qzeros, scales, bits: int, sym: bool = False) -> np.ndarray:
    """GPTQ 4/8-bit -> [N, K] f32 (awq.rs:442-590)."""
    if bits not in (4, 8):
        raise ValueError(f"dequantize_gptq: only 4/8-bit supported, got {bits}")
    qweight, scales = _u32(qweight), _f32(scales)
    pf = 32 // bits
    packed_in, N = qweight.shape
    K = packed_in * pf
    groups, n_s = scales.shape
    if n_s != N:
        raise ValueError(f"GPTQ scales shape {scales.shape} != [{groups}, {N}]")
    if groups == 0 or K % groups:
        raise ValueError(f"quant in_features ({K}) not divisible by scales groups ({groups})")
    if N % pf:
        raise ValueError(f"GPTQ out_features {N} not divisible by pack_factor {pf}")
    qz_ptr = None
    if qzeros is not None:
        qzeros = _u32(qzeros)
        if qzeros.shape != (groups, N // pf):
            raise ValueError(f"GPTQ qzeros shape {qzeros.shape} != [{groups}, {N // pf}]")
        qz_ptr = _p(qzeros)
    out = np.empty((N, K), dtype=np.float32)
    _check(lib().orc_dequantize_gptq(_p(qweight), qz_ptr, _p(scales), C.c_int(bits),
                                     C.c_int(1 if sym else 0), C.c_int64(K), C.c_int64(N),
                                     C.c_int64(K // groups), _p(out)), "gptq")
    return out


def transpose_convert(w_nk, dtype: int) -> np.ndarray:
    """[N,K] f32 -> [K,N] raw bits in dtype: the GPU dequant ops' output layout."""
    w_nk = _f32(w_nk)
    N, K = w_nk.shape
    out = np.empty((K, N), dtype=np.float32 if dtype == F32 else np.uint16)
    lib().orc_transpose_convert(_p(w_nk), C.c_int64(N), C.c_int64(K), _p(out), C.c_int(dtype))
    return out


# ---------------------------------------------------------------- MXFP4 / GGUF
def dequantize_mxfp4_f32(blocks, scales, rows: int, cols: int) -> np.ndarray:
    blocks = np.ascontiguousarray(np.asarray(blocks, dtype=np.uint8)).reshape(-1)
    scales = np.ascontiguousarray(np.asarray(scales, dtype=np.uint8)).reshape(-1)
    out = np.empty((rows, cols), dtype=np.float32)
    rc = lib().orc_dequantize_mxfp4_f32(_p(blocks), C.c_size_t(blocks.size), _p(scales),
                                        C.c_size_t(scales.size), C.c_int64(rows),
                                        C.c_int64(cols), _p(out))
    if rc != 0:
        raise ValueError(f"MXFP4: buffer sizes (blocks {blocks.size}, scales {scales.size}) "
                         f"don't match [{rows}, {cols}]")
    return out


def dequantize_gguf(fmt: int, data, N: int, K: int) -> np.ndarray:
    data = np.ascontiguousarray(np.asarray(data, dtype=np.uint8)).reshape(-1)
    out = np.empty((N, K), dtype=np.float32)
    _check(lib().orc_dequantize_gguf(C.c_int(fmt), _p(data), C.c_size_t(data.size),
                                     C.c_int64(N), C.c_int64(K), _p(out)), "gguf")
    return out


# ---------------------------------------------------------------- matmul
def matmul_nt_f32(x, w, bias=None) -> np.ndarray:
    """y[M,N] = x[M,K] . w[N,K]^T (+ bias), sequential f32 accumulation."""
    x, w = _f32(x), _f32(w)
    M, K = x.shape
    N, K2 = w.shape
    assert K == K2
    b = _f32(bias) if bias is not None else None
    y = np.empty((M, N), dtype=np.float32)
    lib().orc_matmul_nt_f32(_p(x), _p(w), _p(b) if b is not None else None, _p(y),
                            C.c_int64(M), C.c_int64(K), C.c_int64(N))
    return y


def matmul_nt_f64acc(x, w, bias=None) -> np.ndarray:
    x, w = _f32(x), _f32(w)
    M, K = x.shape
    N, _ = w.shape
    b = _f32(bias) if bias is not None else None
    y = np.empty((M, N), dtype=np.float32)
    lib().orc_matmul_nt_f64acc(_p(x), _p(w), _p(b) if b is not None else None, _p(y),
                               C.c_int64(M), C.c_int64(K), C.c_int64(N))
    return y


# ---------------------------------------------------------------- MoE caller
def moe_route(logits, top_k: int, norm_topk: bool = True):
    logits = _f32(logits)
    T, E = logits.shape
    idx = np.empty((T, top_k), dtype=np.uint32)
    vals = np.empty((T, top_k), dtype=np.float32)
    _check(lib().orc_moe_route(_p(logits), C.c_int64(T), C.c_int64(E), C.c_int64(top_k),
                               C.c_int(1 if norm_topk else 0), _p(idx), _p(vals)), "moe_route")
    return idx, vals


def moe_group(top_idx, top_vals, num_experts: int):
    top_idx = np.ascontiguousarray(np.asarray(top_idx, dtype=np.uint32))
    top_vals = _f32(top_vals)
    T, k = top_idx.shape
    offsets = np.empty(num_experts + 1, dtype=np.int64)
    tokens = np.empty(T * k, dtype=np.uint32)
    weights = np.empty(T * k, dtype=np.float32)
    _check(lib().orc_moe_group(_p(top_idx), _p(top_vals), C.c_int64(T), C.c_int64(num_experts),
                               C.c_int64(k), _p(offsets), _p(tokens), _p(weights)), "moe_group")
    return offsets, tokens, weights


def gpt_oss_swiglu(gu, limit: float) -> np.ndarray:
    gu = _f32(gu)
    M, two_i = gu.shape
    h = np.empty((M, two_i // 2), dtype=np.float32)
    lib().orc_gpt_oss_swiglu(_p(gu), C.c_int64(M), C.c_int64(two_i // 2), C.c_float(limit), _p(h))
    return h


def gated_silu(gu) -> np.ndarray:
    gu = _f32(gu)
    M, two_i = gu.shape
    out = np.empty((M, two_i // 2), dtype=np.float32)
    lib().orc_gated_silu(_p(gu), C.c_int64(M), C.c_int64(two_i // 2), _p(out))
    return out


def gated_gelu_tanh(gu) -> np.ndarray:
    gu = _f32(gu)
    M, two_i = gu.shape
    out = np.empty((M, two_i // 2), dtype=np.float32)
    lib().orc_gated_gelu_tanh(_p(gu), C.c_int64(M), C.c_int64(two_i // 2), _p(out))
    return out


def moe_combine(expert_out, offsets, tokens, weights, n_tokens: int) -> np.ndarray:
    expert_out = _f32(expert_out)
    offsets = np.ascontiguousarray(np.asarray(offsets, dtype=np.int64))
    tokens = np.ascontiguousarray(np.asarray(tokens, dtype=np.uint32))
    weights = _f32(weights)
    P, H = expert_out.shape
    out = np.empty((n_tokens, H), dtype=np.float32)
    lib().orc_moe_combine(_p(expert_out), _p(offsets), _p(tokens), _p(weights), C.c_int64(len(offsets) - 1),
                          C.c_int64(n_tokens), C.c_int64(H), _p(out))
    return out
