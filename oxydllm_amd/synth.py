"""Synthetic packed-quant checkpoints in the on-disk layouts the kernels consume.

Host-side numpy only.  Packers follow the layouts of the reference
(``src/common/awq.rs:1-17, 23``; ``src/common/mxfp4.rs:1-9``; ggml block
structs in ``src/common/quant_kernels.metal:792-795, 1100-1103, 1228-1233,
1681-1686``).  The seeded generators reproduce the value distributions the
benchmark configurations are stated on.
"""
from __future__ import annotations

import numpy as np

AWQ_PACK_ORDER = (0, 2, 4, 6, 1, 3, 5, 7)

GGUF_Q4_0, GGUF_Q8_0, GGUF_Q4_K, GGUF_Q6_K = 0, 1, 2, 3
GGUF_Q4_1, GGUF_Q5_0, GGUF_Q5_1, GGUF_Q2_K, GGUF_Q3_K, GGUF_Q5_K = 4, 5, 6, 7, 8, 9
GGUF_BLOCK_LAYOUT = {GGUF_Q4_0: (32, 18), GGUF_Q8_0: (32, 34),
                     GGUF_Q4_K: (256, 144), GGUF_Q6_K: (256, 210),
                     GGUF_Q4_1: (32, 20), GGUF_Q5_0: (32, 22), GGUF_Q5_1: (32, 24),
                     GGUF_Q2_K: (256, 84), GGUF_Q3_K: (256, 110), GGUF_Q5_K: (256, 176)}
GGUF_NAMES = {GGUF_Q4_0: "Q4_0", GGUF_Q8_0: "Q8_0", GGUF_Q4_K: "Q4_K", GGUF_Q6_K: "Q6_K",
              GGUF_Q4_1: "Q4_1", GGUF_Q5_0: "Q5_0", GGUF_Q5_1: "Q5_1", GGUF_Q2_K: "Q2_K",
              GGUF_Q3_K: "Q3_K", GGUF_Q5_K: "Q5_K"}
# byte offsets of the f16 fields (d, then m / dmin where the format has one) in a block
GGUF_F16_FIELDS = {GGUF_Q4_0: (0,), GGUF_Q8_0: (0,), GGUF_Q4_K: (0, 2), GGUF_Q6_K: (208,),
                   GGUF_Q4_1: (0, 2), GGUF_Q5_0: (0,), GGUF_Q5_1: (0, 2), GGUF_Q2_K: (80, 82),
                   GGUF_Q3_K: (108,), GGUF_Q5_K: (0, 2)}


# ------------------------------------------------------------------ packers
def pack_awq(values: np.ndarray) -> np.ndarray:
    """[rows, N] 4-bit values -> int32 [rows, N/8]; slot k holds column 8j+ORDER[k]."""
    values = np.asarray(values)
    rows, n = values.shape
    assert n % 8 == 0
    v = (values.astype(np.uint32) & 0xF).reshape(rows, n // 8, 8)
    word = np.zeros((rows, n // 8), dtype=np.uint32)
    for k, off in enumerate(AWQ_PACK_ORDER):
        word |= v[:, :, off] << np.uint32(4 * k)
    return word.view(np.int32)


def pack_awq_8bit(values: np.ndarray) -> np.ndarray:
    """[rows, N] 8-bit values -> int32 [rows, N/4]; slot k holds column 4j+k."""
    values = np.asarray(values)
    rows, n = values.shape
    assert n % 4 == 0
    v = (values.astype(np.uint32) & 0xFF).reshape(rows, n // 4, 4)
    word = np.zeros((rows, n // 4), dtype=np.uint32)
    for k in range(4):
        word |= v[:, :, k] << np.uint32(8 * k)
    return word.view(np.int32)


def pack_gptq_qweight(values: np.ndarray, bits: int) -> np.ndarray:
    """[K, N] values -> int32 [K/pf, N]; slot s of word (iw, n) holds k = iw*pf + s."""
    values = np.asarray(values)
    k, n = values.shape
    pf = 32 // bits
    assert k % pf == 0
    mask = np.uint32((1 << bits) - 1)
    v = (values.astype(np.uint32) & mask).reshape(k // pf, pf, n)
    word = np.zeros((k // pf, n), dtype=np.uint32)
    for s in range(pf):
        word |= v[:, s, :] << np.uint32(bits * s)
    return word.view(np.int32)


def pack_gptq_qzeros(values: np.ndarray, bits: int) -> np.ndarray:
    """[G, N] stored zero-points -> int32 [G, N/pf]; slot n%pf of word n/pf."""
    values = np.asarray(values)
    g, n = values.shape
    pf = 32 // bits
    assert n % pf == 0
    mask = np.uint32((1 << bits) - 1)
    v = (values.astype(np.uint32) & mask).reshape(g, n // pf, pf)
    word = np.zeros((g, n // pf), dtype=np.uint32)
    for s in range(pf):
        word |= v[:, :, s] << np.uint32(bits * s)
    return word.view(np.int32)


# ------------------------------------------------------------------ seeded configs
def _rng(seed: int) -> np.random.Generator:
    return np.random.Generator(np.random.PCG64(seed))


def awq_checkpoint(K: int, N: int, group_size: int, bits: int = 4, seed: int = 0):
    """Uniform ints in [0, 2^bits), f32 scales ~ U(0.002, 0.02) (cast by the caller).

    Returns (qweight i32, qzeros i32, scales f32 [G,N]).
    """
    r = _rng(seed)
    g = K // group_size
    hi = 1 << bits
    q = r.integers(0, hi, size=(K, N), dtype=np.uint8 if bits == 8 else np.uint8)
    z = r.integers(0, hi, size=(g, N), dtype=np.uint8)
    s = r.uniform(0.002, 0.02, size=(g, N)).astype(np.float32)
    if bits == 4:
        return pack_awq(q), pack_awq(z), s
    return pack_awq_8bit(q), pack_awq_8bit(z), s


def gptq_checkpoint(K: int, N: int, group_size: int, bits: int, seed: int = 0):
    """GPTQ sequential packing; qzeros hold (zero_point - 1) as auto-gptq stores them."""
    r = _rng(seed)
    g = K // group_size
    hi = 1 << bits
    q = r.integers(0, hi, size=(K, N), dtype=np.uint8)
    zp = r.integers(1, hi + 1, size=(g, N), dtype=np.uint16)  # true zero-point in [1, 2^bits]
    s = r.uniform(0.002, 0.02, size=(g, N)).astype(np.float32)
    return pack_gptq_qweight(q, bits), pack_gptq_qzeros(zp - 1, bits), s


def gguf_weight(fmt: int, N: int, K: int, seed: int = 0) -> np.ndarray:
    """Random GGUF block bytes: quant bits uniform, f16 d/dmin ~ U(1e-3, 2e-2)."""
    r = _rng(seed)
    elems, bbytes = GGUF_BLOCK_LAYOUT[fmt]
    nb = N * (K // elems)
    blk = r.integers(0, 256, size=(nb, bbytes), dtype=np.uint8)

    def f16_bytes(n):
        return r.uniform(1e-3, 2e-2, size=n).astype(np.float16).view(np.uint8).reshape(n, 2)

    for off in GGUF_F16_FIELDS[fmt]:
        blk[:, off:off + 2] = f16_bytes(nb)
    return blk.reshape(-1)


def mxfp4_weight(N: int, K: int, seed: int = 0, exp_lo: int = 118, exp_hi: int = 126):
    """blocks u8 [N*K/32*16] uniform, scales u8 [N*K/32] uniform in [exp_lo, exp_hi]."""
    r = _rng(seed)
    nb = K // 32
    blocks = r.integers(0, 256, size=N * nb * 16, dtype=np.uint8)
    scales = r.integers(exp_lo, exp_hi + 1, size=N * nb, dtype=np.uint8)
    return blocks, scales
