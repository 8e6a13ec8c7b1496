"""GPU parity tests for the load-time transforms into the AWQ layout.

compressed_to_awq (awq.rs:187-254), concat_awq_along_out (256-323) and rtn_quantize_awq
(637-742) run as device kernels; every output tensor is compared bit for bit with the CPU
oracle, on the reference's own test constructions (awq.rs:754-835, 1032-1093) and on larger
seeded shapes, and the results are fed to the resident-layer path they exist for.
"""
import sys

import numpy as np
import pytest
import torch

import oracle
from oxydllm_amd import synth
from tests import refgen
from tests.helpers import TORCH_DT, as_f32, assert_close, bits_of, round_x, to_dev

pytestmark = pytest.mark.gpu
ops = None


def setup_module(module):
    from oxydllm_amd import ops as _ops
    module.ops = _ops


def say(msg):
    print(f"[case] {msg}", flush=True)
    sys.stdout.flush()


def host(t):
    return t.cpu().numpy()


def ct_pack(q):
    """signed int4 [out, in] -> compressed-tensors words [out, in/8] (nibble k = q[:, 8c + k] + 8)."""
    packed = np.zeros((q.shape[0], q.shape[1] // 8), np.uint32)
    for k in range(8):
        packed |= ((q[:, k::8] + 8) & 0xF).astype(np.uint32) << np.uint32(4 * k)
    return packed.view(np.int32)


@pytest.mark.parametrize("case", ["reference", "f16 1024x512 g128", "bf16 264x640 g32"])
def test_compressed_to_awq_bit_exact(case):
    say(f"compressed_to_awq {case}")
    if case == "reference":
        q, scale, packed = refgen.compressed_tensors_case()
        tdt = torch.float32
    else:
        dtn, shape, g = case.split()
        out_f, in_f = (int(v) for v in shape.split("x"))
        rng = np.random.default_rng(out_f)
        q = rng.integers(-8, 8, size=(out_f, in_f))
        scale = rng.uniform(0.002, 0.02, size=(out_f, in_f // int(g[1:]))).astype(np.float32)
        packed = ct_pack(q)
        dt = oracle.F16 if dtn == "f16" else oracle.BF16
        tdt = TORCH_DT[dt]
        scale = oracle.round_through(scale, dt)
    want = oracle.compressed_to_awq(packed, scale)
    got = ops.compressed_to_awq(to_dev(packed), to_dev(scale, tdt))
    np.testing.assert_array_equal(host(got[0]), want[0].view(np.int32))
    np.testing.assert_array_equal(host(got[1]), want[1].view(np.int32))
    np.testing.assert_array_equal(as_f32(got[2]), want[2])
    # the converted tensors behave like any AWQ checkpoint: q * scale comes back
    dq = oracle.dequantize_awq(host(got[0]), host(got[1]), as_f32(got[2]))
    expected = q.astype(np.float32) * np.repeat(scale, q.shape[1] // scale.shape[1], axis=1)
    assert np.max(np.abs(dq - expected)) < 1e-6


def test_compressed_to_awq_rejects_like_reference():
    """awq.rs:188-206."""
    say("compressed_to_awq validation")
    q, scale, packed = refgen.compressed_tensors_case()
    with pytest.raises(ops.OxqError, match="weight_scale dim0"):
        ops.compressed_to_awq(to_dev(packed), to_dev(scale[:8]))
    with pytest.raises(ops.OxqError, match="not divisible by scale groups"):
        ops.compressed_to_awq(to_dev(packed), to_dev(np.ones((16, 3), np.float32)))
    with pytest.raises(ops.OxqError, match="not divisible by pack factor"):
        ops.compressed_to_awq(to_dev(packed[:12]), to_dev(scale[:12]))


@pytest.mark.parametrize("dtn", ["f32", "f16", "bf16"])
def test_concat_awq_along_out(dtn):
    """awq.rs:1032-1093: the fused tensors dequantize to the parts' dequants stacked; and a fused
    QKV-like layer's forward equals the separate layers' outputs side by side."""
    say(f"concat_awq_along_out {dtn}")
    parts = refgen.concat_parts()
    tdt = {"f32": torch.float32, "f16": torch.float16, "bf16": torch.bfloat16}[dtn]
    dparts = [(to_dev(p[0]), to_dev(p[1]), to_dev(p[2], tdt)) for p in parts]
    got = ops.concat_awq_along_out(dparts)
    sc_parts = [as_f32(p[2]) for p in dparts]
    want = oracle.concat_awq_along_out([(p[0], p[1], s) for p, s in zip(parts, sc_parts)])
    np.testing.assert_array_equal(host(got[0]), want[0])
    np.testing.assert_array_equal(host(got[1]), want[1])
    np.testing.assert_array_equal(as_f32(got[2]), want[2])
    if dtn == "f32":
        separate = np.concatenate([oracle.dequantize_awq(*p) for p in parts], axis=0)
        np.testing.assert_array_equal(oracle.dequantize_awq(host(got[0]), host(got[1]), as_f32(got[2])), separate)
        return
    # QKV fusion at a resident-layer shape (parts of 512 + 128 + 128 columns)
    dt = oracle.F16 if dtn == "f16" else oracle.BF16
    K, g = 512, 128
    trips = [synth.awq_checkpoint(K, n, g, 4, seed=70 + i) for i, n in enumerate((512, 128, 128))]
    dtr = [(to_dev(t[0]), to_dev(t[1]), to_dev(t[2], tdt)) for t in trips]
    fused = ops.concat_awq_along_out(dtr)
    layer = ops.PackedQuantLinear(4, ops.PACK_OUT, fused[0], fused[1], fused[2], None, tdt)
    assert layer.prepacked
    x = np.random.default_rng(3).standard_normal((5, K)).astype(np.float32)
    y = layer.forward(to_dev(x, tdt))
    ref = np.concatenate([oracle.matmul_nt_f32(round_x(x, dt), oracle.dequantize_awq(
        t[0], t[1], oracle.round_through(t[2], dt))) for t in trips], axis=1)
    assert_close(y, ref, f"fused QKV {dtn}")


def test_concat_awq_rejects_like_reference():
    """awq.rs:264-289, 1095-1110."""
    say("concat validation")
    a = refgen.concat_parts(4, 4, (8,))[0]
    b = refgen.concat_parts(8, 8, (8,))[0]
    da, db = [tuple(to_dev(t) for t in p) for p in (a, b)]
    with pytest.raises(ops.OxqError, match="in_features mismatch at part 1"):
        ops.concat_awq_along_out([da, db])
    c = refgen.concat_parts(8, 4, (8,))[0]
    with pytest.raises(ops.OxqError, match="group_size mismatch at part 1"):
        ops.concat_awq_along_out([db, tuple(to_dev(t) for t in c)])
    with pytest.raises(ops.OxqError, match="no parts"):
        ops.concat_awq_along_out([])


@pytest.mark.parametrize("dtn,shape,group", [("f32", (16, 64), 32), ("f32", (264, 1024), 128), ("f16", (64, 768), 384),
                                             ("bf16", (128, 512), 64), ("f32", (8, 96), 48)])
def test_rtn_quantize_awq_bit_exact(dtn, shape, group):
    """Same integers, zeros and f32 scales as the oracle (awq.rs:637-742), including a flat
    group, a group away from zero, and groups longer than one pass of the kernel."""
    say(f"rtn_quantize_awq {dtn} {shape} g{group}")
    out_f, in_f = shape
    if shape == (16, 64):
        w = refgen.rtn_weight(out_f, in_f)           # the reference's sine weight
    else:
        w = (np.random.default_rng(out_f + in_f).standard_normal(shape) * 0.05).astype(np.float32)
    w[3, :group] = 0.0
    w[5, -group:] = np.abs(w[5, -group:]) + 1.0
    tdt = {"f32": torch.float32, "f16": torch.float16, "bf16": torch.bfloat16}[dtn]
    if dtn != "f32":
        w = oracle.round_through(w, oracle.F16 if dtn == "f16" else oracle.BF16)
    want = oracle.rtn_quantize_awq(w, group)
    got = ops.rtn_quantize_awq(to_dev(w, tdt), group)
    np.testing.assert_array_equal(host(got[0]), want[0].view(np.int32))
    np.testing.assert_array_equal(host(got[1]), want[1].view(np.int32))
    np.testing.assert_array_equal(host(got[2]).view(np.uint32), want[2].view(np.uint32))
    dq = oracle.dequantize_awq(host(got[0]), host(got[1]), host(got[2]))
    rel = np.sqrt(((dq - w).astype(np.float64) ** 2).sum() / (w.astype(np.float64) ** 2).sum())
    assert rel < 0.12   # the reference asks 5 % of its smooth sine weight; Gaussian groups sit near 9 %


def test_rtn_quantized_lm_head_runs_on_the_resident_layer():
    """loader.rs:1060-1076: a tied lm_head is quantized at load and served by the packed layer."""
    say("rtn -> PackedQuantLinear")
    out_f, in_f, g = 1024, 512, 128
    w = (np.random.default_rng(8).standard_normal((out_f, in_f)) * 0.03).astype(np.float32)
    qw, qz, sc = ops.rtn_quantize_awq(to_dev(w, torch.bfloat16), g)
    layer = ops.PackedQuantLinear(4, ops.PACK_OUT, qw, qz, sc.to(torch.bfloat16), None, torch.bfloat16)
    assert layer.prepacked
    x = np.random.default_rng(9).standard_normal((3, in_f)).astype(np.float32)
    y = layer.forward(to_dev(x, torch.bfloat16))
    dq = oracle.dequantize_awq(host(qw), host(qz), oracle.round_through(host(sc), oracle.BF16))
    assert_close(y, oracle.matmul_nt_f32(round_x(x, oracle.BF16), dq), "rtn lm_head forward")
    dense = oracle.matmul_nt_f32(round_x(x, oracle.BF16), oracle.round_through(w, oracle.BF16))
    assert np.abs(as_f32(y) - dense).max() < 0.15 * np.abs(dense).max()


def test_rtn_rejects_like_reference():
    """awq.rs:644-654."""
    say("rtn validation")
    w = to_dev(np.zeros((12, 64), np.float32))
    with pytest.raises(ops.OxqError, match="must be a multiple of 8"):
        ops.rtn_quantize_awq(w, 32)
    with pytest.raises(ops.OxqError, match="not divisible by group_size"):
        ops.rtn_quantize_awq(to_dev(np.zeros((16, 64), np.float32)), 48)


@pytest.mark.parametrize("fmt", [synth.GGUF_Q4_K, synth.GGUF_Q8_0, synth.GGUF_Q5_0, synth.GGUF_Q3_K])
def test_gguf_depermute_qk_rows(fmt):
    """gguf_weights.rs:255-291, 363-405: bytes equal to the oracle's shuffle; the de-interleaved
    tensor dequantizes to the HF-ordered rows; bad geometry is rejected as the reference does."""
    say(f"depermute_qk_rows {synth.GGUF_NAMES[fmt]}")
    n_heads, head_dim, k = 4, 64, 512
    n = n_heads * head_dim
    elems, bbytes = synth.GGUF_BLOCK_LAYOUT[fmt]
    row_bytes = k // elems * bbytes
    hf = synth.gguf_weight(fmt, n, k, seed=31 + fmt).reshape(n, row_bytes)
    permuted = hf.reshape(n_heads, 2, head_dim // 2, row_bytes).swapaxes(1, 2).reshape(-1).copy()
    got = ops.gguf_depermute_qk_rows(to_dev(permuted), k, n, fmt, n_heads, head_dim)
    np.testing.assert_array_equal(host(got), oracle.gguf_depermute_qk_rows(permuted, row_bytes, n_heads, head_dim))
    np.testing.assert_array_equal(host(got).reshape(n, row_bytes), hf)
    np.testing.assert_array_equal(host(ops.gguf_dequantize(got, k, n, fmt)),
                                  oracle.dequantize_gguf(fmt, hf.reshape(-1), n, k))
    with pytest.raises(ops.OxqError, match="incompatible with 3 heads x 64 dims"):
        ops.gguf_depermute_qk_rows(to_dev(permuted), k, n, fmt, 3, 64)
    with pytest.raises(ops.OxqError, match="incompatible with 4 heads x 63 dims"):
        ops.gguf_depermute_qk_rows(to_dev(permuted), k, n, fmt, 4, 63)
