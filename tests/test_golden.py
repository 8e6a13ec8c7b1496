"""The committed fixtures in tests/golden/ (written by tests/golden/make_fixtures.py).

CPU part: the oracle reproduces every stored expected output bit for bit, and the stored
known answers agree with the reference's own closed forms where it has them.
GPU part (marked gpu): the HIP library on the stored inputs - dequantized tiles and transform
outputs bit for bit, products within 2e-3 relative + 1e-2 absolute of the stored
f32-accumulated result (half a bf16 ulp more for bf16 outputs).
"""
import glob
import os
import sys

import numpy as np
import pytest

import oracle
from oxydllm_amd import synth

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def load(name):
    with np.load(os.path.join(GOLDEN, name + ".npz"), allow_pickle=False) as z:
        return {k: z[k] for k in z.files}


def say(msg):
    print(f"[case] {msg}", flush=True)
    sys.stdout.flush()


GGUF = [synth.GGUF_NAMES[f].lower() for f in sorted(synth.GGUF_NAMES)]


# ------------------------------------------------------------------ CPU: oracle == fixtures
def test_fixture_inventory():
    names = sorted(os.path.basename(p)[:-4] for p in glob.glob(os.path.join(GOLDEN, "*.npz")))
    assert len(names) == 24 and all(("gguf_" + g) in names for g in GGUF)


def test_oracle_reproduces_dequant_fixtures():
    f = load("awq4_kat")
    got = oracle.dequantize_awq(f["qweight"], f["qzeros"], f["scales"])
    np.testing.assert_array_equal(got, f["dequant_nk"])
    assert np.max(np.abs(f["dequant_nk"] - f["reference_nk"])) < 1e-6          # awq.rs:1004-1009
    for bits in (4, 8):
        f = load(f"gptq{bits}_kat")
        np.testing.assert_array_equal(oracle.dequantize_gptq(f["qweight"], f["qzeros"], f["scales"], bits),
                                      f["dequant_nk"])
        assert np.max(np.abs(f["dequant_nk"] - f["reference_nk"])) < 1e-5      # awq.rs:1220-1226
    f = load("mxfp4_case")
    np.testing.assert_array_equal(oracle.dequantize_mxfp4_f32(f["blocks"], f["scales"], 10, 64), f["dequant_nk"])
    f = load("f8_block_dequant")
    np.testing.assert_array_equal(oracle.f8_block_dequant_bf16(f["bytes"], f["scales"]), f["dequant_bf16_bits"])
    got = oracle.cast_f8e4m3_to_f32(np.arange(256, dtype=np.uint8))
    np.testing.assert_array_equal(got.view(np.uint32), f["all_bytes_f32"].view(np.uint32))


@pytest.mark.parametrize("name", GGUF)
def test_oracle_reproduces_gguf_fixtures(name):
    f = load("gguf_" + name)
    fmt, n, k = int(f["fmt"][0]), int(f["n"][0]), int(f["k"][0])
    np.testing.assert_array_equal(oracle.dequantize_gguf(fmt, f["weight_bytes"], n, k), f["dequant_nk"])
    np.testing.assert_array_equal(oracle.matmul_nt_f32(f["x"], f["dequant_nk"]), f["y_f32"])


def test_oracle_reproduces_matmul_transform_and_routing_fixtures():
    for name, dt in (("awq4_matmul_f16", oracle.F16), ("awq4_matmul_bf16", oracle.BF16),
                     ("awq8_matmul_f16", oracle.F16), ("awq8_matmul_bf16", oracle.BF16)):
        f = load(name)
        deq = oracle.dequantize_awq if name.startswith("awq4") else oracle.dequantize_awq8
        w = deq(f["qweight"], f["qzeros"], oracle.round_through(f["scales"], dt))
        np.testing.assert_array_equal(oracle.transpose_convert(w, dt), f["dequant_kn_bits"])
        np.testing.assert_array_equal(oracle.matmul_nt_f32(oracle.round_through(f["x"], dt), w), f["y"])
    for bits in (4, 8):
        f = load(f"gptq{bits}_matmul_bf16")
        w = oracle.dequantize_gptq(f["qweight"], f["qzeros"], oracle.round_through(f["scales"], oracle.BF16), bits)
        np.testing.assert_array_equal(oracle.transpose_convert(w, oracle.BF16), f["dequant_kn_bits"])
    f = load("compressed_to_awq")
    got = oracle.compressed_to_awq(f["weight_packed"], f["weight_scale"])
    for g, k in zip(got, ("qweight", "qzeros", "scales")):
        np.testing.assert_array_equal(g, f[k])
    f = load("rtn_quantize_awq")
    got = oracle.rtn_quantize_awq(f["weight"], int(f["group_size"][0]))
    for g, k in zip(got, ("qweight", "qzeros", "scales")):
        np.testing.assert_array_equal(g, f[k])
    f = load("moe_route_group")
    idx, vals = oracle.moe_route(f["logits"], 4, True)
    np.testing.assert_array_equal(idx, f["top_idx"])
    np.testing.assert_array_equal(vals, f["top_vals"])
    off, tok, wts = oracle.moe_group(idx, vals, 32)
    np.testing.assert_array_equal(off, f["offsets"])
    np.testing.assert_array_equal(tok, f["tokens"])
    np.testing.assert_array_equal(wts, f["weights"])


# ------------------------------------------------------------------ GPU: library == fixtures
def _gpu():
    import torch

    from oxydllm_amd import ops
    from tests.helpers import TORCH_DT, as_f32, assert_close, bits_of, to_dev
    return torch, ops, TORCH_DT, as_f32, assert_close, bits_of, to_dev


@pytest.mark.gpu
@pytest.mark.parametrize("name,bits,pack,dt", [("awq4_matmul_f16", 4, "out", oracle.F16),
                                               ("awq4_matmul_bf16", 4, "out", oracle.BF16),
                                               ("awq8_matmul_f16", 8, "out", oracle.F16),
                                               ("awq8_matmul_bf16", 8, "out", oracle.BF16),
                                               ("gptq4_matmul_bf16", 4, "in", oracle.BF16),
                                               ("gptq8_matmul_bf16", 8, "in", oracle.BF16)])
def test_gpu_int_layers_match_fixtures(name, bits, pack, dt):
    torch, ops, TORCH_DT, as_f32, assert_close, bits_of, to_dev = _gpu()
    say(f"golden {name}")
    f = load(name)
    tdt = TORCH_DT[dt]
    qw, qz, sc = to_dev(f["qweight"]), to_dev(f["qzeros"]), to_dev(f["scales"], tdt)
    x = to_dev(f["x"], tdt)
    if pack == "out":
        dq = ops.dequantize_w4(qw, qz, sc) if bits == 4 else ops.dequantize_w8(qw, qz, sc)
        y = ops.w4a16_matmul(x, qw, qz, sc) if bits == 4 else ops.w8a16_matmul(x, qw, qz, sc)
    else:
        dq = ops.dequantize_gptq_packed(qw, qz, sc, bits)
        y = ops.gptq_matmul(x, qw, qz, sc, bits)
    np.testing.assert_array_equal(bits_of(dq), f["dequant_kn_bits"])
    assert_close(y, f["y"], name + " op")
    layer = ops.PackedQuantLinear(bits, ops.PACK_OUT if pack == "out" else ops.PACK_IN, qw, qz, sc, None, tdt)
    assert layer.prepacked
    np.testing.assert_array_equal(bits_of(layer.dequantize()), f["dequant_kn_bits"])
    assert_close(layer.forward(x), f["y"], name + " resident layer")


@pytest.mark.gpu
@pytest.mark.parametrize("name", GGUF)
def test_gpu_gguf_matches_fixtures(name):
    torch, ops, TORCH_DT, as_f32, assert_close, bits_of, to_dev = _gpu()
    say(f"golden gguf {name}")
    f = load("gguf_" + name)
    fmt, n, k = int(f["fmt"][0]), int(f["n"][0]), int(f["k"][0])
    wd = to_dev(f["weight_bytes"])
    got = ops.gguf_dequantize(wd, k, n, fmt).cpu().numpy()
    np.testing.assert_array_equal(got.view(np.uint32), f["dequant_nk"].view(np.uint32))
    assert_close(ops.gguf_quant_matmul(to_dev(f["x"]), wd, k, n, fmt), f["y_f32"], f"gguf {name} f32")


@pytest.mark.gpu
def test_gpu_mxfp4_f8_transforms_and_routing_match_fixtures():
    torch, ops, TORCH_DT, as_f32, assert_close, bits_of, to_dev = _gpu()
    say("golden mxfp4")
    f = load("mxfp4_case")
    bd, sd = to_dev(f["blocks"]), to_dev(f["scales"])
    got = ops.mxfp4_dequantize(bd, sd, 64, 10).cpu().numpy()
    np.testing.assert_array_equal(got.view(np.uint32), f["dequant_nk"].view(np.uint32))
    assert_close(ops.mxfp4_matmul(to_dev(f["x"], torch.bfloat16), bd, sd, 64, 10), f["y"], "mxfp4 case")
    say("golden f8")
    f = load("f8_block_dequant")
    np.testing.assert_array_equal(bits_of(ops.f8_block_dequant_bf16(to_dev(f["bytes"]), to_dev(f["scales"]))),
                                  f["dequant_bf16_bits"])
    cast = ops.cast_f8e4m3_to_f32(to_dev(np.arange(256, dtype=np.uint8))).cpu().numpy()
    nan = np.isnan(f["all_bytes_f32"])
    assert np.array_equal(np.isnan(cast), nan)
    np.testing.assert_array_equal(cast[~nan].view(np.uint32), f["all_bytes_f32"][~nan].view(np.uint32))
    say("golden transforms")
    f = load("compressed_to_awq")
    got = ops.compressed_to_awq(to_dev(f["weight_packed"]), to_dev(f["weight_scale"]))
    np.testing.assert_array_equal(got[0].cpu().numpy().view(np.uint32), f["qweight"])
    np.testing.assert_array_equal(got[1].cpu().numpy().view(np.uint32), f["qzeros"])
    np.testing.assert_array_equal(got[2].cpu().numpy(), f["scales"])
    f = load("rtn_quantize_awq")
    got = ops.rtn_quantize_awq(to_dev(f["weight"]), int(f["group_size"][0]))
    np.testing.assert_array_equal(got[0].cpu().numpy().view(np.uint32), f["qweight"])
    np.testing.assert_array_equal(got[1].cpu().numpy().view(np.uint32), f["qzeros"])
    np.testing.assert_array_equal(got[2].cpu().numpy().view(np.uint32), f["scales"].view(np.uint32))
    say("golden routing")
    f = load("moe_route_group")
    idx, vals = ops.moe_route(to_dev(f["logits"]), 4, True)
    np.testing.assert_array_equal(idx.cpu().numpy(), f["top_idx"])
    np.testing.assert_allclose(vals.cpu().numpy(), f["top_vals"], rtol=1e-6, atol=0)
    off, tok, wts, _ = ops.moe_group(idx, vals, 32)
    np.testing.assert_array_equal(off.cpu().numpy(), f["offsets"])
    np.testing.assert_array_equal(tok.cpu().numpy(), f["tokens"])
