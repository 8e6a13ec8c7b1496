"""Resident GGUF layers (QLinear's strip-major copy of the block bytes) through the C ABI.

oxq_qlinear_new repacks the weights of all ten block formats into strips of 16 rows at load
(linear.rs:225-240 copies the bytes at build); 1 - 4 rows of x then run on that copy.  A bf16 layer of
Q4_0, Q8_0, Q4_K or Q6_K takes the matrix-core layout instead (tests/test_gpu_gguf_mfma.py), on which up
to 32 rows run.  Either repack is pinned bit for bit: the dense dequant read back from the copy must equal
the oracle's dequantize_gguf of the file's bytes.  The GEMV on the copy is held to the f32-accumulated oracle within 2e-3 relative /
1e-2 absolute (plus half a bf16 ulp for bf16 outputs), with f32 and bf16 activations, with and without
bias, on the benchmark's configuration 3, on long and ragged K, and is compared with the kernels on the
file layout; shapes outside the copy's reach and more than 4 rows keep those kernels.
"""
import sys

import numpy as np
import pytest
import torch

import oracle
from oxydllm_amd import synth
from tests.helpers import assert_close, bits_of, gguf_on_matrix_cores, round_x, to_dev, tune

pytestmark = pytest.mark.gpu
ops = None
RES = [synth.GGUF_Q4_0, synth.GGUF_Q8_0, synth.GGUF_Q4_K, synth.GGUF_Q6_K,
       synth.GGUF_Q4_1, synth.GGUF_Q5_0, synth.GGUF_Q5_1, synth.GGUF_Q5_K, synth.GGUF_Q2_K, synth.GGUF_Q3_K]
KQ = (synth.GGUF_Q4_K, synth.GGUF_Q6_K, synth.GGUF_Q5_K, synth.GGUF_Q2_K, synth.GGUF_Q3_K)   # super-blocks of 256
ROWS = 4   # rows of x one pass on the copy takes; f32 rows up to 8 (the reference's GEMV range) take two passes
FMTS = [pytest.param(f, id=synth.GGUF_NAMES[f]) for f in RES]


def setup_module(module):
    from oxydllm_amd import ops as _ops
    module.ops = _ops


def say(msg):
    print(f"[case] {msg}", flush=True)
    sys.stdout.flush()


@pytest.mark.parametrize("fmt", FMTS)
@pytest.mark.parametrize("tdt", [torch.float32, torch.bfloat16], ids=["rotated", "bf16-layer"])
@pytest.mark.parametrize("N,K", [(16, 256), (48, 1024), (160, 2304), (32, 4096)])
def test_resident_copy_dequantizes_bit_exact(fmt, tdt, N, K):
    say(f"resident gguf dequant {synth.GGUF_NAMES[fmt]} N={N} K={K} {tdt}")
    data = synth.gguf_weight(fmt, N, K, seed=7 * N + K + fmt)
    layer = ops.QLinear(fmt, to_dev(data), K, N, None, tdt)
    assert layer.resident
    want = oracle.dequantize_gguf(fmt, data, N, K)
    got = layer.dequantize().cpu().numpy()
    kernel = ops.default_context().last_plan()["kernel"]
    assert ("_mfma_dequant" in kernel) == gguf_on_matrix_cores(fmt, N, K, 1, tdt == torch.bfloat16), kernel
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), "repack changed a weight"


@pytest.mark.parametrize("fmt", FMTS)
@pytest.mark.parametrize("act", ["f32", "bf16"])
def test_resident_gemv_config3(fmt, act):
    """Benchmark configuration 3: M = 1, K = N = 4096."""
    say(f"resident gguf gemv {synth.GGUF_NAMES[fmt]} {act}")
    N = K = 4096
    data = synth.gguf_weight(fmt, N, K, seed=0x0A0D11E8 + fmt)
    w = oracle.dequantize_gguf(fmt, data, N, K)
    x = np.random.default_rng(50 + fmt).standard_normal((1, K)).astype(np.float32)
    tdt = torch.bfloat16 if act == "bf16" else torch.float32
    xd = to_dev(x, tdt)
    xr = round_x(x, oracle.BF16) if act == "bf16" else x
    wd = to_dev(data)
    layer = ops.QLinear(fmt, wd, K, N, None, tdt)
    assert layer.resident
    y = layer.forward(xd)
    plan = ops.default_context().last_plan()
    tag = "_mfma_bf16_mt1" if gguf_on_matrix_cores(fmt, N, K, 1, act == "bf16") else "_res_gemv_"
    assert tag in plan["kernel"] and plan["launches"] == 1 and plan["grid"][0] == N // 16, plan
    assert y.shape == (1, N) and y.dtype == tdt
    assert_close(y, oracle.matmul_nt_f32(xr, w), f"resident {synth.GGUF_NAMES[fmt]} {act}", bf16_out=act == "bf16")
    y0 = ops.gguf_quant_matmul(xd, wd, K, N, fmt)
    assert_close(y, y0.float().cpu().numpy(), "resident against the op on the file layout", bf16_out=act == "bf16")
    assert np.array_equal(bits_of(layer.forward(xd)), bits_of(y)), "run-to-run"


@pytest.mark.parametrize("fmt", FMTS)
def test_resident_gemv_rows_bias_and_shapes(fmt):
    name = synth.GGUF_NAMES[fmt]
    for N, K in [(16, 256), (80, 768), (256, 2048 + 256), (64, 14336), (1008, 1024)]:
        data = synth.gguf_weight(fmt, N, K, seed=N + K + fmt)
        w = oracle.dequantize_gguf(fmt, data, N, K)
        bias = np.random.default_rng(N).standard_normal(N).astype(np.float32)
        for tdt, dt in [(torch.float32, None), (torch.bfloat16, oracle.BF16)]:
            bd = to_dev(bias, tdt)
            br = round_x(bias, dt) if dt is not None else bias
            layer = ops.QLinear(fmt, to_dev(data), K, N, bd, tdt)
            assert layer.resident
            for m in (1, 2, 3, 4, 5, 8):
                say(f"resident gguf {name} N={N} K={K} m={m} {tdt}")
                x = np.random.default_rng(K + m).standard_normal((m, K)).astype(np.float32)
                xr = round_x(x, dt) if dt is not None else x
                y = layer.forward(to_dev(x, tdt))
                kernel = ops.default_context().last_plan()["kernel"]
                if gguf_on_matrix_cores(fmt, N, K, m, dt is not None):
                    assert "_mfma_bf16_mt1" in kernel, (kernel, m, K)
                else:
                    on_copy = "_res_gemv_" in kernel
                    assert on_copy == (m <= ROWS or (m <= 8 and dt is None)), (kernel, m, K)
                assert_close(y, oracle.matmul_nt_f32(xr, w, br), f"resident {name} N={N} K={K} m={m}",
                             bf16_out=dt is not None)


@pytest.mark.parametrize("cap", [2, 3, 5])
def test_workgroups_that_walk_several_strips(cap, monkeypatch):
    """More strips than workgroups (a wide layer; forced here by capping the grid): a workgroup stages x
    once, walks its strips and meets once per group of four - full groups, a partial last group, a single strip."""
    tune("OXQ_GGR_GRID", cap)
    N, K = 16 * 11, 2048
    for fmt in RES:
        data = synth.gguf_weight(fmt, N, K, seed=cap + fmt)
        w = oracle.dequantize_gguf(fmt, data, N, K)
        bias = np.random.default_rng(cap).standard_normal(N).astype(np.float32)
        layer = ops.QLinear(fmt, to_dev(data), K, N, to_dev(bias), torch.float32)
        for m in (1, 3):
            say(f"resident gguf strips per workgroup: cap {cap} {synth.GGUF_NAMES[fmt]} m={m}")
            x = np.random.default_rng(m).standard_normal((m, K)).astype(np.float32)
            y = layer.forward(to_dev(x))
            plan = ops.default_context().last_plan()
            assert "_res_gemv_" in plan["kernel"] and plan["grid"][0] == cap, plan
            assert_close(y, oracle.matmul_nt_f32(x, w, bias), f"cap {cap} fmt {fmt} m={m}")
    tune("OXQ_GGR_GRID", None)
    y1 = layer.forward(to_dev(x))
    assert ops.default_context().last_plan()["grid"][0] == N // 16
    assert np.array_equal(bits_of(y1), bits_of(y)), "the walk does not change a column's sum order"


def test_layers_outside_the_copys_reach_keep_the_file_layout(monkeypatch):
    say("resident gguf: ineligible layers")
    K, N = 512, 96
    for fmt, n, k in [(synth.GGUF_Q2_K, 104, K), (synth.GGUF_Q3_K, N, K), (synth.GGUF_Q4_0, 100, K),
                      (synth.GGUF_Q4_0, N, 416), (synth.GGUF_Q5_1, N, 96), (synth.GGUF_Q6_K, N, 768)]:
        data = synth.gguf_weight(fmt, n, k, seed=5)
        layer = ops.QLinear(fmt, to_dev(data), k, n, None, torch.float32)
        expect = fmt in RES and n % 16 == 0 and k % (256 if fmt in KQ else 128) == 0
        assert layer.resident == expect, (fmt, n, k)
        x = np.random.default_rng(1).standard_normal((1, k)).astype(np.float32)
        y = layer.forward(to_dev(x))
        assert_close(y, oracle.matmul_nt_f32(x, oracle.dequantize_gguf(fmt, data, n, k)), f"fmt {fmt} N={n} K={k}")
        want = oracle.dequantize_gguf(fmt, data, n, k)
        assert np.array_equal(layer.dequantize().cpu().numpy().view(np.uint32), want.view(np.uint32))
    tune("OXQ_PREPACK", 0)
    data = synth.gguf_weight(synth.GGUF_Q4_0, N, K, seed=6)
    assert not ops.QLinear(synth.GGUF_Q4_0, to_dev(data), K, N, None, torch.float32).resident


def test_resident_gemv_replays_in_a_graph():
    fmt, N, K = synth.GGUF_Q4_K, 512, 2048
    say("resident gguf graph replay")
    data = synth.gguf_weight(fmt, N, K, seed=11)
    layer = ops.QLinear(fmt, to_dev(data), K, N, None, torch.float32)
    x = torch.randn((2, K), device="cuda")
    y = torch.empty((2, N), device="cuda")
    layer.forward(x, out=y)
    stream = torch.cuda.Stream()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g, stream=stream):
        layer.forward(x, out=y)
    gen = torch.Generator(device="cuda")
    for i in range(1, 4):
        gen.manual_seed(i)
        x.copy_(torch.randn((2, K), device="cuda", generator=gen))
        layer.forward(x, out=y)
        torch.cuda.synchronize()
        want = bits_of(y).copy()
        y.zero_()
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        assert np.array_equal(bits_of(y), want), f"replay {i}"
