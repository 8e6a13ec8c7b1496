"""Resident bf16 GGUF layers on the matrix-core layout (csrc/gguf_mfma.hip), through the C ABI.

A bf16 QLinear (linear.rs:197-284, the reference's GPU contract: bf16 x and y) of Q4_0, Q4_1, Q5_0, Q5_1, Q8_0, Q4_K,
Q5_K or Q6_K keeps
a copy of its blocks in which a strip of 16 columns and a step of 32 (Q6_K: 16) elements of K are one MFMA whose
rows are rows of x; 1 - 32 rows run on it in one launch.  The arithmetic is the GEMV's at every row count
(quant_kernels.metal:1097-1221, 1681-1838: integer sums, one f32 scale per sub-block): the weights are never
rounded to bf16, which the reference's prefill tiles do above 8 rows (quant_kernels.metal:2315-2640).  Hence
the oracle here is the f32 dequant with an f32 matmul at 2e-3 relative / 1e-2 absolute (plus half a bf16 ulp of
the output) for all rows, and for 9 - 32 rows also the tile oracle within the reference's own bound
(metal_ops.rs:6449-6461).

Shapes cover: the benchmark's 4096 x 4096 (two chunks a wave); one chunk a wave and waves without one
(K = 256 .. 1024, 8-wave workgroups); long K (7 and 14 chunks a wave: the ring's loop with every tail); odd
numbers of super-blocks, so that a wave's share starts in the middle of one; one to four row quads, two row
tiles, ragged rows; bias; a wide layer (768 strips and more), where a workgroup takes four strips, and the
same form forced on a narrow one.  The repack itself is pinned bit for bit in test_gpu_gguf_resident.py.
"""
import sys

import numpy as np
import pytest
import torch

import oracle
from oxydllm_amd import synth
from tests.helpers import as_f32, assert_close, bits_of, gguf_on_matrix_cores, round_x, to_dev, tune

pytestmark = pytest.mark.gpu
ops = None
MC = [synth.GGUF_Q4_0, synth.GGUF_Q8_0, synth.GGUF_Q4_K, synth.GGUF_Q6_K, synth.GGUF_Q4_1, synth.GGUF_Q5_0, synth.GGUF_Q5_1, synth.GGUF_Q5_K]
FMTS = [pytest.param(f, id=synth.GGUF_NAMES[f]) for f in MC]
TAG = {synth.GGUF_Q4_0: "q4_0", synth.GGUF_Q8_0: "q8_0", synth.GGUF_Q4_K: "q4k", synth.GGUF_Q6_K: "q6k",
       synth.GGUF_Q4_1: "q4_1", synth.GGUF_Q5_0: "q5_0", synth.GGUF_Q5_1: "q5_1", synth.GGUF_Q5_K: "q5k"}


def setup_module(module):
    from oxydllm_amd import ops as _ops
    module.ops = _ops


def say(msg):
    print(f"[case] {msg}", flush=True)
    sys.stdout.flush()


def _layer(fmt, N, K, seed, bias=None):
    data = synth.gguf_weight(fmt, N, K, seed=seed)
    layer = ops.QLinear(fmt, to_dev(data), K, N, None if bias is None else to_dev(bias, torch.bfloat16), torch.bfloat16)
    assert layer.resident
    return data, layer


@pytest.mark.parametrize("fmt", FMTS)
@pytest.mark.parametrize("N,K,ns", [(4096, 4096, 1), (16, 256, 1), (48, 768, 1), (64, 1792, 1), (32, 14336, 1), (16, 28672, 1),
                                      (112, 2304 + 256, 1), (12288, 512, 4), (128, 2304 + 256, 4), (64, 14336, 4)])
def test_matrix_core_layer_against_oracle(fmt, N, K, ns):
    name = synth.GGUF_NAMES[fmt]
    tune("OXQ_GGUF_MFMA_NS", ns if N < 12288 else None)
    bias = ((np.arange(N, dtype=np.float32) % 13) - 6) * np.float32(0.25)
    data, layer = _layer(fmt, N, K, seed=N + K + fmt, bias=bias)
    w = oracle.dequantize_gguf(fmt, data, N, K)
    br = round_x(bias, oracle.BF16)
    rows = (1, 4, 8, 9, 16, 32) if N == 4096 else (1, 5, 16, 20) if N == 12288 else (1, 2, 3, 4, 5, 7, 8, 9, 12, 13, 16, 17, 31, 32)
    for m in rows:
        say(f"gguf matrix-core {name} N={N} K={K} m={m}")
        x = np.random.default_rng(K + 3 * m).standard_normal((m, K)).astype(np.float32)
        xd = to_dev(x, torch.bfloat16)
        y = layer.forward(xd)
        plan = ops.default_context().last_plan()
        mt = 2 if m > 16 else 1
        four = ns == 4
        assert plan["kernel"] == f"gguf_{TAG[fmt]}_mfma_bf16_mt{mt}" + ("_n64" if four else "") and plan["launches"] == 1, plan
        assert plan["grid"] == (N // (64 if four else 16), 1, 1), plan
        assert plan["block"][0] == (512 if (K // 128 < 16 or K // 128 >= 64 or mt == 2 or four) else 1024), plan
        xr = round_x(x, oracle.BF16)
        ref = oracle.matmul_nt_f32(xr, w, br)
        assert_close(y, ref, f"matrix-core {name} N={N} K={K} m={m}", bf16_out=True)
        if m > 8:  # what the reference's prefill tiles would give, within the reference's own bound
            tile = oracle.matmul_nt_f32(xr, oracle.round_through(w, oracle.BF16), br)
            assert np.abs(as_f32(y) - tile).max() < 0.06 * np.abs(tile).max() + 1e-2
        assert np.array_equal(bits_of(layer.forward(xd)), bits_of(y)), "run to run"


@pytest.mark.parametrize("fmt", FMTS)
def test_rows_do_not_depend_on_the_batch(fmt):
    """A row's result is the same bits at every row count up to 32: alone, among 8, among 16 (one row tile), among
    32 (two row tiles; the same chunks per wave only where the workgroup has as many waves, so K is short here)."""
    N, K = 64, 1024
    data, layer = _layer(fmt, N, K, seed=21 + fmt)
    x = np.random.default_rng(22).standard_normal((32, K)).astype(np.float32)
    xd = to_dev(x, torch.bfloat16)
    y32 = bits_of(layer.forward(xd))
    y16 = bits_of(layer.forward(xd[:16].contiguous()))
    y8 = bits_of(layer.forward(xd[:8].contiguous()))
    np.testing.assert_array_equal(y16, y32[:16])
    np.testing.assert_array_equal(y8, y32[:8])
    for r in (0, 3, 7, 15, 31):
        say(f"gguf matrix-core {synth.GGUF_NAMES[fmt]} row {r} alone")
        y1 = bits_of(layer.forward(xd[r:r + 1].contiguous()))
        np.testing.assert_array_equal(y1[0], y32[r])


@pytest.mark.parametrize("fmt", FMTS)
def test_switches_and_rows_beyond_the_kernel(fmt):
    """More than 32 rows go to the tile matmul on the file layout; OXQ_GGUF_MFMA_MAX_M moves that bound;
    OXQ_GGUF_MFMA = 0 builds the rotated copy of the vector GEMV instead (1 - 4 rows)."""
    from tests.test_gpu_gguf_mxfp4 import _check_mul_mm
    N, K = 96, 512
    data, layer = _layer(fmt, N, K, seed=31 + fmt)
    w = oracle.dequantize_gguf(fmt, data, N, K)
    x = np.random.default_rng(32).standard_normal((40, K)).astype(np.float32)
    say(f"gguf matrix-core {synth.GGUF_NAMES[fmt]}: 40 rows")
    y = layer.forward(to_dev(x, torch.bfloat16))
    assert "_mul_mm_" in ops.default_context().last_plan()["kernel"]
    _check_mul_mm(y, x, w, "40 rows")
    tune("OXQ_GGUF_MFMA_MAX_M", 8)
    say(f"gguf matrix-core {synth.GGUF_NAMES[fmt]}: bound moved to 8")
    y = layer.forward(to_dev(x[:9], torch.bfloat16))
    assert "_mul_mm_" in ops.default_context().last_plan()["kernel"]
    _check_mul_mm(y, x[:9], w, "9 rows with the bound at 8")
    y = layer.forward(to_dev(x[:8], torch.bfloat16))
    assert "_mfma_bf16_mt1" in ops.default_context().last_plan()["kernel"]
    tune("OXQ_GGUF_MFMA_MAX_M", None)
    tune("OXQ_GGUF_MFMA", 0)
    say(f"gguf matrix-core {synth.GGUF_NAMES[fmt]}: switched off")
    rot = ops.QLinear(fmt, to_dev(data), K, N, None, torch.bfloat16)
    tune("OXQ_GGUF_MFMA", None)
    assert rot.resident
    y4 = rot.forward(to_dev(x[:4], torch.bfloat16))
    assert "_res_gemv_bf16" in ops.default_context().last_plan()["kernel"]
    ref = oracle.matmul_nt_f32(round_x(x[:4], oracle.BF16), w)
    assert_close(y4, ref, "rotated copy of a bf16 layer", bf16_out=True)
    assert_close(layer.forward(to_dev(x[:4], torch.bfloat16)), ref, "matrix-core copy, the same rows", bf16_out=True)
    assert np.array_equal(rot.dequantize().cpu().numpy().view(np.uint32), layer.dequantize().cpu().numpy().view(np.uint32))


def test_f32_layers_keep_the_rotated_copy():
    """f32 activations are the reference's CPU contract (linear.rs:357-372): exact f32 arithmetic on the vector ALU."""
    fmt, N, K = synth.GGUF_Q4_K, 64, 512
    data = synth.gguf_weight(fmt, N, K, seed=41)
    layer = ops.QLinear(fmt, to_dev(data), K, N, None, torch.float32)
    x = np.random.default_rng(42).standard_normal((2, K)).astype(np.float32)
    y = layer.forward(to_dev(x))
    assert "_res_gemv_f32" in ops.default_context().last_plan()["kernel"]
    assert not gguf_on_matrix_cores(fmt, N, K, 2, bf16=False)
    assert_close(y, oracle.matmul_nt_f32(x, oracle.dequantize_gguf(fmt, data, N, K)), "f32 layer")


@pytest.mark.parametrize("fmt", FMTS)
def test_matrix_core_layer_replays_in_a_graph(fmt):
    N, K = 256, 2048
    say(f"gguf matrix-core graph replay {synth.GGUF_NAMES[fmt]}")
    data, layer = _layer(fmt, N, K, seed=51 + fmt)
    x = torch.randn((6, K), device="cuda", dtype=torch.bfloat16)
    y = torch.empty((6, N), device="cuda", dtype=torch.bfloat16)
    layer.forward(x, out=y)
    stream = torch.cuda.Stream()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g, stream=stream):
        layer.forward(x, out=y)
    gen = torch.Generator(device="cuda")
    for i in range(1, 4):
        gen.manual_seed(i)
        x.copy_(torch.randn((6, K), device="cuda", generator=gen).to(torch.bfloat16))
        layer.forward(x, out=y)
        torch.cuda.synchronize()
        want = bits_of(y).copy()
        y.zero_()
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        assert np.array_equal(bits_of(y), want), f"replay {i}"


# ------------------------------------------------------------------ fused gate|up activation
@pytest.mark.parametrize("fmt", FMTS)
@pytest.mark.parametrize("act", ["silu", "gelu_tanh"])
def test_fused_gate_up_activation_gives_the_two_call_bits(fmt, act):
    """ffn.rs:386-413: the fused projection's output goes through gated_silu_fused / gated_gelu_tanh_fused.  The layer
    built with gate_up_act runs that in its epilogue; it must give, bit for bit, what the plain layer followed by
    oxq_gated_activation gives - at every row count the plain layer runs on the same kernel (up to 32), with and
    without bias, one strip and four strips a workgroup.  The paired repack is pinned by the dense dequant."""
    kind = ops.ACT_GATED_SILU if act == "silu" else ops.ACT_GATED_GELU_TANH
    name = synth.GGUF_NAMES[fmt]
    for K, I, ns in [(1024, 64, 1), (2304 + 256, 96, 1), (512, 128, 4)]:
        N = 2 * I
        data = synth.gguf_weight(fmt, N, K, seed=K + I + fmt)
        wd = to_dev(data)
        for with_bias in (False, True):
            bias = ((np.arange(N, dtype=np.float32) % 9) - 4) * np.float32(0.5) if with_bias else None
            bd = None if bias is None else to_dev(bias, torch.bfloat16)
            tune("OXQ_GGUF_MFMA_NS", ns)
            plain = ops.QLinear(fmt, wd, K, N, bd, torch.bfloat16)
            fused = ops.QLinear(fmt, wd, K, N, bd, torch.bfloat16, gate_up_act=kind)
            assert fused.resident and fused.out_features == I
            want = oracle.dequantize_gguf(fmt, data, N, K)
            assert np.array_equal(fused.dequantize().cpu().numpy().view(np.uint32), want.view(np.uint32)), "paired repack"
            for m in (1, 3, 8, 13, 16, 17, 32):
                say(f"gguf fused gate|up {name} {act} K={K} I={I} ns={ns} bias={with_bias} m={m}")
                x = np.random.default_rng(K + m).standard_normal((m, K)).astype(np.float32)
                xd = to_dev(x, torch.bfloat16)
                y = fused.forward(xd)
                plan = ops.default_context().last_plan()
                assert plan["kernel"].endswith("_act") and "_mfma_bf16_mt" in plan["kernel"] and plan["launches"] == 1, plan
                assert tuple(y.shape) == (m, I)
                gu = plain.forward(xd)
                assert "_mfma_bf16_mt" in ops.default_context().last_plan()["kernel"]
                two = ops.gated_activation(gu, kind)
                np.testing.assert_array_equal(bits_of(y), bits_of(two))
            tune("OXQ_GGUF_MFMA_NS", None)


@pytest.mark.parametrize("fmt", [synth.GGUF_Q4_K, synth.GGUF_Q6_K])
def test_fused_gate_up_rows_beyond_a_tile_and_refusals(fmt):
    """More than 32 rows run as row tiles of the same launch: every tile gives what a call on its rows gives (8-wave
    workgroups at this K for every row count, so the sums run in the same order)."""
    K, I = 1024, 64
    N = 2 * I
    data = synth.gguf_weight(fmt, N, K, seed=71 + fmt)
    wd = to_dev(data)
    fused = ops.QLinear(fmt, wd, K, N, None, torch.bfloat16, gate_up_act=ops.ACT_GATED_SILU)
    x = np.random.default_rng(72).standard_normal((70, K)).astype(np.float32)
    xd = to_dev(x, torch.bfloat16)
    say(f"gguf fused gate|up {synth.GGUF_NAMES[fmt]} 70 rows")
    y = bits_of(fused.forward(xd))
    plan = ops.default_context().last_plan()
    assert plan["grid"] == (N // 16, 1, 3) and plan["kernel"].endswith("_mt2_act"), plan
    for r0 in (0, 32):
        np.testing.assert_array_equal(y[r0:r0 + 32], bits_of(fused.forward(xd[r0:r0 + 32].contiguous())))
    g, u = oracle.matmul_nt_f32(round_x(x, oracle.BF16), oracle.dequantize_gguf(fmt, data, N, K)).reshape(70, 2, I).transpose(1, 0, 2)
    g, u = oracle.round_through(g, oracle.BF16), oracle.round_through(u, oracle.BF16)
    with np.errstate(over="ignore"):  # exp overflows to inf where silu is 0
        ref = g / (1.0 + np.exp(-g.astype(np.float64))) * u
    # both factors are rounded to bf16 before the product: where the f32 sums of kernel and oracle fall on either side
    # of a rounding boundary, a whole bf16 ulp of that factor shows in the product
    assert_close(torch.from_numpy(y.view(np.int16)).view(torch.bfloat16), ref.astype(np.float32), "70 rows against the oracle",
                 rtol=2.0 ** -6)
    with pytest.raises(ops.OxqError, match="needs a BF16 layer on the matrix-core copy"):
        ops.QLinear(fmt, wd, K, N, None, torch.float32, gate_up_act=ops.ACT_GATED_SILU)
    with pytest.raises(ops.OxqError, match="needs a BF16 layer on the matrix-core copy"):
        ops.QLinear(synth.GGUF_Q2_K, to_dev(synth.gguf_weight(synth.GGUF_Q2_K, N, K, seed=1)), K, N, None, torch.bfloat16,
                    gate_up_act=ops.ACT_GATED_SILU)
    with pytest.raises(ops.OxqError, match="activation must be"):
        ops.QLinear(fmt, wd, K, N, None, torch.bfloat16, gate_up_act=ops.ACT_GPT_OSS_SWIGLU)
    with pytest.raises(ops.OxqError, match="out dtype"):
        fused.forward(to_dev(x[:2]))


@pytest.mark.parametrize("fmt", FMTS)
@pytest.mark.parametrize("ks", [1, 4])
@pytest.mark.parametrize("N,K", [(576, 512), (1088, 1280), (64, 256)])
def test_prefill_kernel_on_the_matrix_core_copy(fmt, N, K, ks):
    """linear.rs:270-284 forward_prefill: more rows than the integer kernel takes run the tile arithmetic (the
    dequantized weight rounded to bf16, f32 accumulation) from the same copy - a workgroup of 64 rows x eight waves
    of 64 columns, x shared in LDS.  N = 576 and 1088 leave the last group one live wave of eight, N = 64 is one
    wave; m covers a ragged row tile, a whole band of eight row tiles with a remainder (581 rows) and two bands;
    K of 2, 4 and 10 chunks (both ring halves, an odd count, both halves of a K-quant block).  The weights the
    matrix cores see are bit for bit the dense dequant's, so the tile oracle holds at the GEMV tolerance; run to run
    bitwise; a row's bits do not depend on m.  ks = 4: the form for fewer rows - two waves of 64 columns a workgroup,
    the four waves of a column group take every fourth chunk (K of 2 chunks: half of them have none; 10: a ragged
    third round) and meet in LDS."""
    name = synth.GGUF_NAMES[fmt]
    tune("OXQ_GGUF_GEMM_MIN_M", 33)
    tune("OXQ_GGUF_GEMM_KS", ks)
    kname = f"gguf_{TAG[fmt]}_gemm_bf16_r64x" + ("8" if ks == 1 else "2k4")
    bias = ((np.arange(N, dtype=np.float32) % 13) - 6) * np.float32(0.25)
    data, layer = _layer(fmt, N, K, seed=N + K + fmt, bias=bias)
    w = oracle.round_through(oracle.dequantize_gguf(fmt, data, N, K), oracle.BF16)
    x = np.random.default_rng(K + N).standard_normal((1030, K)).astype(np.float32)
    xd = to_dev(x, torch.bfloat16)
    tile_all = oracle.matmul_nt_f32(round_x(x, oracle.BF16), w, round_x(bias, oracle.BF16))
    first = None
    for m in (1030, 33, 64, 65, 300, 581):
        say(f"gguf prefill {name} N={N} K={K} m={m}")
        y = layer.forward(xd[:m])
        plan = ops.default_context().last_plan()
        rt, ng = -(-m // 64), -(-(N // 64) // (8 // ks))
        assert plan["kernel"] == kname and plan["launches"] == 1, plan
        assert plan["grid"][0] == ((rt // 8) * (-(-ng // 8)) * 64 + (rt % 8) * ng if ks == 1 else rt * ng) and plan["block"][0] == 512, plan
        assert tuple(y.shape) == (m, N)
        assert_close(y, tile_all[:m], f"gguf prefill {name} N={N} K={K} m={m}", bf16_out=True)
        assert np.array_equal(bits_of(layer.forward(xd[:m])), bits_of(y)), "run to run"
        if first is None:
            first = bits_of(y)
        else:
            np.testing.assert_array_equal(bits_of(y), first[:m])
    # OXQ_GGUF_GEMM_MIN_M = 0: the tile matmul on the file layout, same arithmetic in another order
    tune("OXQ_GGUF_GEMM_MIN_M", 0)
    y0 = layer.forward(xd[:300])
    assert "_mul_mm_bf16" in ops.default_context().last_plan()["kernel"]
    assert_close(y0, tile_all[:300], f"gguf tile matmul {name}", bf16_out=True)


@pytest.mark.parametrize("fmt", FMTS)
@pytest.mark.parametrize("ks", [1, 4])
@pytest.mark.parametrize("act", ["silu", "gelu_tanh"])
def test_fused_gate_up_activation_at_prefill(fmt, act, ks):
    """The prefill kernel's own activation epilogue (gate and up columns of an output sit in lanes 8 apart of the
    accumulator layout) against the plain layer through the same kernel followed by oxq_gated_activation: the same
    bits, with and without bias; I = 288 leaves the last group one live wave."""
    kind = ops.ACT_GATED_SILU if act == "silu" else ops.ACT_GATED_GELU_TANH
    name = synth.GGUF_NAMES[fmt]
    tune("OXQ_GGUF_GEMM_MIN_M", 33)
    tune("OXQ_GGUF_GEMM_KS", ks)
    kname = f"gguf_{TAG[fmt]}_gemm_bf16_r64x" + ("8" if ks == 1 else "2k4")
    K, I = 512, 288
    N = 2 * I
    data = synth.gguf_weight(fmt, N, K, seed=K + I + fmt)
    wd = to_dev(data)
    xd = to_dev(np.random.default_rng(5).standard_normal((300, K)).astype(np.float32), torch.bfloat16)
    for with_bias in (False, True):
        bias = ((np.arange(N, dtype=np.float32) % 9) - 4) * np.float32(0.5) if with_bias else None
        bd = None if bias is None else to_dev(bias, torch.bfloat16)
        plain = ops.QLinear(fmt, wd, K, N, bd, torch.bfloat16)
        fused = ops.QLinear(fmt, wd, K, N, bd, torch.bfloat16, gate_up_act=kind)
        for m in (33, 65, 300):
            say(f"gguf fused gate|up prefill {name} {act} bias={with_bias} m={m}")
            y = fused.forward(xd[:m])
            plan = ops.default_context().last_plan()
            assert plan["kernel"] == kname + ("_silu" if act == "silu" else "_gelu"), plan
            assert tuple(y.shape) == (m, I) and plan["launches"] == 1
            gu = plain.forward(xd[:m])
            assert ops.default_context().last_plan()["kernel"] == kname
            np.testing.assert_array_equal(bits_of(y), bits_of(ops.gated_activation(gu, kind)))


@pytest.mark.parametrize("fmt", FMTS)
def test_stateless_prefill_op_builds_the_copy_in_the_workspace(fmt):
    """oxq_gguf_quant_mul_mm without a layer or a cached copy: from 1024 rows, where the prefill kernel would take the
    call, the op builds the matrix-core copy in the ctx workspace and runs that kernel (two launches, the layer's
    bits); fewer rows, f32 activations and OXQ_TRANSIENT_REPACK = 0 keep the tile matmul on the file layout."""
    name = synth.GGUF_NAMES[fmt]
    N, K = 128, 512
    tune("OXQ_GGUF_GEMM_MIN_M", 33)
    data, layer = _layer(fmt, N, K, seed=7 + fmt)
    wd = to_dev(data)
    w = oracle.round_through(oracle.dequantize_gguf(fmt, data, N, K), oracle.BF16)
    x = np.random.default_rng(8).standard_normal((1030, K)).astype(np.float32)
    xd = to_dev(x, torch.bfloat16)
    ref = oracle.matmul_nt_f32(round_x(x, oracle.BF16), w)
    for m in (1023, 1024, 1030):
        say(f"gguf stateless prefill {name} m={m}")
        y = ops.gguf_quant_mul_mm(xd[:m], wd, K, N, fmt)
        plan = ops.default_context().last_plan()
        if m >= 1024:
            assert plan["kernel"] == f"gguf_{TAG[fmt]}_gemm_bf16_r64x8" and plan["launches"] == 2, plan
            np.testing.assert_array_equal(bits_of(y), bits_of(layer.forward(xd[:m])))
        else:
            assert "_mul_mm_bf16" in plan["kernel"], plan
        assert_close(y, ref[:m], f"gguf stateless prefill {name} m={m}", bf16_out=True)
    tune("OXQ_TRANSIENT_REPACK", 0)
    ops.gguf_quant_mul_mm(xd, wd, K, N, fmt)
    assert "_mul_mm_bf16" in ops.default_context().last_plan()["kernel"]
    tune("OXQ_TRANSIENT_REPACK", None)
    ops.gguf_quant_mul_mm(to_dev(x), wd, K, N, fmt)
    assert "_gemm_" not in ops.default_context().last_plan()["kernel"]


@pytest.mark.parametrize("fmt", [synth.GGUF_Q4_0, synth.GGUF_Q4_K, synth.GGUF_Q5_K, synth.GGUF_Q6_K])
def test_feed_forward_over_a_fused_gguf_layer(fmt):
    """FeedForward (ffn.rs:386-474) with the fused-activation layer as gate_up_proj gives the bits of the layer built
    over the plain fused projection: through the fused kernel up to 32 rows (where the plain projection runs on the
    same kernel), through the file-layout matmul and the stand-alone activation above."""
    H, I = 512, 256
    gu = to_dev(synth.gguf_weight(fmt, 2 * I, H, seed=81 + fmt))
    dn = to_dev(synth.gguf_weight(fmt, H, I, seed=82 + fmt))
    down = ops.QLinear(fmt, dn, I, H, None, torch.bfloat16)
    plain = ops.QLinear(fmt, gu, H, 2 * I, None, torch.bfloat16)
    fused = ops.QLinear(fmt, gu, H, 2 * I, None, torch.bfloat16, gate_up_act=ops.ACT_GATED_GELU_TANH)
    ff_plain = ops.FeedForward(ops.GATE_UP_FUSED, plain, None, down, I, ops.ACT_GATED_GELU_TANH)
    ff_fused = ops.FeedForward(ops.GATE_UP_FUSED, fused, None, down, I, ops.ACT_GATED_GELU_TANH)
    assert ff_fused.scratch_elems(5) == 5 * 3 * I  # room for the unfused path at many rows
    for m in (1, 8, 32, 33, 100):
        say(f"gguf FeedForward over a fused layer {synth.GGUF_NAMES[fmt]} m={m}")
        x = to_dev(np.random.default_rng(m).standard_normal((m, H)).astype(np.float32) * 0.25, torch.bfloat16)
        np.testing.assert_array_equal(bits_of(ff_fused.forward(x)), bits_of(ff_plain.forward(x)))
    with pytest.raises(ops.OxqError, match="another activation"):
        ops.FeedForward(ops.GATE_UP_FUSED, fused, None, down, I, ops.ACT_GATED_SILU)
    with pytest.raises(ops.OxqError, match="only be the fused gate_up_proj"):
        ops.FeedForward(ops.GATE_UP_SEPARATE, fused, plain, down, I, ops.ACT_GATED_GELU_TANH)
