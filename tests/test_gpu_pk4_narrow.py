"""GPU parity tests for resident 4-bit layers stored in strips of 16 columns.

Layers with few 64-column strips and a long K (attention projections) are kept in 16-column strips: up
to 8 (or 16) rows of x run one workgroup per strip (one launch, K inside the workgroup), more rows run four
strips a workgroup.  Checked against the CPU oracle on shapes that take the layout by themselves and,
with the layout forced, on small ragged ones:
  layer.dequantize()  bit-exact (pins the repack of this layout);
  layer.forward()     2e-3 relative / 1e-2 absolute of the f32-accumulated oracle for every form
                      (single strip, four strips, folded and tile arithmetic, K slices);
  run-to-run          bitwise identical; the wide layout of the same layer agrees within the tolerance.
"""
import sys

import numpy as np
import pytest
import torch

import oracle
from oxydllm_amd import synth
from tests.helpers import TORCH_DT, as_f32, assert_close, bits_of, resident_rounds_weights, round_x, to_dev, tune

pytestmark = pytest.mark.gpu
ops = None


def setup_module(module):
    from oxydllm_amd import ops as _ops
    module.ops = _ops


def say(msg):
    print(f"[case] {msg}", flush=True)
    sys.stdout.flush()


DT = {"f16": oracle.F16, "bf16": oracle.BF16}


def make(kind, K, N, g, seed):
    if kind == "awq":
        return synth.awq_checkpoint(K, N, g, 4, seed=seed), ops.PACK_OUT
    return synth.gptq_checkpoint(K, N, g, 4, seed=seed), ops.PACK_IN


def dense(kind, trip, dt):
    s_r = oracle.round_through(trip[2], dt)
    return oracle.dequantize_awq(trip[0], trip[1], s_r) if kind == "awq" else oracle.dequantize_gptq(trip[0], trip[1], s_r, 4)


def layer_of(trip, pack_dim, dt, bias=None):
    tdt = TORCH_DT[dt]
    b = None if bias is None else to_dev(bias, tdt)
    return ops.PackedQuantLinear(4, pack_dim, to_dev(trip[0]), to_dev(trip[1]), to_dev(trip[2], tdt), b, tdt)


def kernel_of_last_call():
    return ops.default_context().last_plan()


@pytest.mark.parametrize("kind", ["awq", "gptq"])
@pytest.mark.parametrize("dtn", ["f16", "bf16"])
@pytest.mark.parametrize("K,N,g", [(256, 2048, 128), (384, 2112, 128), (1024, 64, 256), (640, 192, 128)])
def test_narrow_layout_forced_on_small_shapes(kind, dtn, K, N, g, monkeypatch):
    """N >= 2048 takes the single-strip form for its first 8 or 16 rows; the narrower ones always run
    four strips a workgroup.  K/128 = 2, 3, 5, 8 blocks over 8 waves: empty waves, odd shares, ring tails."""
    tune("OXQ_PK4_STRIP16", 2)
    dt = DT[dtn]
    trip, pack_dim = make(kind, K, N, g, seed=K + N)
    bias = (np.arange(N, dtype=np.float32) % 13 - 6) * np.float32(0.125)
    layer = layer_of(trip, pack_dim, dt, bias)
    assert layer.prepacked
    w = dense(kind, trip, dt)
    say(f"narrow dequantize {kind} {dtn} K={K} N={N}")
    np.testing.assert_array_equal(bits_of(layer.dequantize()), oracle.transpose_convert(w, dt))
    rng = np.random.default_rng(K * 3 + N)
    for m in (1, 2, 3, 4, 5, 8, 16, 17, 32, 33, 48, 49, 64, 65, 130):
        say(f"narrow forward {kind} {dtn} K={K} N={N} g={g} m={m}")
        x = rng.standard_normal((m, K)).astype(np.float32)
        xd = to_dev(x, TORCH_DT[dt])
        y = layer.forward(xd)
        plan = kernel_of_last_call()
        assert "_n16x" in plan["kernel"], plan
        wide16 = (N // 16 <= 256 and K // 128 <= 32) or ((N // 16) % 256 == 0 and K // 128 <= 64)
        single = N >= 2048 and m <= (16 if wide16 else 8)
        assert plan["kernel"].endswith("x1") == single, plan
        # three row tiles keep the tile form in this layout: the fold's sums do not fit beside the ring
        rounded = resident_rounds_weights(m, dt, kind == "gptq") or (dt == oracle.F16 and 32 < m <= 48)
        assert ("_gs" in plan["kernel"]) == (not rounded), plan
        wr = oracle.round_through(w, dt) if rounded else w
        assert_close(y, oracle.matmul_nt_f32(round_x(x, dt), wr, bias), f"narrow {kind} {dtn} m{m} {plan['kernel']}")
        np.testing.assert_array_equal(bits_of(layer.forward(xd)), bits_of(y))


@pytest.mark.parametrize("ks", [2, 3])
def test_narrow_layout_k_slices(ks, monkeypatch):
    tune("OXQ_PK4_STRIP16", 2)
    tune("OXQ_PK4_KS", ks)
    dt = oracle.F16
    K, N = 1152, 128
    trip, pack_dim = make("awq", K, N, 128, seed=ks)
    bias = (np.arange(N, dtype=np.float32) % 7 - 3) * np.float32(0.25)
    layer = layer_of(trip, pack_dim, dt, bias)
    w = dense("awq", trip, dt)
    rng = np.random.default_rng(ks)
    for m in (1, 7, 40, 64):
        say(f"narrow k-slices ks={ks} m={m}")
        x = rng.standard_normal((m, K)).astype(np.float32)
        y = layer.forward(to_dev(x, torch.float16))
        plan = kernel_of_last_call()
        assert plan["split_k"] == ks and plan["launches"] == 2 and "_n16x4" in plan["kernel"], plan
        wr = oracle.round_through(w, dt) if "_gs" not in plan["kernel"] else w
        assert_close(y, oracle.matmul_nt_f32(round_x(x, dt), wr, bias), f"narrow k-slices m{m}")


@pytest.mark.parametrize("K,N", [(4096, 4096), (4096, 6144), (8192, 2048), (14336, 4096), (4096, 8192), (8192, 4096),
                                 (6144, 4096), (3584, 3584), (2048, 2048), (3072, 5120)])
def test_attention_and_down_projection_shapes_take_the_narrow_layout(K, N, monkeypatch):
    """By shape alone (no switch): one launch up to eight rows, up to 16 on whole rounds of strips and K <= 8192
    (16 waves a workgroup), the wide layout's answer within tolerance."""
    dt = oracle.F16
    trip, pack_dim = make("awq", K, N, 128, seed=N)
    layer = layer_of(trip, pack_dim, dt)
    tune("OXQ_PK4_STRIP16", 0)
    wide = layer_of(trip, pack_dim, dt)
    tune("OXQ_PK4_STRIP16", None)
    w = dense("awq", trip, dt)
    np.testing.assert_array_equal(bits_of(layer.dequantize()), bits_of(wide.dequantize()))
    wide16 = (N // 16 <= 256 and K // 128 <= 32) or ((N // 16) % 256 == 0 and K // 128 <= 64)
    for m in (1, 2, 4, 8, 9, 12, 16, 64):
        say(f"narrow by shape K={K} N={N} m={m}")
        x = np.random.default_rng(m).standard_normal((m, K)).astype(np.float32)
        xd = to_dev(x, torch.float16)
        y = layer.forward(xd)
        plan = kernel_of_last_call()
        assert "_n16x" in plan["kernel"], plan
        if m <= 8:
            assert plan["launches"] == 1 and plan["split_k"] == 1 and plan["grid"][0] == N // 16, plan
            assert plan["block"][0] == 1024, plan   # up to 8 rows: 16 waves, all requests first
        elif m <= 16:
            # 9 - 16 rows: one strip a workgroup on whole rounds of strips and K <= 8192 (16 waves there)
            assert plan["kernel"].endswith("x1") == wide16, plan
            if wide16:
                assert plan["launches"] == 1 and plan["block"][0] == 1024, plan
        yw = wide.forward(xd)
        assert "_n16x" not in kernel_of_last_call()["kernel"]
        wr = oracle.round_through(w, dt) if resident_rounds_weights(m, dt, False) else w
        ref = oracle.matmul_nt_f32(round_x(x, dt), wr)
        assert_close(y, ref, f"narrow by shape m{m}")
        assert_close(yw, ref, f"wide twin m{m}")


@pytest.mark.parametrize("kind", ["awq", "gptq"])
@pytest.mark.parametrize("dtn", ["f16", "bf16"])
def test_sixteen_wave_workgroups_on_a_long_k(kind, dtn, monkeypatch):
    """One or two rows on K >= 8192 run 16 waves a workgroup; 65 blocks leave them uneven shares (4 or 5).
    Up to 8 rows and 8 blocks a wave the waves request their whole share first (a kernel of its own); with
    that switched off the ring kernel takes the same calls."""
    dt = DT[dtn]
    K, N, g = 8192 + 128, 2048, 128
    trip, pack_dim = make(kind, K, N, g, seed=K)
    bias = (np.arange(N, dtype=np.float32) % 11 - 5) * np.float32(0.25)
    layer = layer_of(trip, pack_dim, dt, bias)
    w = dense(kind, trip, dt)
    np.testing.assert_array_equal(bits_of(layer.dequantize()), oracle.transpose_convert(w, dt))
    rng = np.random.default_rng(K)
    for front in (1, 0):
        tune("OXQ_PK4_FRONT", front)
        for m in (1, 2, 3, 4, 5, 8):
            say(f"narrow 16 waves {kind} {dtn} m={m} up-front={front}")
            x = rng.standard_normal((m, K)).astype(np.float32)
            xd = to_dev(x, TORCH_DT[dt])
            y = layer.forward(xd)
            plan = kernel_of_last_call()
            assert plan["kernel"].endswith("_n16x1") and plan["launches"] == 1 and plan["grid"][0] == N // 16, plan
            assert plan["block"][0] == (1024 if m <= (8 if front else 2) else 512), plan
            assert_close(y, oracle.matmul_nt_f32(round_x(x, dt), w, bias), f"narrow 16 waves {kind} {dtn} m{m}")
            np.testing.assert_array_equal(bits_of(layer.forward(xd)), bits_of(y))


def test_shapes_outside_the_rule_keep_the_wide_layout():
    """K beyond 112 blocks, fewer than 128 strips of 16, a layer that fills the chip with 64-column strips, a short K
    (16 - 31 blocks) on more than 5120 columns, a K below 16 blocks; and the short K the rule does take."""
    for K, N in [(14464, 2048), (4096, 1024), (4096, 14336), (2048, 8192), (1920, 2048)]:
        trip, pack_dim = make("awq", K, N, 128, seed=1)
        layer = layer_of(trip, pack_dim, oracle.F16)
        layer.forward(torch.zeros((1, K), device="cuda", dtype=torch.float16))
        assert "_n16x" not in kernel_of_last_call()["kernel"], (K, N)
    for K, N in [(2048, 4096), (3584, 3584), (3968, 5120)]:
        trip, pack_dim = make("awq", K, N, 128, seed=1)
        layer = layer_of(trip, pack_dim, oracle.F16)
        layer.forward(torch.zeros((1, K), device="cuda", dtype=torch.float16))
        assert "_n16x" in kernel_of_last_call()["kernel"], (K, N)
    trip = synth.gptq_checkpoint(4096, 4096, 128, 8, seed=2)
    l8 = ops.PackedQuantLinear(8, ops.PACK_IN, to_dev(trip[0]), to_dev(trip[1]), to_dev(trip[2], torch.float16), None,
                               torch.float16)
    l8.forward(torch.zeros((1, 4096), device="cuda", dtype=torch.float16))
    assert kernel_of_last_call()["kernel"].startswith("pk8_mfma") and "_n16x" not in kernel_of_last_call()["kernel"]
