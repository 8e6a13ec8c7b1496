"""GPU parity tests for resident 4-bit layers on the tile-major (repacked) path.

The layer constructor repacks AWQ / GPTQ 4-bit checkpoints at load; forward
then runs one MFMA kernel for every m.  Checked against the CPU oracle:
  layer.dequantize()  bit-exact against the reference dequant (this pins the
                      repack: every nibble, zero and scale lands where the
                      kernel expects it, since forward consumes the same words
                      with the same arithmetic);
  layer.forward()     2e-3 relative / 1e-2 absolute of the f32-accumulated
                      x . dequant(W)^T (+ bias);
  run-to-run          bitwise identical.
"""
import sys

import numpy as np
import pytest
import torch

import oracle
from oxydllm_amd import synth
from tests import refgen
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


KINDS = ["awq", "gptq", "awq8", "gptq8"]


def bits_of_kind(kind):
    return 8 if kind.endswith("8") else 4


def make(kind, K, N, g, seed):
    bits = bits_of_kind(kind)
    if kind.startswith("awq"):
        return synth.awq_checkpoint(K, N, g, bits, seed=seed), ops.PACK_OUT
    return synth.gptq_checkpoint(K, N, g, bits, seed=seed), ops.PACK_IN


def dense(kind, trip, dt):
    s_r = oracle.round_through(trip[2], dt)
    if kind == "awq":
        return oracle.dequantize_awq(trip[0], trip[1], s_r)
    if kind == "awq8":
        return oracle.dequantize_awq8(trip[0], trip[1], s_r)
    return oracle.dequantize_gptq(trip[0], trip[1], s_r, bits_of_kind(kind))


def layer_of(trip, pack_dim, dt, bias=None, bits=4):
    tdt = TORCH_DT[dt]
    b = None if bias is None else to_dev(bias, tdt)
    return ops.PackedQuantLinear(bits, pack_dim, to_dev(trip[0]), to_dev(trip[1]), to_dev(trip[2], tdt), b, tdt)


@pytest.mark.parametrize("kind", KINDS)
@pytest.mark.parametrize("dtn,K,N,g", [("f16", 256, 128, 128), ("bf16", 256, 128, 128), ("f16", 512, 192, 128),
                                       ("bf16", 1280, 64, 128), ("f16", 1024, 320, 256)])
def test_repacked_dequantize_bit_exact(kind, dtn, K, N, g):
    dt = DT[dtn]
    say(f"pk4 dequantize {kind} {dtn} K={K} N={N} g={g}")
    trip, pack_dim = make(kind, K, N, g, seed=K + N + g)
    layer = layer_of(trip, pack_dim, dt, bits=bits_of_kind(kind))
    assert layer.prepacked
    want = oracle.transpose_convert(dense(kind, trip, dt), dt)
    got = layer.dequantize()
    assert got.shape == (K, N) and got.dtype == TORCH_DT[dt]
    np.testing.assert_array_equal(bits_of(got), want)


def test_repacked_dequantize_reference_generators():
    """The reference's own closed-form triplets (metal_ops.rs:3668-3716, 4001-4060)."""
    say("pk4 dequantize reference triplets")
    for kind, trip, pack_dim in [("awq", refgen.build_awq_triplet(256, 128, 128), ops.PACK_OUT),
                                 ("gptq", refgen.build_gptq_triplet(4, 256, 128, 128), ops.PACK_IN),
                                 ("awq8", refgen.build_w8a16_triplet(256, 128, 128), ops.PACK_OUT),
                                 ("gptq8", refgen.build_gptq_triplet(8, 256, 128, 128), ops.PACK_IN)]:
        for dtn in ("f16", "bf16"):
            dt = DT[dtn]
            layer = layer_of(trip, pack_dim, dt, bits=bits_of_kind(kind))
            assert layer.prepacked
            want = oracle.transpose_convert(dense(kind, trip, dt), dt)
            np.testing.assert_array_equal(bits_of(layer.dequantize()), want)


@pytest.mark.parametrize("kind", KINDS)
@pytest.mark.parametrize("dtn", ["f16", "bf16"])
@pytest.mark.parametrize("K,N,g", [(256, 128, 128), (512, 192, 128), (1280, 64, 128), (2048, 256, 256), (1152, 128, 128)])
def test_repacked_forward_all_m(kind, dtn, K, N, g):
    """m sweeps every row-tile count (1..4 tiles of 16), partial tiles and m > 64; K/g covers
    fewer groups than waves (2), counts not divisible by 8 (10, 9: an odd number of
    128-row blocks per wave) and an even split."""
    dt = DT[dtn]
    trip, pack_dim = make(kind, K, N, g, seed=7 * K + N)
    bias = (np.arange(N, dtype=np.float32) % 11 - 5) * np.float32(0.125)
    layer = layer_of(trip, pack_dim, dt, bias, bits=bits_of_kind(kind))
    assert layer.prepacked
    w = dense(kind, trip, dt)
    rng = np.random.default_rng(K + N)
    for m in (1, 2, 5, 8, 9, 16, 17, 33, 48, 49, 64, 65, 130):
        say(f"pk4 forward {kind} {dtn} K={K} N={N} g={g} m={m}")
        x = rng.standard_normal((m, K)).astype(np.float32)
        ref = oracle.matmul_nt_f32(round_x(x, dt), w, bias)
        y = layer.forward(to_dev(x, TORCH_DT[dt]))
        assert y.shape == (m, N)
        if not resident_rounds_weights(m, dt, kind.startswith("gptq")):
            # the fused-GEMV range: the dequantized weight is never rounded
            assert_close(y, ref, f"pk4 {kind} {dtn} m{m}")
        else:
            # the tile-GEMM range rounds B to the activation type before the matrix unit
            # (mpp_gemm.metal:115-184): compare with that, and with the reference's own
            # bound against the unrounded weights (metal_ops.rs:3713-3716)
            tile = oracle.matmul_nt_f32(round_x(x, dt), oracle.round_through(w, dt), bias)
            assert_close(y, tile, f"pk4 {kind} {dtn} m{m} vs rounded-tile oracle")
            assert np.abs(as_f32(y) - ref).max() < 0.06 * np.abs(ref).max() + 1e-2


def front_rule(K, ks, m, bits=4):
    """The launcher's rule for a single row tile: "front" = 16 waves (4-bit: the whole share of two blocks
    requested up front, 8-bit: one block at a time), "line" = 8 waves, the ring as straight-line code (up to
    8 blocks a wave), "" = the ring kernel."""
    bslice = -(-(K // 128) // ks)
    share8, xq = -(-bslice // 8), -(-m // 4)
    if m > 16:
        return ""
    if bits == 4:
        return "front" if bslice == 32 and xq <= 2 else "line" if share8 <= 8 else ""
    if bslice == 32 and ks == 1:
        return "front"
    return "line" if bslice % 8 == 0 and share8 in (1, 2, 3, 4, 5, 6, 8) else ""


@pytest.mark.parametrize("kind,strip16", [(k, s16) for k in KINDS for s16 in (0, 2) if not (s16 and k.endswith("8"))])
@pytest.mark.parametrize("dtn", ["f16", "bf16"])
@pytest.mark.parametrize("rows", [64, 128])
@pytest.mark.parametrize("K,N,g", [(512, 576, 128), (1280, 1088, 128), (256, 64, 128)])
def test_prefill_rows_by_eight_strips(kind, dtn, rows, K, N, g, strip16):
    """The prefill decomposition (a workgroup = 64 or 128 rows x eight strips, x shared in LDS, a strip per
    wave): N = 576 and 1088 leave the last group one live strip of eight, N = 64 a single group of one; m covers
    one ragged row tile, whole bands of eight row tiles with a ragged remainder (581 rows: 8 + 2 tiles of 64,
    5 of 128; 1100: 16 + 2, 8 + 1) and a band alone; K of 2, 4 and 10 blocks.  Against the tile-GEMM oracle
    (mpp_gemm.metal:115-184: B rounded to the activation type), the reference's own bound against the
    unrounded weights (metal_ops.rs:3713-3716), run to run bitwise, and rows of y independent of m.  Both resident
    layouts: 64-column strips (4- and 8-bit) and (strip16 = 2) the 16-column strips of narrow layers, whose kernel
    rings whole blocks in two halves (K of 2, 4 and 10 blocks: both halves, and an odd count)."""
    bits = bits_of_kind(kind)  # (16-column strips are a 4-bit layout)
    tune("OXQ_PK4_STRIP16", strip16)
    tune("OXQ_PK4_GEMM_ROWS", rows)
    kname = f"pk{bits}_gemm_{dtn}_r{rows}x8" + ("_n16" if strip16 else "")
    dt = DT[dtn]
    trip, pack_dim = make(kind, K, N, g, seed=K + 5 * N)
    bias = (np.arange(N, dtype=np.float32) % 13 - 6) * np.float32(0.125)
    layer = layer_of(trip, pack_dim, dt, bias, bits=bits)
    assert layer.prepacked
    w = dense(kind, trip, dt)
    wt = oracle.round_through(w, dt)
    rng = np.random.default_rng(K + N + rows)
    x_all = rng.standard_normal((1100, K)).astype(np.float32)
    xd_all = to_dev(x_all, TORCH_DT[dt])
    tile_all = oracle.matmul_nt_f32(round_x(x_all, dt), wt, bias)
    ref_all = oracle.matmul_nt_f32(round_x(x_all, dt), w, bias)
    first = None
    for m in (1100, 65, 128, 300, 512, 581, 1024):
        say(f"pk4 prefill {kind} {dtn} r{rows} K={K} N={N} m={m}")
        xd = xd_all[:m]
        y = layer.forward(xd)
        plan = ops.default_context().last_plan()
        rt, ng = -(-m // rows), -(-(N // 64) // 8)
        assert plan["kernel"] == kname, plan
        assert plan["grid"][0] == (rt // 8) * (-(-ng // 8)) * 64 + (rt % 8) * ng and plan["launches"] == 1, plan
        assert y.shape == (m, N)
        assert_close(y, tile_all[:m], f"pk4 prefill {kind} {dtn} r{rows} m{m}")
        assert np.abs(as_f32(y) - ref_all[:m]).max() < 0.06 * np.abs(ref_all[:m]).max() + 1e-2
        np.testing.assert_array_equal(bits_of(layer.forward(xd)), bits_of(y))
        if first is None:
            first = bits_of(y)
        else:
            # a row's result does not depend on how many rows ride along or on which tile it falls
            np.testing.assert_array_equal(bits_of(y), first[:m])
    # without a bias, into a caller's buffer that holds other values
    plain = layer_of(trip, pack_dim, dt, None, bits=bits)
    out = torch.full((300, N), 7.0, device="cuda", dtype=TORCH_DT[dt])
    plain.forward(xd_all[:300], out=out)
    assert ops.default_context().last_plan()["kernel"] == kname
    assert_close(out, tile_all[:300] - bias[None, :], f"pk4 prefill {kind} {dtn} no bias")


@pytest.mark.parametrize("kind,strip16", [(k, s16) for k in KINDS for s16 in (0, 2) if not (s16 and k.endswith("8"))])
@pytest.mark.parametrize("dtn", ["f16", "bf16"])
@pytest.mark.parametrize("K,N,g", [(512, 576, 128), (1280, 1088, 128), (256, 64, 128), (4096, 128, 128)])
def test_prefill_two_strips_with_k_split(kind, dtn, K, N, g, strip16):
    """The form for 65 to a few hundred rows: a workgroup = 64 rows x two strips, the four waves of a strip take every
    fourth block of K and wave kq finishes row tile kq from the four partial tiles in LDS.  N = 576 and 1088 leave
    the last workgroup one live strip; K of 2 blocks (half the waves have none), 4 (one round), 10 (a ragged third
    round: both ring halves of the 16-column layout, and an odd count) and 32; ragged row tiles.  Both resident
    layouts.  Against the tile-GEMM oracle, run to run bitwise, rows independent of m."""
    bits = bits_of_kind(kind)
    tune("OXQ_PK4_STRIP16", strip16)
    tune("OXQ_PK4_GEMM_KS", 4)
    n16 = "_n16" if strip16 else ""
    dt = DT[dtn]
    trip, pack_dim = make(kind, K, N, g, seed=K + 7 * N)
    bias = (np.arange(N, dtype=np.float32) % 13 - 6) * np.float32(0.125)
    layer = layer_of(trip, pack_dim, dt, bias, bits=bits)
    w = dense(kind, trip, dt)
    wt = oracle.round_through(w, dt)
    rng = np.random.default_rng(K + N)
    x_all = rng.standard_normal((330, K)).astype(np.float32)
    xd_all = to_dev(x_all, TORCH_DT[dt])
    tile_all = oracle.matmul_nt_f32(round_x(x_all, dt), wt, bias)
    ref_all = oracle.matmul_nt_f32(round_x(x_all, dt), w, bias)
    first = None
    for m in (330, 65, 128, 200):
        say(f"pk{bits} prefill two strips {kind} {dtn} K={K} N={N} m={m}")
        y = layer.forward(xd_all[:m])
        plan = ops.default_context().last_plan()
        assert plan["kernel"] == f"pk{bits}_gemm_{dtn}_r64x2k4{n16}" and plan["launches"] == 1, plan
        assert plan["grid"][0] == -(-m // 64) * -(-(N // 64) // 2) and plan["block"][0] == 512, plan
        assert_close(y, tile_all[:m], f"pk{bits} two strips {kind} {dtn} m{m}")
        assert np.abs(as_f32(y) - ref_all[:m]).max() < 0.06 * np.abs(ref_all[:m]).max() + 1e-2
        np.testing.assert_array_equal(bits_of(layer.forward(xd_all[:m])), bits_of(y))
        if first is None:
            first = bits_of(y)
        else:
            np.testing.assert_array_equal(bits_of(y), first[:m])
    if N % 128 == 0 and N >= 128 and not strip16:
        # the same layer as a fused gate|up projection: the activation epilogue on the summed tile
        kind_id = ops.ACT_GATED_SILU
        tdt = TORCH_DT[dt]
        fused = ops.PackedQuantLinear(bits, pack_dim, to_dev(trip[0]), to_dev(trip[1]), to_dev(trip[2], tdt), to_dev(bias, tdt), tdt,
                                      gate_up_act=kind_id)
        y = fused.forward(xd_all[:200])
        assert ops.default_context().last_plan()["kernel"] == f"pk{bits}_gemm_{dtn}_r64x2k4_silu"
        np.testing.assert_array_equal(bits_of(y), bits_of(ops.gated_activation(layer.forward(xd_all[:200]), kind_id)))


def test_prefill_takes_over_where_it_fills_the_chip():
    """With the switches at their defaults a 4096 x 14336 layer moves from the split-K tiles (one row tile) to
    workgroups of two strips with K split inside (128 rows: 224 of them), then to 64-row and 128-row workgroups of
    eight strips as m grows (512 rows are 224 workgroups of 64 rows, 1000 rows 224 of 128), OXQ_PK4_GEMM_MIN_M = 0
    keeps the split-K tiles, and the two agree within the tolerance of one f16 rounding of y."""
    K, N, g = 4096, 14336, 128
    trip, pack_dim = make("awq", K, N, g, seed=11)
    layer = layer_of(trip, pack_dim, oracle.F16, None)
    rng = np.random.default_rng(5)
    xd = to_dev(rng.standard_normal((1000, K)).astype(np.float32), torch.float16)
    for m, kern in [(64, "pk4_mfma_f16_mt4"), (128, "pk4_gemm_f16_r64x2k4"), (256, "pk4_gemm_f16_r64x2k4"), (512, "pk4_gemm_f16_r64x8"),
                    (1000, "pk4_gemm_f16_r128x8")]:
        say(f"pk4 prefill rule m={m}")
        y = layer.forward(xd[:m])
        plan = ops.default_context().last_plan()
        assert plan["kernel"].startswith(kern), (m, plan)
        tune("OXQ_PK4_GEMM_MIN_M", 0)
        y0 = layer.forward(xd[:m])
        assert ops.default_context().last_plan()["kernel"].startswith("pk4_mfma_f16_mt4")
        tune("OXQ_PK4_GEMM_MIN_M", None)
        a, b = y.float(), y0.float()
        assert bool(((a - b).abs() <= 2.0 ** -9 * b.abs() + 2e-2).all()), (m, float((a - b).abs().max()))


@pytest.mark.parametrize("kind", ["awq", "gptq"])
@pytest.mark.parametrize("dtn", ["f16", "bf16"])
@pytest.mark.parametrize("K,N,g,ks", [(2048, 256, 128, 1), (4096 + 640, 128, 128, 1), (6144, 64, 128, 1),
                                      (4096, 192, 256, 1), (128 * 21, 64, 128, 1), (4096, 128, 128, 3),
                                      (8192, 64, 128, 1), (8192 - 384, 128, 128, 1), (5120, 128, 128, 1),
                                      (7168, 64, 128, 1), (9216, 64, 128, 1), (1024, 128, 128, 1), (768, 64, 128, 1)])
def test_whole_share_requested_up_front(kind, dtn, K, N, g, ks, monkeypatch):
    """A single row tile of a 4-bit layer runs straight-line kernels: 16 waves that request everything first
    for 32 blocks and up to 8 rows, otherwise 8 waves with one or two blocks in flight for up to 8 blocks a wave.
    16, 37, 48, 32 and 21 blocks (2, 4 or 5, 6, 4 or 2 each, 2 or 3), three K slices of 11, 64 blocks (8 each),
    61 (7 or 8), 40 (5 each), 56 (7: the kernel for 8 with a block of zeros), 8 and 6 blocks (one or none) and
    72 (9: the ring); against the oracle, against the ring kernel within the tolerance, run to run bitwise."""
    tune("OXQ_PK4_STRIP16", 0)   # these small N would take the 16-column layout
    tune("OXQ_PK4_KS", ks)    # and few strips would cut K by themselves
    dt = DT[dtn]
    trip, pack_dim = make(kind, K, N, g, seed=K + 3 * N)
    bias = (np.arange(N, dtype=np.float32) % 9 - 4) * np.float32(0.25)
    layer = layer_of(trip, pack_dim, dt, bias)
    w = dense(kind, trip, dt)
    rng = np.random.default_rng(K)
    for m in (1, 2, 4, 5, 8, 9, 16):
        say(f"pk4 up-front {kind} {dtn} K={K} N={N} ks={ks} m={m}")
        x = rng.standard_normal((m, K)).astype(np.float32)
        xd = to_dev(x, TORCH_DT[dt])
        ref = oracle.matmul_nt_f32(round_x(x, dt), w, bias)
        y = layer.forward(xd)
        plan = ops.default_context().last_plan()
        assert "_n16x" not in plan["kernel"] and plan["split_k"] == ks, plan
        form = front_rule(K, ks, m)
        assert plan["block"][0] == (1024 if form == "front" else 512), (plan, m)
        assert plan["kernel"].endswith("_gs" + ("_" + form if form else "")), (plan, m, form)
        assert_close(y, ref, f"pk4 up-front {kind} {dtn} m{m}")
        np.testing.assert_array_equal(bits_of(layer.forward(xd)), bits_of(y))
        tune("OXQ_PK4_FRONT", 0)
        y0 = layer.forward(xd)
        plan = ops.default_context().last_plan()
        assert plan["block"][0] == 512 and plan["kernel"].endswith("_gs"), plan
        tune("OXQ_PK4_FRONT", None)
        assert_close(y0, ref, f"pk4 ring {kind} {dtn} m{m}")


@pytest.mark.parametrize("kind", ["awq8", "gptq8"])
@pytest.mark.parametrize("dtn", ["f16", "bf16"])
@pytest.mark.parametrize("K,N,g,ks", [(1024, 128, 128, 1), (2048, 64, 128, 1), (5120, 64, 128, 1), (8192, 64, 128, 1),
                                      (4096, 128, 256, 2), (7168, 64, 128, 1), (4096 + 640, 64, 128, 1),
                                      (9216, 64, 128, 1), (4096, 64, 128, 1), (8192, 128, 128, 2)])
def test_eight_bit_single_row_tile_in_straight_line_code(kind, dtn, K, N, g, ks, monkeypatch):
    """8-bit layers take the 8-wave straight-line kernel where every wave's share is whole and the kernel exists
    for it (1 - 6 or 8 blocks): 8, 16, 40 and 64 blocks and two K slices of 16; 32 blocks in one slice run 16
    waves; 56 (7 each), 37 (uneven) and 72 (9 each) keep the ring.  Against the oracle, run to run bitwise, and
    the ring kernel on the same calls."""
    tune("OXQ_PK4_KS", ks)
    dt = DT[dtn]
    trip, pack_dim = make(kind, K, N, g, seed=K + 5 * N)
    bias = (np.arange(N, dtype=np.float32) % 9 - 4) * np.float32(0.25)
    layer = layer_of(trip, pack_dim, dt, bias, bits=8)
    w = dense(kind, trip, dt)
    rng = np.random.default_rng(K + 1)
    for m in (1, 3, 4, 7, 8, 12, 16):
        say(f"pk8 straight-line {kind} {dtn} K={K} N={N} ks={ks} m={m}")
        x = rng.standard_normal((m, K)).astype(np.float32)
        xd = to_dev(x, TORCH_DT[dt])
        ref = oracle.matmul_nt_f32(round_x(x, dt), w, bias)
        y = layer.forward(xd)
        plan = ops.default_context().last_plan()
        form = front_rule(K, ks, m, bits=8)
        assert plan["kernel"].startswith("pk8_mfma") and plan["split_k"] == ks, plan
        assert plan["block"][0] == (1024 if form == "front" else 512), (plan, m)
        assert plan["kernel"].endswith("_gs" + ("_" + form if form else "")), (plan, m, form)
        assert_close(y, ref, f"pk8 straight-line {kind} {dtn} m{m}")
        np.testing.assert_array_equal(bits_of(layer.forward(xd)), bits_of(y))
        tune("OXQ_PK4_FRONT", 0)
        y0 = layer.forward(xd)
        assert ops.default_context().last_plan()["kernel"].endswith("_gs")
        tune("OXQ_PK4_FRONT", None)
        assert_close(y0, ref, f"pk8 ring {kind} {dtn} m{m}")


@pytest.mark.parametrize("kind", ["awq", "gptq", "gptq8"])
@pytest.mark.parametrize("dtn", ["f16", "bf16"])
@pytest.mark.parametrize("K,N,g,ks", [(4096, 128, 128, 1), (8192, 64, 128, 2), (8064, 64, 128, 2), (5120, 64, 128, 1),
                                      (6144, 64, 128, 1), (8192, 64, 128, 1)])
def test_two_to_four_row_tiles_in_straight_line_code(kind, dtn, K, N, g, ks, monkeypatch):
    """17 - 64 rows on K slices of 32 or 40 blocks (4-bit: also 48 and 64) run the block loop as straight-line
    code (four to eight blocks a wave); 63 blocks in two slices leave one wave of the second slice a block short.  Against the
    oracle of the form the row count takes, run to run bitwise, and against the looping kernel."""
    tune("OXQ_PK4_STRIP16", 0)
    tune("OXQ_PK4_KS", ks)
    dt = DT[dtn]
    trip, pack_dim = make(kind, K, N, g, seed=K + N)
    bias = (np.arange(N, dtype=np.float32) % 9 - 4) * np.float32(0.25)
    bits = bits_of_kind(kind)
    layer = layer_of(trip, pack_dim, dt, bias, bits=bits)
    w0 = dense(kind, trip, dt)
    rng = np.random.default_rng(K + 2)
    for m in (17, 24, 32, 33, 48, 49, 57, 64):
        say(f"pk4 two to four tiles, straight line {kind} {dtn} K={K} ks={ks} m={m}")
        x = rng.standard_normal((m, K)).astype(np.float32)
        xd = to_dev(x, TORCH_DT[dt])
        y = layer.forward(xd)
        plan = ops.default_context().last_plan()
        assert any(t in plan["kernel"] for t in ("_mt2", "_mt3", "_mt4")) and plan["split_k"] == ks, plan
        w = w0 if "_gs" in plan["kernel"] else oracle.round_through(w0, dt)
        ref = oracle.matmul_nt_f32(round_x(x, dt), w, bias)
        assert_close(y, ref, f"pk4 four tiles {kind} {dtn} m{m}")
        np.testing.assert_array_equal(bits_of(layer.forward(xd)), bits_of(y))
        tune("OXQ_PK4_FRONT", 0)
        y0 = layer.forward(xd)
        tune("OXQ_PK4_FRONT", None)
        assert_close(y0, ref, f"pk4 four tiles, loop {kind} {dtn} m{m}")
        if m > 48 and bits == 4 and ks == 1 and K in (4096, 5120):
            # the 49 - 64-row kernel (x straight into LDS, weights up front) shares the ring kernel's arithmetic, K
            # split and summation order: the same bits
            tune("OXQ_PK4_T64", 0)
            y1 = layer.forward(xd)
            tune("OXQ_PK4_T64", None)
            np.testing.assert_array_equal(bits_of(y1), bits_of(y))


@pytest.mark.parametrize("kind", KINDS)
@pytest.mark.parametrize("dtn", ["f16", "bf16"])
@pytest.mark.parametrize("K,N,g,ks", [(1280, 128, 128, 3), (2048, 64, 256, 2), (1152, 192, 128, 9), (512, 64, 128, 4)])
def test_repacked_forward_k_slices(kind, dtn, K, N, g, ks, monkeypatch):
    """Layers with few column strips also cut K into slices (grid.y) whose f32 partial tiles a
    second launch adds in slice order.  Forced here on small shapes: slices of unequal size
    (10 groups in 3 slices), fewer groups than waves per slice, one group per slice, bias
    applied once by the reduction."""
    dt = DT[dtn]
    tune("OXQ_PK4_KS", ks)
    trip, pack_dim = make(kind, K, N, g, seed=K + N + ks)
    bias = (np.arange(N, dtype=np.float32) % 7 - 3) * np.float32(0.25)
    layer = layer_of(trip, pack_dim, dt, bias, bits=bits_of_kind(kind))
    assert layer.prepacked
    w = dense(kind, trip, dt)
    rng = np.random.default_rng(K + ks)
    groups = K // 128  # slices are cut in blocks of 128 rows of K
    per = -(-groups // min(ks, groups))
    for m in (1, 7, 16, 40, 64, 100):
        say(f"pk4 k-slices {kind} {dtn} K={K} N={N} g={g} ks={ks} m={m}")
        x = rng.standard_normal((m, K)).astype(np.float32)
        xd = to_dev(x, TORCH_DT[dt])
        y = layer.forward(xd)
        plan = ops.default_context().last_plan()
        assert plan["split_k"] == -(-groups // per) and plan["launches"] == 2
        wr = oracle.round_through(w, dt) if resident_rounds_weights(m, dt, kind.startswith("gptq")) else w
        assert_close(y, oracle.matmul_nt_f32(round_x(x, dt), wr, bias), f"pk4 k-slices m{m}")
        np.testing.assert_array_equal(bits_of(layer.forward(xd)), bits_of(y))


@pytest.mark.parametrize("m", [1, 16, 64])
@pytest.mark.parametrize("K,N", [(4096, 14336), (14336, 4096)])
def test_repacked_forward_config1(m, K, N):
    """Benchmark config 1 (both orientations), f16, and bitwise run-to-run determinism."""
    dt = oracle.F16
    say(f"pk4 forward config1 m={m} K={K} N={N}")
    trip = synth.awq_checkpoint(K, N, 128, 4, seed=0x0A0D11E6)
    layer = layer_of(trip, ops.PACK_OUT, dt)
    assert layer.prepacked
    x = np.random.default_rng(30 + m).standard_normal((m, K)).astype(np.float32)
    ref = oracle.matmul_nt_f32(round_x(x, dt), dense("awq", trip, dt))
    xd = to_dev(x, torch.float16)
    y = layer.forward(xd)
    assert_close(y, ref, f"pk4 config1 m{m} {K}x{N}")
    first = bits_of(y)
    for _ in range(5):
        np.testing.assert_array_equal(bits_of(layer.forward(xd)), first)


@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("dtn", ["f16", "bf16"])
def test_repacked_forward_biased_activations(dtn, bits):
    """m <= 16 feeds bias + q to the matrix cores and removes the bias with the row sums of x:
    activations with a large mean and with outliers are where that cancellation is hardest."""
    dt = DT[dtn]
    K, N = 4096, 256
    kind = "awq8" if bits == 8 else "awq"
    trip, pack_dim = make(kind, K, N, 128, seed=4242)
    layer = layer_of(trip, pack_dim, dt, bits=bits)
    w = dense(kind, trip, dt)
    rng = np.random.default_rng(77)
    cases = {"mean 3": 3.0 + 0.1 * rng.standard_normal((4, K)),
             "positive": np.abs(rng.standard_normal((4, K))) * 2.0,
             "outliers": rng.standard_normal((4, K)) * np.where(rng.random((4, K)) < 0.01, 60.0, 1.0)}
    for name, x in cases.items():
        say(f"pk4 forward {dtn} biased activations: {name}")
        x = x.astype(np.float32)
        ref = oracle.matmul_nt_f32(round_x(x, dt), w)
        assert_close(layer.forward(to_dev(x, TORCH_DT[dt])), ref, f"pk4 {dtn} {name}")


@pytest.mark.parametrize("bits", [4, 8])
def test_repacked_forward_config2_gptq(bits):
    """Benchmark config 2 (GPTQ 4- and 8-bit, K=5120, N=13824, g=128), bf16."""
    dt = oracle.BF16
    K, N = 5120, 13824
    trip = synth.gptq_checkpoint(K, N, 128, bits, seed=0x0A0D11E7)
    layer = layer_of(trip, ops.PACK_IN, dt, bits=bits)
    assert layer.prepacked
    w = dense("gptq8" if bits == 8 else "gptq", trip, dt)
    for m in (1, 8, 24):
        say(f"pk4 forward config2 m={m}")
        x = np.random.default_rng(40 + m).standard_normal((m, K)).astype(np.float32)
        wr = oracle.round_through(w, dt) if resident_rounds_weights(m, dt, True) else w
        ref = oracle.matmul_nt_f32(round_x(x, dt), wr)
        assert_close(layer.forward(to_dev(x, torch.bfloat16)), ref, f"pk{bits} config2 m{m}", bf16_out=True)


def test_ineligible_layers_keep_checkpoint_layout():
    """N not a multiple of 64, g < 128 and 8-bit layers are not repacked and still match."""
    say("pk4 ineligible shapes")
    dt = oracle.F16
    for K, N, g in [(192, 104, 64), (256, 128, 32), (256, 128, 64)]:
        trip = refgen.build_awq_triplet(K, N, g)
        layer = layer_of(trip, ops.PACK_OUT, dt)
        assert not layer.prepacked
        x = refgen.batch_x(3, K)
        ref = oracle.matmul_nt_f32(round_x(x, dt), dense("awq", trip, dt))
        assert_close(layer.forward(to_dev(x, torch.float16)), ref, f"raw layout {K}x{N} g{g}")
        want = oracle.transpose_convert(dense("awq", trip, dt), dt)
        np.testing.assert_array_equal(bits_of(layer.dequantize()), want)
    trip8 = refgen.build_gptq_triplet(8, 256, 128, 64)
    l8 = ops.PackedQuantLinear(8, ops.PACK_IN, to_dev(trip8[0]), to_dev(trip8[1]),
                               to_dev(trip8[2], torch.float16), None, torch.float16)
    assert not l8.prepacked


def test_repacked_layer_survives_freed_checkpoint_tensors():
    """The layer owns its copy: overwrite the caller's tensors after construction."""
    say("pk4 ownership")
    dt = oracle.F16
    K, N, g = 512, 256, 128
    trip, pack_dim = make("awq", K, N, g, seed=99)
    qw, qz, sc = to_dev(trip[0]), to_dev(trip[1]), to_dev(trip[2], torch.float16)
    layer = ops.PackedQuantLinear(4, pack_dim, qw, qz, sc, None, torch.float16)
    assert layer.prepacked
    qw.zero_(), qz.zero_(), sc.zero_()
    torch.cuda.synchronize()
    x = refgen.batch_x(4, K)
    ref = oracle.matmul_nt_f32(round_x(x, dt), dense("awq", trip, dt))
    assert_close(layer.forward(to_dev(x, torch.float16)), ref, "pk4 after source cleared")


@pytest.mark.parametrize("kind", KINDS)
@pytest.mark.parametrize("dtn", ["f16", "bf16"])
@pytest.mark.parametrize("act", ["silu", "gelu"])
@pytest.mark.parametrize("K,I,g", [(256, 64, 128), (512, 96, 128), (1024, 32, 256)])
def test_fused_gate_up_activation(kind, dtn, act, K, I, g):
    """The gate|up layer with the activation in its epilogue (ffn.rs:386-400) against the two-call
    path it replaces, bit for bit, and against the oracle's gated activation.  Its dense dequant is the plain layer's: the column order of the
    resident copy is internal."""
    dt = DT[dtn]
    N = 2 * I
    trip, pack_dim = make(kind, K, N, g, seed=3 * K + I)
    bias = (np.arange(N, dtype=np.float32) % 7 - 3) * np.float32(0.0625)
    bits = bits_of_kind(kind)
    tdt = TORCH_DT[dt]
    kind_id = ops.ACT_GATED_SILU if act == "silu" else ops.ACT_GATED_GELU_TANH
    for b in (None, bias):
        plain = layer_of(trip, pack_dim, dt, b, bits=bits)
        bd = None if b is None else to_dev(b, tdt)
        fused = ops.PackedQuantLinear(bits, pack_dim, to_dev(trip[0]), to_dev(trip[1]), to_dev(trip[2], tdt), bd, tdt,
                                      gate_up_act=kind_id)
        assert fused.prepacked and (fused.in_features, fused.out_features) == (K, I)
        np.testing.assert_array_equal(bits_of(fused.dequantize()), bits_of(plain.dequantize()))
        w = dense(kind, trip, dt)
        rng = np.random.default_rng(K + I)
        for m in (1, 3, 16, 17, 33, 48, 49, 64, 100):
            say(f"gate|up {kind} {dtn} {act} K={K} I={I} m={m} bias={b is not None}")
            x = rng.standard_normal((m, K)).astype(np.float32)
            xd = to_dev(x, tdt)
            y = fused.forward(xd)
            assert y.shape == (m, I)
            gu = plain.forward(xd)
            two = ops.gated_activation(gu, kind_id)
            np.testing.assert_array_equal(bits_of(y), bits_of(two))
            # the projection itself against the oracle matmul, then the activation on the projection's
            # own 16-bit output (a last-place difference in a factor would otherwise be amplified by
            # the gate function's slope: |g|^2 ulp in GeLU's tail)
            wr = oracle.round_through(w, dt) if resident_rounds_weights(m, dt, kind.startswith("gptq")) else w
            assert_close(gu, oracle.matmul_nt_f32(round_x(x, dt), wr, b), f"gate|up projection {kind} {dtn} m{m}")
            ref = oracle.gated_silu(as_f32(gu)) if act == "silu" else oracle.gated_gelu_tanh(as_f32(gu))
            assert_close(y, ref, f"gate|up {kind} {dtn} {act} m{m}")


@pytest.mark.parametrize("kind", KINDS)
@pytest.mark.parametrize("dtn", ["f16", "bf16"])
@pytest.mark.parametrize("act", ["silu", "gelu"])
@pytest.mark.parametrize("rows", [64, 128])
def test_fused_gate_up_activation_at_prefill(kind, dtn, act, rows):
    """The prefill kernel's own activation epilogue (gate and up columns of an output sit in lanes 8 apart of the
    accumulator layout): bit for bit the plain layer through the same kernel followed by the activation kernel,
    with and without bias, ragged row tiles, a last strip group of one strip (I = 288: nine strips)."""
    tune("OXQ_PK4_GEMM_ROWS", rows)
    dt = DT[dtn]
    tdt = TORCH_DT[dt]
    K, I, g = 512, 288, 128
    trip, pack_dim = make(kind, K, 2 * I, g, seed=17)
    bias = (np.arange(2 * I, dtype=np.float32) % 7 - 3) * np.float32(0.0625)
    kind_id = ops.ACT_GATED_SILU if act == "silu" else ops.ACT_GATED_GELU_TANH
    rng = np.random.default_rng(rows)
    xd = to_dev(rng.standard_normal((581, K)).astype(np.float32), tdt)
    bits = bits_of_kind(kind)
    for b in (None, bias):
        plain = layer_of(trip, pack_dim, dt, b, bits=bits)
        bd = None if b is None else to_dev(b, tdt)
        fused = ops.PackedQuantLinear(bits, pack_dim, to_dev(trip[0]), to_dev(trip[1]), to_dev(trip[2], tdt), bd, tdt,
                                      gate_up_act=kind_id)
        for m in (65, 300, 581):
            say(f"gate|up prefill {kind} {dtn} {act} r{rows} m={m} bias={b is not None}")
            y = fused.forward(xd[:m])
            plan = ops.default_context().last_plan()
            assert plan["kernel"] == f"pk{bits}_gemm_{dtn}_r{rows}x8_{act}" and plan["launches"] == 1, plan
            assert y.shape == (m, I)
            gu = plain.forward(xd[:m])
            assert ops.default_context().last_plan()["kernel"] == f"pk{bits}_gemm_{dtn}_r{rows}x8"
            np.testing.assert_array_equal(bits_of(y), bits_of(ops.gated_activation(gu, kind_id)))
            ref = oracle.gated_silu(as_f32(gu)) if act == "silu" else oracle.gated_gelu_tanh(as_f32(gu))
            assert_close(y, ref, f"gate|up prefill {kind} {dtn} {act} m{m}")


def test_fused_gate_up_benchmark_shape_and_refusals():
    K, I, g = 4096, 14336, 128
    trip = synth.awq_checkpoint(K, 2 * I, g, 4, seed=11)
    args = (4, ops.PACK_OUT, to_dev(trip[0]), to_dev(trip[1]), to_dev(trip[2], torch.float16), None, torch.float16)
    plain = ops.PackedQuantLinear(*args)
    fused = ops.PackedQuantLinear(*args, gate_up_act=ops.ACT_GATED_SILU)
    rng = np.random.default_rng(2)
    for m in (1, 16, 64, 300, 1000):  # 300 rows: 64-row workgroups of the prefill kernel, 1000: 128-row
        x = to_dev(rng.standard_normal((m, K)).astype(np.float32), torch.float16)
        y = fused.forward(x)
        assert ops.default_context().last_plan()["kernel"].endswith("_silu")
        assert ops.default_context().last_plan()["kernel"].startswith("pk4_gemm_f16_r") == (m > 64)
        assert ops.default_context().last_plan()["launches"] == 1
        np.testing.assert_array_equal(bits_of(y), bits_of(ops.gated_activation(plain.forward(x), ops.ACT_GATED_SILU)))
        with pytest.raises(ops.OxqError):
            fused.forward(x, out=torch.empty((m, 2 * I), dtype=torch.float16, device="cuda"))
    # a layer that cannot be made resident has no fused form; a non-gated activation kind is refused
    odd = synth.awq_checkpoint(192, 128, 64, 4, seed=1)
    with pytest.raises(ops.OxqError) as e:
        ops.PackedQuantLinear(4, ops.PACK_OUT, to_dev(odd[0]), to_dev(odd[1]), to_dev(odd[2], torch.float16), None,
                              torch.float16, gate_up_act=ops.ACT_GATED_SILU)
    assert e.value.status == -11
    with pytest.raises(ops.OxqError) as e:
        ops.PackedQuantLinear(*args, gate_up_act=ops.ACT_GPT_OSS_SWIGLU)
    assert e.value.status == -1
