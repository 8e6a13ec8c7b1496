"""GPU parity tests for the GGUF block-quant GEMV and the MXFP4 expert GEMV.

GGUF: no golden vectors exist in the reference (its tests quantize with the
third-party candle QTensor, metal_ops.rs:6405-6417); inputs here are seeded
random block bytes (benchmark config 3) and the oracle is the ggml-format
restatement pinned in test_oracle_kat.py.  Dequant is compared bit for bit,
GEMV at 2e-3 rel / 1e-2 abs of the f32-accumulated oracle.
MXFP4: generators of metal_ops.rs:6622-6670 plus benchmark config 4.
"""
import sys

import numpy as np
import pytest
import torch

import oracle
from oxydllm_amd import synth
from tests import refgen
from tests.helpers import RTOL, ATOL, as_f32, assert_close, bits_of, gguf_on_matrix_cores, round_x, to_dev, tune

pytestmark = pytest.mark.gpu
ops = None
FMTS = [pytest.param(f, id=synth.GGUF_NAMES[f]) for f in sorted(synth.GGUF_NAMES)]


def setup_module(module):
    from oxydllm_amd import ops as _ops
    module.ops = _ops


def say(msg):
    print(f"[case] {msg}", flush=True)
    sys.stdout.flush()


# ------------------------------------------------------------------ GGUF
@pytest.mark.parametrize("fmt", FMTS)
def test_gguf_dequant_bit_exact(fmt):
    say(f"gguf dequant {synth.GGUF_NAMES[fmt]}")
    N, K = 37, 1024
    data = synth.gguf_weight(fmt, N, K, seed=40 + fmt)
    want = oracle.dequantize_gguf(fmt, data, N, K)
    got = ops.gguf_dequantize(to_dev(data), K, N, fmt)
    np.testing.assert_array_equal(got.cpu().numpy().view(np.uint32), want.view(np.uint32))


@pytest.mark.parametrize("fmt", FMTS)
@pytest.mark.parametrize("act", ["f32", "bf16"])
def test_gguf_gemv_config3(fmt, act):
    """Benchmark config 3: M=1, K=N=4096, x~N(0,1) f32 (and the reference's bf16 contract)."""
    say(f"gguf gemv {synth.GGUF_NAMES[fmt]} {act}")
    N = K = 4096
    data = synth.gguf_weight(fmt, N, K, seed=0x0A0D11E8 + fmt)
    w = oracle.dequantize_gguf(fmt, data, N, K)
    x = np.random.default_rng(50 + fmt).standard_normal((1, K)).astype(np.float32)
    if act == "bf16":
        xd, xr = to_dev(x, torch.bfloat16), round_x(x, oracle.BF16)
    else:
        xd, xr = to_dev(x), x
    ref = oracle.matmul_nt_f32(xr, w)
    y = ops.gguf_quant_matmul(xd, to_dev(data), K, N, fmt)
    assert y.shape == (1, N) and y.dtype == xd.dtype
    assert_close(y, ref, f"gguf {synth.GGUF_NAMES[fmt]} {act}")


@pytest.mark.parametrize("fmt", FMTS)
def test_gguf_gemv_batch_and_odd_n(fmt):
    """metal_ops.rs:6544-6617 (M in {2,4,8}) and 6471-6536 (odd N: 1001)."""
    elems, _ = synth.GGUF_BLOCK_LAYOUT[fmt]
    N, K = 1001, 4 * 256
    data = synth.gguf_weight(fmt, N, K, seed=60 + fmt)
    w = oracle.dequantize_gguf(fmt, data, N, K)
    wd = to_dev(data)
    for m in (1, 2, 4, 8):
        say(f"gguf batch {synth.GGUF_NAMES[fmt]} m={m} N={N}")
        x = np.random.default_rng(70 + m).standard_normal((m, K)).astype(np.float32)
        ref = oracle.matmul_nt_f32(round_x(x, oracle.BF16), w)
        y = ops.gguf_quant_matmul(to_dev(x, torch.bfloat16), wd, K, N, fmt)
        assert_close(y, ref, f"gguf batch m{m}")


def _check_mul_mm(y, x, w, what, bias=None):
    """The tile matmul rounds every dequantized weight to bf16 before the matrix unit
    (quant_kernels.metal:2315-2640 write `(bfloat)` tiles): 2e-3 / 1e-2 against that, and the
    reference's own bound (metal_ops.rs:6449-6461) against the unrounded weights."""
    xr = round_x(x, oracle.BF16)
    tile = oracle.matmul_nt_f32(xr, oracle.round_through(w, oracle.BF16), bias)
    assert_close(y, tile, what + " vs bf16-tile oracle", bf16_out=True)
    ref = oracle.matmul_nt_f32(xr, w, bias)
    assert np.abs(as_f32(y) - ref).max() < 0.06 * np.abs(ref).max() + 1e-2


@pytest.mark.parametrize("fmt", FMTS)
@pytest.mark.parametrize("m", [9, 33, 70])
def test_gguf_mul_mm(fmt, m):
    """metal_ops.rs:6387-6463: M in {9, 33, 70}."""
    say(f"gguf mul_mm {synth.GGUF_NAMES[fmt]} m={m}")
    N, K = 200, 512
    data = synth.gguf_weight(fmt, N, K, seed=80 + fmt)
    w = oracle.dequantize_gguf(fmt, data, N, K)
    x = np.random.default_rng(90 + m).standard_normal((m, K)).astype(np.float32)
    y = ops.gguf_quant_mul_mm(to_dev(x, torch.bfloat16), to_dev(data), K, N, fmt)
    assert "mul_mm" in ops.default_context().last_plan()["kernel"]
    _check_mul_mm(y, x, w, f"gguf mul_mm m{m}")
    with pytest.raises(ops.OxqError, match=r"out of \[1, 8\]"):
        ops.gguf_quant_matmul(to_dev(x, torch.bfloat16), to_dev(data), K, N, fmt)


@pytest.mark.parametrize("fmt", FMTS)
@pytest.mark.parametrize("mt,ks", [(4, 1), (1, 1), (2, 1), (4, 3), (2, 5), (1, 2)])
def test_gguf_mul_mm_ragged(fmt, mt, ks, monkeypatch):
    """Odd N (1001: partial row tile, unaligned output rows and a tensor whose last 16-byte
    chunk is partial; 1000 where K is split, which needs N % 4 == 0), m = 150 (token tiles
    with a partial last one), and for the 32-element formats a K that is not a multiple of the
    256-element stage.  The launcher picks tokens per tile and K slices from the grid size;
    every choice is forced over the same ragged shape."""
    elems, _ = synth.GGUF_BLOCK_LAYOUT[fmt]
    N, K, m = (1001 if ks == 1 else 1000), (1024 if elems == 256 else 1120), 150
    say(f"gguf mul_mm ragged {synth.GGUF_NAMES[fmt]} K={K} N={N} mt {mt} ks {ks}")
    tune("OXQ_GGUF_MM_MT", mt)
    tune("OXQ_GGUF_MM_KS", ks)
    data = synth.gguf_weight(fmt, N, K, seed=130 + fmt)
    w = oracle.dequantize_gguf(fmt, data, N, K)
    x = np.random.default_rng(131).standard_normal((m, K)).astype(np.float32)
    bias = np.linspace(-2, 2, N).astype(np.float32)
    layer = ops.QLinear(fmt, to_dev(data), K, N, to_dev(bias, torch.bfloat16), torch.bfloat16)
    y = layer.forward(to_dev(x, torch.bfloat16))
    plan = ops.default_context().last_plan()
    stages = -(-K // 256)
    per_slice = -(-stages // min(ks, stages))
    slices = -(-stages // per_slice)
    assert plan["kernel"].endswith(f"mul_mm_bf16_mt{mt}") and plan["split_k"] == slices
    assert plan["launches"] == (2 if slices > 1 else 1)
    _check_mul_mm(y, x, w, f"gguf mul_mm ragged {synth.GGUF_NAMES[fmt]}", round_x(bias, oracle.BF16))
    y2 = layer.forward(to_dev(x, torch.bfloat16))
    assert torch.equal(y.view(torch.int16), y2.view(torch.int16))


def test_gguf_mul_mm_f32_activations_keep_f32_weights():
    """f32 activations (the reference's CPU contract) never round the weights."""
    fmt, N, K, m = synth.GGUF_Q4_K, 96, 512, 20
    say("gguf mul_mm f32")
    data = synth.gguf_weight(fmt, N, K, seed=140)
    w = oracle.dequantize_gguf(fmt, data, N, K)
    x = np.random.default_rng(141).standard_normal((m, K)).astype(np.float32)
    y = ops.gguf_quant_mul_mm(to_dev(x), to_dev(data), K, N, fmt)
    assert_close(y, oracle.matmul_nt_f32(x, w), "gguf mul_mm f32")


@pytest.mark.parametrize("fmt", FMTS)
def test_gguf_gemv_single_row_wave_per_weight_row(fmt, monkeypatch):
    """One activation row: every wave fetches its own weight row (six 16-byte chunks a lane at most, the
    activations in one batch of four).  Shapes at and past those limits, a last workgroup with fewer rows
    than waves, rows that start off 16-byte boundaries and a tensor whose size is no multiple of 16; the
    result must equal the jointly staged kernel's bit for bit (same arithmetic in the same order) and the
    oracle within tolerance."""
    elems, bbytes = synth.GGUF_BLOCK_LAYOUT[fmt]
    shapes = [(13, 256), (8, 2 * elems if elems == 256 else 96), (37, 4096), (21, 5632), (9, 8192)]
    for N, K in shapes:
        if K % elems:
            continue
        for dt in (torch.float32, torch.bfloat16):
            say(f"gguf wave-per-row {synth.GGUF_NAMES[fmt]} N={N} K={K} {dt}")
            data = synth.gguf_weight(fmt, N, K, seed=N + K + fmt)
            w = oracle.dequantize_gguf(fmt, data, N, K)
            x = np.random.default_rng(N * 7 + K).standard_normal((1, K)).astype(np.float32)
            xd, wd = to_dev(x, dt), to_dev(data)
            xr = x if dt == torch.float32 else round_x(x, oracle.BF16)
            tune("OXQ_GGUF_PW", 1)
            y = ops.gguf_quant_matmul(xd, wd, K, N, fmt)
            assert_close(y, oracle.matmul_nt_f32(xr, w), f"gguf wave-per-row {synth.GGUF_NAMES[fmt]} {N}x{K}")
            tune("OXQ_GGUF_PW", 0)
            joint = ops.gguf_quant_matmul(xd, wd, K, N, fmt)
            np.testing.assert_array_equal(bits_of(y), bits_of(joint))
    tune("OXQ_GGUF_PW", None)


@pytest.mark.parametrize("fmt", FMTS)
def test_gguf_gemv_long_rows(fmt, monkeypatch):
    """K = 8192 with 8 activation rows does not fit the staged variant's LDS budget in one pass: the rows go
    through it in passes of as many as fit; the direct one-wave-per-row kernel (shapes that never fit, here
    forced) must agree as well."""
    N, K, m = 160, 8192, 8
    say(f"gguf long rows {synth.GGUF_NAMES[fmt]}")
    data = synth.gguf_weight(fmt, N, K, seed=120 + fmt)
    w = oracle.dequantize_gguf(fmt, data, N, K)
    x = np.random.default_rng(121).standard_normal((m, K)).astype(np.float32)
    ref = oracle.matmul_nt_f32(x, w)
    y = ops.gguf_quant_matmul(to_dev(x), to_dev(data), K, N, fmt)   # f32 activations: always the GEMV kernels
    plan = ops.default_context().last_plan()
    assert plan["kernel"].endswith("gemv_f32_lds") and plan["launches"] in (2, 4, 8), plan
    assert_close(y, ref, f"gguf long rows {synth.GGUF_NAMES[fmt]}")
    tune("OXQ_FORCE_GENERIC", 1)
    y = ops.gguf_quant_matmul(to_dev(x), to_dev(data), K, N, fmt)
    kernel = ops.default_context().last_plan()["kernel"]
    assert kernel.endswith("gemv_f32") and not kernel.endswith("_lds")
    assert_close(y, ref, f"gguf long rows, wave per row {synth.GGUF_NAMES[fmt]}")
    tune("OXQ_FORCE_GENERIC", None)
    # bf16 rows of the decode range take the staged GEMV up to 2 rows and the tile matmul with
    # unrounded (hi + lo) weights from 3: both are held to the unrounded oracle
    for mb in (2, 3, 8):
        xb = x[:mb]
        yb = ops.gguf_quant_matmul(to_dev(xb, torch.bfloat16), to_dev(data), K, N, fmt)
        kernel = ops.default_context().last_plan()["kernel"]
        assert ("gemv" in kernel) if mb <= 2 else kernel.endswith("mul_mm_bf16_mt1_f32w")
        assert_close(yb, oracle.matmul_nt_f32(round_x(xb, oracle.BF16), w), f"gguf decode rows m={mb}")


def test_qlinear_layer_bias_and_routing():
    """linear.rs:324-351: decode vs prefill routing, out dtype, bias."""
    say("QLinear")
    fmt, N, K = synth.GGUF_Q4_K, 96, 512
    data = synth.gguf_weight(fmt, N, K, seed=99)
    w = oracle.dequantize_gguf(fmt, data, N, K)
    bias = np.linspace(-1, 1, N).astype(np.float32)
    layer = ops.QLinear(fmt, to_dev(data), K, N, to_dev(bias, torch.bfloat16), torch.bfloat16)
    for shape in [(1, K), (2, 4, K), (3, 5, K), (5, 8, K)]:
        m = int(np.prod(shape[:-1]))
        x = np.random.default_rng(m).standard_normal((m, K)).astype(np.float32)
        y = layer.forward(to_dev(x.reshape(shape), torch.bfloat16))
        assert tuple(y.shape) == shape[:-1] + (N,)
        if m <= 8 or gguf_on_matrix_cores(fmt, N, K, m):  # the matrix-core copy keeps the GEMV's unrounded weights
            ref = oracle.matmul_nt_f32(round_x(x, oracle.BF16), w, round_x(bias, oracle.BF16))
            assert_close(y.reshape(m, N), ref, f"QLinear {shape}")
        else:  # prefill: the tile matmul
            _check_mul_mm(y.reshape(m, N), x, w, f"QLinear {shape}", round_x(bias, oracle.BF16))


# ------------------------------------------------------------------ MXFP4
def test_mxfp4_dequant_bit_exact():
    say("mxfp4 dequant")
    n, k = 64, 2880
    blocks, scales = synth.mxfp4_weight(n, k, seed=7, exp_lo=0, exp_hi=254)
    blocks[:16] = np.arange(16, dtype=np.uint8) * 17  # every code in both nibbles
    scales[3] = 255                                   # E8M0 NaN encoding (mxfp4.rs:26-29)
    want = oracle.dequantize_mxfp4_f32(blocks, scales, n, k)
    got = ops.mxfp4_dequantize(to_dev(blocks), to_dev(scales), k, n).cpu().numpy()
    nan = np.isnan(want)
    assert nan.any() and np.array_equal(np.isnan(got), nan)
    np.testing.assert_array_equal(got.view(np.uint32)[~nan], want.view(np.uint32)[~nan])


@pytest.mark.parametrize("m", [1, 4, 8, 33])
def test_mxfp4_matmul_reference_case(m):
    """metal_ops.rs:6622-6670: n=10 (unaligned), k=64, M in {1,4,8,33}."""
    say(f"mxfp4 matmul m={m}")
    n, k = 10, 64
    blocks, scales = refgen.mxfp4_case(n, k)
    w = oracle.dequantize_mxfp4_f32(blocks, scales, n, k)
    x = refgen.mxfp4_x(m, k)
    ref = oracle.matmul_nt_f32(round_x(x, oracle.BF16), w)
    y = ops.mxfp4_matmul(to_dev(x, torch.bfloat16), to_dev(blocks), to_dev(scales), k, n)
    assert y.shape == (m, n) and y.dtype == torch.bfloat16
    assert_close(y, ref, f"mxfp4 m{m}")


def _config4(seed=0x0A0D11E9):
    E, top_k, hidden, inter, T = 32, 4, 2880, 2880, 8
    rng = np.random.default_rng(seed)
    gu_b, gu_s = synth.mxfp4_weight(E * 2 * inter, hidden, seed=seed + 1)
    dn_b, dn_s = synth.mxfp4_weight(E * hidden, inter, seed=seed + 2)
    gu_bias = (rng.standard_normal((E, 2 * inter)) * 0.1).astype(np.float32)
    dn_bias = (rng.standard_normal((E, hidden)) * 0.1).astype(np.float32)
    x = rng.standard_normal((T, hidden)).astype(np.float32)
    logits = rng.standard_normal((T, E)).astype(np.float32)
    return dict(E=E, top_k=top_k, hidden=hidden, inter=inter, T=T, gu_b=gu_b, gu_s=gu_s, dn_b=dn_b,
                dn_s=dn_s, gu_bias=gu_bias, dn_bias=dn_bias, x=x, logits=logits)


@pytest.mark.parametrize("m,n,k", [(17, 10, 64), (33, 100, 96), (150, 1000, 1120), (150, 1001, 2880), (64, 5760, 2880)])
def test_mxfp4_mul_mm(m, n, k, monkeypatch):
    """m > 16 runs the tile matmul (metal_ops.rs:6197-6223 switches to mul_mm above 8 rows).
    E2M1 x E8M0 is exact in bf16, so the tile form matches the unrounded oracle; shapes cover
    the reference's n = 10, k = 64 case, partial row and token tiles, K that is not a multiple
    of the 256-element stage, odd N, and split K (forced for the small shapes)."""
    say(f"mxfp4 mul_mm m={m} n={n} k={k}")
    blocks, scales = synth.mxfp4_weight(n, k, seed=m + n)
    w = oracle.dequantize_mxfp4_f32(blocks, scales, n, k)
    x = np.random.default_rng(m).standard_normal((m, k)).astype(np.float32)
    ref = oracle.matmul_nt_f32(round_x(x, oracle.BF16), w)
    bd, sd, xd = to_dev(blocks), to_dev(scales), to_dev(x, torch.bfloat16)
    y = ops.mxfp4_matmul(xd, bd, sd, k, n)
    plan = ops.default_context().last_plan()
    assert plan["kernel"].startswith("mxfp4_mul_mm_bf16")
    assert_close(y, ref, f"mxfp4 mul_mm {m}x{n}x{k}")
    if n % 4 == 0 and k >= 512:
        tune("OXQ_MXFP4_MM_KS", 3)
        y3 = ops.mxfp4_matmul(xd, bd, sd, k, n)
        assert ops.default_context().last_plan()["split_k"] > 1
        assert_close(y3, ref, f"mxfp4 mul_mm split {m}x{n}x{k}")
    # the decode kernel on the same rows agrees within the tolerance as well
    tune("OXQ_MXFP4_MM", 0)
    y0 = ops.mxfp4_matmul(xd, bd, sd, k, n)
    assert "gemv" in ops.default_context().last_plan()["kernel"]
    assert_close(y0, ref, f"mxfp4 gemv form {m}x{n}x{k}")


@pytest.mark.parametrize("T,E,top_k,N,K", [(64, 8, 2, 200, 320), (300, 4, 2, 130, 576), (40, 32, 4, 64, 64)])
def test_mxfp4_moe_prefill_grouped(T, E, top_k, N, K, monkeypatch):
    """Grouped tile matmul: many routed pairs per expert (prefill).  Experts with no, few and
    more than one tile of tokens; gathered rows (gate_up) and identity rows (down)."""
    say(f"mxfp4 moe prefill T={T} E={E} top{top_k} N={N} K={K}")
    rng = np.random.default_rng(T + E)
    logits = rng.standard_normal((T, E)).astype(np.float32)
    logits[:, 1] = -30.0  # expert 1 never routed
    idx, vals = oracle.moe_route(logits, top_k, True)
    offsets, tokens, _ = oracle.moe_group(idx, vals, E)
    n_pairs = int(offsets[-1])
    nb = K // 32
    blocks, scales = synth.mxfp4_weight(E * N, K, seed=E)
    bias = rng.standard_normal((E, N)).astype(np.float32) * 0.1
    x = rng.standard_normal((T, K)).astype(np.float32)
    xb, bb = round_x(x, oracle.BF16), round_x(bias, oracle.BF16)
    ref = np.zeros((n_pairs, N), np.float32)
    for e in range(E):
        lo, hi = int(offsets[e]), int(offsets[e + 1])
        if hi > lo:
            w = oracle.dequantize_mxfp4_f32(blocks[e * N * nb * 16:(e + 1) * N * nb * 16],
                                            scales[e * N * nb:(e + 1) * N * nb], N, K)
            ref[lo:hi] = oracle.matmul_nt_f32(xb[tokens[lo:hi]], w, bb[e])
    off_d, tok_d = to_dev(offsets.astype(np.int32)), to_dev(tokens.astype(np.int32))
    tune("OXQ_MXFP4_MM", 1)
    y = ops.mxfp4_moe_matmul(to_dev(x, torch.bfloat16), to_dev(blocks), to_dev(scales),
                             to_dev(bias, torch.bfloat16), off_d, tok_d, K, N)
    assert ops.default_context().last_plan()["kernel"].startswith("mxfp4_moe_mul_mm_bf16")
    assert_close(y, ref, "moe prefill gathered")
    xp = x[tokens]  # identity rows: one activation row per pair
    y2 = ops.mxfp4_moe_matmul(to_dev(xp, torch.bfloat16), to_dev(blocks), to_dev(scales),
                              to_dev(bias, torch.bfloat16), off_d, None, K, N)
    assert_close(y2, ref, "moe prefill identity rows")
    tune("OXQ_MXFP4_MM", 0)
    y0 = ops.mxfp4_moe_matmul(to_dev(x, torch.bfloat16), to_dev(blocks), to_dev(scales),
                              to_dev(bias, torch.bfloat16), off_d, tok_d, K, N)
    assert "gemv" in ops.default_context().last_plan()["kernel"]
    assert_close(y0, ref, "moe prefill through the decode kernel")


def test_mxfp4_moe_config4():
    """Benchmark config 4: 32 experts, top-4, hidden 2880, gate_up N=5760, down K=2880, 8 tokens.
    Routing lists come from the oracle's restatement of moe.rs:466-607."""
    c = _config4()
    E, H, I = c["E"], c["hidden"], c["inter"]
    idx, vals = oracle.moe_route(c["logits"], c["top_k"], True)
    offsets, tokens, _ = oracle.moe_group(idx, vals, E)
    n_pairs = int(offsets[-1])
    assert n_pairs == c["T"] * c["top_k"]
    say(f"mxfp4 moe gate_up: {int((np.diff(offsets) > 0).sum())} active experts, {n_pairs} pairs")
    xb = round_x(c["x"], oracle.BF16)
    gub = round_x(c["gu_bias"], oracle.BF16)
    dnb = round_x(c["dn_bias"], oracle.BF16)
    nb = H // 32

    # oracle, per active expert (Mxfp4Linear::forward = x.W^T + bias, mxfp4.rs:119-154)
    ref_gu = np.zeros((n_pairs, 2 * I), np.float32)
    ref_dn = np.zeros((n_pairs, H), np.float32)
    h_in = np.random.default_rng(5).standard_normal((n_pairs, I)).astype(np.float32)
    hb = round_x(h_in, oracle.BF16)
    for e in range(E):
        lo, hi = int(offsets[e]), int(offsets[e + 1])
        if hi == lo:
            continue
        wg = oracle.dequantize_mxfp4_f32(c["gu_b"][e * 2 * I * nb * 16:(e + 1) * 2 * I * nb * 16],
                                         c["gu_s"][e * 2 * I * nb:(e + 1) * 2 * I * nb], 2 * I, H)
        ref_gu[lo:hi] = oracle.matmul_nt_f32(xb[tokens[lo:hi]], wg, gub[e])
        wd = oracle.dequantize_mxfp4_f32(c["dn_b"][e * H * nb * 16:(e + 1) * H * nb * 16],
                                         c["dn_s"][e * H * nb:(e + 1) * H * nb], H, I)
        ref_dn[lo:hi] = oracle.matmul_nt_f32(hb[lo:hi], wd, dnb[e])

    off_d = to_dev(offsets.astype(np.int32))
    tok_d = to_dev(tokens.astype(np.int32))
    y = ops.mxfp4_moe_matmul(to_dev(c["x"], torch.bfloat16), to_dev(c["gu_b"]), to_dev(c["gu_s"]),
                             to_dev(c["gu_bias"], torch.bfloat16), off_d, tok_d, H, 2 * I)
    assert y.shape == (n_pairs, 2 * I)
    assert_close(y, ref_gu, "moe gate_up")
    say("mxfp4 moe down")
    y2 = ops.mxfp4_moe_matmul(to_dev(h_in, torch.bfloat16), to_dev(c["dn_b"]), to_dev(c["dn_s"]),
                              to_dev(c["dn_bias"], torch.bfloat16), off_d, None, I, H)
    assert_close(y2, ref_dn, "moe down")

    # one expert through the layer type equals its slice of the grouped launch
    e = int(np.argmax(np.diff(offsets)))
    lo, hi = int(offsets[e]), int(offsets[e + 1])
    say(f"Mxfp4Linear expert {e} rows {hi - lo}")
    lay = ops.Mxfp4Linear(to_dev(c["gu_b"][e * 2 * I * nb * 16:(e + 1) * 2 * I * nb * 16]),
                          to_dev(c["gu_s"][e * 2 * I * nb:(e + 1) * 2 * I * nb]),
                          to_dev(c["gu_bias"][e], torch.bfloat16), H, 2 * I)
    ys = lay.forward(to_dev(c["x"][tokens[lo:hi]], torch.bfloat16))
    assert_close(ys, ref_gu[lo:hi], "Mxfp4Linear")
    assert torch.equal(ys, y[lo:hi])


# ------------------------------------------------------------------ mixture-of-experts glue
@pytest.mark.parametrize("dt", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("T,E,k,norm", [(8, 32, 4, True), (1, 128, 8, True), (70, 64, 2, False), (5, 300, 6, True)])
def test_moe_route_matches_oracle(dt, T, E, k, norm):
    """moe.rs:466-486.  Expert ids must agree exactly, gate values to 1e-5 relative (device expf)."""
    say(f"moe route {dt} T={T} E={E} k={k}")
    rng = np.random.default_rng(T * E + k)
    logits = (rng.standard_normal((T, E)) * 2).astype(np.float32)
    ld = to_dev(logits, dt)
    lg = ld.float().cpu().numpy()  # what the kernel sees after the dtype cast
    ridx, rvals = oracle.moe_route(lg, k, norm)
    idx, vals = ops.moe_route(ld, k, norm)
    np.testing.assert_array_equal(idx.cpu().numpy().astype(np.uint32), ridx)
    np.testing.assert_allclose(vals.cpu().numpy(), rvals, rtol=1e-5, atol=1e-7)


def test_moe_route_ties_keep_expert_order():
    """Stable descending sort: equal scores keep ascending expert order (arg_sort_last_dim)."""
    say("moe route ties")
    logits = np.zeros((3, 16), np.float32)
    logits[1, [5, 9, 2]] = 1.0
    logits[2, :] = np.arange(16) % 4
    ridx, _ = oracle.moe_route(logits, 4, True)
    idx, _ = ops.moe_route(to_dev(logits), 4, True)
    np.testing.assert_array_equal(idx.cpu().numpy().astype(np.uint32), ridx)
    np.testing.assert_array_equal(ridx[0], [0, 1, 2, 3])


@pytest.mark.parametrize("E,k", [(32, 4), (200, 6)])
def test_moe_route_rows_without_an_order_stay_in_range(E, k):
    """A NaN or +inf logit makes every probability of its row NaN.  A stable sort leaves such a row in index
    order (the oracle, like arg_sort_last_dim, then returns experts 0..k-1 with NaN weights); the device must
    do the same: ids inside [0, E), so that grouping still places every pair."""
    say(f"moe route NaN rows E={E} k={k}")
    rng = np.random.default_rng(E)
    logits = rng.standard_normal((6, E)).astype(np.float32)
    logits[1, E // 2] = np.nan
    logits[3, 0] = np.nan
    logits[4, E - 1] = np.inf
    ridx, rvals = oracle.moe_route(logits, k, True)
    for r in (1, 3, 4):
        np.testing.assert_array_equal(ridx[r], np.arange(k))
        assert np.isnan(rvals[r]).all()
    for fn in (lambda: ops.moe_route(to_dev(logits), k, True), lambda: ops.moe_route_group(to_dev(logits), k, True)[:2]):
        idx, vals = fn()
        idx, vals = idx.cpu().numpy(), vals.cpu().numpy()
        np.testing.assert_array_equal(idx.astype(np.uint32), ridx)
        np.testing.assert_array_equal(np.isnan(vals), np.isnan(rvals))
        ok = ~np.isnan(rvals)
        np.testing.assert_allclose(vals[ok], rvals[ok], rtol=1e-5, atol=1e-7)
    _, _, off, tok, _, pos = ops.moe_route_group(to_dev(logits), k, True)
    roff, rtok, _ = oracle.moe_group(ridx, rvals, E)
    np.testing.assert_array_equal(off.cpu().numpy(), roff.astype(np.int32))
    np.testing.assert_array_equal(tok.cpu().numpy(), rtok.astype(np.int32))
    assert sorted(pos.cpu().numpy().ravel().tolist()) == list(range(6 * k))


@pytest.mark.parametrize("T,E,k", [(8, 32, 4), (1, 32, 4), (16, 64, 4), (5, 200, 3), (13, 256, 5), (257, 16, 2),
                                   (1000, 256, 8)])
def test_moe_group_matches_oracle(T, E, k):
    """moe.rs:563-590: integer work, compared exactly."""
    say(f"moe group T={T} E={E} k={k}")
    rng = np.random.default_rng(T + E)
    logits = rng.standard_normal((T, E)).astype(np.float32)
    ridx, rvals = oracle.moe_route(logits, k, True)
    roff, rtok, rw = oracle.moe_group(ridx, rvals, E)
    off, tok, w, pos = ops.moe_group(to_dev(ridx.astype(np.int32)), to_dev(rvals), E)
    np.testing.assert_array_equal(off.cpu().numpy(), roff.astype(np.int32))
    np.testing.assert_array_equal(tok.cpu().numpy(), rtok.astype(np.int32))
    np.testing.assert_array_equal(w.cpu().numpy(), rw)
    pos = pos.cpu().numpy()
    assert sorted(pos.ravel().tolist()) == list(range(T * k))
    np.testing.assert_array_equal(rtok[pos.ravel()], np.repeat(np.arange(T), k))
    np.testing.assert_array_equal(rw[pos.ravel()], rvals.ravel())


@pytest.mark.parametrize("T,E,k,norm", [(8, 32, 4, True), (1, 32, 4, True), (16, 64, 4, False), (5, 200, 3, True),
                                         (64, 16, 1, True), (13, 256, 5, True), (17, 32, 4, True), (300, 8, 2, False)])
def test_moe_route_group_equals_the_two_calls(T, E, k, norm):
    """moe.rs:466-486 + 563-590 in one call: identical outputs to route followed by group, as one launch up to
    64 pairs and as the two launches beyond."""
    say(f"moe_route_group T={T} E={E} k={k}")
    logits = torch.from_numpy(np.random.default_rng(T * E + k).standard_normal((T, E)).astype(np.float32)).cuda()
    for dt in (torch.float32, torch.bfloat16):
        lg = logits.to(dt)
        idx, vals = ops.moe_route(lg, k, norm)
        want = (idx, vals) + tuple(ops.moe_group(idx, vals, E))
        got = ops.moe_route_group(lg, k, norm)
        assert ops.default_context().last_plan()["kernel"] == ("moe_route_group" if T * k <= 64 else "moe_group")
        for a, b, name in zip(got, want, ("top_idx", "top_vals", "expert_offsets", "token_ids", "pair_weights", "pair_pos")):
            assert a.dtype == b.dtype and a.shape == b.shape, name
            assert torch.equal(a.view(torch.int32), b.view(torch.int32)), name
    with pytest.raises(ops.OxqError, match="top_k"):
        ops.moe_route_group(logits, E + 1)


@pytest.mark.parametrize("dt", [torch.float32, torch.bfloat16, torch.float16])
def test_gated_activations_match_oracle(dt, monkeypatch):
    tune("OXQ_ACT_VEC", 1)      # the 8-outputs-a-thread kernel at test sizes too
    """ffn_kernels.metal:19-242 and moe.rs:152-173: f32 math, one rounding to the tensor dtype."""
    say(f"gated activations {dt}")
    rng = np.random.default_rng(3)
    odt = {torch.float32: None, torch.bfloat16: oracle.BF16, torch.float16: oracle.F16}[dt]
    for rows, half in [(7, 96), (5, 37), (3, 8), (2, 20)]:   # whole 16-byte pieces per half (8 outputs a thread) and not
        gu = (rng.standard_normal((rows, 2 * half)) * 3).astype(np.float32)
        gd = to_dev(gu, dt)
        gr = gd.float().cpu().numpy()
        for kind, ref in [(ops.ACT_GATED_SILU, oracle.gated_silu(gr)), (ops.ACT_GATED_GELU_TANH, oracle.gated_gelu_tanh(gr)),
                          (ops.ACT_GPT_OSS_SWIGLU, oracle.gpt_oss_swiglu(gr, 7.0))]:
            y = ops.gated_activation(gd, kind, 7.0)
            assert y.shape == (rows, half) and y.dtype == dt
            assert_close(y, ref, f"gated act {kind} {dt} {rows}x{half}", rtol=1e-5 if odt is None else RTOL,
                         atol=1e-5 if odt is None else ATOL, bf16_out=dt == torch.bfloat16)
            if half % 8 == 0 and dt != torch.float32:
                # the same rows inside a wider, odd-width tensor take the one-output-a-thread kernel: same bits
                wide = torch.zeros((rows, 2 * (half + 1)), dtype=dt, device="cuda")
                if kind == ops.ACT_GPT_OSS_SWIGLU:
                    wide[:, :2 * half] = gd
                else:
                    wide[:, :half] = gd[:, :half]
                    wide[:, half + 1:2 * half + 1] = gd[:, half:]
                y1 = ops.gated_activation(wide, kind, 7.0)[:, :half]
                assert torch.equal(y.view(torch.int16), y1.contiguous().view(torch.int16))
    gu = (rng.standard_normal((7, 2 * 96)) * 3).astype(np.float32)
    with pytest.raises(ops.OxqError, match="2 \\* intermediate_size"):
        ops.gated_activation(to_dev(gu[:, :191].copy(), dt), ops.ACT_GATED_SILU)


@pytest.mark.parametrize("dt", [torch.float32, torch.bfloat16, torch.float16])
def test_two_tensor_activations_match_oracle_and_the_fused_tensor_form(dt):
    """metal_ops.rs:1252/1271 (ffn_kernels.metal:72-110, 164-200): act(gate) * up over separate tensors equals
    the oracle and, bit for bit, the [gate | up] form on the concatenation; errors as metal_ops.rs:649-662."""
    say(f"two-tensor activations {dt}")
    rng = np.random.default_rng(8)
    for shape in [(5, 96), (3, 2, 77), (1, 1), (0, 8)]:
        g = (rng.standard_normal(shape) * 3).astype(np.float32)
        u = (rng.standard_normal(shape) * 3).astype(np.float32)
        if g.size:
            g.flat[0] = -90.0  # silu underflows towards -0 here: the sign of the product must survive
        gd, ud = to_dev(g, dt), to_dev(u, dt)
        both = torch.cat([gd, ud], dim=-1)
        br = both.float().cpu().numpy()
        for fn, kind, ref in [(ops.silu_mul, ops.ACT_GATED_SILU, oracle.gated_silu),
                              (ops.gelu_tanh_mul, ops.ACT_GATED_GELU_TANH, oracle.gated_gelu_tanh)]:
            y = fn(gd, ud)
            assert y.shape == gd.shape and y.dtype == dt
            if g.size:
                lo = dt != torch.float32
                want = ref(br.reshape(-1, br.shape[-1])).reshape(shape)
                assert_close(y, want, f"{fn.__name__} {dt} {shape}", rtol=RTOL if lo else 1e-5,
                             atol=ATOL if lo else 1e-5, bf16_out=dt == torch.bfloat16)
                ints = torch.int32 if dt == torch.float32 else torch.int16
                same = ops.gated_activation(both, kind)
                assert torch.equal(y.reshape(-1).view(ints), same.reshape(-1).view(ints))
            else:
                assert y.numel() == 0
    g, u = to_dev(np.ones((2, 8), np.float32), dt), to_dev(np.ones((2, 8), np.float32), dt)
    with pytest.raises(ops.OxqError, match="shape mismatch"):
        ops.silu_mul(g, u[:, :4].contiguous())
    with pytest.raises(ops.OxqError, match="both inputs must be contiguous"):
        ops.gelu_tanh_mul(g, u.t().contiguous().t())
    other = torch.float16 if dt != torch.float16 else torch.bfloat16
    with pytest.raises(ops.OxqError, match="dtype mismatch"):
        ops.silu_mul(g, u.to(other))
    with pytest.raises(ops.OxqError, match="no two-tensor form"):
        ops.activation_mul(g, u, ops.ACT_GPT_OSS_SWIGLU)


def test_moe_step_config4_end_to_end():
    """Benchmark config 4 as one device-side pipeline: route -> group -> gate_up -> GPT-OSS SwiGLU ->
    down -> combine, against the oracle restating moe.rs:466-607 + 152-173 step by step (each
    intermediate rounded to bf16 where the device stores bf16)."""
    c = _config4()
    E, H, I, T, k = c["E"], c["hidden"], c["inter"], c["T"], c["top_k"]
    say("moe step end to end")
    nb = H // 32
    xb = round_x(c["x"], oracle.BF16)
    gub, dnb = round_x(c["gu_bias"], oracle.BF16), round_x(c["dn_bias"], oracle.BF16)
    ridx, rvals = oracle.moe_route(c["logits"], k, True)
    roff, rtok, rw = oracle.moe_group(ridx, rvals, E)
    P = T * k
    gu_ref = np.zeros((P, 2 * I), np.float32)
    for e in range(E):
        lo, hi = int(roff[e]), int(roff[e + 1])
        if hi > lo:
            wg = oracle.dequantize_mxfp4_f32(c["gu_b"][e * 2 * I * nb * 16:(e + 1) * 2 * I * nb * 16],
                                             c["gu_s"][e * 2 * I * nb:(e + 1) * 2 * I * nb], 2 * I, H)
            gu_ref[lo:hi] = oracle.matmul_nt_f32(xb[rtok[lo:hi]], wg, gub[e])
    h_ref = round_x(oracle.gpt_oss_swiglu(round_x(gu_ref, oracle.BF16), 7.0), oracle.BF16)
    dn_ref = np.zeros((P, H), np.float32)
    for e in range(E):
        lo, hi = int(roff[e]), int(roff[e + 1])
        if hi > lo:
            wd = oracle.dequantize_mxfp4_f32(c["dn_b"][e * H * nb * 16:(e + 1) * H * nb * 16],
                                             c["dn_s"][e * H * nb:(e + 1) * H * nb], H, I)
            dn_ref[lo:hi] = oracle.matmul_nt_f32(h_ref[lo:hi], wd, dnb[e])
    out_ref = oracle.moe_combine(round_x(dn_ref, oracle.BF16), roff, rtok, rw, T)

    xd = to_dev(c["x"], torch.bfloat16)
    idx, vals = ops.moe_route(to_dev(c["logits"]), k, True)
    off, tok, w, pos = ops.moe_group(idx, vals, E)
    np.testing.assert_array_equal(off.cpu().numpy(), roff.astype(np.int32))
    gu = ops.mxfp4_moe_matmul(xd, to_dev(c["gu_b"]), to_dev(c["gu_s"]), to_dev(c["gu_bias"], torch.bfloat16),
                              off, tok, H, 2 * I)
    h = ops.gated_activation(gu, ops.ACT_GPT_OSS_SWIGLU, 7.0)
    # the same two steps as one launch: bit-identical
    h1 = ops.mxfp4_moe_gate_up_swiglu(xd, to_dev(c["gu_b"]), to_dev(c["gu_s"]), to_dev(c["gu_bias"], torch.bfloat16),
                                      off, tok, H, 2 * I, 7.0)
    plan = ops.default_context().last_plan()
    assert plan["kernel"].endswith("_swiglu") and plan["launches"] == 1, plan
    np.testing.assert_array_equal(h1.view(torch.int16).cpu().numpy(), h.view(torch.int16).cpu().numpy())
    dn = ops.mxfp4_moe_matmul(h, to_dev(c["dn_b"]), to_dev(c["dn_s"]), to_dev(c["dn_bias"], torch.bfloat16),
                              off, None, I, H)
    out = ops.moe_combine(dn, pos, vals)
    assert out.shape == (T, H) and out.dtype == torch.bfloat16
    # three bf16 roundings sit between the oracle's and the device's intermediates: compare with the
    # reference's own end-to-end bound (moe.rs:705-788: 1e-3 * max + 1e-3, widened for bf16 storage)
    err = np.abs(out.float().cpu().numpy() - out_ref)
    assert err.max() < 2e-2 * np.abs(out_ref).max() + 1e-2, err.max()


@pytest.mark.parametrize("dtn", ["bf16", "f16"])
@pytest.mark.parametrize("T,H,k", [(700, 768, 4), (260, 2880, 4), (1200, 512, 8), (300, 2884, 4)])
def test_moe_combine_at_prefill_sizes(dtn, T, H, k):
    """moe.rs:592-605 at prefill sizes: from 2^19 outputs on, 16-bit types and H a multiple of 8 take eight columns a
    thread (16-byte loads and stores); the sums run in slot order in f32 either way, so the result equals the slot
    loop restated in torch bit for bit, and the scalar kernel's (an output buffer that starts 8 bytes off a 16-byte
    boundary takes that one).  H = 2884 is not a multiple of 8: the scalar kernel."""
    tdt = torch.bfloat16 if dtn == "bf16" else torch.float16
    say(f"moe combine {dtn} T={T} H={H} k={k}")
    g = torch.Generator(device="cpu").manual_seed(T + H)
    P = T * k
    eo = torch.randn((P, H), generator=g).to(tdt).cuda()
    pos = torch.randperm(P, generator=g).to(torch.int32).view(T, k).cuda()
    vals = torch.rand((T, k), generator=g).cuda()
    out = ops.moe_combine(eo, pos, vals)
    vec = H % 8 == 0
    assert ops.default_context().last_plan()["kernel"] == ("moe_combine_x8" if vec else "moe_combine")
    acc = torch.zeros((T, H), device="cuda", dtype=torch.float32)
    for s in range(k):  # fmaf(w, v, acc) in slot order; the product of a 16-bit value and an f32 weight needs the fma
        acc = torch.addcmul(acc.double(), vals[:, s:s + 1].double(), eo[pos[:, s].long()].double()).float()
    want = acc.to(tdt)
    assert torch.equal(out.view(torch.int16), want.view(torch.int16))
    buf = torch.zeros(T * H + 4, device="cuda", dtype=tdt)
    off = buf[4:].view(T, H)
    ops.moe_combine(eo, pos, vals, out=off)
    assert ops.default_context().last_plan()["kernel"] == "moe_combine"
    assert torch.equal(off.view(torch.int16), out.view(torch.int16))


@pytest.mark.parametrize("E,N,K,counts,bias", [(4, 64, 64, (1, 0, 3, 2), True), (3, 38, 96, (5, 1, 0), False),
                                               (2, 6, 32, (9, 4), True), (5, 130, 160, (0, 0, 2, 0, 1), True)])
def test_mxfp4_moe_gate_up_swiglu_fused(E, N, K, counts, bias, monkeypatch):
    """Fused gate_up + GPT-OSS SwiGLU against the two calls it replaces (bit for bit) on ragged shapes:
    idle experts, more than four pairs per expert (two passes over the tokens), a row count that is not
    a multiple of 16, with and without bias, gathered and direct rows; and the declined case (tile
    matmul sizes), where the wrapper makes the two calls."""
    rng = np.random.default_rng(E * 100 + N)
    blocks = np.concatenate([synth.mxfp4_weight(N, K, seed=10 + e)[0] for e in range(E)])
    scales = np.concatenate([synth.mxfp4_weight(N, K, seed=10 + e)[1] for e in range(E)])
    b = to_dev(rng.standard_normal((E, N)).astype(np.float32), torch.bfloat16) if bias else None
    offsets = np.concatenate([[0], np.cumsum(counts)]).astype(np.int32)
    P = int(offsets[-1])
    T = 6
    tok = rng.integers(0, T, size=P).astype(np.int32)
    x = to_dev(rng.standard_normal((T, K)).astype(np.float32) * 2.0, torch.bfloat16)
    bd, sd, od, td = to_dev(blocks), to_dev(scales), to_dev(offsets), to_dev(tok)
    for gather in (True, False):
        xs = x if gather else x[torch.from_numpy(tok).long().cuda()].contiguous()
        tk = td if gather else None
        say(f"fused swiglu E={E} N={N} K={K} gather={gather}")
        tune("OXQ_MXFP4_MM", 0)
        two = ops.gated_activation(ops.mxfp4_moe_matmul(xs, bd, sd, b, od, tk, K, N), ops.ACT_GPT_OSS_SWIGLU, 7.0)
        one = ops.mxfp4_moe_gate_up_swiglu(xs, bd, sd, b, od, tk, K, N, 7.0)
        assert ops.default_context().last_plan()["kernel"].endswith("_swiglu")
        assert one.shape == (P, N // 2)
        np.testing.assert_array_equal(one.view(torch.int16).cpu().numpy(), two.view(torch.int16).cpu().numpy())
        tune("OXQ_MXFP4_MM", 1)      # the tile matmul declines the fused form
        alt = ops.mxfp4_moe_gate_up_swiglu(xs, bd, sd, b, od, tk, K, N, 7.0)
        assert ops.default_context().last_plan()["kernel"] == "gpt_oss_swiglu"
        assert_close(alt, as_f32(two), "declined path", bf16_out=True)
    with pytest.raises(ops.OxqError):                # odd n cannot be interleaved pairs
        ops.mxfp4_moe_gate_up_swiglu(x, bd, sd, None, od, td, K, N - 1, 7.0, out=torch.empty((P, N // 2), dtype=torch.bfloat16, device="cuda"))
