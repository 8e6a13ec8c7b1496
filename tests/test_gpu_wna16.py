"""GPU parity tests for the AWQ / GPTQ path, through the C ABI.

Every kernel result is compared with the CPU oracle on identical inputs:
  dequantized tiles  bit-exact (integer compare of the 16-bit patterns);
  GEMV / GEMM        2e-3 relative / 1e-2 absolute of the f32-accumulated
                     x_f32 . dequant(W)^T, the tolerance the task states
                     (the reference's own tests use 0.06*max|ref| + 1e-2,
                     metal_ops.rs:3713-3716).
Shapes and generators are the reference's (metal_ops.rs:3668-4712, 5005-5055)
plus the seeded benchmark configurations.
"""
import sys

import numpy as np
import pytest
import torch

import oracle
from oxydllm_amd import synth
from tests import refgen
from tests.helpers import RTOL, ATOL, TORCH_DT, as_f32, assert_close, bits_of, round_x, to_dev, resident_rounds_weights, tune

pytestmark = pytest.mark.gpu
ops = None


def setup_module(module):
    global ops
    from oxydllm_amd import ops as _ops
    module.ops = _ops


def say(msg):
    print(f"[case] {msg}", flush=True)
    sys.stdout.flush()


DT = {"f16": oracle.F16, "bf16": oracle.BF16}


def awq_ref(qw, qz, sc, x, dt, bits=4):
    """Oracle result: x (rounded to dt) . dequant(W with scales rounded to dt)^T, f32."""
    s_r = oracle.round_through(sc, dt)
    w = oracle.dequantize_awq(qw, qz, s_r) if bits == 4 else oracle.dequantize_awq8(qw, qz, s_r)
    return oracle.matmul_nt_f32(round_x(x, dt), w), w


def gptq_ref(qw, qz, sc, x, dt, bits):
    s_r = oracle.round_through(sc, dt)
    w = oracle.dequantize_gptq(qw, qz, s_r, bits)
    return oracle.matmul_nt_f32(round_x(x, dt), w), w


def dev_triplet(qw, qz, sc, dt):
    return to_dev(qw), to_dev(qz), to_dev(sc, TORCH_DT[dt])


# ------------------------------------------------------------------ AWQ GEMV
@pytest.mark.parametrize("dtn,K,N,g", [("bf16", 256, 128, 128), ("bf16", 256, 128, 64),
                                       ("bf16", 512, 256, 128), ("f16", 256, 128, 64),
                                       ("f16", 512, 256, 32), ("bf16", 192, 104, 64)])
def test_w4a16_gemv_reference_shapes(dtn, K, N, g):
    """metal_ops.rs:3895-3924 (+ an N that is not a multiple of 32 and g=32 for the generic kernel)."""
    dt = DT[dtn]
    say(f"w4a16 gemv {dtn} K={K} N={N} g={g}")
    qw, qz, sc = refgen.build_awq_triplet(K, N, g)
    x = refgen.x_gemv(K)
    ref, _ = awq_ref(qw, qz, sc, x, dt)
    y = ops.w4a16_matmul(to_dev(x, TORCH_DT[dt]), *dev_triplet(qw, qz, sc, dt))
    assert y.shape == (1, N) and y.dtype == TORCH_DT[dt]
    assert_close(y, ref, f"w4a16 {dtn} {K}x{N} g{g}")


@pytest.mark.parametrize("dtn,m", [("bf16", 2), ("bf16", 4), ("bf16", 8), ("f16", 3), ("f16", 5),
                                   ("f16", 7)])
def test_w4a16_gemv_batch(dtn, m):
    """metal_ops.rs:3820-3835: K=256, N=128, g=64."""
    dt = DT[dtn]
    say(f"w4a16 batch {dtn} m={m}")
    K, N, g = 256, 128, 64
    qw, qz, sc = refgen.build_awq_triplet(K, N, g)
    x = refgen.batch_x(m, K)
    ref, _ = awq_ref(qw, qz, sc, x, dt)
    y = ops.w4a16_matmul(to_dev(x, TORCH_DT[dt]), *dev_triplet(qw, qz, sc, dt))
    assert_close(y, ref, f"w4a16 batch {dtn} m{m}")


@pytest.mark.parametrize("dtn,K,N,g,m", [("bf16", 256, 128, 128, 1), ("f16", 256, 128, 64, 1),
                                         ("bf16", 256, 128, 64, 2), ("bf16", 256, 128, 64, 5),
                                         ("bf16", 256, 128, 64, 8)])
def test_w8a16_gemv(dtn, K, N, g, m):
    """metal_ops.rs:4110-4124, 3838-3856."""
    dt = DT[dtn]
    say(f"w8a16 {dtn} K={K} N={N} g={g} m={m}")
    qw, qz, sc, _ = refgen.build_w8a16_triplet(K, N, g)
    x = refgen.x_gemv(K) if m == 1 else refgen.batch_x(m, K)
    ref, _ = awq_ref(qw, qz, sc, x, dt, bits=8)
    y = ops.w8a16_matmul(to_dev(x, TORCH_DT[dt]), *dev_triplet(qw, qz, sc, dt))
    assert_close(y, ref, f"w8a16 {dtn} m{m}")


@pytest.mark.parametrize("dtn", ["f16", "bf16"])
@pytest.mark.parametrize("m", [1, 4, 8])
def test_w4a16_seeded_config0(dtn, m):
    """Benchmark config 0: K=N=4096, g=128, x~N(0,1), q,z uniform, s~U(0.002,0.02)."""
    dt = DT[dtn]
    say(f"w4a16 config0 {dtn} m={m}")
    K, N, g = 4096, 4096, 128
    qw, qz, sc = synth.awq_checkpoint(K, N, g, 4, seed=0x0A0D11E5)
    x = np.random.default_rng(1 + m).standard_normal((m, K)).astype(np.float32)
    ref, _ = awq_ref(qw, qz, sc, x, dt)
    y = ops.w4a16_matmul(to_dev(x, TORCH_DT[dt]), *dev_triplet(qw, qz, sc, dt))
    assert_close(y, ref, f"config0 {dtn} m{m}")
    # forced generic kernel must agree as well (same oracle)


@pytest.mark.parametrize("K,N", [(4096, 14336), (14336, 4096)])
def test_w4a16_seeded_config1_gemv(K, N):
    """Benchmark config 1 shapes at M in {1, 4}, f16."""
    dt = oracle.F16
    g = 128
    qw, qz, sc = synth.awq_checkpoint(K, N, g, 4, seed=0x0A0D11E6)
    d = dev_triplet(qw, qz, sc, dt)
    s_r = oracle.round_through(sc, dt)
    w = oracle.dequantize_awq(qw, qz, s_r)
    for m in (1, 4):
        say(f"w4a16 config1 K={K} N={N} m={m}")
        x = np.random.default_rng(10 + m).standard_normal((m, K)).astype(np.float32)
        ref = oracle.matmul_nt_f32(round_x(x, dt), w)
        y = ops.w4a16_matmul(to_dev(x, torch.float16), *d)
        assert_close(y, ref, f"config1 {K}x{N} m{m}")


@pytest.mark.parametrize("m", [1, 4])
def test_w4a16_bitwise_deterministic(m):
    """metal_ops.rs:4563-4625: 48 runs bit-identical, K=3072 N=128 g=64."""
    say(f"w4a16 determinism m={m}")
    K, N, g = 3072, 128, 64
    qw, qz, sc = refgen.build_awq_triplet(K, N, g)
    d = dev_triplet(qw, qz, sc, oracle.BF16)
    x = to_dev(refgen.batch_x(m, K), torch.bfloat16)
    first = bits_of(ops.w4a16_matmul(x, *d))
    for _ in range(47):
        np.testing.assert_array_equal(bits_of(ops.w4a16_matmul(x, *d)), first)
    # and at the benchmark shape, where K is split across many workgroups
    K, N, g = 4096, 14336, 128
    qw, qz, sc = synth.awq_checkpoint(K, N, g, 4, seed=3)
    d = dev_triplet(qw, qz, sc, oracle.F16)
    x = to_dev(np.random.default_rng(4).standard_normal((m, K)).astype(np.float32), torch.float16)
    first = bits_of(ops.w4a16_matmul(x, *d))
    for _ in range(15):
        np.testing.assert_array_equal(bits_of(ops.w4a16_matmul(x, *d)), first)


# ------------------------------------------------------------------ dequant (bit-exact)
@pytest.mark.parametrize("dtn,K,N,g", [("bf16", 256, 128, 128), ("f16", 256, 128, 64),
                                       ("f16", 4096, 4096, 128), ("bf16", 192, 104, 32)])
def test_dequantize_w4_bit_exact(dtn, K, N, g):
    """metal_ops.rs:3927-3940; tiles must equal the reference dequant bit for bit."""
    dt = DT[dtn]
    say(f"dequantize_w4 {dtn} K={K} N={N} g={g}")
    if K >= 4096:
        qw, qz, sc = synth.awq_checkpoint(K, N, g, 4, seed=5)
    else:
        qw, qz, sc = refgen.build_awq_triplet(K, N, g)
    w = oracle.dequantize_awq(qw, qz, oracle.round_through(sc, dt))
    want = oracle.transpose_convert(w, dt)
    got = ops.dequantize_w4(*dev_triplet(qw, qz, sc, dt))
    assert got.shape == (K, N) and got.dtype == TORCH_DT[dt]
    np.testing.assert_array_equal(bits_of(got), want)


@pytest.mark.parametrize("dtn", ["bf16", "f16"])
def test_dequantize_w8_bit_exact(dtn):
    """metal_ops.rs:4127-4132."""
    dt = DT[dtn]
    say(f"dequantize_w8 {dtn}")
    qw, qz, sc, _ = refgen.build_w8a16_triplet(256, 128, 128)
    w = oracle.dequantize_awq8(qw, qz, oracle.round_through(sc, dt))
    got = ops.dequantize_w8(*dev_triplet(qw, qz, sc, dt))
    np.testing.assert_array_equal(bits_of(got), oracle.transpose_convert(w, dt))


@pytest.mark.parametrize("dtn,bits,K,N,g", [("bf16", 8, 256, 128, 128), ("f16", 4, 256, 128, 64),
                                            ("bf16", 4, 5120, 1024, 128)])
def test_dequantize_gptq_bit_exact(dtn, bits, K, N, g):
    """metal_ops.rs:4303-4308."""
    dt = DT[dtn]
    say(f"dequantize_gptq {dtn} bits={bits} K={K} N={N}")
    if K > 1000:
        qw, qz, sc = synth.gptq_checkpoint(K, N, g, bits, seed=6)
    else:
        qw, qz, sc = refgen.build_gptq_triplet(bits, K, N, g)
    w = oracle.dequantize_gptq(qw, qz, oracle.round_through(sc, dt), bits)
    got = ops.dequantize_gptq_packed(*dev_triplet(qw, qz, sc, dt), bits)
    assert got.shape == (K, N)
    np.testing.assert_array_equal(bits_of(got), oracle.transpose_convert(w, dt))


# ------------------------------------------------------------------ GPTQ GEMV
@pytest.mark.parametrize("dtn,bits,K,N,g", [("bf16", 4, 256, 128, 128), ("bf16", 8, 256, 128, 128),
                                            ("f16", 4, 256, 128, 64), ("f16", 8, 512, 136, 32)])
def test_gptq_gemv_reference_shapes(dtn, bits, K, N, g):
    """metal_ops.rs:4279-4301."""
    dt = DT[dtn]
    say(f"gptq gemv {dtn} bits={bits} K={K} N={N} g={g}")
    qw, qz, sc = refgen.build_gptq_triplet(bits, K, N, g)
    x = refgen.x_gemv(K, 17, 8.0, 0.02)
    ref, _ = gptq_ref(qw, qz, sc, x, dt, bits)
    y = ops.gptq_matmul(to_dev(x, TORCH_DT[dt]), *dev_triplet(qw, qz, sc, dt), bits)
    assert_close(y, ref, f"gptq{bits} {dtn}")


@pytest.mark.parametrize("dtn,bits,ms", [("bf16", 4, (2, 4, 8)), ("bf16", 8, (2, 5, 8)), ("f16", 4, (3,))])
def test_gptq_gemv_batch(dtn, bits, ms):
    """metal_ops.rs:4650-4676."""
    dt = DT[dtn]
    K, N, g = 256, 128, 64
    qw, qz, sc = refgen.build_gptq_triplet(bits, K, N, g)
    d = dev_triplet(qw, qz, sc, dt)
    for m in ms:
        say(f"gptq batch {dtn} bits={bits} m={m}")
        x = refgen.batch_x(m, K)
        ref, _ = gptq_ref(qw, qz, sc, x, dt, bits)
        y = ops.gptq_matmul(to_dev(x, TORCH_DT[dt]), *d, bits)
        assert_close(y, ref, f"gptq{bits} batch m{m}")


@pytest.mark.parametrize("bits", [4, 8])
def test_gptq_seeded_config2(bits):
    """Benchmark config 2: K=5120, N=13824, g=128, M in {1, 8}, f16, stored zero = zp-1."""
    dt = oracle.F16
    K, N, g = 5120, 13824, 128
    qw, qz, sc = synth.gptq_checkpoint(K, N, g, bits, seed=0x0A0D11E7)
    d = dev_triplet(qw, qz, sc, dt)
    w = oracle.dequantize_gptq(qw, qz, oracle.round_through(sc, dt), bits)
    for m in (1, 8):
        say(f"gptq config2 bits={bits} m={m}")
        x = np.random.default_rng(20 + m).standard_normal((m, K)).astype(np.float32)
        ref = oracle.matmul_nt_f32(round_x(x, dt), w)
        y = ops.gptq_matmul(to_dev(x, torch.float16), *d, bits)
        assert_close(y, ref, f"config2 gptq{bits} m{m}")
    first = bits_of(ops.gptq_matmul(to_dev(x, torch.float16), *d, bits))
    for _ in range(7):
        np.testing.assert_array_equal(bits_of(ops.gptq_matmul(to_dev(x, torch.float16), *d, bits)), first)


# ------------------------------------------------------------------ tile GEMM (MFMA)
def _tile_ref(w_f32, x, dt):
    """x . T(dequant)^T: the B tile is rounded to the activation type before the
    matrix unit (mpp_gemm.metal:115-184), f32 accumulate."""
    return oracle.matmul_nt_f32(round_x(x, dt), oracle.round_through(w_f32, dt))


@pytest.mark.parametrize("dtn,m,K,N,g", [("bf16", 70, 192, 104, 64), ("bf16", 70, 160, 104, 32),
                                         ("f16", 16, 256, 128, 64), ("f16", 33, 512, 256, 128),
                                         ("bf16", 64, 256, 1024, 128), ("f16", 9, 256, 128, 64),
                                         ("f16", 130, 256, 640, 64)])
def test_mpp_quant_matmul_partial_tiles(dtn, m, K, N, g):
    """metal_ops.rs:5005-5055 (partial tiles 70x192x104 g64, 70x160x104 g32) and more."""
    dt = DT[dtn]
    say(f"tile gemm {dtn} m={m} K={K} N={N} g={g}")
    qw, qz, sc = refgen.build_awq_triplet(K, N, g)
    x = refgen.batch_x(m, K)
    ref_exact, w = awq_ref(qw, qz, sc, x, dt)
    y = ops.mpp_quant_matmul(to_dev(x, TORCH_DT[dt]), *dev_triplet(qw, qz, sc, dt), 4, ops.PACK_OUT)
    assert y.shape == (m, N)
    assert_close(y, _tile_ref(w, x, dt), f"tile {dtn} m{m} vs rounded-tile oracle")
    # and the reference's own bound against the unrounded weights
    tol = 0.06 * np.abs(ref_exact).max() + 1e-2
    assert np.abs(as_f32(y) - ref_exact).max() < tol


@pytest.mark.parametrize("m", [16, 64])
@pytest.mark.parametrize("K,N", [(4096, 14336), (14336, 4096)])
def test_mpp_quant_matmul_config1(m, K, N):
    """Benchmark config 1 at M in {16, 64}, f16: against the unrounded f32 oracle."""
    dt = oracle.F16
    say(f"tile gemm config1 m={m} K={K} N={N}")
    qw, qz, sc = synth.awq_checkpoint(K, N, 128, 4, seed=0x0A0D11E6)
    x = np.random.default_rng(30 + m).standard_normal((m, K)).astype(np.float32)
    ref, _ = awq_ref(qw, qz, sc, x, dt)
    d = dev_triplet(qw, qz, sc, dt)
    xd = to_dev(x, torch.float16)
    y = ops.mpp_quant_matmul(xd, *d, 4, ops.PACK_OUT)
    assert_close(y, ref, f"tile config1 m{m} {K}x{N}")
    first = bits_of(y)
    for _ in range(5):
        np.testing.assert_array_equal(bits_of(ops.mpp_quant_matmul(xd, *d, 4, ops.PACK_OUT)), first)


def test_maybe_mpp_quant_matmul_routing():
    say("maybe_mpp routing")
    qw, qz, sc = refgen.build_awq_triplet(256, 128, 64)
    d = dev_triplet(qw, qz, sc, oracle.F16)
    assert ops.maybe_mpp_quant_matmul(to_dev(refgen.batch_x(4, 256), torch.float16), *d, 4,
                                      ops.PACK_OUT) is None
    y = ops.maybe_mpp_quant_matmul(to_dev(refgen.batch_x(16, 256), torch.float16), *d, 4, ops.PACK_OUT)
    assert y is not None and y.shape == (16, 128)
    # GPTQ and 8-bit go through the chunked GEMV fallback and still match
    qw, qz, sc = refgen.build_gptq_triplet(4, 256, 128, 64)
    x = refgen.batch_x(20, 256)
    ref, _ = gptq_ref(qw, qz, sc, x, oracle.BF16, 4)
    y = ops.mpp_quant_matmul(to_dev(x, torch.bfloat16), *dev_triplet(qw, qz, sc, oracle.BF16), 4,
                             ops.PACK_IN)
    assert_close(y, ref, "gptq tile fallback")


# ------------------------------------------------------------------ layer
@pytest.mark.parametrize("m", [12, 20])
def test_packed_quant_linear_chunk_invariance(m):
    """metal_ops.rs:4679-4712: m > 8 through the layer equals the rows computed singly."""
    say(f"PackedQuantLinear m={m}")
    K, N, g = 256, 128, 64
    dt = oracle.BF16
    for bits, pack_dim, trip in [(4, ops.PACK_OUT, refgen.build_awq_triplet(K, N, g)),
                                 (4, ops.PACK_IN, refgen.build_gptq_triplet(4, K, N, g)),
                                 (8, ops.PACK_IN, refgen.build_gptq_triplet(8, K, N, g))]:
        d = dev_triplet(*trip, dt)
        layer = ops.PackedQuantLinear(bits, pack_dim, *d, None, torch.bfloat16)
        x = to_dev(refgen.batch_x(m, K), torch.bfloat16)
        y = as_f32(layer.forward(x))
        rows = np.concatenate([as_f32(layer.forward(x[i:i + 1].contiguous())) for i in range(m)])
        if pack_dim == ops.PACK_OUT:
            ref, w = awq_ref(*trip, refgen.batch_x(m, K), dt)
            assert_close(y, _tile_ref(w, refgen.batch_x(m, K), dt), "layer tile", bf16_out=True)
        else:
            ref, _ = gptq_ref(*trip, refgen.batch_x(m, K), dt, bits)
            assert_close(y, ref, "layer gptq", bf16_out=True)
        assert_close(rows, ref, "layer rows", bf16_out=True)
        assert np.abs(y - rows).max() < 0.06 * np.abs(ref).max() + 1e-2


def test_packed_quant_linear_bias_and_leading_dims():
    """linear.rs:482-533: [..., K] input, bias broadcast-added (linear.rs:688-787 on the CPU side)."""
    say("PackedQuantLinear bias")
    K, N, g = 512, 256, 128
    dt = oracle.F16
    trip = refgen.build_awq_triplet(K, N, g)
    bias = (np.arange(N, dtype=np.float32) % 7 - 3) * np.float32(0.25)
    layer = ops.PackedQuantLinear(4, ops.PACK_OUT, *dev_triplet(*trip, dt), to_dev(bias, torch.float16),
                                  torch.float16)
    assert (layer.in_features, layer.out_features) == (K, N)
    w = oracle.dequantize_awq(trip[0], trip[1], oracle.round_through(trip[2], dt))
    for shape in [(1, K), (2, 3, K), (4, 8, K)]:
        m = int(np.prod(shape[:-1]))
        x = refgen.batch_x(m, K)
        y = layer.forward(to_dev(x.reshape(shape), torch.float16))
        assert tuple(y.shape) == shape[:-1] + (N,)
        ref = oracle.matmul_nt_f32(round_x(x, dt), w, bias)
        assert_close(y.reshape(m, N), ref, f"layer bias {shape}")
    with pytest.raises(ops.OxqError, match="input last dim"):
        layer.forward(to_dev(refgen.batch_x(1, K - 32), torch.float16))


# ------------------------------------------------------------------ 8-bit fast kernels
@pytest.mark.parametrize("method", ["awq", "gptq"])
@pytest.mark.parametrize("dtn", ["f16", "bf16"])
@pytest.mark.parametrize("K,N,g", [(256, 128, 128), (1024, 96, 256), (1280, 544, 128), (5120, 1024, 128)])
def test_8bit_fast_gemv(method, dtn, K, N, g, monkeypatch):
    """The 8-bit stateless ops on the checkpoint layout run the same fast kernels as the 4-bit
    ones (word = 4 columns / 4 consecutive k); every m of the decode range, ragged column tiles
    (N = 96, 544), several K slices, and the generic kernel on the same inputs as a second opinion."""
    dt = DT[dtn]
    make = synth.awq_checkpoint if method == "awq" else synth.gptq_checkpoint
    qw, qz, sc = make(K, N, g, 8, seed=K + N)
    d = dev_triplet(qw, qz, sc, dt)
    s_r = oracle.round_through(sc, dt)
    w = oracle.dequantize_awq8(qw, qz, s_r) if method == "awq" else oracle.dequantize_gptq(qw, qz, s_r, 8)
    op = (lambda x: ops.w8a16_matmul(x, *d)) if method == "awq" else (lambda x: ops.gptq_matmul(x, *d, 8))
    rng = np.random.default_rng(K * 3 + N)
    tune("OXQ_GPTQ_TILE", 0)  # this test is about the dot-product kernels (the tile kernel: test_gpu_gptq_tile.py)
    for m in (1, 2, 3, 4, 7, 8):
        say(f"8-bit fast {method} {dtn} K={K} N={N} g={g} m={m}")
        x = rng.standard_normal((m, K)).astype(np.float32)
        xd = to_dev(x, TORCH_DT[dt])
        tune("OXQ_FORCE_GENERIC", None)
        y = op(xd)
        kern = ops.default_context().last_plan()["kernel"]
        assert kern.startswith(f"{method}8_gemv_fast_{dtn}"), kern
        assert_close(y, oracle.matmul_nt_f32(round_x(x, dt), w), f"{method}8 fast {dtn} m{m}")
        np.testing.assert_array_equal(bits_of(op(xd)), bits_of(y))          # run-to-run
        tune("OXQ_FORCE_GENERIC", 1)
        yg = op(xd)
        assert "generic" in ops.default_context().last_plan()["kernel"]
        # two roundings of nearly equal sums may land one output ulp apart
        assert_close(y, as_f32(yg), f"{method}8 fast vs generic {dtn} m{m}", rtol=RTOL + (2.0 ** -7 if dtn == "bf16" else 2.0 ** -10))


@pytest.mark.parametrize("method,bits", [("gptq", 4), ("gptq", 8), ("awq", 8)])
@pytest.mark.parametrize("dtn", ["f16", "bf16"])
def test_stateless_tile_op_on_layouts_without_a_tile_kernel(method, bits, dtn, monkeypatch):
    """mpp_quant_matmul on GPTQ / 8-bit AWQ checkpoint tensors.  GPTQ runs its own tile kernel on the
    checkpoint layout (one launch); with that switched off, and for 8-bit AWQ, the tile-major copy is built
    in the ctx workspace and the resident-layer kernel runs on it (two launches); with that switch off too
    the call falls back to GEMV passes of 8 rows.  All against the oracle; a following 4-bit AWQ call on the
    same ctx (which uses the workspace for K slices) still gives the right answer."""
    dt = DT[dtn]
    K, N, g = 1024, 384, 128
    make = synth.awq_checkpoint if method == "awq" else synth.gptq_checkpoint
    qw, qz, sc = make(K, N, g, bits, seed=bits + K)
    d = dev_triplet(qw, qz, sc, dt)
    s_r = oracle.round_through(sc, dt)
    w = oracle.dequantize_awq8(qw, qz, s_r) if method == "awq" else oracle.dequantize_gptq(qw, qz, s_r, bits)
    pd = ops.PACK_OUT if method == "awq" else ops.PACK_IN
    rng = np.random.default_rng(5)
    for m in (9, 16, 17, 64, 100):
        say(f"transient repack {method}{bits} {dtn} m={m}")
        x = rng.standard_normal((m, K)).astype(np.float32)
        xd = to_dev(x, TORCH_DT[dt])
        tune("OXQ_TRANSIENT_REPACK", None)
        if method == "gptq":
            tune("OXQ_GPTQ_TILE", None)
            y = ops.mpp_quant_matmul(xd, *d, bits, pd)
            plan = ops.default_context().last_plan()
            assert plan["kernel"].startswith(f"gptq{bits}_tile_{dtn}") and plan["launches"] == 1, plan
            # the tile kernel keeps the unrounded weight up to 32 rows (the reach of the reference's GEMV)
            wr = oracle.round_through(w, dt) if m > 32 else w
            assert_close(y, oracle.matmul_nt_f32(round_x(x, dt), wr), f"{method}{bits} {dtn} m{m} (tile kernel on the checkpoint layout)")
            tune("OXQ_GPTQ_TILE", 0)
        y = ops.mpp_quant_matmul(xd, *d, bits, pd)
        plan = ops.default_context().last_plan()
        assert plan["kernel"].startswith(f"pk{bits}_mfma_{dtn}") and plan["launches"] == 2, plan
        wr = oracle.round_through(w, dt) if resident_rounds_weights(m, dt, method == "gptq") else w
        assert_close(y, oracle.matmul_nt_f32(round_x(x, dt), wr), f"{method}{bits} {dtn} m{m} (repacked in the workspace)")
        tune("OXQ_TRANSIENT_REPACK", 0)
        y2 = ops.mpp_quant_matmul(xd, *d, bits, pd)
        assert "gemv" in ops.default_context().last_plan()["kernel"]
        assert_close(y2, oracle.matmul_nt_f32(round_x(x, dt), w), f"{method}{bits} {dtn} m{m} (GEMV passes)")
    tune("OXQ_TRANSIENT_REPACK", None)
    aw = synth.awq_checkpoint(2048, 128, 128, 4, seed=3)
    ad = dev_triplet(*aw, dt)
    wa = oracle.dequantize_awq(aw[0], aw[1], oracle.round_through(aw[2], dt))
    xa = rng.standard_normal((32, 2048)).astype(np.float32)
    ya = ops.mpp_quant_matmul(to_dev(xa, TORCH_DT[dt]), *ad, 4, ops.PACK_OUT)
    assert_close(ya, oracle.matmul_nt_f32(round_x(xa, dt), oracle.round_through(wa, dt)), "awq4 after a repacked call")


@pytest.mark.parametrize("method", ["awq", "gptq"])
@pytest.mark.parametrize("dtn", ["f16", "bf16"])
def test_stateless_tile_op_repacks_at_prefill_sizes(method, dtn):
    """mpp_quant_matmul at prefill sizes: the kernels of the resident layout run at two to six times the rate of
    those on the checkpoint layout, so from 640 rows (bf16 AWQ: 80) the op builds the tile-major copy in the ctx
    workspace and runs them (two launches); below that, and with OXQ_TRANSIENT_REPACK = 0, the checkpoint-layout
    kernel.  Both against the tile oracle."""
    dt = DT[dtn]
    K, N, g = 512, 640, 128
    make = synth.awq_checkpoint if method == "awq" else synth.gptq_checkpoint
    qw, qz, sc = make(K, N, g, 4, seed=K + N)
    d = dev_triplet(qw, qz, sc, dt)
    s_r = oracle.round_through(sc, dt)
    w = oracle.dequantize_awq(qw, qz, s_r) if method == "awq" else oracle.dequantize_gptq(qw, qz, s_r, 4)
    wt = oracle.round_through(w, dt)
    pd = ops.PACK_OUT if method == "awq" else ops.PACK_IN
    own = "awq4_mfma_pipe" if method == "awq" else "gptq4_tile"
    first = 80 if (method, dtn) == ("awq", "bf16") else 640
    x = np.random.default_rng(6).standard_normal((700, K)).astype(np.float32)
    xd = to_dev(x, TORCH_DT[dt])
    ref = oracle.matmul_nt_f32(round_x(x, dt), wt)
    for m in (64, first - 1, first, 700):
        say(f"prefill repack {method} {dtn} m={m}")
        y = ops.mpp_quant_matmul(xd[:m], *d, 4, pd)
        plan = ops.default_context().last_plan()
        if m >= first:
            assert plan["kernel"].startswith("pk4_") and plan["launches"] == 2, (m, plan)
        else:
            assert plan["kernel"].startswith(own), (m, plan)
        assert_close(y, ref[:m], f"{method} {dtn} m{m}")
        tune("OXQ_TRANSIENT_REPACK", 0)
        y0 = ops.mpp_quant_matmul(xd[:m], *d, 4, pd)
        assert ops.default_context().last_plan()["kernel"].startswith(own)
        assert_close(y0, ref[:m], f"{method} {dtn} m{m} on the checkpoint layout")
        tune("OXQ_TRANSIENT_REPACK", None)


# ------------------------------------------------------------------ split-K: fused sum against the second launch
@pytest.mark.parametrize("route", ["awq4", "awq8", "gptq4", "gptq8", "awq4_generic", "gptq4_generic"])
@pytest.mark.parametrize("dtn", ["f16", "bf16"])
def test_splitk_fused_and_two_launch_sums_give_the_same_bits(route, dtn, monkeypatch):
    """The K slices' partial sums are added in slice order either by the last workgroup to arrive (mode 1,
    relaxed device-scope accesses and an arrival counter) or by a second launch (mode 2, plain stores and a
    kernel boundary).  Both must give the same bits on every GEMV route, for every row count."""
    dt = DT[dtn]
    bits = 8 if route.endswith("8") else 4
    gptq = route.startswith("gptq")
    generic = route.endswith("generic")
    K, N, g = (2048, 1024, 128) if not generic else (1024, 328, 32)
    qw, qz, sc = (synth.gptq_checkpoint if gptq else synth.awq_checkpoint)(K, N, g, bits, seed=77)
    d = dev_triplet(qw, qz, sc, dt)
    ctxs = {}
    for mode in (1, 2):
        ctxs[mode] = ops.Context()
        tune("OXQ_SPLITK_MODE", mode, ctx=ctxs[mode])
        tune("OXQ_GPTQ_TILE", 0, ctx=ctxs[mode])  # the GPTQ tile kernel keeps K inside the workgroup: nothing to sum
    for m in (1, 3, 8):
        if m > 1 and dtn == "f16" and bits == 4 and not gptq:
            continue  # f16 batches on 4-bit AWQ run the tile kernel, which always sums with the second launch
        say(f"split-K modes {route} {dtn} m={m}")
        x = np.random.default_rng(m).standard_normal((m, K)).astype(np.float32)
        xd = to_dev(x, TORCH_DT[dt])
        outs, plans = {}, {}
        for mode in (1, 2):
            if gptq:
                outs[mode] = ops.gptq_matmul(xd, *d, bits, ctx=ctxs[mode])
            elif bits == 8:
                outs[mode] = ops.w8a16_matmul(xd, *d, ctx=ctxs[mode])
            else:
                outs[mode] = ops.w4a16_matmul(xd, *d, ctx=ctxs[mode])
            plans[mode] = ctxs[mode].last_plan()
        torch.cuda.synchronize()
        assert plans[1]["kernel"] == plans[2]["kernel"] and plans[1]["split_k"] == plans[2]["split_k"] > 1, plans
        assert ("generic" in plans[1]["kernel"]) == generic, plans[1]
        assert plans[1]["launches"] == 1 and plans[2]["launches"] == 2, plans
        assert np.array_equal(bits_of(outs[1]), bits_of(outs[2])), f"{route} {dtn} m={m}: fused and two-launch sums differ"
        ref = (gptq_ref(qw, qz, sc, x, dt, bits) if gptq else awq_ref(qw, qz, sc, x, dt, bits))[0]
        assert_close(outs[1], ref, f"split-K {route} {dtn} m={m}")
    for c in ctxs.values():
        c.close()
