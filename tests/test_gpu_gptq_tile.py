"""The GPTQ tile kernel on the checkpoint layout (csrc/gptq_tile.hip), through the stateless ops of the C ABI:
gptq_matmul up to 8 rows (metal_ops.rs:2281-2303), mpp_quant_matmul from 9 rows on (metal_ops.rs:2748-2797).

Against the oracle's dense dequant (awq.rs:442-590) and f32 matmul: with the unrounded weight up to 32 rows
(the reach of the reference's fused GEMV, linear.rs:450-480), with the weight rounded to the activation type
above (the reference's staged GEMM, mpp_gemm.metal:115-184).  Shapes cover every code path of the kernel:
K = 4096 and 5120 (4 and 5 blocks a wave, straight-line code), other K through the block loop with one block a
wave, uneven shares, waves without a block and an odd number of blocks a wave; K slices (few strips and 32 blocks
or more) with and without them forced off; one, two and four row tiles with ragged last tiles and several row-tile
workgroups; groups larger than a block; bias; both bit widths and types.
"""
import sys

import numpy as np
import pytest
import torch

import oracle
from oxydllm_amd import synth
from tests.helpers import TORCH_DT, assert_close, bits_of, round_x, to_dev, tune

pytestmark = pytest.mark.gpu
DT = {"f16": oracle.F16, "bf16": oracle.BF16}


def say(msg):
    print(f"[case] {msg}", flush=True)
    sys.stdout.flush()


def _run(ops, xd, d, bits, m):
    if m <= 8:
        return ops.gptq_matmul(xd, *d, bits)
    return ops.mpp_quant_matmul(xd, *d, bits, ops.PACK_IN)


@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("dtn", ["f16", "bf16"])
@pytest.mark.parametrize("K,N,g", [(4096, 128, 128), (5120, 64, 128), (1024, 192, 128), (1152, 64, 128),
                                   (2816, 128, 128), (2048, 128, 256), (2048, 64, 1024)])
def test_gptq_tile_against_oracle(bits, dtn, K, N, g):
    from oxydllm_amd import ops
    dt = DT[dtn]
    qw, qz, sc = synth.gptq_checkpoint(K, N, g, bits, seed=K + N + g + bits)
    d = (to_dev(qw), to_dev(qz), to_dev(sc, TORCH_DT[dt]))
    w = oracle.dequantize_gptq(qw, qz, oracle.round_through(sc, dt), bits)
    w_r = oracle.round_through(w, dt)
    rng = np.random.default_rng(K * 7 + N)
    tune("OXQ_GPTQ_TILE", 2)  # also where the dot-product kernel would keep a narrow layer's few rows
    for m in (1, 3, 8, 16, 17, 32, 33, 64, 65, 130):
        say(f"gptq tile bits={bits} {dtn} K={K} N={N} g={g} m={m}")
        x = rng.standard_normal((m, K)).astype(np.float32)
        xd = to_dev(x, TORCH_DT[dt])
        y = _run(ops, xd, d, bits, m)
        plan = ops.default_context().last_plan()
        mt = 4 if m > 32 else (m + 15) // 16
        assert plan["kernel"] == f"gptq{bits}_tile_{dtn}_mt{mt}", plan
        # these layers have few strips: from 32 blocks of K on they are cut into K slices, added by a second launch
        tiles = (N // 64) * -(-m // (16 * mt))
        ks = max(1, min(256 // tiles, K // 128 // 8)) if K // 128 >= 32 and tiles <= 96 else 1
        assert plan["split_k"] == ks and plan["launches"] == (2 if ks > 1 else 1), plan
        assert plan["grid"] == (N // 64, -(-m // (16 * mt)), ks), plan
        ref = oracle.matmul_nt_f32(round_x(x, dt), w_r if m > 32 else w)
        assert_close(y, ref, f"gptq{bits} tile {dtn} {K}x{N} g{g} m{m}")
        np.testing.assert_array_equal(bits_of(_run(ops, xd, d, bits, m)), bits_of(y))  # run to run


@pytest.mark.parametrize("bits", [4, 8])
def test_gptq_tile_rows_do_not_depend_on_the_batch(bits):
    """A row's result is the same bits whatever rows stand beside it, as long as the form (folded up to 32 rows,
    tile above) is the same: rows of a 32-row call against one-row calls, rows of a 100-row call against a
    40-row call."""
    from oxydllm_amd import ops
    K, N, g = 4096, 128, 128
    qw, qz, sc = synth.gptq_checkpoint(K, N, g, bits, seed=91)
    d = (to_dev(qw), to_dev(qz), to_dev(sc, torch.float16))
    x = np.random.default_rng(92).standard_normal((100, K)).astype(np.float32)
    xd = to_dev(x, torch.float16)
    tune("OXQ_GPTQ_TILE", 2)
    y32 = bits_of(_run(ops, xd[:32].contiguous(), d, bits, 32))
    for r in (0, 15, 16, 31):
        say(f"gptq tile row {r} alone, bits={bits}")
        y1 = bits_of(_run(ops, xd[r:r + 1].contiguous(), d, bits, 1))
        np.testing.assert_array_equal(y1[0], y32[r])
    y100 = bits_of(_run(ops, xd, d, bits, 100))
    y40 = bits_of(_run(ops, xd[:40].contiguous(), d, bits, 40))
    np.testing.assert_array_equal(y40, y100[:40])


@pytest.mark.parametrize("bits", [4, 8])
def test_gptq_tile_many_row_tiles_and_bias(bits):
    """300 rows are five row-tile workgroups a strip, the last one ragged; the bias is added once, after the
    waves' sum."""
    from oxydllm_amd import ops
    dt = oracle.BF16
    K, N, g, m = 1024, 128, 128, 300
    qw, qz, sc = synth.gptq_checkpoint(K, N, g, bits, seed=5 + bits)
    bias = ((np.arange(N, dtype=np.float32) % 11) - 5) * np.float32(0.125)
    layer = ops.PackedQuantLinear(bits, ops.PACK_IN, to_dev(qw), to_dev(qz), to_dev(sc, torch.bfloat16),
                                  to_dev(bias, torch.bfloat16), torch.bfloat16)
    tune("OXQ_PREPACK", 0)  # a layer that keeps the checkpoint layout forwards through the stateless ops
    plain = ops.PackedQuantLinear(bits, ops.PACK_IN, to_dev(qw), to_dev(qz), to_dev(sc, torch.bfloat16),
                                  to_dev(bias, torch.bfloat16), torch.bfloat16)
    x = np.random.default_rng(17).standard_normal((m, K)).astype(np.float32)
    xd = to_dev(x, torch.bfloat16)
    say(f"gptq tile bits={bits} m={m} with bias, through a layer on the checkpoint layout")
    y = plain.forward(xd)
    plan = ops.default_context().last_plan()
    assert plan["kernel"] == f"gptq{bits}_tile_bf16_mt4" and plan["grid"] == (N // 64, 5, 1), plan
    w = oracle.round_through(oracle.dequantize_gptq(qw, qz, oracle.round_through(sc, dt), bits), dt)
    assert_close(y, oracle.matmul_nt_f32(round_x(x, dt), w, oracle.round_through(bias, dt)), f"gptq{bits} tile m{m} bias")
    # the resident layer's tile form is the same arithmetic in the same order of K blocks per wave only when the
    # waves' shares agree; its result stays within the tolerance of this one
    assert_close(y, layer.forward(xd).float().cpu().numpy(), f"gptq{bits} tile vs resident m{m}")


@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("dtn", ["f16", "bf16"])
def test_gptq_tile_k_slices_and_straight_line_code_agree(bits, dtn):
    """K = 4096 and 5120 on a layer of few strips: by default K slices (the block loop, partial tiles added by the
    second launch); with one slice forced the straight-line kernels.  Both against the oracle, and the sliced sum
    run to run bitwise."""
    from oxydllm_amd import ops
    dt = DT[dtn]
    for K in (4096, 5120):
        N, g = 128, 128
        qw, qz, sc = synth.gptq_checkpoint(K, N, g, bits, seed=K + bits)
        d = (to_dev(qw), to_dev(qz), to_dev(sc, TORCH_DT[dt]))
        w = oracle.dequantize_gptq(qw, qz, oracle.round_through(sc, dt), bits)
        rng = np.random.default_rng(K)
        tune("OXQ_GPTQ_TILE", 2)
        for m in (1, 8, 16, 32, 64):
            x = rng.standard_normal((m, K)).astype(np.float32)
            xd = to_dev(x, TORCH_DT[dt])
            ref = oracle.matmul_nt_f32(round_x(x, dt), oracle.round_through(w, dt) if m > 32 else w)
            for ks in (None, 1, 3):
                say(f"gptq tile bits={bits} {dtn} K={K} m={m} slices={ks}")
                tune("OXQ_GPTQ_TILE_KS", ks)
                y = _run(ops, xd, d, bits, m)
                plan = ops.default_context().last_plan()
                want_ks = {None: min(256 // 2, K // 128 // 8), 1: 1, 3: 3}[ks]
                assert plan["split_k"] == want_ks and plan["launches"] == (2 if want_ks > 1 else 1), plan
                assert_close(y, ref, f"gptq{bits} tile {dtn} K{K} m{m} ks{ks}")
                np.testing.assert_array_equal(bits_of(_run(ops, xd, d, bits, m)), bits_of(y))
            tune("OXQ_GPTQ_TILE_KS", None)
