"""Seeded random shapes through every matmul route, against the oracle.

The fixed-shape tests pick sizes that name a boundary; these draw ragged M, N and K from a seeded
generator so that a tile, strip or slice edge nobody thought of still gets a case.  Tolerance as in
the other parity tests: 2e-3 relative / 1e-2 absolute on the f32-accumulated product.
"""
import os

import numpy as np
import pytest
import torch

import oracle
from oxydllm_amd import ops, synth
from tests.helpers import assert_close, round_x, to_dev, resident_rounds_weights, tune

pytestmark = pytest.mark.gpu


def _kernel():
    return ops.default_context().last_plan()["kernel"]


def test_gguf_random_shapes():
    rng = np.random.default_rng(12345)
    for it in range(40):
        fmt = int(rng.integers(0, 10))
        elems, _ = synth.GGUF_BLOCK_LAYOUT[fmt]
        K = int(rng.integers(1, 9)) * 256 if elems == 256 else int(rng.integers(1, 40)) * 32
        N = int(rng.integers(1, 300))
        M = int(rng.choice([1, 2, 3, 5, 8, 9, 15, 16, 17, 31, 33, 64, 65, 100, 129]))
        data = synth.gguf_weight(fmt, N, K, seed=it)
        w = oracle.dequantize_gguf(fmt, data, N, K)
        x = rng.standard_normal((M, K)).astype(np.float32)
        bias = rng.standard_normal(N).astype(np.float32)
        layer = ops.QLinear(fmt, to_dev(data), K, N, to_dev(bias, torch.bfloat16), torch.bfloat16)
        y = layer.forward(to_dev(x, torch.bfloat16))
        # rows above the hi+lo range multiply bf16-rounded weights, as the reference's mul_mm does
        wr = w if M <= 8 else oracle.round_through(w, oracle.BF16)
        ref = oracle.matmul_nt_f32(round_x(x, oracle.BF16), wr, round_x(bias, oracle.BF16))
        assert_close(y, ref, f"gguf fmt{fmt} M{M} N{N} K{K} {_kernel()}", bf16_out=True)


def test_mxfp4_random_shapes():
    rng = np.random.default_rng(2345)
    for it in range(30):
        K = int(rng.integers(1, 60)) * 32
        N = int(rng.integers(1, 300))
        M = int(rng.choice([1, 3, 8, 9, 16, 17, 33, 64, 65, 130]))
        blocks, scales = synth.mxfp4_weight(N, K, seed=it)
        w = oracle.dequantize_mxfp4_f32(blocks, scales, N, K)
        x = rng.standard_normal((M, K)).astype(np.float32)
        y = ops.mxfp4_matmul(to_dev(x, torch.bfloat16), to_dev(blocks), to_dev(scales), K, N)
        ref = oracle.matmul_nt_f32(round_x(x, oracle.BF16), w)
        assert_close(y, ref, f"mxfp4 M{M} N{N} K{K} {_kernel()}")


def test_f8_random_shapes():
    rng = np.random.default_rng(345)
    for it in range(30):
        s_r, s_c = int(rng.integers(1, 5)), int(rng.integers(1, 9))
        K = s_c * int(rng.choice([32, 64, 128, 24, 16]))
        N = s_r * int(rng.integers(1, 80))
        M = int(rng.choice([1, 2, 3, 8, 9, 17, 64, 70]))
        b = rng.integers(0, 256, size=(N, K), dtype=np.uint8)
        b = np.where((b & 0x7F) == 0x7F, b ^ 0x08, b).astype(np.uint8)   # no NaN encodings
        sc = rng.uniform(0.05, 1.5, size=(s_r, s_c)).astype(np.float32)
        w = oracle.widen_to_f32(oracle.f8_block_dequant_bf16(b, sc), oracle.BF16)
        x = rng.standard_normal((M, K)).astype(np.float32)
        y = ops.f8_matmul(to_dev(x, torch.bfloat16), to_dev(b), to_dev(sc))
        ref = oracle.matmul_nt_f32(round_x(x, oracle.BF16), w)
        assert_close(y, ref, f"f8 M{M} N{N} K{K} {_kernel()}")


def test_resident_layer_random_shapes(monkeypatch):
    rng = np.random.default_rng(45)
    for it in range(30):
        bits = int(rng.choice([4, 8]))
        gptq = bool(rng.integers(0, 2))
        g = int(rng.choice([128, 256]))
        K = g * int(rng.integers(1, 20))
        N = 64 * int(rng.integers(1, 12))
        M = int(rng.choice([1, 4, 16, 17, 40, 64, 90]))
        dt, tdt = (oracle.F16, torch.float16) if rng.integers(0, 2) else (oracle.BF16, torch.bfloat16)
        make = synth.gptq_checkpoint if gptq else synth.awq_checkpoint
        qw, qz, sc = make(K, N, g, bits, seed=it)[:3]
        s_r = oracle.round_through(sc, dt)
        if gptq:
            w = oracle.dequantize_gptq(qw, qz, s_r, bits)
        elif bits == 4:
            w = oracle.dequantize_awq(qw, qz, s_r)
        else:
            w = oracle.dequantize_awq8(qw, qz, s_r)
        if rng.integers(0, 2):
            tune("OXQ_PK4_KS", int(rng.integers(2, 6)))
        else:
            tune("OXQ_PK4_KS", None)
        layer = ops.PackedQuantLinear(bits, ops.PACK_IN if gptq else ops.PACK_OUT, to_dev(qw), to_dev(qz),
                                      to_dev(sc, tdt), None, tdt)
        assert layer.prepacked
        x = rng.standard_normal((M, K)).astype(np.float32)
        y = layer.forward(to_dev(x, tdt))
        plan = ops.default_context().last_plan()
        wr = oracle.round_through(w, dt) if resident_rounds_weights(M, dt, bool(gptq)) else w
        ref = oracle.matmul_nt_f32(round_x(x, dt), wr)
        assert_close(y, ref, f"pk{bits} gptq={gptq} M{M} N{N} K{K} g{g} ks{plan['split_k']} {plan['kernel']}")
