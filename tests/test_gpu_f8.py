"""GPU parity tests for the block-scaled F8E4M3 path (cast, dense dequant, GEMV, tile matmul).

Generators and shapes are the reference's own (metal_ops.rs:2991-3035, 4310-4450); the dense
dequant and the cast are compared bit for bit with the oracle, the products within 2e-3
relative + 1e-2 absolute (+ half a bf16 ulp for the bf16 output) of the f32-accumulated
x . dequant(W)^T, and run to run bit for bit.
"""
import sys

import numpy as np
import pytest
import torch

import oracle
from tests import refgen
from tests.helpers import as_f32, assert_close, bits_of, round_x, to_dev

pytestmark = pytest.mark.gpu
ops = None


def setup_module(module):
    from oxydllm_amd import ops as _ops
    module.ops = _ops


def say(msg):
    print(f"[case] {msg}", flush=True)
    sys.stdout.flush()


def dense(b, scales):
    return oracle.widen_to_f32(oracle.f8_block_dequant_bf16(b, scales), oracle.BF16)


def test_cast_every_byte():
    """metal_ops.rs:2991-3035, over all 256 encodings (the two NaN bytes compared as NaN)."""
    say("f8 cast")
    b = np.tile(np.arange(256, dtype=np.uint8), 5).reshape(5, 256)
    got = ops.cast_f8e4m3_to_f32(to_dev(b)).cpu().numpy()
    want = oracle.cast_f8e4m3_to_f32(b)
    nan = np.isnan(want)
    assert got.shape == b.shape and np.array_equal(np.isnan(got), nan)
    np.testing.assert_array_equal(got[~nan].view(np.uint32), want[~nan].view(np.uint32))


@pytest.mark.parametrize("case", ["reference", "all bytes", "1000x384"])
def test_block_dequant_bit_exact(case):
    """metal_ops.rs:4310-4375."""
    say(f"f8 block dequant {case}")
    if case == "reference":
        b, scales = refgen.f8_dequant_case()
    elif case == "all bytes":
        b = np.arange(256, dtype=np.uint8).reshape(4, 64)
        scales = np.array([[0.37, 1.5], [3.0, 0.011]], np.float32)
    else:
        rng = np.random.default_rng(5)
        b = rng.integers(0, 256, size=(1000, 384), dtype=np.uint8)
        b = np.where((b & 0x7F) == 0x7F, b ^ 0x08, b).astype(np.uint8)
        scales = rng.uniform(0.01, 2.0, size=(8, 3)).astype(np.float32)
    want = oracle.f8_block_dequant_bf16(b, scales)
    got = bits_of(ops.f8_block_dequant_bf16(to_dev(b), to_dev(scales)))
    nan = np.isnan(oracle.widen_to_f32(want, oracle.BF16))
    assert np.array_equal(np.isnan(oracle.widen_to_f32(got, oracle.BF16)), nan)
    np.testing.assert_array_equal(got[~nan], want[~nan])


@pytest.mark.parametrize("out_f,in_f,s_r,s_c,m", [(512, 2048, 4, 16, 1), (2048, 512, 16, 4, 1), (512, 2048, 4, 16, 4),
                                                  (96, 160, 3, 5, 2), (96, 168, 3, 7, 3), (1001, 1024, 1, 8, 8)])
def test_gemv_parity_and_determinism(out_f, in_f, s_r, s_c, m):
    """metal_ops.rs:4378-4450 (shapes 1-4; 5: a block width of 24 that 16-byte chunks straddle;
    6: odd out_features, a single scale row)."""
    say(f"f8 gemv {out_f}x{in_f} scales {s_r}x{s_c} m={m}")
    b, scales, x = refgen.f8_gemv_case(out_f, in_f, s_r, s_c, m)
    ref = oracle.matmul_nt_f32(round_x(x, oracle.BF16), dense(b, scales))
    bd, sd, xd = to_dev(b), to_dev(scales), to_dev(x, torch.bfloat16)
    y = ops.f8_gemv(xd, bd, sd)
    assert y.shape == (m, out_f) and y.dtype == torch.bfloat16
    assert_close(y, ref, f"f8 gemv {out_f}x{in_f} m{m}")
    assert np.abs(as_f32(y) - ref).max() < 0.02 * max(1.0, np.abs(ref).max())   # the reference's bound
    first = bits_of(y)
    for _ in range(8):
        np.testing.assert_array_equal(bits_of(ops.f8_gemv(xd, bd, sd)), first)


@pytest.mark.parametrize("out_f,in_f,s_r,s_c,m", [(512, 2048, 4, 16, 9), (2048, 512, 16, 4, 64), (1000, 1120, 8, 35, 150),
                                                  (96, 160, 3, 5, 20), (768, 2048, 6, 16, 33)])
def test_matmul_any_m(out_f, in_f, s_r, s_c, m):
    """moe.rs:106-113: beyond 8 rows the reference dequantizes and multiplies; here the tile
    matmul decodes the same bf16 weights on the fly (shape 3: partial tiles and a K that is not
    a multiple of the 256-element stage; shape 4: 32-wide blocks; the last: K split forced)."""
    say(f"f8 matmul {out_f}x{in_f} m={m}")
    b, scales, x = refgen.f8_gemv_case(out_f, in_f, s_r, s_c, m)
    ref = oracle.matmul_nt_f32(round_x(x, oracle.BF16), dense(b, scales))
    bd, sd, xd = to_dev(b), to_dev(scales), to_dev(x, torch.bfloat16)
    y = ops.f8_matmul(xd, bd, sd)
    assert ops.default_context().last_plan()["kernel"].startswith("f8_mul_mm_bf16")
    assert_close(y, ref, f"f8 matmul {out_f}x{in_f} m{m}")
    np.testing.assert_array_equal(bits_of(ops.f8_matmul(xd, bd, sd)), bits_of(y))
    # rows taken 8 at a time by the GEMV agree within the same tolerance
    chunks = torch.cat([ops.f8_gemv(xd[i:i + 8].contiguous(), bd, sd) for i in range(0, m, 8)])
    assert_close(chunks, ref, "f8 gemv in chunks")


def test_matmul_small_m_and_narrow_blocks_use_the_gemv():
    say("f8 matmul routing")
    b, scales, x = refgen.f8_gemv_case(96, 168, 3, 7, 20)   # 24-wide blocks: no tile matmul
    y = ops.f8_matmul(to_dev(x, torch.bfloat16), to_dev(b), to_dev(scales))
    plan = ops.default_context().last_plan()
    assert plan["kernel"] == "f8_gemv_bf16_bytes" and plan["launches"] == 3
    assert_close(y, oracle.matmul_nt_f32(round_x(x, oracle.BF16), dense(b, scales)), "f8 matmul via gemv")


def test_validation_like_reference():
    """metal_ops.rs:5589-5613, 5703-5731."""
    say("f8 validation")
    b, scales, x = refgen.f8_gemv_case(96, 160, 3, 5, 2)
    bd, sd, xd = to_dev(b), to_dev(scales), to_dev(x, torch.bfloat16)
    with pytest.raises(ops.OxqError, match=r"scale grid \[5, 5\] does not tile weight \[96, 160\]"):
        ops.f8_block_dequant_bf16(bd, to_dev(np.ones((5, 5), np.float32)))
    with pytest.raises(ops.OxqError, match="expected U8 bytes and F32 scales"):
        ops.f8_block_dequant_bf16(bd, sd.to(torch.bfloat16))
    with pytest.raises(ops.OxqError, match="x must be BF16"):
        ops.f8_gemv(xd.to(torch.float16), bd, sd)
    with pytest.raises(ops.OxqError, match=r"m must be 1\.\.=8"):
        ops.f8_gemv(to_dev(np.zeros((9, 160), np.float32), torch.bfloat16), bd, sd)
    with pytest.raises(ops.OxqError, match="incompatible with in_features 160"):
        ops.f8_gemv(to_dev(np.zeros((2, 128), np.float32), torch.bfloat16), bd, sd)
