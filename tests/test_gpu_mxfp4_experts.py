"""Resident MXFP4 experts (oxq_mxfp4_experts_*) through the C ABI.

The handle repacks the stacked expert tensors tile-major at construction.  The repack is pinned bit for
bit: the dense dequant read back from the copy must equal the oracle's dequantize_mxfp4_f32 of the
checkpoint bytes (mxfp4.rs:35-64).  The grouped GEMV on the copy is held to the f32-accumulated oracle
(moe.rs:593-605 over Mxfp4Linear::forward) within 2e-3 relative / 1e-2 absolute, plus half a bf16 ulp
for the bf16 output, on the reference's generator shape (metal_ops.rs:6626-6631), ragged shapes, idle
experts, more pairs per expert than one pass takes, and the benchmark's configuration 4.
"""
import sys

import numpy as np
import pytest
import torch

import oracle
from oxydllm_amd import synth
from tests.helpers import assert_close, bits_of, round_x, to_dev, tune

pytestmark = pytest.mark.gpu


def say(msg):
    print(f"[case] {msg}", flush=True)
    sys.stdout.flush()


def _experts(E, N, K, seed, bias=True):
    blocks, scales = synth.mxfp4_weight(E * N, K, seed=seed)
    b = (np.random.default_rng(seed + 1).standard_normal((E, N)).astype(np.float32) * 0.1) if bias else None
    return blocks, scales, b


def _dense(blocks, scales, e, N, K):
    nb = K // 32
    return oracle.dequantize_mxfp4_f32(blocks[e * N * nb * 16:(e + 1) * N * nb * 16], scales[e * N * nb:(e + 1) * N * nb], N, K)


def _lists(counts):
    """expert_offsets and token ids for the given number of pairs per expert (tokens 0, 1, 2, ... in turn)."""
    offsets = np.zeros(len(counts) + 1, np.int32)
    offsets[1:] = np.cumsum(counts)
    n_tok = max(1, max(counts))
    tokens = np.concatenate([np.arange(c, dtype=np.int32) % n_tok for c in counts]) if offsets[-1] else np.zeros(0, np.int32)
    return offsets, tokens.astype(np.int32), n_tok


@pytest.mark.parametrize("E,N,K", [(3, 16, 64), (2, 48, 96), (4, 80, 2880), (2, 64, 32), (1, 10, 64)])
def test_experts_dequantize_is_bit_exact(E, N, K):
    from oxydllm_amd import ops
    say(f"experts dequant E={E} N={N} K={K}")
    blocks, scales, _ = _experts(E, N, K, seed=E * N + K, bias=False)
    if N == 16:  # the reference's own generator (metal_ops.rs:6626-6631) on a tile-aligned shape
        i = np.arange(blocks.size, dtype=np.int64)
        blocks = ((37 * i + 11) & 255).astype(np.uint8)
        scales = (125 + np.arange(scales.size) % 5).astype(np.uint8)
    ex = ops.Mxfp4Experts(to_dev(blocks), to_dev(scales), None, E, K, N)
    assert ex.resident == (N % 16 == 0)
    for e in range(E):
        got = ex.dequantize(e).cpu().numpy()
        want = _dense(blocks, scales, e, N, K)
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), f"expert {e}: repack changed a weight"


@pytest.mark.parametrize("E,N,K,counts", [
    (3, 16, 64, [1, 0, 2]),
    (4, 48, 96, [4, 1, 0, 3]),
    (5, 80, 160, [0, 0, 5, 9, 1]),        # more pairs than one pass of 4 takes
    (2, 64, 2880, [2, 3]),
    (6, 128, 512, [0, 0, 0, 0, 0, 1]),
    # chunk counts with a straight-line kernel of their own (16, 23, 24, 32 chunks of four blocks), a ragged
    # last chunk beside them (2848 = 89 blocks) and the looping kernel on either side (22 and 25 chunks)
    (2, 32, 2048, [1, 5]),
    (2, 48, 3072, [3, 2]),
    (1, 32, 4096, [6]),
    (2, 32, 2848, [4, 1]),
    (2, 32, 2816, [1, 2]),
    (2, 32, 3200, [2, 4]),
])
@pytest.mark.parametrize("gather", [True, False])
def test_experts_matmul_matches_oracle_and_the_stateless_op(E, N, K, counts, gather):
    from oxydllm_amd import ops
    say(f"experts matmul E={E} N={N} K={K} counts={counts} gather={gather}")
    tune("OXQ_MXFP4_GEMM_MIN_PAIRS", 0)  # the decode kernel at every pair count, also where the tiles would take over
    blocks, scales, bias = _experts(E, N, K, seed=7 * E + N)
    offsets, tokens, n_tok = _lists(counts)
    n_pairs = int(offsets[-1])
    x = np.random.default_rng(K).standard_normal((n_tok, K)).astype(np.float32)
    xb, bb = round_x(x, oracle.BF16), round_x(bias, oracle.BF16)
    ref = np.zeros((n_pairs, N), np.float32)
    for e in range(E):
        lo, hi = int(offsets[e]), int(offsets[e + 1])
        if hi > lo:
            ref[lo:hi] = oracle.matmul_nt_f32(xb[tokens[lo:hi]], _dense(blocks, scales, e, N, K), bb[e])
    bd, sd, biasd = to_dev(blocks), to_dev(scales), to_dev(bias, torch.bfloat16)
    ex = ops.Mxfp4Experts(bd, sd, biasd, E, K, N)
    assert ex.resident
    off_d = to_dev(offsets)
    if gather:
        xd, tok_d = to_dev(x, torch.bfloat16), to_dev(tokens)
    else:
        xd, tok_d = to_dev(x[tokens], torch.bfloat16), None
    y = ex.matmul(xd, off_d, tok_d)
    plan = ops.default_context().last_plan()
    assert plan["kernel"].startswith("mxfp4_experts_gemv_bf16") and plan["launches"] == 1, plan
    assert_close(y, ref, "experts matmul")
    y0 = ops.mxfp4_moe_matmul(xd, bd, sd, biasd, off_d, tok_d, K, N)
    assert_close(y, y0.float().cpu().numpy(), "experts matmul against the stateless op", bf16_out=True)
    # run-to-run determinism
    assert np.array_equal(bits_of(ex.matmul(xd, off_d, tok_d)), bits_of(y))


@pytest.mark.parametrize("E,N,K,counts", [(3, 32, 64, [2, 0, 1]), (4, 96, 2880, [1, 4, 0, 6])])
def test_experts_gate_up_swiglu_equals_the_two_calls(E, N, K, counts):
    from oxydllm_amd import ops
    say(f"experts swiglu E={E} N={N} K={K}")
    tune("OXQ_MXFP4_GEMM_MIN_PAIRS", 0)
    blocks, scales, bias = _experts(E, N, K, seed=N + K)
    offsets, tokens, n_tok = _lists(counts)
    x = np.random.default_rng(1).standard_normal((n_tok, K)).astype(np.float32) * 2
    ex = ops.Mxfp4Experts(to_dev(blocks), to_dev(scales), to_dev(bias, torch.bfloat16), E, K, N)
    xd, off_d, tok_d = to_dev(x, torch.bfloat16), to_dev(offsets), to_dev(tokens)
    fused = ex.gate_up_swiglu(xd, off_d, tok_d, 7.0)
    assert ops.default_context().last_plan()["kernel"].endswith("_swiglu")
    gu = ex.matmul(xd, off_d, tok_d)
    two = ops.gated_activation(gu, ops.ACT_GPT_OSS_SWIGLU, 7.0)
    assert np.array_equal(bits_of(fused), bits_of(two))
    want = oracle.gpt_oss_swiglu(gu.float().cpu().numpy(), 7.0)
    assert_close(fused, want, "swiglu on the resident copy")


@pytest.mark.parametrize("E,N,K,counts", [
    (3, 80, 2880, [70, 0, 130]),      # 22.5 chunks; five tiles: a wave with one live tile of its four
    (2, 192, 96, [5, 64]),            # three blocks: one chunk, cut off; a whole row tile and a sliver
    (4, 64, 512, [1, 65, 0, 128]),    # four chunks; an idle expert
    (2, 640, 1280, [33, 200]),        # ten chunks: both ring halves; two column groups, the second two waves wide
])
@pytest.mark.parametrize("rows", [16, 32, 64, 128])
@pytest.mark.parametrize("gather", [True, False])
def test_experts_prefill_kernel_on_the_copy(E, N, K, counts, rows, gather):
    """Many pairs an expert: tiles of 16 - 128 of an expert's pairs x the waves' four tiles of 16 weight rows, x
    gathered through the token list straight into LDS, whole K in a wave's accumulators.  Against the
    f32-accumulated oracle on the dense dequant (the weights are exact in bf16, so this is the tile matmul's
    arithmetic too), run to run bitwise, and with the fused SwiGLU epilogue bit-identical to matmul + activation."""
    from oxydllm_amd import ops
    say(f"experts prefill E={E} N={N} K={K} counts={counts} rows={rows} gather={gather}")
    tune("OXQ_MXFP4_GEMM_MIN_PAIRS", 1)
    tune("OXQ_MXFP4_GEMM_ROWS", rows)
    blocks, scales, bias = _experts(E, N, K, seed=3 * E + N)
    offsets, tokens, n_tok = _lists(counts)
    n_pairs = int(offsets[-1])
    x = np.random.default_rng(K + 1).standard_normal((n_tok, K)).astype(np.float32)
    xb, bb = round_x(x, oracle.BF16), round_x(bias, oracle.BF16)
    ref = np.zeros((n_pairs, N), np.float32)
    for e in range(E):
        lo, hi = int(offsets[e]), int(offsets[e + 1])
        if hi > lo:
            ref[lo:hi] = oracle.matmul_nt_f32(xb[tokens[lo:hi]], _dense(blocks, scales, e, N, K), bb[e])
    bd, sd, biasd = to_dev(blocks), to_dev(scales), to_dev(bias, torch.bfloat16)
    ex = ops.Mxfp4Experts(bd, sd, biasd, E, K, N)
    assert ex.resident
    off_d = to_dev(offsets)
    if gather:
        xd, tok_d = to_dev(x, torch.bfloat16), to_dev(tokens)
    else:
        xd, tok_d = to_dev(x[tokens], torch.bfloat16), None
    y = ex.matmul(xd, off_d, tok_d)
    plan = ops.default_context().last_plan()
    kname = f"mxfp4_experts_gemm_bf16_r{rows}x8"
    assert plan["kernel"] == kname and plan["launches"] == 1, plan
    assert plan["grid"][0] == -(-(N // 16) // 32) and plan["grid"][1] == n_pairs // rows + E, plan
    assert_close(y, ref, "experts prefill matmul")
    assert np.array_equal(bits_of(ex.matmul(xd, off_d, tok_d)), bits_of(y))
    # without a bias, into a buffer that holds other values
    plain = ops.Mxfp4Experts(bd, sd, None, E, K, N)
    out = torch.full((n_pairs, N), 3.0, device="cuda", dtype=torch.bfloat16)
    plain.matmul(xd, off_d, tok_d, out=out)
    assert ops.default_context().last_plan()["kernel"] == kname
    assert_close(out, ref - np.repeat(bb, counts, axis=0), "experts prefill matmul, no bias")
    if rows == 32:
        # an output that starts at an odd element (the tiles store two neighbouring outputs as one word): the tile
        # matmul on the caller's tensors takes the call
        buf = torch.zeros(n_pairs * N + 1, device="cuda", dtype=torch.bfloat16)
        ex.matmul(xd, off_d, tok_d, out=buf[1:].view(n_pairs, N))
        assert "mul_mm" in ops.default_context().last_plan()["kernel"], ops.default_context().last_plan()
        assert_close(buf[1:].view(n_pairs, N), ref, "experts prefill matmul, odd output address")
    # interleaved gate / up rows with the clamped SwiGLU in the epilogue
    fused = ex.gate_up_swiglu(xd * 2, off_d, tok_d, 7.0)
    assert ops.default_context().last_plan()["kernel"] == kname + "_swiglu"
    two = ops.gated_activation(ex.matmul(xd * 2, off_d, tok_d), ops.ACT_GPT_OSS_SWIGLU, 7.0)
    assert np.array_equal(bits_of(fused), bits_of(two))


def test_experts_fall_back_where_the_copy_does_not_apply(monkeypatch):
    from oxydllm_amd import ops
    say("experts fallback")
    E, N, K = 2, 10, 64   # the reference's n = 10: not a whole tile of 16 rows
    blocks, scales, bias = _experts(E, N, K, seed=3)
    offsets, tokens, n_tok = _lists([2, 1])
    x = np.random.default_rng(2).standard_normal((n_tok, K)).astype(np.float32)
    bd, sd, biasd = to_dev(blocks), to_dev(scales), to_dev(bias, torch.bfloat16)
    ex = ops.Mxfp4Experts(bd, sd, biasd, E, K, N)
    assert not ex.resident
    y = ex.matmul(to_dev(x, torch.bfloat16), to_dev(offsets), to_dev(tokens))
    y0 = ops.mxfp4_moe_matmul(to_dev(x, torch.bfloat16), bd, sd, biasd, to_dev(offsets), to_dev(tokens), K, N)
    assert np.array_equal(bits_of(y), bits_of(y0))
    # the prefill kernel switched off: many pairs per expert take the tile matmul on the checkpoint layout, same
    # result as the stateless op
    tune("OXQ_MXFP4_GEMM_MIN_PAIRS", 0)
    E, N, K = 2, 64, 128
    blocks, scales, bias = _experts(E, N, K, seed=4)
    offsets, tokens, n_tok = _lists([20, 13])
    x = np.random.default_rng(3).standard_normal((n_tok, K)).astype(np.float32)
    bd, sd, biasd = to_dev(blocks), to_dev(scales), to_dev(bias, torch.bfloat16)
    ex = ops.Mxfp4Experts(bd, sd, biasd, E, K, N)
    assert ex.resident
    y = ex.matmul(to_dev(x, torch.bfloat16), to_dev(offsets), to_dev(tokens))
    assert "mul_mm" in ops.default_context().last_plan()["kernel"]
    y0 = ops.mxfp4_moe_matmul(to_dev(x, torch.bfloat16), bd, sd, biasd, to_dev(offsets), to_dev(tokens), K, N)
    assert np.array_equal(bits_of(y), bits_of(y0))
    tune("OXQ_PREPACK", 0)
    assert not ops.Mxfp4Experts(bd, sd, biasd, E, K, N).resident


def test_experts_config4_decode_step():
    """Benchmark configuration 4: 32 experts, top-4, 8 tokens, hidden 2880, gate_up 5760 rows, down 2880."""
    from oxydllm_amd import ops
    E, top_k, H, I, T = 32, 4, 2880, 2880, 8
    rng = np.random.default_rng(0x0A0D11E9)
    logits = rng.standard_normal((T, E)).astype(np.float32)
    idx, vals = oracle.moe_route(logits, top_k, True)
    offsets, tokens, _ = oracle.moe_group(idx, vals, E)
    offsets, tokens = offsets.astype(np.int32), tokens.astype(np.int32)
    n_pairs = T * top_k
    say(f"experts config 4: {int((np.diff(offsets) > 0).sum())} active experts")
    gu_b, gu_s = synth.mxfp4_weight(E * 2 * I, H, seed=1)
    dn_b, dn_s = synth.mxfp4_weight(E * H, I, seed=2)
    gu_bias = rng.standard_normal((E, 2 * I)).astype(np.float32) * 0.1
    dn_bias = rng.standard_normal((E, H)).astype(np.float32) * 0.1
    x = rng.standard_normal((T, H)).astype(np.float32)
    h_in = rng.standard_normal((n_pairs, I)).astype(np.float32)
    xb, hb = round_x(x, oracle.BF16), round_x(h_in, oracle.BF16)
    gub, dnb = round_x(gu_bias, oracle.BF16), round_x(dn_bias, oracle.BF16)
    ref_gu = np.zeros((n_pairs, 2 * I), np.float32)
    ref_dn = np.zeros((n_pairs, H), np.float32)
    for e in range(E):
        lo, hi = int(offsets[e]), int(offsets[e + 1])
        if hi > lo:
            ref_gu[lo:hi] = oracle.matmul_nt_f32(xb[tokens[lo:hi]], _dense(gu_b, gu_s, e, 2 * I, H), gub[e])
            ref_dn[lo:hi] = oracle.matmul_nt_f32(hb[lo:hi], _dense(dn_b, dn_s, e, H, I), dnb[e])
    gu = ops.Mxfp4Experts(to_dev(gu_b), to_dev(gu_s), to_dev(gu_bias, torch.bfloat16), E, H, 2 * I)
    dn = ops.Mxfp4Experts(to_dev(dn_b), to_dev(dn_s), to_dev(dn_bias, torch.bfloat16), E, I, H)
    assert gu.resident and dn.resident
    off_d, tok_d = to_dev(offsets), to_dev(tokens)
    y = gu.matmul(to_dev(x, torch.bfloat16), off_d, tok_d)
    assert_close(y, ref_gu, "experts gate_up")
    y2 = dn.matmul(to_dev(h_in, torch.bfloat16), off_d, None)
    assert_close(y2, ref_dn, "experts down")
    for e in (0, 17, 31):
        assert np.array_equal(gu.dequantize(e).cpu().numpy().view(np.uint32), _dense(gu_b, gu_s, e, 2 * I, H).view(np.uint32))
