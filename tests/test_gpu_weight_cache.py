"""GPU tests of the opt-in weight cache behind the stateless ops.

With the cache on, w4a16_matmul / w8a16_matmul / gptq_matmul / mpp_quant_matmul remember their weight
tensors by address, build the resident layers' tile-major copy on the first call and run the
resident-layer kernel afterwards.  Checked here:
  * the result is bit for bit what PackedQuantLinear.forward gives on the same tensors, and within
    2e-3 relative / 1e-2 absolute of the f32-accumulated oracle;
  * forgetting, eviction by size and shapes the resident layout does not cover fall back to the
    checkpoint-layout kernels;
  * a first call inside a graph capture allocates nothing (it takes the usual path), a warmed call
    is captured and replays with the eager bits.
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


def _trip(kind, K, N, g, seed):
    bits = 8 if kind.endswith("8") else 4
    if kind.startswith("awq"):
        return synth.awq_checkpoint(K, N, g, bits, seed=seed), ops.PACK_OUT, bits
    return synth.gptq_checkpoint(K, N, g, bits, seed=seed), ops.PACK_IN, bits


def _dense(kind, trip, dt):
    s_r = oracle.round_through(trip[2], dt)
    if kind == "awq":
        return oracle.dequantize_awq(trip[0], trip[1], s_r)
    if kind == "awq8":
        return oracle.dequantize_awq8(trip[0], trip[1], s_r)
    return oracle.dequantize_gptq(trip[0], trip[1], s_r, 8 if kind.endswith("8") else 4)


def _op(kind, ctx, x, dev, bits, pack_dim, out, tile=False):
    if tile:
        return ops.mpp_quant_matmul(x, dev[0], dev[1], dev[2], bits, pack_dim, out=out, ctx=ctx)
    if kind == "awq":
        return ops.w4a16_matmul(x, dev[0], dev[1], dev[2], out=out, ctx=ctx)
    if kind == "awq8":
        return ops.w8a16_matmul(x, dev[0], dev[1], dev[2], out=out, ctx=ctx)
    return ops.gptq_matmul(x, dev[0], dev[1], dev[2], bits, out=out, ctx=ctx)


@pytest.mark.parametrize("kind", ["awq", "awq8", "gptq", "gptq8"])
@pytest.mark.parametrize("dtn", ["f16", "bf16"])
def test_cached_op_equals_resident_layer_and_oracle(kind, dtn):
    dt = {"f16": oracle.F16, "bf16": oracle.BF16}[dtn]
    tdt = TORCH_DT[dt]
    K, N, g = 1024, 512, 128
    trip, pack_dim, bits = _trip(kind, K, N, g, seed=77)
    dev = (to_dev(trip[0]), to_dev(trip[1]), to_dev(trip[2], tdt))
    ctx = ops.Context()
    layer = ops.PackedQuantLinear(bits, pack_dim, dev[0], dev[1], dev[2], None, tdt, ctx=ctx)
    assert layer.prepacked
    w = _dense(kind, trip, dt)
    try:
        for m, tile in [(1, False), (5, False), (8, False), (33, True), (64, True)]:
            say(f"weight cache {kind} {dtn} m={m} tile={tile}")
            xh = round_x(np.random.default_rng(m).standard_normal((m, K)).astype(np.float32), dt)
            x = to_dev(xh, tdt)
            y0 = torch.empty((m, N), device="cuda", dtype=tdt)
            ctx.set_weight_cache(0)
            _op(kind, ctx, x, dev, bits, pack_dim, y0, tile)
            plain = ctx.last_plan()["kernel"]
            ctx.set_weight_cache(64 << 20)
            y1 = torch.empty_like(y0)
            _op(kind, ctx, x, dev, bits, pack_dim, y1, tile)           # builds the copy (or finds it)
            assert ctx.last_plan()["kernel"].startswith(f"pk{bits}_mfma"), ctx.last_plan()
            y2 = torch.empty_like(y0)
            _op(kind, ctx, x, dev, bits, pack_dim, y2, tile)           # served from the copy
            assert ctx.last_plan()["kernel"].startswith(f"pk{bits}_mfma")
            assert ctx.last_plan()["launches"] <= 2
            yl = layer.forward(x)
            torch.cuda.synchronize()
            np.testing.assert_array_equal(bits_of(y1), bits_of(yl))
            np.testing.assert_array_equal(bits_of(y2), bits_of(yl))
            wk = oracle.round_through(w, dt) if resident_rounds_weights(m, dt, kind.startswith("gptq")) else w
            assert_close(y1, oracle.matmul_nt_f32(xh, wk), f"{kind} {dtn} cached m={m} (uncached: {plain})")
        nbytes, entries = ctx.weight_cache_usage()
        assert entries == 1 and nbytes >= K * N * bits // 8
    finally:
        ctx.close()


def test_forget_evict_and_ineligible_shapes():
    K, N, g = 512, 256, 128
    tdt = torch.float16
    ctx = ops.Context()
    try:
        trips = [synth.awq_checkpoint(K, N, g, 4, seed=s) for s in (1, 2)]
        devs = [(to_dev(t[0]), to_dev(t[1]), to_dev(t[2], tdt)) for t in trips]
        x = torch.randn((2, K), device="cuda", dtype=tdt)
        y = torch.empty((2, N), device="cuda", dtype=tdt)
        ref = []
        for d in devs:
            ops.w4a16_matmul(x, *d, out=y, ctx=ctx)
            torch.cuda.synchronize()
            ref.append(as_f32(y).copy())
        assert not ctx.last_plan()["kernel"].startswith("pk4")

        one = (K // 128) * (N // 64) * (1024 + 64) * 4          # bytes of one copy
        say("weight cache: room for one copy, two weights in turn: the first stays, the second keeps its own kernel")
        ctx.set_weight_cache(one + 256)
        for rnd in range(3):
            for i, (d, r) in enumerate(zip(devs, ref)):
                ops.w4a16_matmul(x, *d, out=y, ctx=ctx)
                # evicting the copy the next call asks for would rebuild one on every call
                assert ctx.last_plan()["kernel"].startswith("pk4") == (i == 0), (rnd, i, ctx.last_plan()["kernel"])
                torch.cuda.synchronize()
                np.testing.assert_allclose(as_f32(y), r, rtol=2e-3, atol=1e-2)
                assert ctx.weight_cache_usage()[1] == 1
        say("weight cache: a weight that keeps coming alone takes the room")
        for _ in range(4):
            ops.w4a16_matmul(x, *devs[1], out=y, ctx=ctx)
        assert ctx.last_plan()["kernel"].startswith("pk4")
        torch.cuda.synchronize()
        np.testing.assert_allclose(as_f32(y), ref[1], rtol=2e-3, atol=1e-2)
        assert ctx.weight_cache_usage()[1] == 1

        say("weight cache: forget one, forget all")
        ctx.set_weight_cache(8 * one)
        for d in devs:
            ops.w4a16_matmul(x, *d, out=y, ctx=ctx)
        assert ctx.weight_cache_usage()[1] == 2
        ctx.forget_weights(devs[0][0])
        assert ctx.weight_cache_usage()[1] == 1
        ctx.forget_weights(None)
        assert ctx.weight_cache_usage() == (0, 0)

        say("weight cache: a new weight at a forgotten address is rebuilt")
        devs[0][0].copy_(devs[1][0]), devs[0][1].copy_(devs[1][1]), devs[0][2].copy_(devs[1][2])
        ops.w4a16_matmul(x, *devs[0], out=y, ctx=ctx)
        torch.cuda.synchronize()
        np.testing.assert_allclose(as_f32(y), ref[1], rtol=2e-3, atol=1e-2)

        say("weight cache: a shape outside the resident layout keeps its kernel")
        t3 = synth.awq_checkpoint(256, 96, 64, 4, seed=3)      # group 64, N % 64 != 0
        d3 = (to_dev(t3[0]), to_dev(t3[1]), to_dev(t3[2], tdt))
        x3 = torch.randn((1, 256), device="cuda", dtype=tdt)
        y3 = torch.empty((1, 96), device="cuda", dtype=tdt)
        before = ctx.weight_cache_usage()
        ops.w4a16_matmul(x3, *d3, out=y3, ctx=ctx)
        assert not ctx.last_plan()["kernel"].startswith("pk4")
        assert ctx.weight_cache_usage() == before

        say("weight cache: a copy larger than the limit is not made")
        ctx.forget_weights(None)
        ctx.set_weight_cache(one - 256)
        ops.w4a16_matmul(x, *devs[1], out=y, ctx=ctx)
        assert not ctx.last_plan()["kernel"].startswith("pk4")
        assert ctx.weight_cache_usage() == (0, 0)
    finally:
        ctx.close()


@pytest.mark.parametrize("fmt", [synth.GGUF_Q4_0, synth.GGUF_Q8_0, synth.GGUF_Q4_K, synth.GGUF_Q6_K, synth.GGUF_Q5_0,
                                 synth.GGUF_Q5_K])
def test_cached_gguf_op_equals_the_resident_layer(fmt):
    N, K = 256, 2048
    data = synth.gguf_weight(fmt, N, K, seed=90 + fmt)
    wd = to_dev(data)
    w = oracle.dequantize_gguf(fmt, data, N, K)
    ctx = ops.Context()
    layer = ops.QLinear(fmt, wd, K, N, None, torch.float32, ctx=ctx)
    assert layer.resident
    try:
        for m in (1, 3, 6, 8):
            say(f"weight cache gguf {synth.GGUF_NAMES[fmt]} m={m}")
            x = np.random.default_rng(m).standard_normal((m, K)).astype(np.float32)
            xd = to_dev(x)
            ctx.set_weight_cache(0)
            ops.gguf_quant_matmul(xd, wd, K, N, fmt, ctx=ctx)
            assert "_res_" not in ctx.last_plan()["kernel"]
            ctx.set_weight_cache(64 << 20)
            y1 = ops.gguf_quant_matmul(xd, wd, K, N, fmt, ctx=ctx)
            y2 = ops.gguf_quant_matmul(xd, wd, K, N, fmt, ctx=ctx)
            assert "_res_gemv_" in ctx.last_plan()["kernel"] and ctx.last_plan()["launches"] == (m + 3) // 4
            yl = layer.forward(xd)
            torch.cuda.synchronize()
            np.testing.assert_array_equal(bits_of(y1), bits_of(yl))
            np.testing.assert_array_equal(bits_of(y2), bits_of(y1))
            assert_close(y1, oracle.matmul_nt_f32(x, w), f"cached gguf op m={m}")
            nbytes, entries = ctx.weight_cache_usage()   # setting the limit to 0 above dropped the copy
            assert entries == 1 and nbytes >= data.nbytes
        ops.gguf_quant_matmul(to_dev(x[:1]), wd, K, N, fmt, ctx=ctx)
        assert ctx.weight_cache_usage()[1] == 1
        ctx.forget_weights(wd)
        assert ctx.weight_cache_usage() == (0, 0)
    finally:
        ctx.close()


@pytest.mark.parametrize("fmt", [synth.GGUF_Q4_0, synth.GGUF_Q8_0, synth.GGUF_Q4_K, synth.GGUF_Q6_K])
def test_cached_gguf_op_with_bf16_activations_runs_on_the_matrix_core_copy(fmt):
    """bf16 activations: the cache holds the matrix-core copy of a bf16 QLinear; the decode op (1 - 8 rows) and the
    prefill op (up to 32 rows) run on it with the layer's bits.  f32 calls on the same bytes keep the rotated copy:
    two entries."""
    N, K = 64, 1024
    data = synth.gguf_weight(fmt, N, K, seed=95 + fmt)
    wd = to_dev(data)
    w = oracle.dequantize_gguf(fmt, data, N, K)
    layer = ops.QLinear(fmt, wd, K, N, None, torch.bfloat16)
    nbytes = (data.size + 255) // 256 * 256
    ctx = ops.Context()
    try:
        ctx.set_weight_cache(1 << 22)
        for m, op in [(1, ops.gguf_quant_matmul), (8, ops.gguf_quant_matmul), (9, ops.gguf_quant_mul_mm), (32, ops.gguf_quant_mul_mm)]:
            say(f"weight cache gguf bf16 {synth.GGUF_NAMES[fmt]} m={m}")
            x = np.random.default_rng(m).standard_normal((m, K)).astype(np.float32)
            xd = to_dev(x, torch.bfloat16)
            y = op(xd, wd, K, N, fmt, ctx=ctx)
            assert "_mfma_bf16_mt" in ctx.last_plan()["kernel"], ctx.last_plan()
            np.testing.assert_array_equal(bits_of(y), bits_of(layer.forward(xd)))
            assert_close(y, oracle.matmul_nt_f32(round_x(x, oracle.BF16), w), f"cached gguf bf16 op m={m}", bf16_out=True)
        assert ctx.weight_cache_usage() == (nbytes, 1)
        x33 = to_dev(x[:1].repeat(33, 0), torch.bfloat16)
        ops.gguf_quant_mul_mm(x33, wd, K, N, fmt, ctx=ctx)
        assert "_mul_mm_" in ctx.last_plan()["kernel"]  # more rows than the integer kernel takes: the file layout
        ctx.set_tuning("OXQ_GGUF_GEMM_MIN_M", 33)       # or, where it pays, the prefill kernel on the same copy
        y33 = ops.gguf_quant_mul_mm(x33, wd, K, N, fmt, ctx=ctx)
        assert "_gemm_bf16_r64x8" in ctx.last_plan()["kernel"] and ctx.weight_cache_usage() == (nbytes, 1)
        tune("OXQ_GGUF_GEMM_MIN_M", 33)
        np.testing.assert_array_equal(bits_of(y33), bits_of(layer.forward(x33)))
        tune("OXQ_GGUF_GEMM_MIN_M", None)
        ctx.set_tuning("OXQ_GGUF_GEMM_MIN_M", None)
        ops.gguf_quant_matmul(to_dev(x[:2]), wd, K, N, fmt, ctx=ctx)
        assert "_res_gemv_f32" in ctx.last_plan()["kernel"]
        assert ctx.weight_cache_usage() == (2 * nbytes, 2)
    finally:
        ctx.close()


def test_cached_mxfp4_moe_op_runs_on_the_resident_experts_copy():
    """The grouped MXFP4 op with the cache on: the stacked expert tensors get the resident experts' tile-major copy on
    the first call; decode sizes then run its GEMV, many pairs an expert its tiles, with the handle's bits and the
    fused SwiGLU; forgetting the blocks goes back to the checkpoint-layout kernels."""
    E, N, K = 4, 96, 2880
    blocks, scales = synth.mxfp4_weight(E * N, K, seed=77)
    bias = np.random.default_rng(78).standard_normal((E, N)).astype(np.float32) * 0.1
    bd, sd, biasd = to_dev(blocks), to_dev(scales), to_dev(bias, torch.bfloat16)
    ex = ops.Mxfp4Experts(bd, sd, biasd, E, K, N)
    nb = K // 32
    want_bytes = E * (N // 16) * nb * 256 + E * (N // 16) * -(-(-(-nb // 4)) // 4) * 256
    ctx = ops.Context()
    try:
        ctx.set_weight_cache(1 << 24)
        for counts, kern in [([1, 0, 2, 1], "mxfp4_experts_gemv_bf16_t4"), ([20, 0, 13, 7], "mxfp4_experts_gemm_bf16_r16x8"),
                             ([70, 1, 40, 30], "mxfp4_experts_gemm_bf16_r32x8")]:
            say(f"weight cache mxfp4 moe counts={counts}")
            offsets = np.zeros(E + 1, np.int32)
            offsets[1:] = np.cumsum(counts)
            n_tok = max(counts)
            tokens = np.concatenate([np.arange(c, dtype=np.int32) % n_tok for c in counts]).astype(np.int32)
            x = np.random.default_rng(sum(counts)).standard_normal((n_tok, K)).astype(np.float32)
            xd, off_d, tok_d = to_dev(x, torch.bfloat16), to_dev(offsets), to_dev(tokens)
            y = ops.mxfp4_moe_matmul(xd, bd, sd, biasd, off_d, tok_d, K, N, ctx=ctx)
            assert ctx.last_plan()["kernel"] == kern, ctx.last_plan()
            np.testing.assert_array_equal(bits_of(y), bits_of(ex.matmul(xd, off_d, tok_d)))
            ref = np.zeros((int(offsets[-1]), N), np.float32)
            xb, bb = round_x(x, oracle.BF16), round_x(bias, oracle.BF16)
            for e in range(E):
                lo, hi = int(offsets[e]), int(offsets[e + 1])
                if hi > lo:
                    w = oracle.dequantize_mxfp4_f32(blocks[e * N * nb * 16:(e + 1) * N * nb * 16], scales[e * N * nb:(e + 1) * N * nb], N, K)
                    ref[lo:hi] = oracle.matmul_nt_f32(xb[tokens[lo:hi]], w, bb[e])
            assert_close(y, ref, f"cached mxfp4 moe op {counts}")
            h = ops.mxfp4_moe_gate_up_swiglu(xd, bd, sd, biasd, off_d, tok_d, K, N, 7.0, ctx=ctx)
            assert ctx.last_plan()["kernel"] == kern + "_swiglu"
            np.testing.assert_array_equal(bits_of(h), bits_of(ex.gate_up_swiglu(xd, off_d, tok_d, 7.0)))
        assert ctx.weight_cache_usage() == (want_bytes, 1)
        ctx.forget_weights(bd)
        assert ctx.weight_cache_usage() == (0, 0)
        ctx.set_weight_cache(0)
        ops.mxfp4_moe_matmul(xd, bd, sd, biasd, off_d, tok_d, K, N, ctx=ctx)
        assert "experts" not in ctx.last_plan()["kernel"]
    finally:
        ctx.close()


def test_capture_allocates_nothing_and_replays_the_cached_kernel():
    K, N, g, m = 2048, 512, 128, 4
    tdt = torch.float16
    trip = synth.awq_checkpoint(K, N, g, 4, seed=9)
    dev = (to_dev(trip[0]), to_dev(trip[1]), to_dev(trip[2], tdt))
    x = torch.randn((m, K), device="cuda", dtype=tdt)
    y = torch.empty((m, N), device="cuda", dtype=tdt)
    ctx = ops.Context()
    try:
        ctx.set_weight_cache(64 << 20)
        ops.w4a16_matmul(x, *dev, out=y, ctx=ctx)                # warm the kernels' one-time set-up
        ctx.forget_weights(None)
        stream = torch.cuda.Stream()
        say("weight cache: first sight of a weight during capture")
        g1 = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g1, stream=stream):
            ops.w4a16_matmul(x, *dev, out=y, ctx=ctx)
            missed = ctx.last_plan()["kernel"]
        assert not missed.startswith("pk4"), missed
        assert ctx.weight_cache_usage() == (0, 0)

        ops.w4a16_matmul(x, *dev, out=y, ctx=ctx)                # eager: builds the copy
        torch.cuda.synchronize()
        assert ctx.weight_cache_usage()[1] == 1
        say("weight cache: warmed call captured and replayed")
        g2 = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g2, stream=stream):
            ops.w4a16_matmul(x, *dev, out=y, ctx=ctx)
            assert ctx.last_plan()["kernel"].startswith("pk4")
        gen = torch.Generator(device="cuda")
        for i in range(1, 5):
            gen.manual_seed(i)
            x.copy_(torch.randn((m, K), device="cuda", dtype=tdt, generator=gen))
            y.zero_()
            ops.w4a16_matmul(x, *dev, out=y, ctx=ctx)
            torch.cuda.synchronize()
            want = bits_of(y).copy()
            y.zero_()
            torch.cuda.synchronize()
            g2.replay()
            torch.cuda.synchronize()
            np.testing.assert_array_equal(bits_of(y), want, err_msg=f"replay {i}")

        say("weight cache: the copy a captured graph holds survives a smaller limit and other weights")
        one = ctx.weight_cache_usage()[0]
        ctx.set_weight_cache(256)                                  # would drop every copy that is not held
        assert ctx.weight_cache_usage() == (one, 1)
        ctx.set_weight_cache(one + 256)                            # room for one: a second weight would evict it
        trip2 = synth.awq_checkpoint(K, N, g, 4, seed=10)
        dev2 = (to_dev(trip2[0]), to_dev(trip2[1]), to_dev(trip2[2], tdt))
        y2 = torch.empty((m, N), device="cuda", dtype=tdt)
        for _ in range(5):
            ops.w4a16_matmul(x, *dev2, out=y2, ctx=ctx)
            assert not ctx.last_plan()["kernel"].startswith("pk4")
        assert ctx.weight_cache_usage() == (one, 1)
        y.zero_()
        ops.w4a16_matmul(x, *dev, out=y, ctx=ctx)
        torch.cuda.synchronize()
        want = bits_of(y).copy()
        y.zero_()
        torch.cuda.synchronize()
        g2.replay()
        torch.cuda.synchronize()
        np.testing.assert_array_equal(bits_of(y), want, err_msg="replay after the limit shrank")
        del g2                                                     # forgetting the weight invalidates the graph
        ctx.forget_weights(dev[0])
        assert ctx.weight_cache_usage() == (0, 0)
    finally:
        ctx.close()
