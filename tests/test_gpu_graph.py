"""HIP-graph capture of the hot path: a captured forward must give the eager result on every
replay, with eager work and synchronizations between replays (captured memset nodes have given
wrong results on replays after the first on this platform, so nothing here may rely on them;
the library's launch paths record kernels only).
"""
import sys

import numpy as np
import pytest
import torch

from oxydllm_amd import synth
from tests.helpers import bits_of, to_dev

pytestmark = pytest.mark.gpu
ops = None


def setup_module(module):
    from oxydllm_amd import ops as _ops
    module.ops = _ops


def say(msg):
    print(f"[case] {msg}", flush=True)
    sys.stdout.flush()


def replay_matches_eager(name, fn, make_inputs, out):
    """fn() writes `out` from the current inputs; make_inputs(i) rewrites the inputs in place."""
    say(f"graph {name}")
    make_inputs(0)
    fn()                                  # warm-up: one-time attribute calls happen outside the capture
    torch.cuda.synchronize()
    stream = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=stream):
        fn()
    for i in range(1, 5):
        make_inputs(i)                    # new activations in the same buffers
        out.zero_()
        fn()                              # eager reference for these inputs
        torch.cuda.synchronize()
        want = bits_of(out).copy()
        out.zero_()                       # eager work between the replays
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        np.testing.assert_array_equal(bits_of(out), want, err_msg=f"{name}: replay {i}")


@pytest.mark.parametrize("K,N,m", [(4096, 1024, 1), (4096, 1024, 64), (8192, 512, 16)])
def test_resident_layer_forward_in_a_graph(K, N, m):
    """(8192, 512): 8 strips, so K is cut into slices and the call is two launches."""
    trip = synth.awq_checkpoint(K, N, 128, 4, seed=K + N)
    layer = ops.PackedQuantLinear(4, ops.PACK_OUT, to_dev(trip[0]), to_dev(trip[1]),
                                  to_dev(trip[2], torch.float16), None, torch.float16)
    x = torch.empty((m, K), device="cuda", dtype=torch.float16)
    y = torch.empty((m, N), device="cuda", dtype=torch.float16)
    gen = torch.Generator(device="cuda")

    def inputs(i):
        gen.manual_seed(100 + i)
        x.copy_(torch.randn((m, K), device="cuda", generator=gen).to(torch.float16))
    replay_matches_eager(f"pk4 {K}x{N} m={m}", lambda: layer.forward(x, out=y), inputs, y)
    if (K, N) == (8192, 512):
        assert ops.default_context().last_plan()["launches"] == 2


def test_checkpoint_layout_ops_in_a_graph():
    """The stateless W4A16 op: split-K with the fused last-arriver reduction (counters return to
    zero by themselves) and with the separate reduction launch."""
    K, N = 4096, 2048
    trip = synth.awq_checkpoint(K, N, 128, 4, seed=5)
    qw, qz, sc = to_dev(trip[0]), to_dev(trip[1]), to_dev(trip[2], torch.float16)
    for m in (1, 8):
        x = torch.empty((m, K), device="cuda", dtype=torch.float16)
        y = torch.empty((m, N), device="cuda", dtype=torch.float16)

        def inputs(i, x=x, m=m):
            x.copy_(torch.randn((m, K), device="cuda").to(torch.float16) * (1 + i))
        replay_matches_eager(f"w4a16 op m={m}", lambda: ops.w4a16_matmul(x, qw, qz, sc, out=y), inputs, y)


def test_block_quant_paths_in_a_graph():
    K, N = 2048, 1024
    data = to_dev(synth.gguf_weight(synth.GGUF_Q4_K, N, K, seed=9))
    blocks, scales = synth.mxfp4_weight(N, K, seed=10)
    bd, sd = to_dev(blocks), to_dev(scales)
    for m in (1, 6, 40):
        x = torch.empty((m, K), device="cuda", dtype=torch.bfloat16)
        y = torch.empty((m, N), device="cuda", dtype=torch.bfloat16)

        def inputs(i, x=x, m=m):
            x.copy_(torch.randn((m, K), device="cuda").to(torch.bfloat16) * (1 + 0.5 * i))
        layer = ops.QLinear(synth.GGUF_Q4_K, data, K, N, None, torch.bfloat16)
        replay_matches_eager(f"gguf q4_k m={m}", lambda: layer.forward(x, out=y), inputs, y)
        replay_matches_eager(f"mxfp4 m={m}", lambda: ops.mxfp4_matmul(x, bd, sd, K, N, out=y), inputs, y)


def test_fused_epilogues_and_workspace_repack_in_a_graph():
    """The gate|up layer with the activation in its epilogue, the GPTQ tile kernel on the checkpoint layout,
    the stateless tile op that builds its tile-major copy in the ctx workspace (the workspace rewritten on
    every replay), and the expert GEMV with the fused SwiGLU."""
    gen = torch.Generator(device="cuda")
    K, I = 1024, 256
    trip = synth.awq_checkpoint(K, 2 * I, 128, 4, seed=3)
    layer = ops.PackedQuantLinear(4, ops.PACK_OUT, to_dev(trip[0]), to_dev(trip[1]), to_dev(trip[2], torch.float16),
                                  None, torch.float16, gate_up_act=ops.ACT_GATED_SILU)
    for m in (1, 40):
        x = torch.empty((m, K), device="cuda", dtype=torch.float16)
        y = torch.empty((m, I), device="cuda", dtype=torch.float16)

        def inputs(i, x=x, m=m):
            gen.manual_seed(300 + i)
            x.copy_(torch.randn((m, K), device="cuda", generator=gen).to(torch.float16))
        replay_matches_eager(f"gate|up silu m={m}", lambda: layer.forward(x, out=y), inputs, y)

    for bits in (4, 8):
        gq = synth.gptq_checkpoint(K, 384, 128, bits, seed=bits)
        d = (to_dev(gq[0]), to_dev(gq[1]), to_dev(gq[2], torch.float16))
        for m in (2, 24):
            x = torch.empty((m, K), device="cuda", dtype=torch.float16)
            y = torch.empty((m, 384), device="cuda", dtype=torch.float16)

            def inputs(i, x=x, m=m):
                gen.manual_seed(400 + i)
                x.copy_(torch.randn((m, K), device="cuda", generator=gen).to(torch.float16))
            if m <= 8:
                fn = lambda: ops.gptq_matmul(x, *d, bits, out=y)
            else:
                fn = lambda: ops.mpp_quant_matmul(x, *d, bits, ops.PACK_IN, out=y)
            replay_matches_eager(f"gptq{bits} m={m}", fn, inputs, y)
            if m > 8:
                plan = ops.default_context().last_plan()
                assert plan["kernel"].startswith(f"gptq{bits}_tile") and plan["launches"] == 1, plan

    # 8-bit AWQ above 8 rows has no tile kernel on the checkpoint layout: the op repacks into the ctx
    # workspace and runs the resident-layer kernel on the copy (two launches, the workspace rewritten on
    # every replay)
    aq = synth.awq_checkpoint(K, 384, 128, 8, seed=11)
    d = (to_dev(aq[0]), to_dev(aq[1]), to_dev(aq[2], torch.float16))
    m = 24
    x = torch.empty((m, K), device="cuda", dtype=torch.float16)
    y = torch.empty((m, 384), device="cuda", dtype=torch.float16)

    def inputs(i):
        gen.manual_seed(500 + i)
        x.copy_(torch.randn((m, K), device="cuda", generator=gen).to(torch.float16))
    replay_matches_eager(f"awq8 m={m}", lambda: ops.mpp_quant_matmul(x, *d, 8, ops.PACK_OUT, out=y), inputs, y)
    assert ops.default_context().last_plan()["launches"] == 2

    E, N, Kx = 3, 64, 96
    blocks = torch.from_numpy(np.concatenate([synth.mxfp4_weight(N, Kx, seed=e)[0] for e in range(E)])).cuda()
    scales = torch.from_numpy(np.concatenate([synth.mxfp4_weight(N, Kx, seed=e)[1] for e in range(E)])).cuda()
    offsets = to_dev(np.array([0, 2, 2, 5], np.int32))
    tok = to_dev(np.array([0, 3, 1, 2, 3], np.int32))
    x = torch.empty((4, Kx), device="cuda", dtype=torch.bfloat16)
    y = torch.empty((5, N // 2), device="cuda", dtype=torch.bfloat16)

    def inputs(i):
        gen.manual_seed(500 + i)
        x.copy_(torch.randn((4, Kx), device="cuda", generator=gen).to(torch.bfloat16))
    replay_matches_eager("mxfp4 gate_up + swiglu",
                         lambda: ops.mxfp4_moe_gate_up_swiglu(x, blocks, scales, None, offsets, tok, Kx, N, 7.0, out=y),
                         inputs, y)


def test_resident_experts_in_a_graph():
    """The MoE decode step on resident experts: gate_up with the SwiGLU in its epilogue, then down,
    captured together; the token lists stay, the activations change between replays."""
    gen = torch.Generator(device="cuda")
    E, H, I = 4, 128, 96
    gu = [synth.mxfp4_weight(2 * I, H, seed=10 + e) for e in range(E)]
    dn = [synth.mxfp4_weight(H, I, seed=20 + e) for e in range(E)]
    gub = torch.from_numpy(np.concatenate([g[0] for g in gu])).cuda(), torch.from_numpy(np.concatenate([g[1] for g in gu])).cuda()
    dnb = torch.from_numpy(np.concatenate([d[0] for d in dn])).cuda(), torch.from_numpy(np.concatenate([d[1] for d in dn])).cuda()
    gu_bias = (torch.randn((E, 2 * I), device="cuda") * 0.1).to(torch.bfloat16)
    dn_bias = (torch.randn((E, H), device="cuda") * 0.1).to(torch.bfloat16)
    gu_ex = ops.Mxfp4Experts(gub[0], gub[1], gu_bias, E, H, 2 * I)
    dn_ex = ops.Mxfp4Experts(dnb[0], dnb[1], dn_bias, E, I, H)
    assert gu_ex.resident and dn_ex.resident
    offsets = to_dev(np.array([0, 3, 3, 4, 6], np.int32))
    tok = to_dev(np.array([0, 1, 2, 1, 0, 2], np.int32))
    x = torch.empty((3, H), device="cuda", dtype=torch.bfloat16)
    h = torch.empty((6, I), device="cuda", dtype=torch.bfloat16)
    y = torch.empty((6, H), device="cuda", dtype=torch.bfloat16)

    def inputs(i):
        gen.manual_seed(600 + i)
        x.copy_(torch.randn((3, H), device="cuda", generator=gen).to(torch.bfloat16))

    def step():
        gu_ex.gate_up_swiglu(x, offsets, tok, 7.0, out=h)
        assert ops.default_context().last_plan()["kernel"].startswith("mxfp4_experts_gemv")
        dn_ex.matmul(h, offsets, None, out=y)
    replay_matches_eager("resident experts: gate_up + swiglu, down", step, inputs, y)
