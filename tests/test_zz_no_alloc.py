"""The allocation-free entry point, oxq_w4a16_matmul_static, through the C ABI.

It is a variant of oxq_w4a16_matmul whose split-K partial sums live in the library's static device
array.  The test holds it to the existing entry point's output, bit for bit (same kernels, same
slice order), on two calls in a row - the second on a smaller input, so that anything the first call
left in the array would show - and to the oracle within the path's tolerance.  The size limit and the
plan-only route are checked too.
"""
import sys

import numpy as np
import pytest
import torch

import oracle
from oxydllm_amd import _lib, synth
from tests.helpers import TORCH_DT, assert_close, bits_of, fake, round_x, to_dev, tune

pytestmark = pytest.mark.gpu


def say(msg):
    print(f"[case] {msg}", flush=True)
    sys.stdout.flush()


def _case(ops, dt, m, K, N, g, seed):
    qw, qz, sc = synth.awq_checkpoint(K, N, g, 4, seed=seed)
    x = np.random.default_rng(seed + 1).standard_normal((m, K)).astype(np.float32)
    tdt = TORCH_DT[dt]
    d = (to_dev(qw), to_dev(qz), to_dev(sc, tdt))
    xd = to_dev(x, tdt)
    w = oracle.dequantize_awq(qw, qz, oracle.round_through(sc, dt))
    ref = oracle.matmul_nt_f32(round_x(x, dt), w)
    return d, xd, ref


@pytest.mark.parametrize("dtn", ["f16", "bf16"])
def test_static_scratch_matches_workspace_entry_point_two_calls(dtn):
    from oxydllm_amd import ops
    dt = {"f16": oracle.F16, "bf16": oracle.BF16}[dtn]
    ctx = ops.default_context()
    # first call: 8 K slices over 14336 columns; second call: a smaller problem right after it
    for (m, K, N, g, seed) in [(1, 4096, 14336, 128, 101), (1, 1024, 2048, 128, 202),
                               (5, 2048, 4096, 128, 303), (2, 512, 256, 64, 404)]:
        say(f"static scratch {dtn} m={m} K={K} N={N} g={g}")
        d, xd, ref = _case(ops, dt, m, K, N, g, seed)
        want = ops.w4a16_matmul(xd, *d, ctx=ctx)
        plan_ws = ctx.last_plan()
        out = torch.full((m, N), float("nan"), dtype=TORCH_DT[dt], device="cuda")
        got = ops.w4a16_matmul_static(xd, *d, out=out, ctx=ctx)
        plan_st = ctx.last_plan()
        torch.cuda.synchronize()
        assert plan_st["kernel"] == plan_ws["kernel"] and plan_st["split_k"] == plan_ws["split_k"]
        assert np.array_equal(bits_of(got), bits_of(want)), f"{dtn} m={m} {K}x{N}: bits differ from oxq_w4a16_matmul"
        assert_close(got, ref, f"static {dtn} m={m} {K}x{N}")
        # what the entry point is for: it runs under stream capture (an allocation there fails the capture) and
        # leaves the device's free memory as it found it; every replay gives the eager bits
        free0 = torch.cuda.mem_get_info()[0]
        graph, stream = torch.cuda.CUDAGraph(), torch.cuda.Stream()
        with torch.cuda.graph(graph, stream=stream):
            ops.w4a16_matmul_static(xd, *d, out=out, ctx=ctx)
        for rep in range(3):
            out.fill_(float("nan"))
            torch.cuda.synchronize()
            graph.replay()
            torch.cuda.synchronize()
            assert np.array_equal(bits_of(out), bits_of(want)), f"{dtn} m={m} {K}x{N}: replay {rep} differs"
        # an instantiated graph may take a 2 MiB chunk of device memory for its own bookkeeping; the workspace the
        # other entry point would allocate for these shapes is 64 MiB
        assert torch.cuda.mem_get_info()[0] >= free0 - (8 << 20), "device memory was allocated"
        del graph


def test_static_scratch_rejects_oversize_and_plans_without_gpu_memory(monkeypatch):
    from oxydllm_amd import ops
    lib = _lib.load()
    plan = ops.Context(plan_only=True)
    # The library's own slicing keeps the partial sums of any shape within a few MiB; one K slice per
    # group (a tuning switch) on 8 rows x 131072 columns asks for 32 x 8 x 131072 x 4 bytes = 128 MiB,
    # which the 16 MiB array cannot hold: refused on the host, nothing is enqueued.
    tune("OXQ_GEMV_GPW", 1, ctx=plan)
    K, N, g, m = 4096, 131072, 128, 8
    args = (fake((m, K), _lib.BF16), fake((K, N // 8), _lib.I32), fake((K // g, N // 8), _lib.I32),
            fake((K // g, N), _lib.BF16), fake((m, N), _lib.BF16))
    rc = lib.oxq_w4a16_matmul_static(plan.handle, None, *[_lib.C.byref(a) for a in args])
    msg = lib.oxq_last_error().decode()
    assert rc == -10, (rc, msg)  # OXQ_ERR_WORKSPACE
    assert "static scratch" in msg and "16777216" in msg, msg
    tune("OXQ_GEMV_GPW", None, ctx=plan)
    # a plan-only ctx answers without a device
    small = (fake((1, 4096), _lib.F16, device=0), fake((4096, 512), _lib.I32, device=0), fake((32, 512), _lib.I32, device=0),
             fake((32, 4096), _lib.F16, device=0), fake((1, 4096), _lib.F16, device=0))
    rc = lib.oxq_w4a16_matmul_static(plan.handle, None, *[_lib.C.byref(a) for a in small])
    assert rc == 0, lib.oxq_last_error().decode()
    assert plan.last_plan()["launches"] >= 1
