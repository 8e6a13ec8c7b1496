"""Two engine threads on one GPU, each with its own context and stream.

The reference runs one engine-loop thread per model (engine_loop.rs:672-675) and
keeps its pipeline caches behind a mutex (metal_ops.rs:1367-1403).  The library's
contract is the same shape: a context (split-K workspace, last plan, last error)
belongs to one thread, while everything process-wide (the per-kernel shared-memory
limits raised on first use) must tolerate concurrent callers.  Each thread here
builds its own layers and runs them in a loop while the other does the same with
other sizes; every result must equal, bit for bit, what the same layer returned
when it ran alone.
"""
import sys
import threading

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


def _engine(seed, rows, ctx):
    """A down-projection-shaped AWQ layer (K slices + reduce: uses the context's workspace)
    and a GGUF Q4_K layer (staged GEMV: dynamic shared memory), with their inputs."""
    K, N = 8192, 256
    trip = synth.awq_checkpoint(K, N, 128, 4, seed=seed)
    awq = ops.PackedQuantLinear(4, ops.PACK_OUT, to_dev(trip[0]), to_dev(trip[1]),
                                to_dev(trip[2], torch.float16), None, torch.float16, ctx=ctx)
    Kg, Ng = 1024, 512
    gg = ops.QLinear(synth.GGUF_Q4_K, to_dev(synth.gguf_weight(synth.GGUF_Q4_K, Ng, Kg, seed=seed)), Kg, Ng,
                     None, torch.bfloat16, ctx=ctx)
    rng = np.random.default_rng(seed)
    xs = [to_dev(rng.standard_normal((m, K)).astype(np.float32), torch.float16) for m in rows]
    xg = to_dev(rng.standard_normal((1, Kg)).astype(np.float32), torch.bfloat16)
    return awq, gg, xs, xg


def test_two_contexts_two_threads_bitwise():
    say("threads: two contexts, two streams, interleaved row counts")
    # different row-tile counts per thread, in opposite order: the two threads ask for
    # different shared-memory sizes of the same kernels at the same time
    plans = [(11, (1, 64, 16, 40, 3)), (23, (64, 1, 40, 16, 130))]
    engines, alone = [], []
    for seed, rows in plans:
        ctx = ops.Context()
        awq, gg, xs, xg = _engine(seed, rows, ctx)
        want = [bits_of(awq.forward(x)) for x in xs] + [bits_of(gg.forward(xg))]
        engines.append((ctx, awq, gg, xs, xg))
        alone.append(want)
    torch.cuda.synchronize()

    errors = []
    start = threading.Barrier(len(engines))

    def run(i):
        try:
            ctx, awq, gg, xs, xg = engines[i]
            stream = torch.cuda.Stream()
            start.wait()
            with torch.cuda.stream(stream):
                for it in range(40):
                    got = [awq.forward(x) for x in xs] + [gg.forward(xg)]
                    stream.synchronize()
                    for k, (g, w) in enumerate(zip(got, alone[i])):
                        if not np.array_equal(bits_of(g), w):
                            errors.append(f"thread {i} iteration {it} output {k} differs")
                            return
        except Exception as e:  # surfaced below: an exception in a thread would otherwise pass silently
            errors.append(f"thread {i}: {type(e).__name__}: {e}")

    threads = [threading.Thread(target=run, args=(i,)) for i in range(len(engines))]
    for t in threads:
        t.start()
    for t in threads:
        t.join(timeout=100)
    assert not any(t.is_alive() for t in threads), "engine thread did not finish"
    assert not errors, errors
