"""The bench-only entry points of include/oxq_bench.h: they are measurement aids with no counterpart in the
reference, but bench.py's calibration fields rest on them, so what they read and that they end is checked."""
import sys

import numpy as np
import pytest
import torch

from oxydllm_amd import _lib
from tests.helpers import fake

pytestmark = pytest.mark.gpu


def say(msg):
    print(f"[case] {msg}", flush=True)
    sys.stdout.flush()


def _xor_words(a: np.ndarray) -> int:
    return int(np.bitwise_xor.reduce(a.view(np.uint32)))


@pytest.mark.parametrize("nontemporal", [False, True])
def test_bare_reads_read_every_byte(nontemporal):
    """The checksum word of a workgroup is the xor of all 32-bit words of its span, for the read in passes and
    for the read that requests everything first (8 and 16 waves)."""
    from oxydllm_amd import ops
    wgs, span = 28, 128 * 1024
    host = np.random.default_rng(3).integers(0, 256, wgs * span, dtype=np.uint8)
    src = torch.from_numpy(host).cuda()
    want = np.array([_xor_words(host[i * span:(i + 1) * span]) for i in range(wgs)], dtype=np.uint32)
    sums = torch.zeros(wgs, dtype=torch.int32, device="cuda")
    say(f"calib_read nontemporal={nontemporal}")
    ops.calib_read(src, wgs, nontemporal, sums)
    torch.cuda.synchronize()
    np.testing.assert_array_equal(sums.cpu().numpy().view(np.uint32), want)
    for waves in (8, 16):
        say(f"read_upfront waves={waves} nontemporal={nontemporal}")
        sums.zero_()
        ops.read_upfront(src, wgs, waves, nontemporal, sums)
        torch.cuda.synchronize()
        np.testing.assert_array_equal(sums.cpu().numpy().view(np.uint32), want)


def test_empty_launch_and_two_streams_run():
    from oxydllm_amd import ops
    say("empty launch 224 x 1024, 64 KiB of LDS")
    ops.empty_launch(224, 1024, 65536)
    w = torch.randint(0, 256, (8 * 128 * 1024,), dtype=torch.uint8, device="cuda")
    x = torch.randint(0, 256, (64 * 1024,), dtype=torch.uint8, device="cuda")
    sums = torch.zeros(8, dtype=torch.int32, device="cuda")
    for which in (1, 2, 3):
        say(f"two streams which={which}")
        ops.two_streams(w, x, 8, which, sums)
    torch.cuda.synchronize()


def test_grid_barrier_completes_and_gives_up_when_told_to():
    """Every workgroup takes one ticket per launch; with the default limit nobody gives up; with a limit of one
    poll (forced from the host) the launch still ends, whatever the error word then says."""
    from oxydllm_amd import ops
    state = torch.zeros(2, dtype=torch.int32, device="cuda")
    for threads in (512, 1024):
        for rep in range(3):
            say(f"grid barrier 224 x {threads}, launch {rep}")
            ops.grid_barrier(224, threads, state)
    torch.cuda.synchronize()
    counter, err = (int(v) for v in state.cpu().numpy())
    assert counter == 6 * 224 and err == 0, (counter, err)
    say("grid barrier with a spin limit of one poll")
    ops.grid_barrier(224, 1024, state, spin_limit=1)
    torch.cuda.synchronize()
    counter, err = (int(v) for v in state.cpu().numpy())
    assert counter == 7 * 224 and err in (0, 1), (counter, err)


def test_grid_barrier_refuses_grids_that_are_not_resident_at_once():
    from oxydllm_amd import ops
    lib = _lib.load()
    ctx = ops.default_context()
    state = torch.zeros(2, dtype=torch.int32, device="cuda")
    for wgs, threads in ((100000, 1024), (257, 1024), (513, 512)):
        rc = lib.oxq_bench_grid_barrier(ctx.handle, None, wgs, threads, _lib.C.byref(ops.desc_struct(state)), 1 << 10)
        assert rc == -1, (wgs, threads, rc, lib.oxq_last_error().decode())  # OXQ_ERR_ARG
    torch.cuda.synchronize()
    assert int(state[0].item()) == 0
