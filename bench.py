#!/usr/bin/env python3
"""Benchmark of the quantized-weight matmul path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--all]

Workload (BASELINE.json configs[1]): AWQ W4A16, K=4096, N=14336, g=128, f16
activations/scales, at M = 1 (GEMV), 16 and 64 (MFMA tile GEMM).  A "step" is
one call of the hot path at M=1 on synthetic inputs already resident in HBM;
consecutive steps rotate over enough weight copies (> 256 MB) that no step finds
its weights in L2 or the memory-side cache.  The K timed steps are replayed from
one HIP graph so that host launch overhead is not what is measured.

Prints ONE JSON line: `value` is the M=1 throughput in GB/s of algorithmic
bytes (packed weights + zeros + scales + x + y per call); the M=16 / M=64
results, in GB/s and TFLOP/s, ride along in `cases`.  `roofline` describes the
dominant kernel (the M=1 GEMV, HBM-bound); `cpu_baseline` times the CPU oracle's
restatement of the reference's CPU path (dequantize at load, then a dense f32
x.W^T per call, linear.rs:40-79, 597-600) on this machine's cores.
`roofline.bare_read_us` / `bare_read_nt_us` / `bare_read_best_us` are plain reads of the same
packed weights with no arithmetic (in passes, plain / nontemporal; everything requested first),
`roofline.empty_launch_us` an empty kernel of the same launch shape.
`other_configs` holds one compact row per case of BASELINE configs 0, 2, 3 and 4,
each with its own roofline fraction and a CPU baseline per configuration.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0       # MI355X HBM3E
MFMA_F16_PEAK_TFLOPS = 2500.0
K, N, G = 4096, 14336, 128
SAMPLES = 11                # timed replays per case; the median is reported
MIN_TIMED_STEPS = 200       # launches inside one event pair (short runs are timed as one longer graph)
SPINUP_MS = 30.0            # untimed replays ahead of the samples of every case


def algo_bytes(M: int, k: int = K, n: int = N, g: int = G, bits: int = 4) -> int:
    """Algorithmic bytes per call: packed weights + zeros + scales + x + y (16-bit)."""
    w = k * n * bits // 8
    z = (k // g) * n * bits // 8
    s = (k // g) * n * 2
    return w + z + s + M * k * 2 + M * n * 2


def time_graph(fn_of_step, steps: int, warmup: int, stream):
    """Capture `steps` consecutive calls into one HIP graph, replay it SAMPLES times, each
    replay timed with HIP events recorded on the stream the kernels run on.  Returns the
    medians (wall_ms, event_ms) for `steps` calls."""
    import torch
    for i in range(warmup):
        fn_of_step(i)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=stream):
        for i in range(steps):
            fn_of_step(i)
    torch.cuda.synchronize()
    graph.replay()          # untimed replay (first replay uploads the graph)
    torch.cuda.synchronize()
    # Untimed: keep the GPU busy for SPINUP_MS before sampling.  A replay of 20 steps lasts 0.2 ms; from
    # idle, that is over before the clocks have come up, and a short run would time the ramp.
    t_spin = time.perf_counter()
    while (time.perf_counter() - t_spin) * 1e3 < SPINUP_MS:
        for _ in range(8):
            graph.replay()
        torch.cuda.synchronize()
    cur = torch.cuda.current_stream()
    reps = max(1, -(-MIN_TIMED_STEPS // steps))
    # Short graphs: the event pair times one graph of reps * steps launches (the same calls, the step index
    # running on), so that the gap between two graph launches (several microseconds: 0.2 - 0.4 us a step at 20
    # steps) is not booked as kernel time.  The host-clock figure stays one replay of `steps` launches.
    timed = graph
    if reps > 1:
        timed = torch.cuda.CUDAGraph()
        with torch.cuda.graph(timed, stream=stream):
            for i in range(reps * steps):
                fn_of_step(i)
        torch.cuda.synchronize()
        timed.replay()
        torch.cuda.synchronize()
    walls, evs = [], []
    for _ in range(SAMPLES):   # median of SAMPLES replays of the same `steps` launches
        ev0 = torch.cuda.Event(enable_timing=True)
        ev1 = torch.cuda.Event(enable_timing=True)
        # (a) the host's clock around one replay, synchronized on both sides: `steps` launches plus
        # the host's graph-launch latency (about 12 us, a large share of a 20-step replay)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        graph.replay()
        torch.cuda.synchronize()
        walls.append((time.perf_counter() - t0) * 1e3)
        # (b) HIP events on the launch stream, with untimed replays directly ahead: the timed replay
        # is enqueued while the GPU is still busy, so the first kernel starts when the event before it
        # completes and the launch latency is not counted as kernel time.  The event pair itself costs a
        # few microseconds, which 20 steps would carry as +0.4 us per step: the pair spans at least
        # MIN_TIMED_STEPS launches (`reps` times `steps`) and its time is divided by `reps`, i.e. each sample
        # is the mean time of `steps` launches.
        graph.replay()
        graph.replay()
        ev0.record(cur)
        timed.replay()
        ev1.record(cur)
        torch.cuda.synchronize()
        evs.append(ev0.elapsed_time(ev1) / reps)
    return float(np.median(walls)), float(np.median(evs))


def cpu_baseline(qw, qz, sc, x_f32):
    """Reference CPU path restated by the oracle: dequantize once (load time), then per
    call a dense f32 y = x.W^T over the [N,K] f32 weight.  Bounded sample."""
    import oracle
    cores = int(os.environ.get("OMP_NUM_THREADS", os.cpu_count() or 1))
    t0 = time.perf_counter()
    w = oracle.dequantize_awq(qw, qz, oracle.round_through(sc, oracle.F16))
    t_deq = time.perf_counter() - t0
    xr = oracle.round_through(x_f32, oracle.F16)
    oracle.matmul_nt_f32(xr, w)  # warm
    calls, t_total = 0, 0.0
    while t_total < 4.0 and calls < 200:
        t0 = time.perf_counter()
        oracle.matmul_nt_f32(xr, w)
        t_total += time.perf_counter() - t0
        calls += 1
    per_call = t_total / calls
    return {
        "value": round(algo_bytes(1) / per_call / 1e9, 3),
        "unit": "GB/s",
        "cores": cores,
        "kind": "port",
        "sample": (f"{calls} calls of the dense f32 GEMV over the dequantized {N}x{K} weight "
                   f"({per_call * 1e3:.2f} ms/call, OpenMP over rows); one-time dequant-at-load "
                   f"{t_deq:.2f} s not included; GB/s counts the same packed-weight bytes as `value`"),
        "ms_per_call": round(per_call * 1e3, 3),
        "dequant_at_load_s": round(t_deq, 3),
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=400)
    ap.add_argument("--warmup", type=int, default=40)
    ap.add_argument("--copies", type=int, default=16, help="weight copies rotated to defeat caches")
    ap.add_argument("--no-cpu", action="store_true", help="skip the cpu_baseline leg")
    ap.add_argument("--skip-ops", action="store_true", help="skip the checkpoint-layout op cases")
    ap.add_argument("--no-hot", action="store_true",
                    help="skip the same-weights-every-call (cache-resident) timings, so that a profiler "
                         "run sees only the launches `value` is computed from plus the warm-up")
    ap.add_argument("--no-others", action="store_true",
                    help="skip the compact rows for BASELINE configs 0, 2, 3 and 4 (`other_configs`)")
    ap.add_argument("--no-bare-read", action="store_true",
                    help="skip the plain-read calibration (`roofline.bare_read_us`)")
    ap.add_argument("--all", action="store_true",
                    help="also the long list: prefill sizes, fused FFN entry, F8, all ten GGUF formats (`extra_configs`)")
    ap.add_argument("--prefill-only", action="store_true",
                    help="only the resident layers at prefill sizes (the first part of --all), as one JSON line "
                         "{\"prefill\": [...]}: a short run for a profiler")
    ap.add_argument("--moe-only", action="store_true",
                    help="only config 4's MXFP4 mixture-of-experts rows of --all (decode step, prefill layer steps), as one "
                         "JSON line {\"moe\": [...]}: a short run for a profiler")
    ap.add_argument("--calib-copy", action="store_true",
                    help="first run a plain 256 MiB device copy 4 times: a kernel of known HBM "
                         "traffic to scale rocprofv3 FETCH_SIZE / WRITE_SIZE readings with")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: this build has no multi-GPU path (--gpus must be 1)")

    import torch
    if not torch.cuda.is_available():
        sys.exit("bench.py needs a GPU")
    from oxydllm_amd import _lib
    if not os.path.exists(_lib.LIB_PATH):  # load what is built; build only if nothing is
        from oxydllm_amd import build
        build.build(force=False)
    from oxydllm_amd import ops, synth

    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    ctx = ops.default_context()
    stream = torch.cuda.Stream()

    if args.calib_copy:
        src = torch.empty(256 << 20, dtype=torch.uint8, device=dev).fill_(1)
        dst = torch.empty_like(src)
        for _ in range(4):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    if args.moe_only:
        import bench_extra
        print(json.dumps({"moe": bench_extra.run_moe(ops, ctx, stream, args.steps, args.warmup, time_graph)}), flush=True)
        return
    if args.prefill_only:
        import bench_extra
        rows = bench_extra.run_prefill(ops, ctx, stream, args.steps, args.warmup, time_graph)
        for r in rows:
            print(f"[bench] {r['case']}: {r['us_per_call']} us, {r['TFLOP_per_s']} TFLOP/s "
                  f"({r['mfma_frac']:.3f} of the dense MFMA peak), {r['kernel']}", file=sys.stderr, flush=True)
        print(json.dumps({"prefill": rows}), flush=True)
        return

    qw, qz, sc = synth.awq_checkpoint(K, N, G, 4, seed=0x0A0D11E6)
    copies = max(1, args.copies)
    qw_d = [torch.from_numpy(qw).to(dev) for _ in range(copies)]
    qz_d = [torch.from_numpy(qz).to(dev) for _ in range(copies)]
    sc_d = [torch.from_numpy(sc).to(dev, torch.float16) for _ in range(copies)]
    rng = np.random.default_rng(1)
    x_host = {m: rng.standard_normal((m, K)).astype(np.float32) for m in (1, 16, 64)}
    x_d = {m: torch.from_numpy(v).to(dev, torch.float16) for m, v in x_host.items()}
    y_d = {m: torch.empty((m, N), dtype=torch.float16, device=dev) for m in (1, 16, 64)}

    # The hot path as the reference's model code enters it: PackedQuantLinear::forward on a
    # resident layer (linear.rs:482-533).  The layer repacks its weights tile-major at load.
    layers = [ops.PackedQuantLinear(4, ops.PACK_OUT, qw_d[c], qz_d[c], sc_d[c], None, torch.float16, ctx=ctx)
              for c in range(copies)]

    def run_case(m, fn_cold, fn_hot, k=K, n=N):
        fn_cold(0)
        plan = ctx.last_plan()
        wall_ms, ev_ms = time_graph(fn_cold, args.steps, args.warmup, stream)
        # same weights every call: the 30 MB stay in the 256 MB memory-side cache
        hot_ms = float("nan") if args.no_hot else time_graph(fn_hot, args.steps, args.warmup, stream)[1]
        us = ev_ms * 1e3 / args.steps
        b = algo_bytes(m, k, n)
        flops = 2.0 * m * k * n
        return {
            "M": m, "K": k, "N": n, "kernel": plan["kernel"], "grid": list(plan["grid"]), "split_k": plan["split_k"],
            "launches": plan["launches"],
            "us_per_call": round(us, 3), "us_per_call_wall": round(wall_ms * 1e3 / args.steps, 3),
            "us_per_call_hot_cache": None if args.no_hot else round(hot_ms * 1e3 / args.steps, 3),
            "algorithmic_bytes": b, "GB_per_s": round(b / us / 1e3, 1),
            "hbm_frac": round(b / us / 1e3 / HBM_PEAK_GBS, 4),
            "TFLOP_per_s": round(flops / us / 1e6, 2),
            "mfma_frac": round(flops / us / 1e6 / MFMA_F16_PEAK_TFLOPS, 4),
        }

    cases, op_cases = [], []
    for m in (1, 16, 64):
        cases.append(run_case(m, lambda i, m=m: layers[i % copies].forward(x_d[m], out=y_d[m]),
                              lambda i, m=m: layers[0].forward(x_d[m], out=y_d[m])))
        print(f"[bench] layer M={m}: {cases[-1]}", file=sys.stderr, flush=True)
    # The stateless ops on the checkpoint layout (metal_ops.rs w4a16_matmul / mpp_quant_matmul).
    for m in (() if args.skip_ops else (1, 16, 64)):
        if m <= 8:
            def op(c, m=m):
                ops.w4a16_matmul(x_d[m], qw_d[c], qz_d[c], sc_d[c], out=y_d[m], ctx=ctx)
        else:
            def op(c, m=m):
                ops.mpp_quant_matmul(x_d[m], qw_d[c], qz_d[c], sc_d[c], 4, ops.PACK_OUT, out=y_d[m], ctx=ctx)
        op_cases.append(run_case(m, lambda i, op=op: op(i % copies), lambda i, op=op: op(0)))
        print(f"[bench] op M={m}: {op_cases[-1]}", file=sys.stderr, flush=True)
    # The same op calls with the ctx's opt-in weight cache on: the first call on a weight builds the
    # resident layers' tile-major copy (outside the timed region and outside any capture), later calls
    # find the weight by its address and run the resident-layer kernel.
    cached_op_cases = []
    if not args.skip_ops:
        ctx.set_weight_cache(2 << 30)
        for m in (1, 16, 64):
            if m <= 8:
                def op(c, m=m):
                    ops.w4a16_matmul(x_d[m], qw_d[c], qz_d[c], sc_d[c], out=y_d[m], ctx=ctx)
            else:
                def op(c, m=m):
                    ops.mpp_quant_matmul(x_d[m], qw_d[c], qz_d[c], sc_d[c], 4, ops.PACK_OUT, out=y_d[m], ctx=ctx)
            for c in range(copies):
                op(c)
            torch.cuda.synchronize()
            cached_op_cases.append(run_case(m, lambda i, op=op: op(i % copies), lambda i, op=op: op(0)))
            print(f"[bench] op with weight cache M={m}: {cached_op_cases[-1]}", file=sys.stderr, flush=True)
        ctx.set_weight_cache(0)
        ctx.forget_weights(None)

    # The same weight shape the other way round (the MLP's down projection, BASELINE configs[1]
    # names both orientations): 64 column strips, so K is also cut into slices.
    down_cases = []
    if not args.skip_ops:
        kd, nd = N, K
        dq = synth.awq_checkpoint(kd, nd, G, 4, seed=0x0A0D11E6 + 1)
        dlayers = [ops.PackedQuantLinear(4, ops.PACK_OUT, torch.from_numpy(dq[0]).to(dev),
                                         torch.from_numpy(dq[1]).to(dev),
                                         torch.from_numpy(dq[2]).to(dev, torch.float16), None, torch.float16,
                                         ctx=ctx) for _ in range(copies)]
        for m in (1, 16, 64):
            xd = torch.randn((m, kd), device=dev, dtype=torch.float16)
            yd = torch.empty((m, nd), device=dev, dtype=torch.float16)
            down_cases.append(run_case(m, lambda i, xd=xd, yd=yd: dlayers[i % copies].forward(xd, out=yd),
                                       lambda i, xd=xd, yd=yd: dlayers[0].forward(xd, out=yd), kd, nd))
            print(f"[bench] down-projection layer M={m}: {down_cases[-1]}", file=sys.stderr, flush=True)
        del dlayers

    # What the machine does with the same bytes and launch shape when there is no arithmetic (include/oxq_bench.h):
    #  * empty_launch_us: an empty kernel of the M = 1 kernel's launch shape - the period of back-to-back launches;
    #  * bare_read_us / bare_read_nt_us: 224 workgroups of 512 threads read the packed weights in passes, eight loads
    #    in flight a lane (plain / nontemporal);
    #  * bare_read_best_us: the same bytes with every lane's whole share requested before the first wait, as the
    #    M <= 16 kernels request their weights - the best of 8 and 16 waves a workgroup, nontemporal.
    bare, streams = {}, None
    if not args.no_bare_read:
        nbytes_w = K * N // 2
        pool = torch.empty(copies * nbytes_w, dtype=torch.uint8, device=dev).random_(0, 256)
        sums = torch.empty(256, dtype=torch.int32, device=dev)
        m1 = cases[0]
        _, ev = time_graph(lambda i: ops.empty_launch(m1["grid"][0], 1024 if "front" in m1["kernel"] else 512, 65536, ctx=ctx),
                           args.steps, args.warmup, stream)
        bare["empty_launch_us"] = round(ev * 1e3 / args.steps, 3)
        # the same launch shape with one grid barrier in it (bounded spin): what a persistent kernel would pay per
        # layer boundary instead of a launch
        bar_state = torch.zeros(2, dtype=torch.int32, device=dev)
        _, ev = time_graph(lambda i: ops.grid_barrier(m1["grid"][0], 1024 if "front" in m1["kernel"] else 512, bar_state,
                                                      ctx=ctx), args.steps, args.warmup, stream)
        bare["grid_barrier_launch_us"] = round(ev * 1e3 / args.steps, 3) if int(bar_state[1].item()) == 0 else None
        for nt in (0, 1):
            def rd(i, nt=nt):
                c = i % copies
                ops.calib_read(pool[c * nbytes_w:(c + 1) * nbytes_w], N // 64, bool(nt), sums, ctx=ctx)
            _, ev = time_graph(rd, args.steps, args.warmup, stream)
            bare["bare_read_nt_us" if nt else "bare_read_us"] = round(ev * 1e3 / args.steps, 3)
        best = {}
        for waves in (8, 16):
            def rd(i, waves=waves):
                c = i % copies
                ops.read_upfront(pool[c * nbytes_w:(c + 1) * nbytes_w], N // 64, waves, True, sums, ctx=ctx)
            _, ev = time_graph(rd, args.steps, args.warmup, stream)
            best[waves] = round(ev * 1e3 / args.steps, 3)
        bare["bare_read_best_us"] = min(best.values())
        bare["bare_read_best_waves"] = min(best, key=best.get)
        bare["bare_read_upfront_us_by_waves"] = best
        # the M = 64 kernel's two request streams, alone and together: the strip's weights (cold) and the 64 rows of x
        # that every workgroup reads whole (512 KB, L2 hits), the latter straight into LDS as that kernel does it
        xs = torch.empty(64 * K * 2, dtype=torch.uint8, device=dev).random_(0, 256)
        streams = {}
        for which, key in ((1, "weights_us"), (2, "x_64_rows_us"), (3, "both_us")):
            def rd(i, which=which):
                c = i % copies
                ops.two_streams(pool[c * nbytes_w:(c + 1) * nbytes_w], xs, N // 64, which, sums, ctx=ctx)
            _, ev = time_graph(rd, args.steps, args.warmup, stream)
            streams[key] = round(ev * 1e3 / args.steps, 3)
        bare["bare_read_bytes"] = nbytes_w
        bare["bare_read_workgroups"] = N // 64
        print(f"[bench] plain read of {nbytes_w} B by {N // 64} workgroups: {bare}", file=sys.stderr, flush=True)
        print(f"[bench] two request streams a compute unit (M = 64): {streams}", file=sys.stderr, flush=True)
        del pool, xs

    c1 = cases[0]
    # HBM bytes per launch of the M=1 kernel, measured offline with rocprofv3 --pmc (FETCH_SIZE, WRITE_SIZE) and
    # recorded in the committed profile summary - which names the kernel it measured: a summary of another
    # kernel than the one this run timed gives no traffic figure.
    traffic, traffic_kernel = None, None
    tpath = os.path.join(ROOT, "profiles", "pk4_mfma_m1_K4096_N14336_pmc.txt")
    if os.path.exists(tpath):
        for line in open(tpath):
            if line.startswith("hbm_bytes_per_launch:"):
                try:
                    traffic = int(float(line.split(":", 1)[1].split()[0]))
                except ValueError:
                    traffic = None
            elif line.startswith("kernel_of_traffic:"):
                traffic_kernel = line.split(":", 1)[1].strip()
    if traffic_kernel != c1["kernel"]:
        traffic = None
    result = {
        "metric": "int4 GEMV/GEMM HBM GB/s (% peak) + TFLOPS at M=1/16/64, K=4096 N=14336",
        "value": c1["GB_per_s"],
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(c1["us_per_call_wall"] / 1e3, 6),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f16",
        "data": "synthetic",
        "config": {"workload": "AWQ W4A16 M=1, K=4096 N=14336 g=128, f16 in/out, f32 accumulate "
                               "(BASELINE configs[1]) through PackedQuantLinear.forward on a resident layer; "
                               "M=16/64 in `cases`; the stateless checkpoint-layout ops in "
                               "`cases_checkpoint_layout_ops`",
                   "weight_copies_rotated": copies, "timing": f"HIP graph of max(1, ceil({MIN_TIMED_STEPS}/steps)) x `steps` launches; {SAMPLES} samples, each one "
                             f"HIP-event pair around one replay, divided by that factor; median"},
        "roofline": {"bound": "hbm", "achieved": c1["GB_per_s"], "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(c1["GB_per_s"] / HBM_PEAK_GBS, 4), "traffic": traffic,
                     "kernel": c1["kernel"], "algorithmic_bytes_per_launch": c1["algorithmic_bytes"],
                     "us_per_launch": c1["us_per_call"], **bare},
        "roofline_m64": {"bound": "mfma", "achieved": cases[2]["TFLOP_per_s"],
                         "peak": MFMA_F16_PEAK_TFLOPS, "unit": "TFLOP/s",
                         "frac": cases[2]["mfma_frac"], "traffic": None,
                         "kernel": cases[2]["kernel"], "hbm_frac": cases[2]["hbm_frac"],
                         "us_per_launch": cases[2]["us_per_call"], "request_streams_us": streams},
        "cases": cases,
        "cases_down_projection_K14336_N4096": down_cases,
        "cases_checkpoint_layout_ops": op_cases,
        "cases_checkpoint_layout_ops_weight_cache": cached_op_cases,
    }
    del layers, qw_d, qz_d, sc_d
    torch.cuda.empty_cache()
    if not args.no_others:
        import bench_configs
        result["other_configs"] = bench_configs.run(ops, ctx, stream, args.steps, args.warmup, time_graph,
                                                    with_cpu=not args.no_cpu)
        for r in result["other_configs"]:
            print(f"[bench] {r['config']}: {r['case']}: {r['us_per_call']} us, {r['GB_per_s']} GB/s "
                  f"({r['roofline']['frac']:.3f} of HBM peak), {r['kernel']}", file=sys.stderr, flush=True)
    if args.all:
        import bench_extra
        result["extra_configs"] = bench_extra.run(ops, ctx, stream, args.steps, args.warmup, time_graph)
    if not args.no_cpu:
        result["cpu_baseline"] = cpu_baseline(qw, qz, sc, x_host[1])
    else:
        result["cpu_baseline"] = None
    print(json.dumps(result), flush=True)


if __name__ == "__main__":
    main()
