"""One compact row per remaining benchmark configuration, for the default ``bench.py`` run.

Config 0: AWQ W4A16 GEMV, M=1, K=N=4096, g=128 (the reference's CPU-runnable case).
Config 2: GPTQ 4- and 8-bit, K=5120, N=13824, g=128, M in {1, 8}.
Config 3: GGUF Q4_0 / Q8_0 / Q4_K / Q6_K GEMV, M=1, K=N=4096, f32 activations.
Config 4: MXFP4 MoE expert GEMV, 32 experts, top-4, 8 decode tokens, hidden 2880.

Every row carries the kernel's time per call from a HIP-graph replay on cold weights (copies
rotated past the 256 MB memory-side cache), GB/s of algorithmic bytes, its fraction of the 8 TB/s
HBM roofline, and - once per configuration - a CPU baseline: the oracle's restatement of what the
reference does on the CPU for that layer type, timed on this machine's cores on a bounded sample.
"""
from __future__ import annotations

import os
import time

import numpy as np
import torch

from oxydllm_amd import synth

HBM_PEAK_GBS = 8000.0


def _copies_for(nbytes: int, want_total: int = 400 << 20, cap: int = 24) -> int:
    return int(max(2, min(cap, -(-want_total // max(1, nbytes)))))


MFMA_PEAK_TFLOPS = 2500.0  # dense f16 / bf16


def _row(config, case, fn_of_step, steps, warmup, stream, time_graph, nbytes, flops, ctx, mfma=False):
    """mfma: price the row against the dense 16-bit MFMA peak (tile GEMMs at 64 rows) instead of HBM."""
    fn_of_step(0)
    plan = ctx.last_plan()
    _, ev_ms = time_graph(fn_of_step, steps, warmup, stream)
    us = ev_ms * 1e3 / steps
    gbs = nbytes / us / 1e3
    tf = flops / us / 1e6
    roof = ({"bound": "mfma", "achieved": round(tf, 2), "peak": MFMA_PEAK_TFLOPS, "unit": "TFLOP/s",
             "frac": round(tf / MFMA_PEAK_TFLOPS, 4)} if mfma else
            {"bound": "hbm", "achieved": round(gbs, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
             "frac": round(gbs / HBM_PEAK_GBS, 4)})
    return {"config": config, "case": case, "kernel": plan["kernel"], "launches": plan["launches"],
            "us_per_call": round(us, 3), "algorithmic_bytes": int(nbytes), "GB_per_s": round(gbs, 1),
            "TFLOP_per_s": round(tf, 3), "roofline": roof}


def _cached_row(config, case, call, nc, steps, warmup, stream, time_graph, nbytes, flops, ctx, mfma=False):
    """`call(c)` on weight copy c with the ctx's opt-in weight cache on: every copy is seen once
    outside the timed region (that call builds its tile-major copy), the timed calls find it."""
    ctx.set_weight_cache(2 << 30)
    try:
        for c in range(nc):
            call(c)
        torch.cuda.synchronize()
        return _row(config, case, lambda i: call(i % nc), steps, warmup, stream, time_graph, nbytes, flops, ctx, mfma)
    finally:
        ctx.set_weight_cache(0)


def _time_cpu(fn, budget_s: float, max_calls: int):
    fn()  # warm
    calls, total = 0, 0.0
    while total < budget_s and calls < max_calls:
        t0 = time.perf_counter()
        fn()
        total += time.perf_counter() - t0
        calls += 1
    return total / calls, calls


def _cores() -> int:
    return int(os.environ.get("OMP_NUM_THREADS", os.cpu_count() or 1))


def _cpu_dense(w_nk, x_f32, nbytes, what, budget_s=2.0):
    """Reference CPU path of an AWQ / GPTQ layer (linear.rs:40-79, 582-601): the weight was
    dequantized at load; a call is a dense f32 x.W^T."""
    import oracle
    per, calls = _time_cpu(lambda: oracle.matmul_nt_f32(x_f32, w_nk), budget_s, 200)
    return {"value": round(nbytes / per / 1e9, 3), "unit": "GB/s", "cores": _cores(), "kind": "port",
            "ms_per_call": round(per * 1e3, 3),
            "sample": f"{calls} calls of the dense f32 GEMV over the weight dequantized at load ({what}); "
                      "GB/s counts the packed-weight bytes the GPU rows count"}


def run(ops, ctx, stream, steps, warmup, time_graph, with_cpu=True):
    import oracle
    dev = torch.device("cuda:0")
    rows = []

    # ---- config 0 --------------------------------------------------------------------------------------
    K = N = 4096
    G = 128
    qw, qz, sc = synth.awq_checkpoint(K, N, G, 4, seed=0x0A0D11E5)
    wbytes = qw.nbytes + qz.nbytes + sc.size * 2
    nc = _copies_for(wbytes, cap=48)
    d = [(torch.from_numpy(qw).to(dev), torch.from_numpy(qz).to(dev), torch.from_numpy(sc).to(dev, torch.float16))
         for _ in range(nc)]
    layers = [ops.PackedQuantLinear(4, ops.PACK_OUT, *c, None, torch.float16, ctx=ctx) for c in d]
    xh = np.random.default_rng(10).standard_normal((1, K)).astype(np.float32)
    x = torch.from_numpy(xh).to(dev, torch.float16)
    y = torch.empty((1, N), device=dev, dtype=torch.float16)
    nb = wbytes + K * 2 + N * 2
    r = _row("cfg0", f"awq4 M=1 K={K} N={N} g={G} f16, PackedQuantLinear.forward (resident layer)",
             lambda i: layers[i % nc].forward(x, out=y), steps, warmup, stream, time_graph, nb, 2.0 * K * N, ctx)
    if with_cpu:
        w = oracle.dequantize_awq(qw, qz, oracle.round_through(sc, oracle.F16))
        r["cpu_baseline"] = _cpu_dense(w, oracle.round_through(xh, oracle.F16), nb, f"{N}x{K} f32")
        del w
    rows.append(r)
    rows.append(_row("cfg0", f"awq4 M=1 K={K} N={N} g={G} f16, w4a16_matmul op (checkpoint layout)",
                     lambda i: ops.w4a16_matmul(x, *d[i % nc], out=y, ctx=ctx), steps, warmup, stream, time_graph,
                     nb, 2.0 * K * N, ctx))
    rows.append(_cached_row("cfg0", f"awq4 M=1 K={K} N={N} g={G} f16, w4a16_matmul op with the ctx weight cache on",
                            lambda c: ops.w4a16_matmul(x, *d[c], out=y, ctx=ctx), nc, steps, warmup, stream,
                            time_graph, nb, 2.0 * K * N, ctx))
    del d, layers

    # ---- config 2 --------------------------------------------------------------------------------------
    K, N, G = 5120, 13824, 128
    for bits in (4, 8):
        qw, qz, sc = synth.gptq_checkpoint(K, N, G, bits, seed=0x0A0D11E7)
        wbytes = qw.nbytes + qz.nbytes + sc.size * 2
        nc = _copies_for(wbytes)
        d = [(torch.from_numpy(qw).to(dev), torch.from_numpy(qz).to(dev), torch.from_numpy(sc).to(dev, torch.float16))
             for _ in range(nc)]
        layers = [ops.PackedQuantLinear(bits, ops.PACK_IN, *c, None, torch.float16, ctx=ctx) for c in d]
        first = True
        for m in (1, 8, 64):  # 64 rows: the prefill tile op on the same tensors (mpp_quant_matmul)
            xh = np.random.default_rng(20 + m).standard_normal((m, K)).astype(np.float32)
            x = torch.from_numpy(xh).to(dev, torch.float16)
            y = torch.empty((m, N), device=dev, dtype=torch.float16)
            nb = wbytes + m * K * 2 + m * N * 2
            r = _row("cfg2", f"gptq{bits} M={m} K={K} N={N} g={G} f16, PackedQuantLinear.forward (resident layer)",
                     lambda i, x=x, y=y: layers[i % nc].forward(x, out=y), steps, warmup, stream, time_graph, nb,
                     2.0 * m * K * N, ctx, m >= 64)
            if with_cpu and first and bits == 4:
                w = oracle.dequantize_gptq(qw, qz, oracle.round_through(sc, oracle.F16), bits)
                r["cpu_baseline"] = _cpu_dense(w, oracle.round_through(xh, oracle.F16), nb,
                                               f"{N}x{K} f32; the 8-bit layer runs the same dense matmul")
                del w
            first = False
            rows.append(r)
            if m <= 8:
                opn, op = "gptq_matmul", (lambda t, x=x, y=y, bits=bits: ops.gptq_matmul(x, *t, bits, out=y, ctx=ctx))
            else:
                opn, op = "mpp_quant_matmul", (lambda t, x=x, y=y, bits=bits: ops.mpp_quant_matmul(x, *t, bits, ops.PACK_IN,
                                                                                                 out=y, ctx=ctx))
            rows.append(_row("cfg2", f"gptq{bits} M={m} K={K} N={N} g={G} f16, {opn} op (checkpoint layout)",
                             lambda i, op=op: op(d[i % nc]), steps, warmup, stream, time_graph, nb, 2.0 * m * K * N, ctx,
                             m >= 64))
            rows.append(_cached_row("cfg2", f"gptq{bits} M={m} K={K} N={N} g={G} f16, {opn} op with the ctx "
                                            "weight cache on",
                                    lambda c, op=op: op(d[c]), nc, steps, warmup, stream, time_graph, nb,
                                    2.0 * m * K * N, ctx, m >= 64))
        del d, layers

    # ---- config 3 --------------------------------------------------------------------------------------
    K = N = 4096
    for fmt in (synth.GGUF_Q4_0, synth.GGUF_Q8_0, synth.GGUF_Q4_K, synth.GGUF_Q6_K):
        data = synth.gguf_weight(fmt, N, K, seed=0x0A0D11E8 + fmt)
        nc = _copies_for(data.nbytes, cap=48)
        d = [torch.from_numpy(data).to(dev) for _ in range(nc)]
        xh = np.random.default_rng(30).standard_normal((1, K)).astype(np.float32)
        x = torch.from_numpy(xh).to(dev)
        y = torch.empty((1, N), device=dev, dtype=torch.float32)
        nb = data.nbytes + K * 4 + N * 4
        r = _row("cfg3", f"gguf {synth.GGUF_NAMES[fmt]} M=1 K={K} N={N} f32 activations, gguf_quant_matmul op",
                 lambda i, d=d, nc=nc, fmt=fmt: ops.gguf_quant_matmul(x, d[i % nc], K, N, fmt, out=y, ctx=ctx),
                 steps, warmup, stream, time_graph, nb, 2.0 * K * N, ctx)
        # what reading the same block bytes costs when nothing else is done (64 KiB per workgroup)
        wgs = data.nbytes // 65536
        sums = torch.zeros(wgs, device=dev, dtype=torch.int32)
        _, ev = time_graph(lambda i, d=d, nc=nc: ops.calib_read(d[i % nc].view(torch.uint8).reshape(-1)[:wgs * 65536],
                                                               wgs, True, sums, ctx=ctx), steps, warmup, stream)
        r["bare_read_nt_us"] = round(ev * 1e3 / steps, 3)
        r["bare_read_workgroups"] = wgs
        if with_cpu:
            def cpu_call(fmt=fmt, data=data):
                oracle.matmul_nt_f32(xh, oracle.dequantize_gguf(fmt, data, N, K))
            per, calls = _time_cpu(cpu_call, 1.5, 50)
            r["cpu_baseline"] = {"value": round(nb / per / 1e9, 3), "unit": "GB/s", "cores": _cores(), "kind": "port",
                                 "ms_per_call": round(per * 1e3, 3),
                                 "sample": f"{calls} calls of block dequant + f32 dot per row (restatement; candle's "
                                           "QMatMul, which the reference calls on the CPU, is not available here)"}
        layers = [ops.QLinear(fmt, d[i], K, N, None, torch.float32, ctx=ctx) for i in range(nc)]
        rr = _row("cfg3", f"gguf {synth.GGUF_NAMES[fmt]} M=1 K={K} N={N} f32 activations, QLinear.forward (resident "
                          "strip-major copy of the blocks)",
                  lambda i, layers=layers, nc=nc: layers[i % nc].forward(x, out=y), steps, warmup, stream, time_graph,
                  nb, 2.0 * K * N, ctx)
        rr["bare_read_nt_us"] = r["bare_read_nt_us"]
        rows.append(rr)
        rows.append(r)
        del layers
        # bf16 activations (the reference's GPU contract, linear.rs:250-284): a bf16 layer keeps the matrix-core
        # copy of the four formats; 1, 8 (the decode op's limit) and 16 rows
        layers = [ops.QLinear(fmt, d[i], K, N, None, torch.bfloat16, ctx=ctx) for i in range(nc)]
        for m in (1, 8, 16):
            xb = torch.randn((m, K), device=dev, dtype=torch.bfloat16)
            yb = torch.empty((m, N), device=dev, dtype=torch.bfloat16)
            rb = _row("cfg3", f"gguf {synth.GGUF_NAMES[fmt]} M={m} K={K} N={N} bf16 activations, QLinear.forward (resident "
                              "matrix-core copy of the blocks)",
                      lambda i, layers=layers, nc=nc, xb=xb, yb=yb: layers[i % nc].forward(xb, out=yb), steps, warmup, stream,
                      time_graph, data.nbytes + m * (K + N) * 2, 2.0 * m * K * N, ctx)
            rb["bare_read_nt_us"] = r["bare_read_nt_us"]
            rows.append(rb)
        del layers
        rc = _cached_row("cfg3", f"gguf {synth.GGUF_NAMES[fmt]} M=1 K={K} N={N} f32 activations, gguf_quant_matmul op "
                                 "with the ctx weight cache on",
                         lambda c, d=d, fmt=fmt: ops.gguf_quant_matmul(x, d[c], K, N, fmt, out=y, ctx=ctx),
                         nc, steps, warmup, stream, time_graph, nb, 2.0 * K * N, ctx)
        rc["bare_read_nt_us"] = r["bare_read_nt_us"]
        rows.append(rc)
        ctx.forget_weights(None)
        del d

    # ---- config 4 --------------------------------------------------------------------------------------
    E, top_k, H, I, T = 32, 4, 2880, 2880, 8
    rng = np.random.default_rng(0x0A0D11E9)
    logits = rng.standard_normal((T, E)).astype(np.float32)
    top_idx, top_vals = oracle.moe_route(logits, top_k, True)
    offsets, tokens, _w = oracle.moe_group(top_idx, top_vals, E)
    offsets = np.asarray(offsets, np.int32)
    tokens = np.asarray(tokens, np.int32)
    active = int(np.count_nonzero(np.diff(offsets)))
    n_pairs = T * top_k
    gu_b, gu_s = synth.mxfp4_weight(E * 2 * I, H, seed=1)
    dn_b, dn_s = synth.mxfp4_weight(E * H, I, seed=2)
    gub = torch.from_numpy(gu_b).to(dev), torch.from_numpy(gu_s).to(dev)
    dnb = torch.from_numpy(dn_b).to(dev), torch.from_numpy(dn_s).to(dev)
    gu_bias = torch.randn((E, 2 * I), device=dev, dtype=torch.bfloat16) * 0.1
    dn_bias = torch.randn((E, H), device=dev, dtype=torch.bfloat16) * 0.1
    xh = rng.standard_normal((T, H)).astype(np.float32)
    x = torch.from_numpy(xh).to(dev, torch.bfloat16)
    h = torch.randn((n_pairs, I), device=dev, dtype=torch.bfloat16)
    off_d, tok_d = torch.from_numpy(offsets).to(dev), torch.from_numpy(tokens).to(dev)
    y_gu = torch.empty((n_pairs, 2 * I), device=dev, dtype=torch.bfloat16)
    y_dn = torch.empty((n_pairs, H), device=dev, dtype=torch.bfloat16)
    per_expert = (2 * I * (H // 32) * 17 + 2 * I * 2) + (H * (I // 32) * 17 + H * 2)
    nb = active * per_expert + T * H * 2 + n_pairs * (2 * I + I + H) * 2
    flops = 2.0 * n_pairs * (2 * I * H + H * I)

    # the experts as the model holds them: resident (repacked tile-major at load, moe.rs:366-417)
    gu_res = ops.Mxfp4Experts(gub[0], gub[1], gu_bias, E, H, 2 * I, ctx=ctx)
    dn_res = ops.Mxfp4Experts(dnb[0], dnb[1], dn_bias, E, I, H, ctx=ctx)

    def step(i):
        gu_res.matmul(x, off_d, tok_d, out=y_gu)
        dn_res.matmul(h, off_d, None, out=y_dn)
    r = _row("cfg4", f"mxfp4 expert GEMVs of one MoE decode step: gate_up + down over {active} active experts of {E}, "
                     f"{n_pairs} (token, expert) pairs, bf16, resident experts", step, steps, warmup, stream, time_graph, nb,
             flops, ctx)
    r["launches"] = 2
    r["note"] = ("no copy rotation: the active experts' weights (about 13.2 MB each) exceed the 256 MB "
                 "memory-side cache by themselves")
    if with_cpu:
        # mxfp4.rs:158-168: the CPU path dequantizes the expert's blocks on every call, then a dense matmul
        gu_rows, dn_rows = 2 * I, H
        gub_h = gu_b.reshape(E, -1), gu_s.reshape(E, -1)
        dnb_h = dn_b.reshape(E, -1), dn_s.reshape(E, -1)

        def cpu_step():
            for e in range(E):
                n_e = int(offsets[e + 1] - offsets[e])
                if n_e == 0:
                    continue
                xe = xh[tokens[offsets[e]:offsets[e + 1]]]
                wg = oracle.dequantize_mxfp4_f32(gub_h[0][e], gub_h[1][e], gu_rows, H)
                oracle.matmul_nt_f32(xe, wg)
                wd = oracle.dequantize_mxfp4_f32(dnb_h[0][e], dnb_h[1][e], dn_rows, I)
                oracle.matmul_nt_f32(np.ascontiguousarray(xe[:, :I]), wd)
        per, calls = _time_cpu(cpu_step, 3.0, 20)
        r["cpu_baseline"] = {"value": round(nb / per / 1e9, 3), "unit": "GB/s", "cores": _cores(), "kind": "port",
                             "ms_per_call": round(per * 1e3, 3),
                             "sample": f"{calls} MoE steps: per active expert, dequantize_mxfp4_f32 of gate_up and down "
                                       "followed by a dense f32 matmul over its tokens (Mxfp4Linear's CPU path)"}
    rows.append(r)

    def step_ops(i):
        ops.mxfp4_moe_matmul(x, gub[0], gub[1], gu_bias, off_d, tok_d, H, 2 * I, out=y_gu, ctx=ctx)
        ops.mxfp4_moe_matmul(h, dnb[0], dnb[1], dn_bias, off_d, None, I, H, out=y_dn, ctx=ctx)
    r1 = _row("cfg4", "the same step through the stateless mxfp4_moe_matmul op (checkpoint layout)", step_ops, steps,
              warmup, stream, time_graph, nb, flops, ctx)
    r1["launches"] = 2
    rows.append(r1)
    ctx.set_weight_cache(1 << 30)  # the op remembers the stacked expert tensors by address: the resident experts' copy
    step_ops(0)
    r1c = _row("cfg4", "the same step through the stateless mxfp4_moe_matmul op with the ctx weight cache on", step_ops, steps,
               warmup, stream, time_graph, nb, flops, ctx)
    r1c["launches"] = 2
    rows.append(r1c)
    ctx.set_weight_cache(0)

    logits_d = torch.from_numpy(logits).to(dev)
    out_d = torch.empty((T, H), device=dev, dtype=torch.bfloat16)
    h_d = torch.empty((n_pairs, I), device=dev, dtype=torch.bfloat16)

    def full_step(i):
        idx, vals, off, tok, _, pos = ops.moe_route_group(logits_d, top_k, True, ctx=ctx)
        gu_res.gate_up_swiglu(x, off, tok, 7.0, out=h_d)
        dn_res.matmul(h_d, off, None, out=y_dn)
        ops.moe_combine(y_dn, pos, vals, out=out_d, ctx=ctx)
    r2 = _row("cfg4", "mxfp4 MoE layer step on the device: route + group, gate_up with fused SwiGLU, down, combine",
              full_step, steps, warmup, stream, time_graph, nb, flops, ctx)
    r2["launches"] = 4
    rows.append(r2)
    return rows
