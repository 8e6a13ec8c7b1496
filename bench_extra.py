"""Timings of the other benchmark configurations (`bench.py --all`; `--prefill-only`: its first part alone).

Resident AWQ layers at prefill sizes (256 - 4096 rows; 4096 x 14336, 14336 x 4096, 4096 x 4096 and
8192 x 28672, f16 and bf16), GGUF layers and a GGUF FFN at prefill sizes;
GPTQ 4/8-bit GEMV (K=5120, N=13824, g=128, M in {1, 8}); GGUF Q4_0 / Q8_0 / Q4_K /
Q6_K ... GEMV (M=1, K=N=4096, f32 activations) and tile matmul (M=64..2048, bf16); MXFP4
gated GGUF FFN at decode (four launches against the fused gate|up layer's two); MXFP4
MoE expert GEMV (32 experts, top-4, 8 tokens, hidden 2880, gate_up N=5760, down K=2880),
the same layer at 512 tokens, and one expert's gate_up at prefill sizes.  Every case rotates
over enough weight copies to exceed the 256 MB memory-side cache and replays a
HIP graph of `steps` launches.  Returns a list of dicts (GB/s of algorithmic
bytes, TFLOP/s, fraction of the 8 TB/s HBM peak).
"""
from __future__ import annotations

import sys

import numpy as np
import torch

from oxydllm_amd import synth

HBM_PEAK_GBS = 8000.0


def _copies_for(nbytes: int, want_total: int = 400 << 20, cap: int = 24) -> int:
    return int(max(2, min(cap, -(-want_total // max(1, nbytes)))))


def _case(name, fn_of_step, steps, warmup, stream, time_graph, nbytes, flops, ctx):
    fn_of_step(0)
    plan = ctx.last_plan()
    _, ev_ms = time_graph(fn_of_step, steps, warmup, stream)
    us = ev_ms * 1e3 / steps
    print(f"[bench] {name}: {us:.3f} us, {plan['kernel']}", file=sys.stderr, flush=True)  # a long run shows it is alive
    return {"case": name, "kernel": plan["kernel"], "launches": plan["launches"],
            "us_per_call": round(us, 3), "algorithmic_bytes": int(nbytes),
            "GB_per_s": round(nbytes / us / 1e3, 1), "hbm_frac": round(nbytes / us / 1e3 / HBM_PEAK_GBS, 4),
            "TFLOP_per_s": round(flops / us / 1e6, 3)}


def run_prefill(ops, ctx, stream, steps, warmup, time_graph):
    """Config 1's layer, its down projection, an attention projection (both stored in 16-column strips) and a
    70B-class layer at prefill sizes (PackedQuantLinear.forward): the rows x eight strips kernels where the
    launcher chooses them, beside the split-K tiles they replace there."""
    dev = torch.device("cuda:0")
    out = []
    steps, warmup = max(4, steps // 8), max(2, warmup // 8)
    for K, N, rows in ((4096, 14336, (128, 256, 512, 1024, 2048, 4096)), (14336, 4096, (512, 1024, 2048, 4096)),
                       (4096, 4096, (512, 1024, 2048, 4096)), (8192, 28672, (512, 4096))):
        qw, qz, sc = synth.awq_checkpoint(K, N, 128, 4, seed=0x0A0D11F3)
        wbytes = qw.nbytes + qz.nbytes + sc.size * 2
        for tdt, tn in ((torch.float16, "f16"), (torch.bfloat16, "bf16")):
            layer = ops.PackedQuantLinear(4, ops.PACK_OUT, torch.from_numpy(qw).to(dev), torch.from_numpy(qz).to(dev),
                                          torch.from_numpy(sc).to(dev, tdt), None, tdt, ctx=ctx)
            for m in rows:
                x = torch.randn((m, K), device=dev, dtype=tdt)
                y = torch.empty((m, N), device=dev, dtype=tdt)

                def step(i, x=x, y=y, layer=layer):
                    layer.forward(x, out=y)
                nb, fl = wbytes + m * K * 2 + m * N * 2, 2.0 * m * K * N
                r = _case(f"awq4 prefill M={m} K={K} N={N} {tn} (PackedQuantLinear)", step, steps, warmup, stream,
                          time_graph, nb, fl, ctx)
                r["mfma_frac"] = round(r["TFLOP_per_s"] / 2500.0, 4)
                out.append(r)
                if r["kernel"].startswith("pk4_gemm"):
                    ctx.set_tuning("OXQ_PK4_GEMM_MIN_M", 0)
                    r0 = _case(f"awq4 prefill M={m} K={K} N={N} {tn} (split-K tiles, OXQ_PK4_GEMM_MIN_M=0)", step,
                               steps, warmup, stream, time_graph, nb, fl, ctx)
                    ctx.set_tuning("OXQ_PK4_GEMM_MIN_M", None)
                    r0["mfma_frac"] = round(r0["TFLOP_per_s"] / 2500.0, 4)
                    out.append(r0)
            del layer

    # 8-bit layers (config 2's GPTQ shape): the same kernel with two loads a step
    K, N = 5120, 13824
    qw, qz, sc = synth.gptq_checkpoint(K, N, 128, 8, seed=0x0A0D11F7)
    wbytes = qw.nbytes + qz.nbytes + sc.size * 2
    for tdt, tn in ((torch.float16, "f16"), (torch.bfloat16, "bf16")):
        layer = ops.PackedQuantLinear(8, ops.PACK_IN, torch.from_numpy(qw).to(dev), torch.from_numpy(qz).to(dev),
                                      torch.from_numpy(sc).to(dev, tdt), None, tdt, ctx=ctx)
        for m in (512, 2048):
            x = torch.randn((m, K), device=dev, dtype=tdt)
            y = torch.empty((m, N), device=dev, dtype=tdt)

            def step8(i, x=x, y=y, layer=layer):
                layer.forward(x, out=y)
            nb, fl = wbytes + m * K * 2 + m * N * 2, 2.0 * m * K * N
            for label, min_m in (("", None), (" (split-K tiles, OXQ_PK4_GEMM_MIN_M=0)", 0)):
                ctx.set_tuning("OXQ_PK4_GEMM_MIN_M", min_m)
                r = _case(f"gptq8 prefill M={m} K={K} N={N} {tn} (PackedQuantLinear){label}", step8, steps, warmup, stream,
                          time_graph, nb, fl, ctx)
                r["mfma_frac"] = round(r["TFLOP_per_s"] / 2500.0, 4)
                out.append(r)
            ctx.set_tuning("OXQ_PK4_GEMM_MIN_M", None)
        del layer

    # the whole gated FFN of config 1's model (hidden 4096, intermediate 14336, bf16): the gate|up projection with
    # the activation in its epilogue, then the down projection (stored in 16-column strips) - two launches
    H, I = 4096, 14336
    gu = synth.awq_checkpoint(H, 2 * I, 128, 4, seed=0x0A0D11F4)
    dn = synth.awq_checkpoint(I, H, 128, 4, seed=0x0A0D11F5)
    wbytes = sum(t[0].nbytes + t[1].nbytes + t[2].size * 2 for t in (gu, dn))
    tdt = torch.bfloat16

    def lin(t, **kw):
        return ops.PackedQuantLinear(4, ops.PACK_OUT, torch.from_numpy(t[0]).to(dev), torch.from_numpy(t[1]).to(dev),
                                     torch.from_numpy(t[2]).to(dev, tdt), None, tdt, ctx=ctx, **kw)
    ffn = ops.FeedForward(ops.GATE_UP_FUSED, lin(gu, gate_up_act=ops.ACT_GATED_SILU), None, lin(dn), I,
                          ops.ACT_GATED_SILU, ctx=ctx)
    for m in (512, 2048, 4096):
        x = torch.randn((m, H), device=dev, dtype=tdt)
        y = torch.empty((m, H), device=dev, dtype=tdt)
        scratch = torch.empty(max(ffn.scratch_elems(m), 1), device=dev, dtype=tdt)

        def fstep(i, x=x, y=y, scratch=scratch):
            ffn.forward(x, out=y, scratch=scratch)
        nb, fl = wbytes + 2 * m * H * 2 + 2 * m * I * 2, 6.0 * m * H * I
        for label, min_m in (("", None), (" (split-K tiles, OXQ_PK4_GEMM_MIN_M=0)", 0)):
            ctx.set_tuning("OXQ_PK4_GEMM_MIN_M", min_m)
            r = _case(f"awq4 gated FFN prefill M={m} H={H} I={I} bf16 (FeedForward, fused gate|up + down){label}",
                      fstep, steps, warmup, stream, time_graph, nb, fl, ctx)
            r["launches"] = 2
            r["mfma_frac"] = round(r["TFLOP_per_s"] / 2500.0, 4)
            out.append(r)
        ctx.set_tuning("OXQ_PK4_GEMM_MIN_M", None)
    del ffn

    # GGUF layers (bf16 QLinear.forward): the prefill kernel on the layer's matrix-core copy where the launcher
    # chooses it, beside the tile matmul on the file layout
    for fmt in (synth.GGUF_Q4_0, synth.GGUF_Q8_0, synth.GGUF_Q4_K, synth.GGUF_Q6_K):
        for K, N, rows in ((4096, 14336, (512, 2048)), (4096, 4096, (2048, 4096))):
            data = synth.gguf_weight(fmt, N, K, seed=0x0A0D11F6 + fmt)
            layer = ops.QLinear(fmt, torch.from_numpy(data).to(dev), K, N, None, torch.bfloat16, ctx=ctx)
            for m in rows:
                x = torch.randn((m, K), device=dev, dtype=torch.bfloat16)
                y = torch.empty((m, N), device=dev, dtype=torch.bfloat16)

                def gstep(i, x=x, y=y, layer=layer):
                    layer.forward(x, out=y)
                nb, fl = data.nbytes + m * K * 2 + m * N * 2, 2.0 * m * K * N
                for label, min_m in (("", None), (" (tile matmul on the file layout, OXQ_GGUF_GEMM_MIN_M=0)", 0)):
                    ctx.set_tuning("OXQ_GGUF_GEMM_MIN_M", min_m)
                    r = _case(f"gguf {synth.GGUF_NAMES[fmt]} prefill M={m} K={K} N={N} bf16 (QLinear){label}", gstep, steps,
                              warmup, stream, time_graph, nb, fl, ctx)
                    r["mfma_frac"] = round(r["TFLOP_per_s"] / 2500.0, 4)
                    out.append(r)
                ctx.set_tuning("OXQ_GGUF_GEMM_MIN_M", None)
            del layer
    # the whole gated FFN as a GGUF file holds it (Q4_K): fused gate|up with the activation in the epilogue + down
    fmt = synth.GGUF_Q4_K
    gd, ud, dd = (torch.from_numpy(synth.gguf_weight(fmt, n, k, seed=sd)).to(dev) for n, k, sd in ((I, H, 1), (I, H, 2), (H, I, 3)))
    ffn = ops.FeedForward(ops.GATE_UP_FUSED, ops.QLinear(fmt, torch.cat([gd.reshape(-1), ud.reshape(-1)]), H, 2 * I, None,
                                                          torch.bfloat16, ctx=ctx, gate_up_act=ops.ACT_GATED_SILU),
                          None, ops.QLinear(fmt, dd, I, H, None, torch.bfloat16, ctx=ctx), I, ctx=ctx)
    for m in (2048,):
        x = torch.randn((m, H), device=dev, dtype=tdt) * 0.1
        y = torch.empty((m, H), device=dev, dtype=tdt)
        scratch = torch.empty(m * 3 * I, device=dev, dtype=tdt)

        def gfstep(i, x=x, y=y, scratch=scratch):
            ffn.forward(x, out=y, scratch=scratch)
        nb, fl = gd.numel() + ud.numel() + dd.numel() + 2 * m * H * 2, 6.0 * m * H * I
        for label, min_m in (("fused gate|up with the activation + down, on the layers' copies", None),
                             ("tile matmul on the file layout, activation kernel, OXQ_GGUF_GEMM_MIN_M=0", 0)):
            ctx.set_tuning("OXQ_GGUF_GEMM_MIN_M", min_m)
            r = _case(f"gguf Q4_K gated FFN prefill M={m} H={H} I={I} bf16 (FeedForward: {label})", gfstep, steps, warmup,
                      stream, time_graph, nb, fl, ctx)
            r["mfma_frac"] = round(r["TFLOP_per_s"] / 2500.0, 4)
            out.append(r)
        ctx.set_tuning("OXQ_GGUF_GEMM_MIN_M", None)
    del ffn
    return out


def run(ops, ctx, stream, steps, warmup, time_graph):
    dev = torch.device("cuda:0")
    out = run_prefill(ops, ctx, stream, steps, warmup, time_graph)

    # ---- config 2: GPTQ ------------------------------------------------------
    K, N, G = 5120, 13824, 128
    for bits in (4, 8):
        qw, qz, sc = synth.gptq_checkpoint(K, N, G, bits, seed=0x0A0D11E7)
        wbytes = qw.nbytes + qz.nbytes + sc.size * 2
        nc = _copies_for(wbytes)
        d = [(torch.from_numpy(qw).to(dev), torch.from_numpy(qz).to(dev),
              torch.from_numpy(sc).to(dev, torch.float16)) for _ in range(nc)]
        for m in (1, 8):
            x = torch.randn((m, K), device=dev, dtype=torch.float16)
            y = torch.empty((m, N), device=dev, dtype=torch.float16)

            def step(i, x=x, y=y, d=d, bits=bits, nc=nc):
                c = d[i % nc]
                ops.gptq_matmul(x, c[0], c[1], c[2], bits, out=y, ctx=ctx)
            out.append(_case(f"gptq{bits} M={m} K={K} N={N} (gptq_matmul op, checkpoint layout)", step, steps,
                             warmup, stream, time_graph, wbytes + m * K * 2 + m * N * 2, 2.0 * m * K * N, ctx))
        # the same weights as resident layers (PackedQuantLinear.forward, repacked at load)
        layers = [ops.PackedQuantLinear(bits, ops.PACK_IN, c[0], c[1], c[2], None, torch.float16, ctx=ctx)
                  for c in d]
        for m in (1, 8, 64):
            x = torch.randn((m, K), device=dev, dtype=torch.float16)
            y = torch.empty((m, N), device=dev, dtype=torch.float16)

            def lstep(i, x=x, y=y, layers=layers, nc=nc):
                layers[i % nc].forward(x, out=y)
            out.append(_case(f"gptq{bits} M={m} K={K} N={N} (PackedQuantLinear)", lstep, steps, warmup, stream,
                             time_graph, wbytes + m * K * 2 + m * N * 2, 2.0 * m * K * N, ctx))
        del d, layers

    # ---- gated FFN entry: fused gate|up projection (config 1's layer twice over) with the activation
    # in the epilogue, against the projection followed by the activation kernel ------------------------
    K, I, G = 4096, 14336, 128
    qw, qz, sc = synth.awq_checkpoint(K, 2 * I, G, 4, seed=0x0A0D11EF)
    wbytes = qw.nbytes + qz.nbytes + sc.size * 2
    nc = _copies_for(wbytes, cap=6)
    plain, fused = [], []
    for _ in range(nc):
        t = (torch.from_numpy(qw).to(dev), torch.from_numpy(qz).to(dev), torch.from_numpy(sc).to(dev, torch.float16))
        plain.append(ops.PackedQuantLinear(4, ops.PACK_OUT, *t, None, torch.float16, ctx=ctx))
        fused.append(ops.PackedQuantLinear(4, ops.PACK_OUT, *t, None, torch.float16, ctx=ctx,
                                           gate_up_act=ops.ACT_GATED_SILU))
        del t
    for m in (1, 16, 64):
        x = torch.randn((m, K), device=dev, dtype=torch.float16)
        y2 = torch.empty((m, 2 * I), device=dev, dtype=torch.float16)
        y1 = torch.empty((m, I), device=dev, dtype=torch.float16)

        def two(i, x=x, y2=y2, y1=y1):
            plain[i % nc].forward(x, out=y2)
            ops.gated_activation(y2, ops.ACT_GATED_SILU, out=y1, ctx=ctx)

        def one(i, x=x, y1=y1):
            fused[i % nc].forward(x, out=y1)
        nb = wbytes + m * K * 2 + m * I * 2
        r = _case(f"awq4 gate|up + SiLU M={m} K={K} I={I} (projection, then activation kernel)", two, steps, warmup,
                  stream, time_graph, nb + 2 * m * 2 * I * 2, 4.0 * m * K * I, ctx)
        r["launches"] = 2
        out.append(r)
        out.append(_case(f"awq4 gate|up + SiLU M={m} K={K} I={I} (fused epilogue)", one, steps, warmup, stream,
                         time_graph, nb, 4.0 * m * K * I, ctx))
    del plain, fused

    # ---- config 3: GGUF --------------------------------------------------------
    K = N = 4096
    for fmt in sorted(synth.GGUF_NAMES):
        data = synth.gguf_weight(fmt, N, K, seed=0x0A0D11E8 + fmt)
        nc = _copies_for(data.nbytes, cap=48)
        d = [torch.from_numpy(data).to(dev) for _ in range(nc)]
        x = torch.randn((1, K), device=dev, dtype=torch.float32)
        y = torch.empty((1, N), device=dev, dtype=torch.float32)

        def step(i, d=d, nc=nc, fmt=fmt, x=x, y=y):
            ops.gguf_quant_matmul(x, d[i % nc], K, N, fmt, out=y, ctx=ctx)
        out.append(_case(f"gguf {synth.GGUF_NAMES[fmt]} M=1 K={K} N={N} f32", step, steps, warmup, stream,
                         time_graph, data.nbytes + K * 4 + N * 4, 2.0 * K * N, ctx))
        if fmt in (synth.GGUF_Q4_0, synth.GGUF_Q4_K, synth.GGUF_Q6_K, synth.GGUF_Q8_0):
            for m in (64, 512, 2048):  # prefill: the tile matmul, bf16
                xb = torch.randn((m, K), device=dev, dtype=torch.bfloat16)
                yb = torch.empty((m, N), device=dev, dtype=torch.bfloat16)

                def mstep(i, d=d, nc=nc, fmt=fmt, x=xb, y=yb):
                    ops.gguf_quant_mul_mm(x, d[i % nc], K, N, fmt, out=y, ctx=ctx)
                out.append(_case(f"gguf {synth.GGUF_NAMES[fmt]} M={m} K={K} N={N} bf16 mul_mm", mstep, steps,
                                 warmup, stream, time_graph, data.nbytes + m * K * 2 + m * N * 2,
                                 2.0 * m * K * N, ctx))
        del d

    # ---- a gated GGUF FFN at decode (ffn.rs:307-474): the reference's layout (gate, up, activation, down: four
    # launches) against the fused gate|up layer with the activation in its epilogue (two launches)
    H, I = 4096, 14336
    for fmt in (synth.GGUF_Q4_K, synth.GGUF_Q6_K):
        parts = [synth.gguf_weight(fmt, I, H, seed=1), synth.gguf_weight(fmt, I, H, seed=2), synth.gguf_weight(fmt, H, I, seed=3)]
        nb_w = sum(p.nbytes for p in parts)
        nc = 3  # 3 x 100 MB and more: beyond the memory-side cache
        sep, fus = [], []
        for _ in range(nc):
            gd, ud, dd = (torch.from_numpy(p).to(dev) for p in parts)
            down = ops.QLinear(fmt, dd, I, H, None, torch.bfloat16, ctx=ctx)
            sep.append(ops.FeedForward(ops.GATE_UP_SEPARATE, ops.QLinear(fmt, gd, H, I, None, torch.bfloat16, ctx=ctx),
                                       ops.QLinear(fmt, ud, H, I, None, torch.bfloat16, ctx=ctx), down, I, ctx=ctx))
            both = torch.cat([gd.reshape(-1), ud.reshape(-1)])
            fus.append(ops.FeedForward(ops.GATE_UP_FUSED, ops.QLinear(fmt, both, H, 2 * I, None, torch.bfloat16, ctx=ctx,
                                                                      gate_up_act=ops.ACT_GATED_SILU), None, down, I, ctx=ctx))
        for m in (1, 8):
            xb = torch.randn((m, H), device=dev, dtype=torch.bfloat16) * 0.1
            yb = torch.empty((m, H), device=dev, dtype=torch.bfloat16)
            sc = torch.empty(m * 3 * I, device=dev, dtype=torch.bfloat16)
            for tag, ffs, launches in (("gate, up, activation, down", sep, 4), ("fused gate|up with the activation, down", fus, 2)):
                def ffstep(i, ffs=ffs, xb=xb, yb=yb, sc=sc):
                    ffs[i % nc].forward(xb, out=yb, scratch=sc)
                r = _case(f"gguf {synth.GGUF_NAMES[fmt]} FFN {H}/{I} M={m} bf16 SiLU: {tag}", ffstep, steps, warmup, stream,
                          time_graph, nb_w + 2 * m * H * 2, 6.0 * m * H * I, ctx)
                r["launches"] = launches
                out.append(r)
        del sep, fus

    # ---- block-scaled F8E4M3 (sibling path: streamed FP8 experts) -----------------------
    for (n8, k8) in ((4096, 4096), (2048, 512)):
        wb = np.random.default_rng(8).integers(0, 256, size=(n8, k8), dtype=np.uint8)
        wb = np.where((wb & 0x7F) == 0x7F, wb ^ 0x08, wb).astype(np.uint8)
        scl = np.random.default_rng(9).uniform(0.01, 1.0, size=(n8 // 128, k8 // 128)).astype(np.float32)
        nc = _copies_for(wb.nbytes, cap=48)
        d8 = [(torch.from_numpy(wb).to(dev), torch.from_numpy(scl).to(dev)) for _ in range(nc)]
        for m in (1, 8, 256):
            x8 = torch.randn((m, k8), device=dev, dtype=torch.bfloat16)
            y8 = torch.empty((m, n8), device=dev, dtype=torch.bfloat16)

            def fstep(i, d8=d8, nc=nc, x8=x8, y8=y8):
                ops.f8_matmul(x8, d8[i % nc][0], d8[i % nc][1], out=y8, ctx=ctx)
            out.append(_case(f"f8e4m3 block-scaled M={m} K={k8} N={n8} bf16", fstep, steps, warmup, stream,
                             time_graph, wb.nbytes + scl.nbytes + m * (k8 + n8) * 2, 2.0 * m * k8 * n8, ctx))
        del d8

    out.extend(run_moe(ops, ctx, stream, steps, warmup, time_graph))
    return out


def run_moe(ops, ctx, stream, steps, warmup, time_graph):
    """Config 4's MXFP4 mixture-of-experts layer: the decode step through the stateless ops, one expert's projection
    as a plain layer at prefill sizes, and whole layer steps at 512 and 2048 tokens through the stateless ops and on
    the resident experts."""
    dev = torch.device("cuda:0")
    out = []
    # ---- config 4: MXFP4 MoE -----------------------------------------------------
    E, top_k, H, I, T = 32, 4, 2880, 2880, 8
    rng = np.random.default_rng(0x0A0D11E9)
    logits = rng.standard_normal((T, E)).astype(np.float32)
    # routing on the host exactly as moe.rs:466-499, 563-590 (softmax, top-k, token lists)
    p = np.exp(logits - logits.max(1, keepdims=True))
    p /= p.sum(1, keepdims=True)
    top = np.argsort(-p, axis=1, kind="stable")[:, :top_k]
    lists = [[] for _ in range(E)]
    for t in range(T):
        for s in range(top_k):
            lists[int(top[t, s])].append(t)
    offsets = np.zeros(E + 1, np.int32)
    offsets[1:] = np.cumsum([len(l) for l in lists])
    tokens = np.array([t for l in lists for t in l], np.int32)
    active = int(sum(1 for l in lists if l))
    n_pairs = T * top_k
    gu_b, gu_s = synth.mxfp4_weight(E * 2 * I, H, seed=1)
    dn_b, dn_s = synth.mxfp4_weight(E * H, I, seed=2)
    gub = torch.from_numpy(gu_b).to(dev), torch.from_numpy(gu_s).to(dev)
    dnb = torch.from_numpy(dn_b).to(dev), torch.from_numpy(dn_s).to(dev)
    gu_bias = torch.randn((E, 2 * I), device=dev, dtype=torch.bfloat16) * 0.1
    dn_bias = torch.randn((E, H), device=dev, dtype=torch.bfloat16) * 0.1
    x = torch.randn((T, H), device=dev, dtype=torch.bfloat16)
    h = torch.randn((n_pairs, I), device=dev, dtype=torch.bfloat16)
    off_d, tok_d = torch.from_numpy(offsets).to(dev), torch.from_numpy(tokens).to(dev)
    y_gu = torch.empty((n_pairs, 2 * I), device=dev, dtype=torch.bfloat16)
    y_dn = torch.empty((n_pairs, H), device=dev, dtype=torch.bfloat16)

    def step(i):
        ops.mxfp4_moe_matmul(x, gub[0], gub[1], gu_bias, off_d, tok_d, H, 2 * I, out=y_gu, ctx=ctx)
        ops.mxfp4_moe_matmul(h, dnb[0], dnb[1], dn_bias, off_d, None, I, H, out=y_dn, ctx=ctx)
    per_expert = (2 * I * (H // 32) * 17 + 2 * I * 2) + (H * (I // 32) * 17 + H * 2)
    nbytes = active * per_expert + T * H * 2 + n_pairs * (2 * I + I + H) * 2
    r = _case(f"mxfp4 moe step: {active} active experts of {E}, {n_pairs} pairs (gate_up + down)", step,
              steps, warmup, stream, time_graph, nbytes, 2.0 * n_pairs * (2 * I * H + H * I), ctx)
    r["note"] = ("expert weights (443 MB total) are read once per step with no copy rotation: "
                 "about 290 MB of active experts exceed the memory-side cache")
    out.append(r)

    # the whole MoE layer step on the device: route -> group -> gate_up -> SwiGLU -> down -> combine
    logits_d = torch.from_numpy(logits).to(dev)
    out_d = torch.empty((T, H), device=dev, dtype=torch.bfloat16)
    h_d = torch.empty((n_pairs, I), device=dev, dtype=torch.bfloat16)

    def full_step(i):
        idx, vals, off, tok, _, pos = ops.moe_route_group(logits_d, top_k, True, ctx=ctx)
        ops.mxfp4_moe_gate_up_swiglu(x, gub[0], gub[1], gu_bias, off, tok, H, 2 * I, 7.0, out=h_d, ctx=ctx)
        ops.mxfp4_moe_matmul(h_d, dnb[0], dnb[1], dn_bias, off, None, I, H, out=y_dn, ctx=ctx)
        ops.moe_combine(y_dn, pos, vals, out=out_d, ctx=ctx)
    r2 = _case(f"mxfp4 moe layer step on device: route and group in one launch + gate_up with fused swiglu + down + combine "
               f"({E} experts, top-{top_k}, {T} tokens)", full_step, steps, warmup, stream, time_graph, nbytes,
               2.0 * n_pairs * (2 * I * H + H * I), ctx)
    r2["launches"] = 4
    out.append(r2)

    # prefill: one expert's gate_up as a plain layer, and a 512-token MoE layer step
    for m in (64, 256, 1024):
        xm = torch.randn((m, H), device=dev, dtype=torch.bfloat16)
        ym = torch.empty((m, 2 * I), device=dev, dtype=torch.bfloat16)
        nb1 = 2 * I * (H // 32)

        def pstep(i, xm=xm, ym=ym):
            ops.mxfp4_matmul(xm, gub[0][:nb1 * 16], gub[1][:nb1], H, 2 * I, out=ym, ctx=ctx)
        out.append(_case(f"mxfp4 M={m} K={H} N={2 * I} bf16 (mxfp4_matmul, prefill)", pstep, steps, warmup, stream,
                         time_graph, nb1 * 17 + m * (H + 2 * I) * 2, 2.0 * m * H * 2 * I, ctx))
    # a MoE layer step at prefill sizes: through the stateless ops on the checkpoint layout (tile matmul + activation
    # kernel), and on the resident experts (tiles of an expert's pairs on the tile-major copy, SwiGLU in the epilogue)
    gu_res = ops.Mxfp4Experts(gub[0], gub[1], gu_bias, E, H, 2 * I, ctx=ctx)
    dn_res = ops.Mxfp4Experts(dnb[0], dnb[1], dn_bias, E, I, H, ctx=ctx)
    for Tp in (512, 2048):
        logits_p = torch.randn((Tp, E), device=dev, dtype=torch.float32)
        xp = torch.randn((Tp, H), device=dev, dtype=torch.bfloat16)
        np_p = Tp * top_k
        ygu_p = torch.empty((np_p, 2 * I), device=dev, dtype=torch.bfloat16)
        h_p = torch.empty((np_p, I), device=dev, dtype=torch.bfloat16)
        ydn_p = torch.empty((np_p, H), device=dev, dtype=torch.bfloat16)
        out_p = torch.empty((Tp, H), device=dev, dtype=torch.bfloat16)

        def prefill_step(i):
            idx, vals = ops.moe_route(logits_p, top_k, True, ctx=ctx)
            off, tok, _, pos = ops.moe_group(idx, vals, E, ctx=ctx)
            ops.mxfp4_moe_matmul(xp, gub[0], gub[1], gu_bias, off, tok, H, 2 * I, out=ygu_p, ctx=ctx)
            ops.gated_activation(ygu_p, ops.ACT_GPT_OSS_SWIGLU, 7.0, out=h_p, ctx=ctx)
            ops.mxfp4_moe_matmul(h_p, dnb[0], dnb[1], dn_bias, off, None, I, H, out=ydn_p, ctx=ctx)
            ops.moe_combine(ydn_p, pos, vals, out=out_p, ctx=ctx)

        def prefill_step_res(i):
            idx, vals = ops.moe_route(logits_p, top_k, True, ctx=ctx)
            off, tok, _, pos = ops.moe_group(idx, vals, E, ctx=ctx)
            gu_res.gate_up_swiglu(xp, off, tok, 7.0, out=h_p)
            dn_res.matmul(h_p, off, None, out=ydn_p)
            ops.moe_combine(ydn_p, pos, vals, out=out_p, ctx=ctx)
        nbytes = E * per_expert + np_p * (H + 2 * I + I + H) * 2
        fl = 2.0 * np_p * (2 * I * H + H * I)
        r3 = _case(f"mxfp4 moe layer step, prefill: {Tp} tokens, {np_p} pairs over {E} experts (stateless ops, checkpoint layout)",
                   prefill_step, steps, warmup, stream, time_graph, nbytes, fl, ctx)
        r3["launches"] = 6
        r3["mfma_frac"] = round(r3["TFLOP_per_s"] / 2500.0, 4)
        out.append(r3)
        r4 = _case(f"mxfp4 moe layer step, prefill: {Tp} tokens, {np_p} pairs over {E} experts (resident experts, fused SwiGLU)",
                   prefill_step_res, steps, warmup, stream, time_graph, nbytes - np_p * 2 * I * 2 * 2, fl, ctx)
        r4["launches"] = 5
        off0, tok0 = ops.moe_group(*ops.moe_route(logits_p, top_k, True, ctx=ctx), E, ctx=ctx)[:2]
        gu_res.gate_up_swiglu(xp, off0, tok0, 7.0, out=h_p)
        r4["kernel"] = ctx.last_plan()["kernel"]
        r4["mfma_frac"] = round(r4["TFLOP_per_s"] / 2500.0, 4)
        out.append(r4)
        del logits_p, xp, ygu_p, h_p, ydn_p, out_p
    del gu_res, dn_res
    return out
