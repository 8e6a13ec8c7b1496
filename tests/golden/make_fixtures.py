#!/usr/bin/env python3
"""Writes the golden fixtures in this directory (run from the repository root:
`python tests/golden/make_fixtures.py`).

The reference holds no golden files for this path: its known answers are closed-form
generators inside its Rust tests.  Each fixture stores the inputs those generators produce
(tests/refgen.py restates the formulas and cites them) or small seeded random blocks, and the
expected outputs computed by the CPU oracle after it has been pinned by tests/test_oracle_kat.py.
The files are data only (numpy .npz, a few KB each); tests/test_golden.py checks the oracle
against them on the CPU and the HIP library against them on the GPU, so a change in either
shows up as a diff against bytes that are under version control.
"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

import oracle  # noqa: E402
from oxydllm_amd import synth  # noqa: E402
from tests import refgen  # noqa: E402

HERE = os.path.dirname(os.path.abspath(__file__))


def save(name, **arrays):
    path = os.path.join(HERE, name + ".npz")
    np.savez_compressed(path, **arrays)
    print(f"{name}.npz: {os.path.getsize(path)} bytes, " + ", ".join(f"{k}{list(v.shape)}" for k, v in arrays.items()))


def main():
    # AWQ 4-bit known answer (awq.rs:954-1011) and GPTQ 4/8-bit (awq.rs:1170-1283)
    qw, qz, sc, exp = refgen.awq_kat_small()
    save("awq4_kat", qweight=qw, qzeros=qz, scales=sc, dequant_nk=oracle.dequantize_awq(qw, qz, sc), reference_nk=exp)
    for bits in (4, 8):
        qw, qz, sc, exp = refgen.gptq_kat(bits)
        save(f"gptq{bits}_kat", qweight=qw, qzeros=qz, scales=sc,
             dequant_nk=oracle.dequantize_gptq(qw, qz, sc, bits), reference_nk=exp)

    # W4A16 / W8A16 / GPTQ matmul on the reference's generators (metal_ops.rs:3668-3779, 3975-4028, 4134-4183)
    K, N, g = 256, 128, 128
    x = refgen.batch_x(5, K)
    for name, trip, deq in (("awq4", refgen.build_awq_triplet(K, N, g), oracle.dequantize_awq),
                            ("awq8", refgen.build_w8a16_triplet(K, N, g), oracle.dequantize_awq8)):
        for dtn, dt in (("f16", oracle.F16), ("bf16", oracle.BF16)):
            w = deq(trip[0], trip[1], oracle.round_through(trip[2], dt))
            save(f"{name}_matmul_{dtn}", qweight=trip[0], qzeros=trip[1], scales=trip[2], x=x,
                 dequant_kn_bits=oracle.transpose_convert(w, dt),
                 y=oracle.matmul_nt_f32(oracle.round_through(x, dt), w))
    for bits in (4, 8):
        trip = refgen.build_gptq_triplet(bits, K, N, g)
        w = oracle.dequantize_gptq(trip[0], trip[1], oracle.round_through(trip[2], oracle.BF16), bits)
        save(f"gptq{bits}_matmul_bf16", qweight=trip[0], qzeros=trip[1], scales=trip[2], x=x,
             dequant_kn_bits=oracle.transpose_convert(w, oracle.BF16),
             y=oracle.matmul_nt_f32(oracle.round_through(x, oracle.BF16), w))

    # MXFP4: the reference's case n = 10, k = 64 (metal_ops.rs:6626-6631)
    blocks, scales = refgen.mxfp4_case(10, 64)
    w = oracle.dequantize_mxfp4_f32(blocks, scales, 10, 64)
    xm = refgen.mxfp4_x(8, 64)
    save("mxfp4_case", blocks=blocks, scales=scales, x=xm, dequant_nk=w,
         y=oracle.matmul_nt_f32(oracle.round_through(xm, oracle.BF16), w))

    # GGUF: 6 rows of 2 blocks for each of the ten formats, seeded random block bytes
    for fmt in sorted(synth.GGUF_NAMES):
        elems, _ = synth.GGUF_BLOCK_LAYOUT[fmt]
        n, k = 6, 2 * max(elems, 256)
        data = synth.gguf_weight(fmt, n, k, seed=1000 + fmt)
        w = oracle.dequantize_gguf(fmt, data, n, k)
        xg = np.random.default_rng(2000 + fmt).standard_normal((3, k)).astype(np.float32)
        save(f"gguf_{synth.GGUF_NAMES[fmt].lower()}", fmt=np.array([fmt]), n=np.array([n]), k=np.array([k]),
             weight_bytes=data, x=xg, dequant_nk=w, y_f32=oracle.matmul_nt_f32(xg, w))

    # block-scaled F8E4M3 (metal_ops.rs:4320-4329) and the decode of every byte
    b, scl = refgen.f8_dequant_case()
    save("f8_block_dequant", bytes=b, scales=scl, dequant_bf16_bits=oracle.f8_block_dequant_bf16(b, scl),
         all_bytes_f32=oracle.cast_f8e4m3_to_f32(np.arange(256, dtype=np.uint8)))

    # load-time transforms (awq.rs:754-835, 1032-1075)
    q, scale, packed = refgen.compressed_tensors_case()
    cqw, cqz, csc = oracle.compressed_to_awq(packed, scale)
    save("compressed_to_awq", weight_packed=packed, weight_scale=scale, qweight=cqw, qzeros=cqz, scales=csc)
    wr = refgen.rtn_weight(16, 64)
    rqw, rqz, rsc = oracle.rtn_quantize_awq(wr, 32)
    save("rtn_quantize_awq", weight=wr, group_size=np.array([32]), qweight=rqw, qzeros=rqz, scales=rsc)

    # mixture-of-experts routing (moe.rs:466-499, 563-607): 8 tokens, 32 experts, top-4
    logits = np.random.default_rng(0x0A0D11E9).standard_normal((8, 32)).astype(np.float32)
    idx, vals = oracle.moe_route(logits, 4, True)
    offsets, tokens, weights = oracle.moe_group(idx, vals, 32)
    save("moe_route_group", logits=logits, top_idx=idx, top_vals=vals, offsets=offsets, tokens=tokens,
         weights=weights)


if __name__ == "__main__":
    main()
