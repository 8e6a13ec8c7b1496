"""Closed-form input generators taken from the reference's own tests.

Only the formulas are restated (they are the reference's test vectors); each
cites where the reference defines it.  All return numpy arrays.
"""
import numpy as np

from oxydllm_amd import synth


def awq_kat_small():
    """awq.rs:954-1011: K=8, N=16, g=4; returns (qweight, qzeros, scales, expected[N,K])."""
    K, N, g = 8, 16, 4
    G = K // g
    i = np.arange(K)[:, None]
    j = np.arange(N)[None, :]
    iweight = (i * 3 + j * 5 + 1) & 0xF
    gi = np.arange(G)[:, None]
    izero = (gi * 7 + j) & 0xF
    scales = (np.float32(0.01) * (gi + 1).astype(np.float32)
              + np.float32(0.001) * (j + 1).astype(np.float32)).astype(np.float32)
    expected = np.zeros((N, K), dtype=np.float32)
    for ii in range(K):
        for jj in range(N):
            w = int(iweight[ii, jj]) - int(izero[ii // g, jj])
            expected[jj, ii] = np.float32(w) * scales[ii // g, jj]
    return synth.pack_awq(iweight), synth.pack_awq(izero), scales, expected


def gptq_kat(bits):
    """awq.rs:1170-1283: K=32, N=16, g=16; 8-bit and 4-bit variants."""
    K, N, g = 32, 16, 16
    G = K // g
    i = np.arange(K)[:, None]
    j = np.arange(N)[None, :]
    gi = np.arange(G)[:, None]
    if bits == 8:
        iweight = (i * 11 + j * 7) & 0xFF
        izero = (gi * 31 + j * 17 + 1) & 0xFF
        scales = (np.float32(0.02) * (gi + 1).astype(np.float32)
                  + np.float32(0.003) * (j + 1).astype(np.float32)).astype(np.float32)
    else:
        iweight = (i * 3 + j * 5) & 0xF
        izero = (gi * 2 + j) & 0xF
        scales = (np.float32(0.01) * (gi + 1).astype(np.float32)
                  + np.float32(0.002) * (j + 1).astype(np.float32)).astype(np.float32)
    expected = np.zeros((N, K), dtype=np.float32)
    for ii in range(K):
        for jj in range(N):
            q = int(iweight[ii, jj])
            z = int(izero[ii // g, jj]) + 1
            expected[jj, ii] = np.float32(q - z) * scales[ii // g, jj]
    return (synth.pack_gptq_qweight(iweight, bits), synth.pack_gptq_qzeros(izero, bits),
            scales, expected)


def build_awq_triplet(K, N, g):
    """metal_ops.rs:3668-3711: q=(5i+3j+1)&15, z=(7g+j+2)&15, s=0.01+0.003*((g+j)%5)."""
    G = K // g
    i = np.arange(K)[:, None]
    j = np.arange(N)[None, :]
    gi = np.arange(G)[:, None]
    iweight = (i * 5 + j * 3 + 1) & 0xF
    izero = (gi * 7 + j + 2) & 0xF
    scales = (np.float32(0.01) + np.float32(0.003) * ((gi + j) % 5).astype(np.float32))
    return synth.pack_awq(iweight), synth.pack_awq(izero), scales.astype(np.float32)


def build_w8a16_triplet(K, N, g):
    """metal_ops.rs:3975-4028; also returns ref_w [N,K] f32 built from the unpacked ints."""
    G = K // g
    i = np.arange(K)[:, None]
    j = np.arange(N)[None, :]
    gi = np.arange(G)[:, None]
    iweight = (i * 11 + j * 7) & 0xFF
    izero = (gi * 31 + j * 5 + 2) & 0xFF
    scales = (np.float32(0.001) + np.float32(0.0007) * ((gi + j) % 17).astype(np.float32))
    scales = scales.astype(np.float32)
    zfull = np.repeat(izero, g, axis=0)
    sfull = np.repeat(scales, g, axis=0)
    ref_w = ((iweight - zfull).astype(np.float32) * sfull).T.copy()
    return synth.pack_awq_8bit(iweight), synth.pack_awq_8bit(izero), scales, ref_w


def build_gptq_triplet(bits, K, N, g):
    """metal_ops.rs:4134-4183: q=(13i+7o)&mask, z=(31g+17o+1)&mask, s=0.002+0.0005*((g+o)%11)."""
    G = K // g
    mask = (1 << bits) - 1
    i = np.arange(K)[:, None]
    o = np.arange(N)[None, :]
    gi = np.arange(G)[:, None]
    iweight = (i * 13 + o * 7) & mask
    izero = (gi * 31 + o * 17 + 1) & mask
    scales = (np.float32(0.002) + np.float32(0.0005) * ((gi + o) % 11).astype(np.float32))
    return (synth.pack_gptq_qweight(iweight, bits), synth.pack_gptq_qzeros(izero, bits),
            scales.astype(np.float32))


def x_gemv(K, mod=13, off=6.0, step=0.03):
    """metal_ops.rs:3727-3729 (AWQ M=1): ((i % 13) - 6) * 0.03; GPTQ uses (17, 8, 0.02)."""
    i = np.arange(K)
    return (((i % mod).astype(np.float32) - np.float32(off)) * np.float32(step)).reshape(1, K)


def batch_x(M, K):
    """metal_ops.rs:3771-3779: ((i % 17) - 8) * 0.03 over the flat [M*K] index."""
    i = np.arange(M * K)
    return (((i % 17).astype(np.float32) - np.float32(8.0)) * np.float32(0.03)).reshape(M, K)


def mxfp4_case(n=10, k=64):
    """metal_ops.rs:6626-6631: blocks=(37i+11)&255, scales=125+i%5."""
    nb = k // 32
    blocks = ((np.arange(n * nb * 16) * 37 + 11) & 0xFF).astype(np.uint8)
    scales = (125 + (np.arange(n * nb) % 5)).astype(np.uint8)
    return blocks, scales


def mxfp4_x(m, k):
    """metal_ops.rs:6642: ((i % 13) - 6) * 0.05."""
    i = np.arange(m * k)
    return (((i % 13).astype(np.float32) - np.float32(6.0)) * np.float32(0.05)).reshape(m, k)


def compressed_tensors_case(out_f=16, in_f=64, group=32):
    """awq.rs:756-785: signed int4 q = i % 16 - 8, scale = 0.01 + (i % 7) * 0.003, packed as
    compressed-tensors does (word (o, c) nibble k = q[o][8c + k] + 8)."""
    groups = in_f // group
    q = (np.arange(out_f * in_f) % 16 - 8).reshape(out_f, in_f)
    scale = (np.float32(0.01) + (np.arange(out_f * groups) % 7).astype(np.float32)
             * np.float32(0.003)).reshape(out_f, groups)
    packed = np.zeros((out_f, in_f // 8), np.uint32)
    for k in range(8):
        packed |= ((q[:, k::8] + 8) & 0xF).astype(np.uint32) << np.uint32(4 * k)
    return q, scale, packed.view(np.int32)


def concat_parts(in_features=8, group_size=4, parts_out=(16, 8, 8)):
    """awq.rs:1032-1075: three AWQ parts with q = (i + j + 3 idx) & 15, z = (2 g + j + idx) & 15,
    s = 0.02 (g + 1) + 0.005 (j + 1) + 0.001 idx."""
    groups = in_features // group_size
    parts = []
    for idx, out_f in enumerate(parts_out):
        i, j = np.meshgrid(np.arange(in_features), np.arange(out_f), indexing="ij")
        g, jz = np.meshgrid(np.arange(groups), np.arange(out_f), indexing="ij")
        iw = (i + j + idx * 3) & 0xF
        iz = (g * 2 + jz + idx) & 0xF
        sc = (np.float32(0.02) * (g + 1).astype(np.float32) + np.float32(0.005) * (jz + 1).astype(np.float32)
              + np.float32(0.001) * np.float32(idx)).astype(np.float32)
        parts.append((synth.pack_awq(iw), synth.pack_awq(iz), sc))
    return parts


def rtn_weight(out_f=16, in_f=64):
    """awq.rs:803-806: sin(0.013 i)."""
    return np.sin(np.arange(out_f * in_f, dtype=np.float32) * np.float32(0.013)).astype(np.float32).reshape(out_f, in_f)


def f8_dequant_case(rows=8, cols=256):
    """metal_ops.rs:4320-4329: bytes (37 i + 11) & 255 with the NaN encodings S.1111.111 moved
    off (b ^ 0x08), scale grid [2, 2] = 0.5 + 0.75 i."""
    b = ((np.arange(rows * cols, dtype=np.int64) * 37 + 11) & 0xFF).astype(np.uint8)
    b = np.where((b & 0x7F) == 0x7F, b ^ 0x08, b).astype(np.uint8)
    scales = (np.float32(0.5) + np.arange(4, dtype=np.float32) * np.float32(0.75)).reshape(2, 2)
    return b.reshape(rows, cols), scales


def f8_gemv_case(out_f, in_f, s_r, s_c, m):
    """metal_ops.rs:4388-4396: bytes (29 i + 13) & 255 (NaN encodings moved off),
    scales 0.2 + (i % 7) * 0.3, x = sin(0.013 i)."""
    b = ((np.arange(out_f * in_f, dtype=np.int64) * 29 + 13) & 0xFF).astype(np.uint8)
    b = np.where((b & 0x7F) == 0x7F, b ^ 0x08, b).astype(np.uint8)
    scales = (np.float32(0.2) + (np.arange(s_r * s_c) % 7).astype(np.float32) * np.float32(0.3)).reshape(s_r, s_c)
    x = np.sin(np.arange(m * in_f, dtype=np.float32) * np.float32(0.013)).astype(np.float32).reshape(m, in_f)
    return b.reshape(out_f, in_f), scales, x
