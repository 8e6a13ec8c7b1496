"""Pins the CPU oracle before anything is compared against it.

Each oracle function is checked against something it was not written from:
the reference's hand-packed known-answer tests, closed forms, IEEE casts done
by numpy/torch, brute force on small inputs, or an independently structured
restatement of the public ggml block formats.
"""
import numpy as np
import pytest
import torch

import oracle
from oxydllm_amd import synth
from tests import refgen


# ------------------------------------------------------------------ conversions
def test_f16_conversion_matches_ieee_rne():
    rng = np.random.default_rng(1)
    vals = np.concatenate([
        rng.standard_normal(20000).astype(np.float32) * np.float32(10.0),
        rng.uniform(-7e4, 7e4, 5000).astype(np.float32),
        (rng.standard_normal(5000) * 1e-5).astype(np.float32),
        (rng.standard_normal(5000) * 1e-7).astype(np.float32),
        np.array([0.0, -0.0, 65504.0, 65519.9, 65520.0, 1e9, -1e9, np.inf, -np.inf,
                  2.0 ** -24, 2.0 ** -25, 2.0 ** -25 * 1.0001, 2.0 ** -14, 1.0009765625,
                  1.00048828125, 1.00146484375], dtype=np.float32),
    ])
    got = oracle.convert_f32(vals, oracle.F16)
    want = vals.astype(np.float16).view(np.uint16)
    np.testing.assert_array_equal(got, want)
    # every f16 bit pattern widens exactly
    allbits = np.arange(65536, dtype=np.uint16)
    wide = oracle.widen_to_f32(allbits, oracle.F16)
    ref = allbits.view(np.float16).astype(np.float32)
    np.testing.assert_array_equal(wide.view(np.uint32), ref.view(np.uint32))


def test_bf16_conversion_matches_torch_rne():
    rng = np.random.default_rng(2)
    vals = np.concatenate([
        rng.standard_normal(30000).astype(np.float32) * np.float32(100.0),
        (rng.standard_normal(5000) * 1e-30).astype(np.float32),
        np.array([0.0, -0.0, 1.00390625, 1.01171875, 3.3895314e38, np.inf, -np.inf],
                 dtype=np.float32),
    ])
    got = oracle.convert_f32(vals, oracle.BF16)
    want = torch.from_numpy(vals).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    np.testing.assert_array_equal(got, want)
    back = oracle.widen_to_f32(got, oracle.BF16)
    ref = torch.from_numpy(vals).to(torch.bfloat16).to(torch.float32).numpy()
    np.testing.assert_array_equal(back.view(np.uint32), ref.view(np.uint32))


# ------------------------------------------------------------------ AWQ / GPTQ KATs
def test_awq_dequant_known_answer():
    """awq.rs:954-1011 dequantize_awq_recovers_original_matrix, tol 1e-6."""
    qw, qz, sc, expected = refgen.awq_kat_small()
    got = oracle.dequantize_awq(qw, qz, sc)
    assert got.shape == (16, 8)
    assert np.max(np.abs(got - expected)) < 1e-6
    np.testing.assert_array_equal(got, expected)  # and in fact bit-equal


def test_awq_hand_packed_word():
    """One word by hand: slot k of the word is column ORDER[k]."""
    # columns 0..7 hold values 1..8 -> slots hold columns 0,2,4,6,1,3,5,7 = 1,3,5,7,2,4,6,8
    word = 0
    for k, v in enumerate([1, 3, 5, 7, 2, 4, 6, 8]):
        word |= v << (4 * k)
    qw = np.array([[word]], dtype=np.uint32)
    qz = np.zeros((1, 1), dtype=np.uint32)
    sc = np.ones((1, 8), dtype=np.float32)
    got = oracle.dequantize_awq(qw, qz, sc)  # [8,1]
    np.testing.assert_array_equal(got[:, 0], np.arange(1, 9, dtype=np.float32))
    assert synth.pack_awq(np.arange(1, 9).reshape(1, 8)).view(np.uint32)[0, 0] == word


def test_awq_accepts_i32_u32_i64():
    """read_packed_to_u32 (awq.rs:158-179)."""
    qw, qz, sc, expected = refgen.awq_kat_small()
    for dt in (np.int32, np.uint32, np.int64):
        a = qw.view(np.uint32).astype(dt) if dt != np.int32 else qw
        b = qz.view(np.uint32).astype(dt) if dt != np.int32 else qz
        np.testing.assert_array_equal(oracle.dequantize_awq(a, b, sc), expected)
    with pytest.raises(TypeError):
        oracle.dequantize_awq(qw.astype(np.float32), qz, sc)


def test_awq_rejects_wrong_shapes():
    """awq.rs:1096-1121: qweight [8,2], qzeros [2,2], scales [2,8] must be rejected."""
    with pytest.raises(ValueError):
        oracle.dequantize_awq(np.zeros((8, 2), np.int32), np.zeros((2, 2), np.int32),
                              np.zeros((2, 8), np.float32))


def test_awq_compressed_tensors_closed_form():
    """awq.rs:754-800: signed int4 q in [-8,7] stored as q+8 with zero 8 gives q*scale."""
    out_f, in_f, group = 16, 64, 32
    groups = in_f // group
    q = (np.arange(out_f * in_f) % 16 - 8).reshape(out_f, in_f)
    scale = (np.float32(0.01) + (np.arange(out_f * groups) % 7).astype(np.float32)
             * np.float32(0.003)).reshape(out_f, groups)
    qweight = synth.pack_awq((q + 8).T)                       # [in, out/8]
    qzeros = synth.pack_awq(np.full((groups, out_f), 8))
    scales = scale.T.copy()                                   # [groups, out]
    dq = oracle.dequantize_awq(qweight, qzeros, scales)
    expected = q.astype(np.float32) * np.repeat(scale, group, axis=1)
    assert np.max(np.abs(dq - expected)) < 1e-6


def test_gguf_depermute_qk_rows_inverts_converter_permute():
    """gguf_weights.rs:363-398: the converter's permute reshape(n_head, 2, hd/2, k).swapaxes(1, 2),
    applied in HF row space, is undone exactly; here with numpy's own reshape/swapaxes as the
    independent statement of that permute, on rows of Q4_K blocks."""
    n_heads, head_dim, k = 2, 8, 512
    n = n_heads * head_dim
    row_bytes = k // 256 * 144
    hf = synth.gguf_weight(synth.GGUF_Q4_K, n, k, seed=77).reshape(n, row_bytes)
    permuted = hf.reshape(n_heads, 2, head_dim // 2, row_bytes).swapaxes(1, 2).reshape(n, row_bytes)
    assert not np.array_equal(permuted, hf)
    restored = oracle.gguf_depermute_qk_rows(permuted.reshape(-1), row_bytes, n_heads, head_dim)
    np.testing.assert_array_equal(restored.reshape(n, row_bytes), hf)
    # the reference's loop form of the same permute (gguf_weights.rs:377-386)
    half = head_dim // 2
    loop = np.empty_like(hf)
    for h in range(n_heads):
        for j in range(head_dim):
            loop[h * head_dim + j] = hf[h * head_dim + (j % 2) * half + j // 2]
    np.testing.assert_array_equal(loop, permuted)


# ------------------------------------------------------------------ block-scaled F8E4M3
def test_f8e4m3_decode_every_byte():
    """metal_ops.rs:2942-2989: the spec decode over all 256 encodings, against torch's own
    float8_e4m3fn cast (an independent implementation) and against the closed form
    (-1)^s 2^(e-7) (1 + m/8), subnormals m/8 2^-6, S.1111.111 = NaN, largest finite 448."""
    import torch
    b = np.arange(256, dtype=np.uint8)
    got = oracle.cast_f8e4m3_to_f32(b)
    ref = torch.from_numpy(b.copy()).view(torch.float8_e4m3fn).to(torch.float32).numpy()
    nan = np.isnan(ref)
    assert list(np.nonzero(nan)[0]) == [0x7F, 0xFF] and np.array_equal(np.isnan(got), nan)
    np.testing.assert_array_equal(got[~nan].view(np.uint32), ref[~nan].view(np.uint32))
    assert got[0x7E] == 448.0 and got[0xFE] == -448.0 and got[0x01] == 2.0 ** -9 and got[0x38] == 1.0
    assert got[0x00] == 0.0 and np.signbit(got[0x80]) and got[0x80] == 0.0


def test_f8_block_dequant_chain():
    """metal_ops.rs:4310-4375: F8 -> F32 -> BF16, F32 scale fold, -> BF16, on the reference's
    bytes and 2 x 2 scale grid, against the same chain written with torch casts."""
    import torch
    b, scales = refgen.f8_dequant_case()
    got = oracle.f8_block_dequant_bf16(b, scales)
    w = torch.from_numpy(b.copy()).view(torch.float8_e4m3fn).to(torch.float32).to(torch.bfloat16).to(torch.float32)
    grid = torch.from_numpy(scales).repeat_interleave(b.shape[0] // 2, 0).repeat_interleave(b.shape[1] // 2, 1)
    want = (w * grid).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    np.testing.assert_array_equal(got, want)
    # the inner bf16 rounding is the identity on E4M3 values (3 mantissa bits)
    vals = oracle.cast_f8e4m3_to_f32(np.arange(256, dtype=np.uint8))
    ok = ~np.isnan(vals)
    np.testing.assert_array_equal(oracle.round_through(vals[ok], oracle.BF16), vals[ok])
    with pytest.raises(ValueError):
        oracle.f8_block_dequant_bf16(b, np.ones((3, 2), np.float32))


# ------------------------------------------------------------------ load-time transforms
def test_compressed_to_awq_matches_direct_dequant():
    """awq.rs:754-800: dequantizing the converted tensors reproduces q * scale exactly; and the
    conversion equals unpacking the nibbles and packing them the AWQ way."""
    q, scale, packed = refgen.compressed_tensors_case()
    out_f, in_f = q.shape
    qw, qz, sc = oracle.compressed_to_awq(packed, scale)
    assert qw.shape == (in_f, out_f // 8) and sc.shape == (scale.shape[1], out_f)
    dq = oracle.dequantize_awq(qw, qz, sc)
    expected = q.astype(np.float32) * np.repeat(scale, in_f // scale.shape[1], axis=1)
    assert np.max(np.abs(dq - expected)) < 1e-6
    np.testing.assert_array_equal(qw.view(np.int32), synth.pack_awq((q + 8).T))
    np.testing.assert_array_equal(qz, np.full_like(qz, 0x88888888))
    np.testing.assert_array_equal(sc, scale.T)
    with pytest.raises(ValueError):
        oracle.compressed_to_awq(packed, scale[:8])


def test_concat_awq_along_out_matches_separate_dequant():
    """awq.rs:1032-1093 and 1095-1110."""
    parts = refgen.concat_parts()
    fused = oracle.concat_awq_along_out(parts)
    assert fused[2].shape == (2, 32)
    separate = np.concatenate([oracle.dequantize_awq(*p) for p in parts], axis=0)
    np.testing.assert_array_equal(oracle.dequantize_awq(*fused), separate)
    with pytest.raises(ValueError):
        oracle.concat_awq_along_out([refgen.concat_parts(4, 4, (8,))[0], refgen.concat_parts(8, 8, (8,))[0]])


def _rtn_numpy(w, group):
    """awq.rs:676-709 with whole-array numpy operations (f32 throughout)."""
    out_f, in_f = w.shape
    g = w.reshape(out_f, in_f // group, group)
    xmin = np.minimum(g.min(axis=2), np.float32(0))
    xmax = np.maximum(g.max(axis=2), np.float32(0))
    flat = (xmax - xmin) < np.float32(1e-12)
    scale = np.where(flat, xmin, (xmax - xmin) / np.float32(15)).astype(np.float32)
    safe = np.where(flat, np.float32(1), scale)

    def rnd(v):  # round half away from zero, as f32::round
        return np.copysign(np.floor(np.abs(v) + np.float32(0.5)), v).astype(np.float32)
    zero = np.where(flat, np.float32(0), np.clip(rnd(-xmin / safe), 0, 15)).astype(np.float32)
    q = np.clip(rnd(g / safe[:, :, None] + zero[:, :, None]), 0, 15)
    q = np.where(flat[:, :, None], np.float32(1), q).astype(np.uint8).reshape(out_f, in_f)
    return q, zero.astype(np.uint8), scale


@pytest.mark.parametrize("shape,group", [((16, 64), 32), ((24, 256), 128), ((8, 96), 48)])
def test_rtn_quantize_awq(shape, group):
    """awq.rs:802-835 (round trip below 5 % relative error) on the reference's sine weight, and
    what the arithmetic fixes: the whole-array restatement gives the same integers; every
    element is reproduced to half a quantization step; an all-zero group stores q = 1, zero = 0,
    scale = 0 and dequantizes to exactly 0."""
    w = refgen.rtn_weight(*shape)
    w[3, :group] = 0.0                       # a flat group
    w[5, group:2 * group] = np.abs(w[5, group:2 * group]) + 1.0   # a group that does not straddle 0
    qw, qz, sc = oracle.rtn_quantize_awq(w, group)
    out_f, in_f = shape
    assert qw.shape == (in_f, out_f // 8) and qz.shape == (in_f // group, out_f // 8) and sc.shape == (in_f // group, out_f)
    dq = oracle.dequantize_awq(qw, qz, sc)
    rel = np.sqrt(((dq - w).astype(np.float64) ** 2).sum() / (w.astype(np.float64) ** 2).sum())
    assert rel < 0.05
    q, z, s = _rtn_numpy(w, group)
    np.testing.assert_array_equal(qw.view(np.int32), synth.pack_awq(q.T))
    np.testing.assert_array_equal(qz.view(np.int32), synth.pack_awq(z.T))
    np.testing.assert_array_equal(sc, s.T)
    step = np.repeat(sc.T, group, axis=1)
    assert np.all(np.abs(dq - w) <= 0.5 * step * (1 + 1e-5) + 1e-7)
    assert np.all(dq[3, :group] == 0.0) and sc[0, 3] == 0.0
    assert np.all((qw[:group, 0] >> 20) & 0xF == 1)   # output row 3 sits in slot 5 (AWQ order[5] = 3)
    with pytest.raises(ValueError):
        oracle.rtn_quantize_awq(w[:7], group)


@pytest.mark.parametrize("bits", [4, 8])
def test_gptq_dequant_known_answer(bits):
    """awq.rs:1170-1283, tol 1e-5."""
    qw, qz, sc, expected = refgen.gptq_kat(bits)
    got = oracle.dequantize_gptq(qw, qz, sc, bits)
    assert got.shape == (16, 32)
    assert np.max(np.abs(got - expected)) < 1e-5
    np.testing.assert_array_equal(got, expected)


@pytest.mark.parametrize("bits", [4, 8])
def test_gptq_symmetric_zero(bits):
    """awq.rs:567, 580-585: no qzeros -> zero+1 = 2^(bits-1)."""
    qw, _, sc, _ = refgen.gptq_kat(bits)
    got = oracle.dequantize_gptq(qw, None, sc, bits)
    pf = 32 // bits
    q = np.zeros((32, 16), dtype=np.int64)
    w = qw.view(np.uint32)
    for i in range(32):
        q[i] = (w[i // pf] >> np.uint32(bits * (i % pf))) & ((1 << bits) - 1)
    want = ((q - (1 << (bits - 1))).astype(np.float32) * np.repeat(sc, 16, axis=0)).T
    np.testing.assert_array_equal(got, want)
    # stored zero 2^(bits-1)-1 with explicit qzeros gives the same matrix
    z = synth.pack_gptq_qzeros(np.full((2, 16), (1 << (bits - 1)) - 1), bits)
    np.testing.assert_array_equal(oracle.dequantize_gptq(qw, z, sc, bits), want)


def test_gptq_rejects_bad_bits():
    qw, qz, sc, _ = refgen.gptq_kat(4)
    with pytest.raises(ValueError):
        oracle.dequantize_gptq(qw, qz, sc, 3)


def test_awq8_matches_reference_generator():
    """metal_ops.rs:3975-4009: ref_w built from the unpacked ints."""
    qw, qz, sc, ref_w = refgen.build_w8a16_triplet(256, 128, 64)
    np.testing.assert_array_equal(oracle.dequantize_awq8(qw, qz, sc), ref_w)


@pytest.mark.parametrize("K,N,g", [(256, 128, 128), (256, 128, 64), (512, 256, 128)])
def test_awq_bruteforce_on_reference_triplets(K, N, g):
    """Brute force per element on the reference's GPU-test generator shapes."""
    qw, qz, sc = refgen.build_awq_triplet(K, N, g)
    got = oracle.dequantize_awq(qw, qz, sc)
    i = np.arange(K)[:, None]
    j = np.arange(N)[None, :]
    q = (i * 5 + j * 3 + 1) & 0xF
    z = np.repeat((np.arange(K // g)[:, None] * 7 + j + 2) & 0xF, g, axis=0)
    want = ((q - z).astype(np.float32) * np.repeat(sc, g, axis=0)).T
    np.testing.assert_array_equal(got, want)


def test_transpose_convert_is_single_rounding():
    qw, qz, sc = refgen.build_awq_triplet(256, 128, 64)
    for dt, npdt in ((oracle.F16, np.float16),):
        s16 = oracle.round_through(sc, dt)
        w = oracle.dequantize_awq(qw, qz, s16)
        kn = oracle.transpose_convert(w, dt)
        np.testing.assert_array_equal(kn, w.T.astype(npdt).view(np.uint16))
    s16 = oracle.round_through(sc, oracle.BF16)
    w = oracle.dequantize_awq(qw, qz, s16)
    kn = oracle.transpose_convert(w, oracle.BF16)
    want = torch.from_numpy(w.T.copy()).to(torch.bfloat16).view(torch.int16).numpy()
    np.testing.assert_array_equal(kn, want.view(np.uint16))


# ------------------------------------------------------------------ MXFP4
def test_mxfp4_known_values():
    """mxfp4.rs:178-197: codes 0..15 at scale 128 (x2)."""
    blocks = [(2 * i) | ((2 * i + 1) << 4) for i in range(8)] + [0] * 8
    out = oracle.dequantize_mxfp4_f32(np.array(blocks, np.uint8), np.array([128], np.uint8), 1, 32)
    exp = np.array([0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0,
                    -0.0, -0.5, -1.0, -1.5, -2.0, -3.0, -4.0, -6.0], np.float32) * 2
    np.testing.assert_array_equal(out[0, :16], exp)
    assert np.signbit(out[0, 8])
    assert np.all(out[0, 16:] == 0.0)


def test_mxfp4_linear_manual_dot():
    """mxfp4.rs:199-214: two rows both dot to 32 with all-ones x."""
    blocks = np.array([0x22] * 16 + [0x44] * 16, np.uint8)
    scales = np.array([127, 126], np.uint8)
    w = oracle.dequantize_mxfp4_f32(blocks, scales, 2, 32)
    y = oracle.matmul_nt_f32(np.ones((1, 32), np.float32), w)
    np.testing.assert_array_equal(y, np.array([[32.0, 32.0]], np.float32))


def test_mxfp4_nan_scale_and_size_check():
    out = oracle.dequantize_mxfp4_f32(np.zeros(16, np.uint8), np.array([255], np.uint8), 1, 32)
    assert np.all(np.isnan(out))
    with pytest.raises(ValueError):
        oracle.dequantize_mxfp4_f32(np.zeros(15, np.uint8), np.array([127], np.uint8), 1, 32)
    with pytest.raises(ValueError):
        oracle.dequantize_mxfp4_f32(np.zeros(16, np.uint8), np.array([127], np.uint8), 1, 33)


def test_mxfp4_e8m0_is_exact_power_of_two():
    for s in (0, 1, 100, 118, 126, 127, 128, 200, 254):
        out = oracle.dequantize_mxfp4_f32(np.full(16, 0x22, np.uint8), np.array([s], np.uint8), 1, 32)
        assert out[0, 0] == np.float32(2.0) ** np.float32(s - 127)


# ------------------------------------------------------------------ GGUF
def _ggml_q4_0(blk):
    d = blk[0:2].view(np.float16).astype(np.float32)[0]
    qs = blk[2:18].astype(np.int32)
    y = np.empty(32, np.float32)
    for j in range(16):  # ggml dequantize_row_q4_0: y[j] low nibble, y[j+16] high nibble
        y[j] = np.float32((qs[j] & 0xF) - 8) * d
        y[j + 16] = np.float32((qs[j] >> 4) - 8) * d
    return y


def _ggml_q8_0(blk):
    d = blk[0:2].view(np.float16).astype(np.float32)[0]
    return blk[2:34].view(np.int8).astype(np.float32) * d


def _k4(j, q):
    if j < 4:
        return q[j] & 63, q[j + 4] & 63
    return (q[j + 4] & 0xF) | ((q[j - 4] >> 6) << 4), (q[j + 4] >> 4) | ((q[j] >> 6) << 4)


def _ggml_q4_k(blk):
    d = blk[0:2].view(np.float16).astype(np.float32)[0]
    dmin = blk[2:4].view(np.float16).astype(np.float32)[0]
    sc = blk[4:16].astype(np.int32)
    q = blk[16:144].astype(np.int32)
    y = []
    is_ = 0
    for j in range(0, 256, 64):  # ggml dequantize_row_q4_K walks 64 elements per 32 bytes
        s1, m1 = _k4(is_, sc)
        s2, m2 = _k4(is_ + 1, sc)
        d1, mm1 = d * np.float32(s1), dmin * np.float32(m1)
        d2, mm2 = d * np.float32(s2), dmin * np.float32(m2)
        qq = q[(j // 64) * 32:(j // 64) * 32 + 32]
        y.extend(d1 * (qq & 0xF).astype(np.float32) - mm1)
        y.extend(d2 * (qq >> 4).astype(np.float32) - mm2)
        is_ += 2
    return np.array(y, np.float32)


def _ggml_q6_k(blk):
    ql = blk[0:128].astype(np.int32)
    qh = blk[128:192].astype(np.int32)
    sc = blk[192:208].view(np.int8).astype(np.int32)
    d = blk[208:210].view(np.float16).astype(np.float32)[0]
    y = np.empty(256, np.float32)
    for n in range(0, 256, 128):  # ggml dequantize_row_q6_K
        h = n // 128
        qlh, qhh, sch = ql[64 * h:], qh[32 * h:], sc[8 * h:]
        for l in range(32):
            is_ = l // 16
            q1 = ((qlh[l] & 0xF) | (((qhh[l] >> 0) & 3) << 4)) - 32
            q2 = ((qlh[l + 32] & 0xF) | (((qhh[l] >> 2) & 3) << 4)) - 32
            q3 = ((qlh[l] >> 4) | (((qhh[l] >> 4) & 3) << 4)) - 32
            q4 = ((qlh[l + 32] >> 4) | (((qhh[l] >> 6) & 3) << 4)) - 32
            y[n + l] = d * np.float32(sch[is_]) * np.float32(q1)
            y[n + l + 32] = d * np.float32(sch[is_ + 2]) * np.float32(q2)
            y[n + l + 64] = d * np.float32(sch[is_ + 4]) * np.float32(q3)
            y[n + l + 96] = d * np.float32(sch[is_ + 6]) * np.float32(q4)
    return y


def _ggml_q4_1(blk):
    d, m = blk[0:4].view(np.float16).astype(np.float32)
    qs = blk[4:20].astype(np.int32)
    y = np.empty(32, np.float32)
    for j in range(16):  # ggml dequantize_row_q4_1
        y[j] = np.float32(qs[j] & 0xF) * d + m
        y[j + 16] = np.float32(qs[j] >> 4) * d + m
    return y


def _ggml_q5(blk, with_min):
    """ggml dequantize_row_q5_0 / q5_1: the fifth bit of element j is bit j of qh, of
    element j + 16 bit j + 16 (written there as (qh >> (j + 12)) & 0x10)."""
    off = 4 if with_min else 2
    d = blk[0:2].view(np.float16).astype(np.float32)[0]
    m = blk[2:4].view(np.float16).astype(np.float32)[0] if with_min else np.float32(0)
    qh = int(blk[off:off + 4].view("<u4")[0])
    qs = blk[off + 4:off + 20].astype(np.int32)
    y = np.empty(32, np.float32)
    for j in range(16):
        xh0 = ((qh >> j) << 4) & 0x10
        xh1 = (qh >> (j + 12)) & 0x10
        x0, x1 = (qs[j] & 0xF) | xh0, (qs[j] >> 4) | xh1
        if with_min:
            y[j], y[j + 16] = np.float32(x0) * d + m, np.float32(x1) * d + m
        else:
            y[j], y[j + 16] = np.float32(x0 - 16) * d, np.float32(x1 - 16) * d
    return y


def _ggml_q2_k(blk):
    scales = blk[0:16].astype(np.int32)
    q = blk[16:80].astype(np.int32)
    d, dmin = blk[80:84].view(np.float16).astype(np.float32)
    y = []
    is_ = 0
    for n in range(0, 256, 128):  # ggml dequantize_row_q2_K
        qq = q[(n // 128) * 32:]
        shift = 0
        for _ in range(4):
            for off in (0, 16):
                sc = scales[is_]
                is_ += 1
                dl, ml = d * np.float32(sc & 0xF), dmin * np.float32(sc >> 4)
                y.extend(dl * ((qq[off:off + 16] >> shift) & 3).astype(np.float32) - ml)
            shift += 2
    return np.array(y, np.float32)


def _ggml_q3_k(blk):
    hm = blk[0:32].astype(np.int32)
    q = blk[32:96].astype(np.int32)
    d = blk[108:110].view(np.float16).astype(np.float32)[0]
    # ggml unpacks the 12 scale bytes with three 32-bit words and two masks
    aux = [int(v) for v in blk[96:108].view("<u4")]
    k1, k2 = 0x03030303, 0x0F0F0F0F
    tmp = aux[2]
    a2 = ((aux[0] >> 4) & k2) | (((tmp >> 4) & k1) << 4)
    a3 = ((aux[1] >> 4) & k2) | (((tmp >> 6) & k1) << 4)
    a0 = (aux[0] & k2) | (((tmp >> 0) & k1) << 4)
    a1 = (aux[1] & k2) | (((tmp >> 2) & k1) << 4)
    scales = np.array([a0, a1, a2, a3], "<u4").view(np.int8).astype(np.int32)
    y = []
    is_, m = 0, 1
    for n in range(0, 256, 128):  # ggml dequantize_row_q3_K
        qq = q[(n // 128) * 32:]
        shift = 0
        for _ in range(4):
            for off in (0, 16):
                dl = d * np.float32(scales[is_] - 32)
                is_ += 1
                low = (qq[off:off + 16] >> shift) & 3
                sub = np.where((hm[off:off + 16] & m) != 0, 0, 4)
                y.extend(dl * (low - sub).astype(np.float32))
            shift += 2
            m <<= 1
    return np.array(y, np.float32)


def _ggml_q5_k(blk):
    d, dmin = blk[0:4].view(np.float16).astype(np.float32)
    sc = blk[4:16].astype(np.int32)
    qh = blk[16:48].astype(np.int32)
    ql = blk[48:176].astype(np.int32)
    y = []
    is_, u1, u2 = 0, 1, 2
    for j in range(0, 256, 64):  # ggml dequantize_row_q5_K
        s1, m1 = _k4(is_, sc)
        s2, m2 = _k4(is_ + 1, sc)
        d1, mm1 = d * np.float32(s1), dmin * np.float32(m1)
        d2, mm2 = d * np.float32(s2), dmin * np.float32(m2)
        qq = ql[(j // 64) * 32:(j // 64) * 32 + 32]
        y.extend(d1 * ((qq & 0xF) + np.where(qh & u1, 16, 0)).astype(np.float32) - mm1)
        y.extend(d2 * ((qq >> 4) + np.where(qh & u2, 16, 0)).astype(np.float32) - mm2)
        is_ += 2
        u1 <<= 2
        u2 <<= 2
    return np.array(y, np.float32)


_GGML = {synth.GGUF_Q4_0: _ggml_q4_0, synth.GGUF_Q8_0: _ggml_q8_0,
         synth.GGUF_Q4_K: _ggml_q4_k, synth.GGUF_Q6_K: _ggml_q6_k,
         synth.GGUF_Q4_1: _ggml_q4_1, synth.GGUF_Q5_0: lambda b: _ggml_q5(b, False),
         synth.GGUF_Q5_1: lambda b: _ggml_q5(b, True), synth.GGUF_Q2_K: _ggml_q2_k,
         synth.GGUF_Q3_K: _ggml_q3_k, synth.GGUF_Q5_K: _ggml_q5_k}


@pytest.mark.parametrize("fmt", sorted(_GGML))
def test_gguf_dequant_matches_ggml_row_loops(fmt):
    """Block formats per the public ggml spec, walked the way ggml's own
    dequantize_row_* loops walk them (not the per-element index formula)."""
    elems, bbytes = synth.GGUF_BLOCK_LAYOUT[fmt]
    N, K = 3, 2 * elems
    data = synth.gguf_weight(fmt, N, K, seed=11 + fmt)
    got = oracle.dequantize_gguf(fmt, data, N, K)
    blocks = data.reshape(N * 2, bbytes)
    want = np.stack([_GGML[fmt](b) for b in blocks]).reshape(N, K)
    np.testing.assert_array_equal(got, want)


def test_gguf_closed_forms():
    # Q4_0 all-zero quants -> -8 d ; Q8_0 quant 1 -> d
    d = np.array([0.0123], np.float16)
    blk = np.zeros(18, np.uint8)
    blk[0:2] = d.view(np.uint8)
    out = oracle.dequantize_gguf(oracle.Q4_0, blk, 1, 32)
    np.testing.assert_array_equal(out, np.full((1, 32), np.float32(-8) * d.astype(np.float32)[0]))
    blk = np.ones(34, np.uint8)
    blk[0:2] = d.view(np.uint8)
    out = oracle.dequantize_gguf(oracle.Q8_0, blk, 1, 32)
    np.testing.assert_array_equal(out, np.full((1, 32), d.astype(np.float32)[0]))
    # Q6_K all-zero ql/qh -> -32 * d * scale[sub-block]
    blk = np.zeros(210, np.uint8)
    blk[192:208] = np.arange(1, 17, dtype=np.uint8)
    blk[208:210] = d.view(np.uint8)
    out = oracle.dequantize_gguf(oracle.Q6_K, blk, 1, 256)[0]
    for j in range(256):
        sub = j // 16
        assert out[j] == d.astype(np.float32)[0] * np.float32(sub + 1) * np.float32(-32)
    # Q4_K: scales bytes give sc=j+1 (j<4), min=0 -> w = d*sc*nib
    blk = np.zeros(144, np.uint8)
    blk[0:2] = d.view(np.uint8)
    blk[2:4] = d.view(np.uint8)
    blk[4:8] = [1, 2, 3, 4]
    blk[16:144] = 0x21  # low nibble 1, high nibble 2
    out = oracle.dequantize_gguf(oracle.Q4_K, blk, 1, 256)[0]
    df = d.astype(np.float32)[0]
    assert np.all(out[0:32] == df * 1 * 1) and np.all(out[32:64] == df * 2 * 2)
    assert np.all(out[64:96] == df * 3 * 1) and np.all(out[96:128] == df * 4 * 2)
    assert np.all(out[128:] == 0)


def test_gguf_closed_forms_more_formats():
    """One element set at a time: which bit of which byte lands on which element, and the
    scale that multiplies it, read off the block layouts without the index formulas."""
    d = np.array([0.5], np.float16)
    mn = np.array([0.25], np.float16)
    # Q4_1: byte 3 = 0xA7 -> element 3 = 7 d + m, element 19 = 10 d + m, the rest m
    blk = np.zeros(20, np.uint8)
    blk[0:2], blk[2:4], blk[4 + 3] = d.view(np.uint8), mn.view(np.uint8), 0xA7
    out = oracle.dequantize_gguf(oracle.Q4_1, blk, 1, 32)[0]
    want = np.full(32, 0.25, np.float32)
    want[3], want[19] = 3.75, 5.25
    np.testing.assert_array_equal(out, want)
    # Q5_0: only qh bit 5 and bit 21 set -> elements 5 and 21 are (16 - 16) d = 0, the rest -16 d
    blk = np.zeros(22, np.uint8)
    blk[0:2] = d.view(np.uint8)
    blk[2:6] = np.array([(1 << 5) | (1 << 21)], "<u4").view(np.uint8)
    out = oracle.dequantize_gguf(oracle.Q5_0, blk, 1, 32)[0]
    want = np.full(32, -8.0, np.float32)
    want[5] = want[21] = 0.0
    np.testing.assert_array_equal(out, want)
    # Q5_1: qh bit 31, qs[15] = 0xF0 -> element 31 = 31 d + m
    blk = np.zeros(24, np.uint8)
    blk[0:2], blk[2:4] = d.view(np.uint8), mn.view(np.uint8)
    blk[4:8] = np.array([1 << 31], "<u4").view(np.uint8)
    blk[8 + 15] = 0xF0
    out = oracle.dequantize_gguf(oracle.Q5_1, blk, 1, 32)[0]
    want = np.full(32, 0.25, np.float32)
    want[31] = 31 * 0.5 + 0.25
    np.testing.assert_array_equal(out, want)
    # Q2_K: scales[i] = (i << 4) | (15 - i): sub-block i of 16 elements has dl = d (15 - i),
    # ml = dmin i; all quants 3 (qs = 0xFF) -> 3 dl - ml
    blk = np.zeros(84, np.uint8)
    blk[0:16] = [(i << 4) | (15 - i) for i in range(16)]
    blk[16:80] = 0xFF
    blk[80:82], blk[82:84] = d.view(np.uint8), mn.view(np.uint8)
    out = oracle.dequantize_gguf(oracle.Q2_K, blk, 1, 256)[0]
    for j in range(256):
        i = j // 16
        assert out[j] == np.float32(3 * 0.5 * (15 - i) - 0.25 * i)
    # Q2_K bit placement: qs[32 + 16 + 2] = 0b01_00_10_11 -> elements 128 + 32 s + 18 = 3, 2, 0, 1
    blk[0:16] = 1  # dl = d, ml = 0
    blk[16:80] = 0
    blk[16 + 32 + 16 + 2] = 0b01001011
    out = oracle.dequantize_gguf(oracle.Q2_K, blk, 1, 256)[0]
    want = np.zeros(256, np.float32)
    want[[128 + 18, 160 + 18, 192 + 18, 224 + 18]] = [1.5, 1.0, 0.0, 0.5]
    np.testing.assert_array_equal(out, want)
    # Q3_K: all scale bits zero -> scale -32; hmask all ones, qs = 0 except one byte
    blk = np.zeros(110, np.uint8)
    blk[0:32] = 0xFF
    blk[32 + 32 + 7] = 0b11100100  # second half, element 7: q = 0, 1, 2, 3 at shifts 0, 2, 4, 6
    blk[108:110] = d.view(np.uint8)
    out = oracle.dequantize_gguf(oracle.Q3_K, blk, 1, 256)[0]
    want = np.zeros(256, np.float32)
    want[[128 + 7, 160 + 7, 192 + 7, 224 + 7]] = np.float32(-16.0) * np.array([0, 1, 2, 3], np.float32)
    np.testing.assert_array_equal(out, want)
    # Q3_K: hmask bit clear subtracts 4; six-bit scale assembled from its two places:
    # sub-block 9 (group 2, k 1): low nibble = scales[1] >> 4, high bits = (scales[9] >> 4) & 3
    blk = np.zeros(110, np.uint8)
    blk[96 + 1] = 0x50        # low nibble of sub-blocks 1 (0) and 9 (5)
    blk[96 + 8 + 1] = 0x20    # high bits of sub-block 9 = 2 -> scale = 5 + 32 - 32 = 5
    blk[108:110] = d.view(np.uint8)
    out = oracle.dequantize_gguf(oracle.Q3_K, blk, 1, 256)[0]
    np.testing.assert_array_equal(out[144:160], np.full(16, 0.5 * 5 * -4, np.float32))
    np.testing.assert_array_equal(out[16:32], np.full(16, 0.5 * -32 * -4, np.float32))
    # Q5_K: sc = j + 1 (j < 4), min = 0; qs = 0x21; qh = 0b0110: bit 1 and 2 set ->
    # sub-block 1 (high nibble 2) gets +16, sub-block 2 (low nibble 1) gets +16
    blk = np.zeros(176, np.uint8)
    blk[0:2], blk[2:4] = d.view(np.uint8), d.view(np.uint8)
    blk[4:8] = [1, 2, 3, 4]
    blk[16:48] = 0b0110
    blk[48:176] = 0x21
    out = oracle.dequantize_gguf(oracle.Q5_K, blk, 1, 256)[0]
    assert np.all(out[0:32] == 0.5 * 1 * 1) and np.all(out[32:64] == 0.5 * 2 * 18)
    assert np.all(out[64:96] == 0.5 * 3 * 17) and np.all(out[96:128] == 0.5 * 4 * 2)
    assert np.all(out[128:] == 0)


def test_gguf_size_checks():
    with pytest.raises(ValueError):
        oracle.dequantize_gguf(oracle.Q4_0, np.zeros(17, np.uint8), 1, 32)
    with pytest.raises(ValueError):
        oracle.dequantize_gguf(oracle.Q4_K, np.zeros(144, np.uint8), 1, 128)


# ------------------------------------------------------------------ matmul / MoE
def test_matmul_against_numpy_float64():
    rng = np.random.default_rng(5)
    x = rng.standard_normal((5, 300)).astype(np.float32)
    w = rng.standard_normal((17, 300)).astype(np.float32)
    b = rng.standard_normal(17).astype(np.float32)
    want = x.astype(np.float64) @ w.astype(np.float64).T + b
    np.testing.assert_allclose(oracle.matmul_nt_f32(x, w, b), want, rtol=1e-5, atol=1e-4)
    np.testing.assert_array_equal(oracle.matmul_nt_f64acc(x, w, b), want.astype(np.float32))
    # transposed-operand mistake would fail this non-square case
    assert oracle.matmul_nt_f32(x, w).shape == (5, 17)


def test_linear_from_awq_matches_dense():
    """linear.rs:688-787 shape: K=4, N=8, g=2, bias; y = x.W^T + b from the dequantized W."""
    K, N, g = 4, 8, 2
    rng = np.random.default_rng(3)
    q = rng.integers(0, 16, (K, N))
    z = rng.integers(0, 16, (K // g, N))
    s = rng.uniform(0.01, 0.1, (K // g, N)).astype(np.float32)
    bias = rng.standard_normal(N).astype(np.float32)
    x = rng.standard_normal((3, K)).astype(np.float32)
    w = oracle.dequantize_awq(synth.pack_awq(q), synth.pack_awq(z), s)
    dense = ((q - np.repeat(z, g, 0)).astype(np.float32) * np.repeat(s, g, 0)).T
    want = x.astype(np.float64) @ dense.astype(np.float64).T + bias
    np.testing.assert_allclose(oracle.matmul_nt_f32(x, w, bias), want, rtol=1e-5, atol=1e-5)


def test_moe_route_nan_row_keeps_index_order():
    """A row whose probabilities are all NaN has no order: numpy's stable argsort, like the oracle's stable
    insertion sort, leaves it as it is, so the chosen experts are 0..k-1 (in range) with NaN weights."""
    logits = np.random.default_rng(3).standard_normal((3, 16)).astype(np.float32)
    logits[1, 7] = np.nan
    idx, vals = oracle.moe_route(logits, 4, True)
    np.testing.assert_array_equal(idx[1], [0, 1, 2, 3])
    assert np.isnan(vals[1]).all() and not np.isnan(vals[[0, 2]]).any()
    offsets, tokens, _ = oracle.moe_group(idx, vals, 16)
    assert offsets[-1] == 12 and sorted(tokens.tolist()) == sorted([0, 1, 2] * 4)


def test_moe_route_matches_numpy():
    rng = np.random.default_rng(7)
    logits = rng.standard_normal((8, 32)).astype(np.float32)
    idx, vals = oracle.moe_route(logits, 4, True)
    p = np.exp(logits - logits.max(1, keepdims=True))
    p /= p.sum(1, keepdims=True)
    order = np.argsort(-p, axis=1, kind="stable")[:, :4]
    np.testing.assert_array_equal(idx, order.astype(np.uint32))
    tv = np.take_along_axis(p, order, 1)
    np.testing.assert_allclose(vals, tv / tv.sum(1, keepdims=True), rtol=1e-5)
    np.testing.assert_allclose(vals.sum(1), 1.0, rtol=1e-5)
    _, raw = oracle.moe_route(logits, 4, False)
    np.testing.assert_allclose(raw, tv, rtol=1e-5)
    offsets, tokens, weights = oracle.moe_group(idx, vals, 32)
    assert offsets[-1] == 32 and offsets[0] == 0
    for e in range(32):
        toks = tokens[offsets[e]:offsets[e + 1]]
        want = [t for t in range(8) if e in idx[t]]
        assert list(toks) == want  # token-major order, like dispatch_sparse
        for t, w_ in zip(toks, weights[offsets[e]:offsets[e + 1]]):
            assert w_ == vals[t, list(idx[t]).index(e)]


def test_gpt_oss_expert_scalar_reference():
    """moe.rs:705-788 gpt_oss_expert_matches_scalar_reference (tol 1e-3*max + 1e-3)."""
    hidden = inter = 32
    limit = np.float32(7.0)
    gu_out, nb = 2 * inter, 1
    gu_blocks = ((np.arange(gu_out * nb * 16) * 23 + 7) & 0xFF).astype(np.uint8)
    gu_scales = (125 + np.arange(gu_out * nb) % 5).astype(np.uint8)
    dn_blocks = ((np.arange(hidden * nb * 16) * 41 + 3) & 0xFF).astype(np.uint8)
    dn_scales = (126 + np.arange(hidden * nb) % 3).astype(np.uint8)
    gu_bias = (np.sin(np.arange(gu_out, dtype=np.float32) * np.float32(0.7)) * 2).astype(np.float32)
    dn_bias = (np.cos(np.arange(hidden, dtype=np.float32) * np.float32(0.3)) * 0.5).astype(np.float32)
    x = (np.sin(np.arange(hidden, dtype=np.float32) * np.float32(0.21)) * 3).astype(np.float32)

    # oracle path: dequant + matmul + swiglu + matmul
    w_gu = oracle.dequantize_mxfp4_f32(gu_blocks, gu_scales, gu_out, hidden)
    w_dn = oracle.dequantize_mxfp4_f32(dn_blocks, dn_scales, hidden, inter)
    gu = oracle.matmul_nt_f32(x[None, :], w_gu, gu_bias)
    h = oracle.gpt_oss_swiglu(gu, float(limit))
    y = oracle.matmul_nt_f32(h, w_dn, dn_bias)[0]

    # independent scalar reference written from the MX spec tables
    lut = [0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0]

    def deq(blocks, scales, rows, cols):
        w = np.zeros((rows, cols))
        for r in range(rows):
            for b in range(cols // 32):
                sc = 2.0 ** (int(scales[r * (cols // 32) + b]) - 127)
                for i in range(16):
                    byte = int(blocks[(r * (cols // 32) + b) * 16 + i])
                    for half, code in enumerate((byte & 0xF, byte >> 4)):
                        v = lut[code & 7] * (-1 if code & 8 else 1)
                        w[r, b * 32 + 2 * i + half] = v * sc
        return w

    wg, wd = deq(gu_blocks, gu_scales, gu_out, hidden), deq(dn_blocks, dn_scales, hidden, inter)
    gate_up = gu_bias + wg @ x
    hh = np.zeros(inter)
    for k in range(inter):
        gate = min(gate_up[2 * k], 7.0)
        up = min(max(gate_up[2 * k + 1], -7.0), 7.0)
        hh[k] = (up + 1.0) * gate * (1.0 / (1.0 + np.exp(-gate * 1.702)))
    expected = dn_bias + wd @ hh
    tol = 1e-3 * np.max(np.abs(expected)) + 1e-3
    assert np.max(np.abs(y - expected)) < tol


def test_gated_activations_match_scipy_and_closed_forms():
    """ffn_kernels.metal:5-17: silu(x) = x / (1 + e^-x); gelu_tanh as the tanh approximation.
    Checked against scipy's expit / numpy tanh in float64 and on closed forms."""
    from scipy.special import expit
    rng = np.random.default_rng(11)
    gu = (rng.standard_normal((5, 64)) * 4).astype(np.float32)
    g, u = gu[:, :32].astype(np.float64), gu[:, 32:].astype(np.float64)
    np.testing.assert_allclose(oracle.gated_silu(gu), g * expit(g) * u, rtol=2e-6, atol=1e-6)
    gel = 0.5 * g * (1 + np.tanh(0.7978845608028654 * (g + 0.044715 * g ** 3)))
    np.testing.assert_allclose(oracle.gated_gelu_tanh(gu), gel * u, rtol=2e-6, atol=1e-6)
    # closed forms: act(0) = 0; large positive gate -> gate * up; large negative -> 0
    probe = np.array([[0.0, 30.0, -30.0, 1.0, 2.0, 3.0, 4.0, 5.0]], np.float32)  # 4 gates | 4 ups
    for fn in (oracle.gated_silu, oracle.gated_gelu_tanh):
        out = fn(probe)[0]
        assert out[0] == 0.0
        np.testing.assert_allclose(out[1], 30.0 * 3.0, rtol=1e-6)
        assert abs(out[2]) < 1e-6


def test_moe_combine_matches_dense_gate_matrix():
    """moe.rs:592-605 restated: the scatter equals out = G . expert_out with the dense
    [n_tokens, n_pairs] gate matrix (a plain matmul, computed in float64)."""
    rng = np.random.default_rng(12)
    T, E, k, H = 9, 16, 3, 24
    idx, vals = oracle.moe_route(rng.standard_normal((T, E)).astype(np.float32), k, True)
    offsets, tokens, weights = oracle.moe_group(idx, vals, E)
    eo = rng.standard_normal((T * k, H)).astype(np.float32)
    G = np.zeros((T, T * k))
    for p_, (t, w_) in enumerate(zip(tokens, weights)):
        G[t, p_] += w_
    np.testing.assert_allclose(oracle.moe_combine(eo, offsets, tokens, weights, T), G @ eo.astype(np.float64),
                               rtol=1e-5, atol=1e-6)
