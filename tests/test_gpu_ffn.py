"""The gated MLP around the quantized projections (ffn.rs:22-474): every gate/up layout against the
layers' own forwards bit for bit and against the oracle chain, built from arrays and from files."""
import numpy as np
import pytest
import torch

import oracle
from oxydllm_amd import checkpoint as ck
from oxydllm_amd import ops, synth
from tests import ggufio as G
from tests.helpers import as_f32, bits_of, round_x, to_dev

pytestmark = pytest.mark.gpu

ODT = {torch.float16: oracle.F16, torch.bfloat16: oracle.BF16}
ACTS = {ops.ACT_GATED_SILU: oracle.gated_silu, ops.ACT_GATED_GELU_TANH: oracle.gated_gelu_tanh}


def say(msg):
    print(f"[ffn] {msg}", flush=True)


def _x(m, k, seed=0):
    return np.random.default_rng(seed).standard_normal((m, k)).astype(np.float32)


def oracle_ffn(x, w_gate, w_up, w_down, act, dt):
    """down(act(gate(x)) * up(x)) with every layer output rounded to the layer dtype, as the reference's
    tensors are between its ops.  Weights are dense [out, in] f32; w_gate None = the ungated layout."""
    r = lambda a: oracle.round_through(a, dt) if dt is not None else a
    xr = r(x)
    up = r(oracle.matmul_nt_f32(xr, w_up))
    if w_gate is None:
        g = up.astype(np.float64)
        a = g / (1.0 + np.exp(-g)) if act == ops.ACT_GATED_SILU else \
            0.5 * g * (1.0 + np.tanh(0.7978845608028654 * (g + 0.044715 * g ** 3)))
        h = r(a.astype(np.float32))
    else:
        gate = r(oracle.matmul_nt_f32(xr, w_gate))
        h = r(ACTS[act](np.concatenate([gate, up], axis=-1)))
    return oracle.matmul_nt_f32(h, w_down)


def close_to_chain(y, ref, what):
    """Three roundings to 16 bits sit between x and y, and a rounding that falls the other way in one
    intermediate moves y by up to an ulp of that intermediate times a weight: the bound is a fraction of
    the output's scale, not of each element."""
    got = as_f32(y)
    scale = np.abs(ref).max() + 1e-6
    err = np.abs(got - ref).max()
    assert err <= 2e-2 * scale, f"{what}: max err {err} vs scale {scale}"


def awq_parts(K, N, g, bits, seed, dt):
    qw, qz, sc = synth.awq_checkpoint(K, N, g, bits, seed=seed)
    s_r = oracle.round_through(sc, ODT[dt])
    dense = oracle.dequantize_awq(qw, qz, s_r) if bits == 4 else oracle.dequantize_awq8(qw, qz, s_r)     # [N, K]
    return (qw, qz, sc), dense


def gptq_parts(K, N, g, bits, seed, dt):
    qw, qz, sc = synth.gptq_checkpoint(K, N, g, bits, seed=seed)
    dense = oracle.dequantize_gptq(qw, qz, oracle.round_through(sc, ODT[dt]), bits)
    return (qw, qz, sc), dense


def packed_layer(raw, bits, pack_dim, dt, act=None):
    qw, qz, sc = raw
    return ops.PackedQuantLinear(bits, pack_dim, to_dev(qw), to_dev(qz), to_dev(sc, dt), None, dt, gate_up_act=act)


@pytest.mark.parametrize("dt", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("act", [ops.ACT_GATED_SILU, ops.ACT_GATED_GELU_TANH])
@pytest.mark.parametrize("method, g", [("awq", 128), ("gptq", 128), ("awq", 64)])
def test_every_gate_up_layout_of_the_packed_quant_mlp(method, g, act, dt):
    """g = 128 layers keep a tile-major copy (the fused projection then carries the activation in its
    matmul); g = 64 layers run on the checkpoint layout.  All layouts must agree with the composition of the
    layers' own forwards bit for bit, since they launch the same kernels."""
    say(f"layouts {method} g={g} act={act} {dt}")
    H, I, bits = 256, 384, 4
    parts = awq_parts if method == "awq" else gptq_parts
    pack_dim = ops.PACK_OUT if method == "awq" else ops.PACK_IN
    gate_raw, w_gate = parts(H, I, g, bits, 1, dt)
    up_raw, w_up = parts(H, I, g, bits, 2, dt)
    down_raw, w_down = parts(I, H, g, bits, 3, dt)
    both_raw = tuple(np.concatenate([a, b], axis=1) for a, b in zip(gate_raw, up_raw))
    if method == "awq":
        want = oracle.concat_awq_along_out([gate_raw, up_raw])
        for a, b in zip(both_raw, want):
            np.testing.assert_array_equal(a, b)
    mk = lambda raw, a=None: packed_layer(raw, bits, pack_dim, dt, a)
    gate, up, down, both = mk(gate_raw), mk(up_raw), mk(down_raw), mk(both_raw)
    assert down.prepacked == (g == 128)
    for m in (1, 5, 16, 40):
        x = to_dev(_x(m, H, seed=m), dt)
        ref = oracle_ffn(_x(m, H, seed=m), w_gate, w_up, w_down, act, ODT[dt])
        # separate
        ff = ops.FeedForward(ops.GATE_UP_SEPARATE, gate, up, down, I, act)
        assert (ff.in_features, ff.out_features) == (H, H) and ff.scratch_elems(m) == 2 * m * I
        y = ff.forward(x)
        two = down.forward(ops.activation_mul(gate.forward(x), up.forward(x), act))
        np.testing.assert_array_equal(bits_of(y), bits_of(two))
        close_to_chain(y, ref, f"separate m={m}")
        # fused, activation as a second launch
        ff = ops.FeedForward(ops.GATE_UP_FUSED, both, None, down, I, act)
        assert ff.scratch_elems(m) == 3 * m * I
        y = ff.forward(x)
        two = down.forward(ops.gated_activation(both.forward(x), act))
        np.testing.assert_array_equal(bits_of(y), bits_of(two))
        close_to_chain(y, ref, f"fused m={m}")
        # fused, activation in the matmul
        if g == 128:
            epi = mk(both_raw, act)
            ff = ops.FeedForward(ops.GATE_UP_FUSED, epi, None, down, I, act)
            assert ff.scratch_elems(m) == m * I
            np.testing.assert_array_equal(bits_of(ff.forward(x)), bits_of(two))
        # ungated
        ff = ops.FeedForward(ops.GATE_UP_SIMPLE, up, None, down, I, act)
        y = ff.forward(x.reshape(1, m, H))
        assert y.shape == (1, m, H)
        close_to_chain(y, oracle_ffn(_x(m, H, seed=m), None, w_up, w_down, act, ODT[dt]), f"simple m={m}")
    if g != 128:
        with pytest.raises(ops.OxqError, match="UNSUPPORTED"):
            mk(both_raw, act)


def test_feed_forward_refusals():
    say("refusals")
    dt, H, I = torch.float16, 256, 384
    gate = packed_layer(awq_parts(H, I, 128, 4, 1, dt)[0], 4, ops.PACK_OUT, dt)
    both_raw = awq_parts(H, 2 * I, 128, 4, 2, dt)[0]
    both = packed_layer(both_raw, 4, ops.PACK_OUT, dt)
    epi = packed_layer(both_raw, 4, ops.PACK_OUT, dt, ops.ACT_GATED_SILU)
    down = packed_layer(awq_parts(I, H, 128, 4, 3, dt)[0], 4, ops.PACK_OUT, dt)
    F = ops.FeedForward
    with pytest.raises(ops.OxqError, match="gate/up out_features must both be"):
        F(ops.GATE_UP_SEPARATE, gate, both, down, I)
    with pytest.raises(ops.OxqError, match="gate_up out_features 384 != 2\\*384"):
        F(ops.GATE_UP_FUSED, gate, None, down, I)
    with pytest.raises(ops.OxqError, match="down_proj in_features 256 != intermediate size 384"):
        F(ops.GATE_UP_SEPARATE, gate, gate, gate, I)
    with pytest.raises(ops.OxqError, match="second projection"):
        F(ops.GATE_UP_FUSED, both, gate, down, I)
    with pytest.raises(ops.OxqError, match="second projection"):
        F(ops.GATE_UP_SEPARATE, gate, None, down, I)
    with pytest.raises(ops.OxqError, match="another activation"):
        F(ops.GATE_UP_FUSED, epi, None, down, I, ops.ACT_GATED_GELU_TANH)
    with pytest.raises(ops.OxqError, match="only be the fused gate_up_proj"):
        F(ops.GATE_UP_SIMPLE, epi, None, down, I)
    with pytest.raises(ops.OxqError, match="down_proj cannot carry"):
        F(ops.GATE_UP_SEPARATE, gate, gate, epi, I)
    with pytest.raises(ops.OxqError, match="activation must be"):
        F(ops.GATE_UP_FUSED, both, None, down, I, ops.ACT_GPT_OSS_SWIGLU)
    with pytest.raises(ops.OxqError, match="unknown gate/up layout"):
        F(7, both, None, down, I)
    ff = F(ops.GATE_UP_FUSED, both, None, down, I)
    x = to_dev(_x(3, H), dt)
    with pytest.raises(ops.OxqError, match="scratch must be a contiguous F16 tensor of at least 3456"):
        ff.forward(x, scratch=torch.empty(3455, dtype=dt, device="cuda"))
    with pytest.raises(ops.OxqError, match="scratch must be"):
        ff.forward(x, scratch=torch.empty(4000, dtype=torch.bfloat16, device="cuda"))
    with pytest.raises(ops.OxqError, match="in_features"):
        ff.forward(to_dev(_x(3, H + 8), dt))


@pytest.mark.parametrize("method", ["awq", "gptq"])
@pytest.mark.parametrize("layout", ["gate+up", "gate_up", "up"])
def test_packed_quant_mlp_from_safetensors(tmp_path, method, layout):
    """ffn.rs:62-68, 200-285: the loader picks the layout from the tensors present; separate gate and up
    tensors are joined into one projection that carries the activation."""
    from safetensors.numpy import save_file
    say(f"safetensors mlp {method} {layout}")
    dt, H, I, g, bits = torch.float16, 256, 384, 128, 4
    parts = awq_parts if method == "awq" else gptq_parts
    gate_raw, w_gate = parts(H, I, g, bits, 1, dt)
    up_raw, w_up = parts(H, I, g, bits, 2, dt)
    down_raw, w_down = parts(I, H, g, bits, 3, dt)
    p = "model.layers.3.mlp"
    tensors = {}

    def put(name, raw):
        for field, a in zip(("qweight", "qzeros", "scales"), raw):
            tensors[f"{p}.{name}.{field}"] = a.astype(np.float16) if field == "scales" else a

    put("down_proj", down_raw)
    if layout == "gate+up":
        put("gate_proj", gate_raw)
        put("up_proj", up_raw)
    elif layout == "gate_up":
        put("gate_up_proj", tuple(np.concatenate([a, b], axis=1) for a, b in zip(gate_raw, up_raw)))
    else:
        put("up_proj", up_raw)
    path = str(tmp_path / "model.safetensors")
    save_file(tensors, path)
    scheme = ck.validate_quantization_config({"quant_method": method, "bits": bits, "group_size": g, "sym": False})
    with ck.ModelWeights.load([path]).with_quant_scheme(scheme) as w:
        ff = w.feed_forward(3, ops.ACT_GATED_SILU, dtype=dt)
        assert ff.intermediate_size == I and (ff.in_features, ff.out_features) == (H, H)
        if layout == "up":
            assert ff.gate_up_kind == ops.GATE_UP_SIMPLE
        else:
            assert ff.gate_up_kind == ops.GATE_UP_FUSED and ff.scratch_elems(2) == 2 * I   # activation in the matmul
        for m in (1, 12, 33):
            x = _x(m, H, seed=m)
            ref = oracle_ffn(x, None if layout == "up" else w_gate, w_up, w_down, ops.ACT_GATED_SILU, oracle.F16)
            close_to_chain(ff.forward(to_dev(x, dt)), ref, f"{method} {layout} m={m}")
        with pytest.raises(KeyError):
            w.feed_forward(4)
    # down_proj packed, nothing else: the mixed-quantization refusal
    save_file({k: v for k, v in tensors.items() if ".down_proj." in k}, path)
    with ck.ModelWeights.load([path]).with_quant_scheme(scheme) as w:
        with pytest.raises(ck.OxqError, match="Mixed quantization"):
            w.feed_forward(3)


@pytest.mark.parametrize("layout", ["separate", "packed", "simple"])
def test_gguf_mlp_from_file(tmp_path, layout):
    """ffn.rs:307-373: blk.{i}.ffn_* kept block-quantized; benchmark config 3's layer at test size."""
    say(f"gguf mlp {layout}")
    H, I = 256, 512
    fg, fu, fd = synth.GGUF_Q4_K, synth.GGUF_Q4_K, synth.GGUF_Q6_K
    gate = synth.gguf_weight(fg, I, H, seed=1)
    up = synth.gguf_weight(fu, I, H, seed=2)
    down = synth.gguf_weight(fd, H, I, seed=3)
    w_gate, w_up, w_down = (oracle.dequantize_gguf(f, b, n, k) for f, b, n, k in
                            ((fg, gate, I, H), (fu, up, I, H), (fd, down, H, I)))
    tensors = [("blk.0.ffn_down.weight", (H, I), G.GGML_OF_QUANT[fd], down.tobytes())]
    if layout == "separate":
        tensors += [("blk.0.ffn_gate.weight", (I, H), G.GGML_OF_QUANT[fg], gate.tobytes()),
                    ("blk.0.ffn_up.weight", (I, H), G.GGML_OF_QUANT[fu], up.tobytes())]
    elif layout == "packed":    # rows of gate, then rows of up, in one tensor
        tensors += [("blk.0.ffn_up.weight", (2 * I, H), G.GGML_OF_QUANT[fu], gate.tobytes() + up.tobytes())]
    else:
        tensors += [("blk.0.ffn_up.weight", (I, H), G.GGML_OF_QUANT[fu], up.tobytes())]
    path = str(tmp_path / "m.gguf")
    G.write_gguf(path, [("general.architecture", G.STRING, "llama")], tensors)
    with ck.GgufWeights.load(path) as w:
        ff = w.feed_forward(0, I, ops.ACT_GATED_SILU)
        # gate and up of one format with the matrix-core copy: fused into one projection by default
        assert ff.gate_up_kind == {"separate": ops.GATE_UP_FUSED, "packed": ops.GATE_UP_FUSED,
                                   "simple": ops.GATE_UP_SIMPLE}[layout]
        assert w.feed_forward(0, I, ops.ACT_GATED_SILU, fuse=False).gate_up_kind == {
            "separate": ops.GATE_UP_SEPARATE, "packed": ops.GATE_UP_FUSED, "simple": ops.GATE_UP_SIMPLE}[layout]
        for m in (1, 6):    # the decode kernels multiply the unrounded dequantized weights
            x = _x(m, H, seed=m)
            ref = oracle_ffn(x, None if layout == "simple" else w_gate, w_up, w_down, ops.ACT_GATED_SILU, oracle.BF16)
            close_to_chain(ff.forward(to_dev(x, torch.bfloat16)), ref, f"gguf {layout} m={m}")
        with pytest.raises(ck.OxqError, match="ffn_down shape mismatch"):
            w.feed_forward(0, I + 32)
        if layout == "separate":
            r = lambda a: oracle.round_through(a, oracle.BF16)
            x = _x(24, H, seed=24)    # the tile kernel multiplies weights rounded to bf16
            ref = oracle_ffn(x, r(w_gate), r(w_up), r(w_down), ops.ACT_GATED_SILU, oracle.BF16)
            close_to_chain(ff.forward(to_dev(x, torch.bfloat16)), ref, "gguf separate m=24")
