"""Checkpoint file -> resident layer -> forward, against the oracle on the same bytes.

The files are written by independent code (the `safetensors` package, the tests' GGUF writer);
the layers are the ones the other parity tests build from in-memory arrays, so these tests cover
the path in between: index, name resolution, upload, device-side transforms.
"""
import numpy as np
import pytest
import torch

import oracle
from oxydllm_amd import checkpoint as ck
from oxydllm_amd import ops, synth
from tests import ggufio as G
from tests import refgen
from tests.helpers import as_f32, assert_close, gguf_on_matrix_cores, round_x, to_dev, resident_rounds_weights

pytestmark = pytest.mark.gpu


def _x(m, k, seed=0):
    return np.random.default_rng(seed).standard_normal((m, k)).astype(np.float32)


def test_gguf_file_to_qlinear(tmp_path):
    shapes = {"blk.0.ffn_up.weight": (synth.GGUF_Q4_K, 96, 512), "blk.0.ffn_down.weight": (synth.GGUF_Q6_K, 64, 256),
              "blk.0.attn_v.weight": (synth.GGUF_Q8_0, 40, 160), "blk.0.attn_q.weight": (synth.GGUF_Q5_0, 64, 96)}
    data = {n: synth.gguf_weight(f, N, K, seed=i) for i, (n, (f, N, K)) in enumerate(shapes.items())}
    path = str(tmp_path / "model.gguf")
    G.write_gguf(path, [("general.architecture", G.STRING, "llama")],
                 [(n, (N, K), G.GGML_OF_QUANT[f], data[n].tobytes()) for n, (f, N, K) in shapes.items()])
    with ck.GgufWeights.load(path) as w:
        for name, (fmt, N, K) in shapes.items():
            layer = w.qlinear(name)
            for m in (1, 5, 24):
                x = _x(m, K, seed=m)
                y = layer.forward(to_dev(x, torch.bfloat16))
                wt = oracle.dequantize_gguf(fmt, data[name], N, K)
                unrounded = m <= 8 or gguf_on_matrix_cores(fmt, N, K, m)
                ref = oracle.matmul_nt_f32(round_x(x, oracle.BF16), wt if unrounded else oracle.round_through(wt, oracle.BF16))
                assert_close(y, ref, f"{name} m={m}", bf16_out=True)
        # q projection with the converter's row interleave undone on the device
        fmt, N, K = shapes["blk.0.attn_q.weight"]
        n_heads, head_dim = 4, 16
        layer = w.qlinear("blk.0.attn_q.weight", depermute=(n_heads, head_dim))
        _, bbytes = synth.GGUF_BLOCK_LAYOUT[fmt]
        fixed = oracle.gguf_depermute_qk_rows(data["blk.0.attn_q.weight"], K // 32 * bbytes, n_heads, head_dim)
        x = _x(3, K, seed=9)
        y = layer.forward(to_dev(x, torch.bfloat16))
        ref = oracle.matmul_nt_f32(round_x(x, oracle.BF16), oracle.dequantize_gguf(fmt, fixed, N, K))
        assert_close(y, ref, "depermuted q", bf16_out=True)
        # the uploaded bytes are the file's bytes
        up = w.get("blk.0.ffn_up.weight").to_device()
        np.testing.assert_array_equal(up.cpu().numpy(), data["blk.0.ffn_up.weight"])
        with pytest.raises(ck.OxqError):
            G.write_gguf(str(tmp_path / "f.gguf"), [], [("dense", (4, 4), 0, b"\0" * 64)])
            with ck.GgufWeights.load(str(tmp_path / "f.gguf")) as d:
                d.qlinear("dense")


@pytest.mark.parametrize("layout", ["separate", "packed"])
def test_gguf_file_to_feed_forward_fuses_gate_and_up(tmp_path, layout):
    """ffn.rs:307-373 FeedForward::load_gguf.  With fuse (the default) a bf16 layer of a format with the matrix-core
    copy becomes one gate|up projection with the activation in its epilogue - separate ffn_gate / ffn_up tensors by
    concatenating their bytes - and gives the bits of the layer built the reference's way; a format without that
    copy keeps its layout."""
    from oxydllm_amd import ops
    H, I = 512, 256
    for fmt, fusable in [(synth.GGUF_Q4_K, True), (synth.GGUF_Q5_0, True), (synth.GGUF_Q2_K, False)]:
        gate, up = synth.gguf_weight(fmt, I, H, seed=1), synth.gguf_weight(fmt, I, H, seed=2)
        down = synth.gguf_weight(fmt, H, I, seed=3)
        G_ = G.GGML_OF_QUANT[fmt]
        if layout == "separate":
            tensors = [("blk.0.ffn_gate.weight", (I, H), G_, gate.tobytes()), ("blk.0.ffn_up.weight", (I, H), G_, up.tobytes())]
        else:
            tensors = [("blk.0.ffn_up.weight", (2 * I, H), G_, gate.tobytes() + up.tobytes())]
        tensors.append(("blk.0.ffn_down.weight", (H, I), G_, down.tobytes()))
        path = str(tmp_path / f"ffn_{fmt}.gguf")
        G.write_gguf(path, [("general.architecture", G.STRING, "llama")], tensors)
        with ck.GgufWeights.load(path) as w:
            ff = w.feed_forward(0, I)
            ref = w.feed_forward(0, I, fuse=False)
            assert ref.gate_up_kind == (ops.GATE_UP_SEPARATE if layout == "separate" else ops.GATE_UP_FUSED)
            assert ff.gate_up_kind == (ops.GATE_UP_FUSED if fusable else ref.gate_up_kind)
            for m in (1, 8, 40):
                x = to_dev(_x(m, H, seed=m) * 0.25, torch.bfloat16)
                y = ff.forward(x)
                np.testing.assert_array_equal(y.view(torch.int16).cpu().numpy(), ref.forward(x).view(torch.int16).cpu().numpy())
            if fusable:
                a = ff._keep[0]
                a.forward(to_dev(_x(2, H, seed=5), torch.bfloat16))
                assert ops.default_context().last_plan()["kernel"].endswith("_act")


@pytest.mark.parametrize("method, bits", [("awq", 4), ("awq", 8), ("gptq", 4), ("gptq", 8)])
def test_safetensors_file_to_packed_linear(tmp_path, method, bits):
    from safetensors.numpy import save_file
    K, N, g = 512, 256, 128
    make = synth.awq_checkpoint if method == "awq" else synth.gptq_checkpoint
    qw, qz, sc = make(K, N, g, bits, seed=bits)
    bias = np.random.default_rng(1).standard_normal(N).astype(np.float16)
    prefix = "model.language_model.layers.0.mlp.gate_proj"      # multimodal nesting, asked for by canonical name
    path = str(tmp_path / "model.safetensors")
    save_file({f"{prefix}.qweight": qw, f"{prefix}.qzeros": qz, f"{prefix}.scales": sc.astype(np.float16),
               f"{prefix}.bias": bias}, path)
    cfg = {"quant_method": method, "bits": bits, "group_size": g, "sym": False}
    scheme = ck.validate_quantization_config(cfg)
    with ck.ModelWeights.load([path]).with_quant_scheme(scheme) as w:
        layer = w.packed_linear("model.layers.0.mlp.gate_proj", dtype=torch.float16)
        assert (layer.in_features, layer.out_features) == (K, N)
        s_r = oracle.round_through(sc, oracle.F16)
        if method == "gptq":
            wt = oracle.dequantize_gptq(qw, qz, s_r, bits)
        else:
            wt = oracle.dequantize_awq(qw, qz, s_r) if bits == 4 else oracle.dequantize_awq8(qw, qz, s_r)
        for m in (1, 7, 40):
            x = _x(m, K, seed=m)
            y = layer.forward(to_dev(x, torch.float16))
            wr = oracle.round_through(wt, oracle.F16) if resident_rounds_weights(m, oracle.F16, method == "gptq") else wt
            ref = oracle.matmul_nt_f32(round_x(x, oracle.F16), wr, bias.astype(np.float32))
            assert_close(y, ref, f"{method}{bits} m={m}")
        assert w.try_get_quant("model.layers.1.mlp.gate_proj") is None


def test_compressed_tensors_file_to_packed_linear(tmp_path):
    from safetensors.numpy import save_file
    out_f, in_f, group = 128, 256, 128
    q, scale, packed = refgen.compressed_tensors_case(out_f, in_f, group)
    path = str(tmp_path / "ct.safetensors")
    save_file({"p.weight_packed": packed, "p.weight_scale": scale.astype(np.float16),
               "p.weight_shape": np.array([out_f, in_f], np.int64)}, path)
    scheme = ck.validate_quantization_config({
        "quant_method": "compressed-tensors", "format": "pack-quantized",
        "config_groups": {"group_0": {"weights": {"num_bits": 4, "symmetric": True, "type": "int", "strategy": "group"}}}})
    with ck.ModelWeights.load([path]).with_quant_scheme(scheme) as w:
        raw = w.try_get_quant("p")
        assert raw.bits == 4 and raw.pack_dim == ops.PACK_OUT
        want = oracle.compressed_to_awq(packed, scale.astype(np.float16))
        for got, exp in zip((raw.qweight, raw.qzeros), want[:2]):
            np.testing.assert_array_equal(got.cpu().numpy().view(np.uint32), np.asarray(exp).view(np.uint32))
        layer = w.packed_linear("p", dtype=torch.float16)
        s16 = oracle.round_through(scale, oracle.F16)
        wt = (q.astype(np.float32) * np.repeat(s16, group, axis=1))          # [out, in]
        x = _x(4, in_f)
        y = layer.forward(to_dev(x, torch.float16))
        assert_close(y, oracle.matmul_nt_f32(round_x(x, oracle.F16), wt), "compressed-tensors")


def test_stacked_mxfp4_experts_from_file(tmp_path):
    from safetensors.torch import save_file
    E, inter, hidden = 4, 64, 128
    rng = np.random.default_rng(5)
    tensors, ref = {}, {}
    for proj, (n, k) in {"gate_up_proj": (2 * inter, hidden), "down_proj": (hidden, inter)}.items():
        bl, sc = zip(*(synth.mxfp4_weight(n, k, seed=10 * e + len(proj)) for e in range(E)))
        blocks = np.stack(bl).reshape(E, n, k // 32, 16)
        scales = np.stack(sc).reshape(E, n, k // 32)
        bias = rng.standard_normal((E, n)).astype(np.float32)
        tensors[f"model.layers.0.mlp.experts.{proj}_blocks"] = torch.from_numpy(blocks)
        tensors[f"model.layers.0.mlp.experts.{proj}_scales"] = torch.from_numpy(scales)
        tensors[f"model.layers.0.mlp.experts.{proj}_bias"] = torch.from_numpy(bias).to(torch.bfloat16)
        ref[proj] = (blocks, scales, round_x(bias, oracle.BF16), n, k)
    path = str(tmp_path / "moe.safetensors")
    save_file(tensors, path)
    with ck.ModelWeights.load([path]) as w:
        ex = w.mxfp4_experts("model.layers.0.mlp")
        assert ex["num_experts"] == E
        for proj, (blocks, scales, bias, n, k) in ref.items():
            p = ex[proj]
            assert (p["out_features"], p["in_features"]) == (n, k)
            # pairs: expert 0 gets rows 0-1, expert 2 gets row 2, experts 1 and 3 none
            offsets = to_dev(np.array([0, 2, 2, 3, 3], np.int32))
            x = _x(3, k, seed=k)
            y = ops.mxfp4_moe_matmul(to_dev(x, torch.bfloat16), p["blocks"], p["scales"], p["bias"], offsets, None, k, n)
            xr = round_x(x, oracle.BF16)
            for row, e in ((0, 0), (1, 0), (2, 2)):
                wt = oracle.dequantize_mxfp4_f32(blocks[e].reshape(-1), scales[e].reshape(-1), n, k)
                assert_close(y[row:row + 1], oracle.matmul_nt_f32(xr[row:row + 1], wt, bias[e]), f"{proj} expert {e}")
        # a blocks tensor of the wrong rank is refused as moe.rs:405-414 refuses it
        bad = dict(tensors)
        bad["model.layers.0.mlp.experts.down_proj_blocks"] = torch.zeros(4, 8, 16, dtype=torch.uint8)
        save_file(bad, str(tmp_path / "bad.safetensors"))
        with ck.ModelWeights.load([str(tmp_path / "bad.safetensors")]) as b:
            with pytest.raises(ck.OxqError):
                b.mxfp4_experts("model.layers.0.mlp")
