"""GGUF / safetensors indexes and the quantization-config rules, on the host (no GPU).

Pins: files written by independent code (the `safetensors` package; a GGUF writer that follows the
published container layout), the reference's own size tests (weights.rs:659-697), and the branch
table of hf_parser.rs:451-585 (fp8 -> no scheme is the reference's own test, hf_parser.rs:765-775).
"""
import json
import struct

import numpy as np
import pytest

from oxydllm_amd import checkpoint as ck
from oxydllm_amd import synth
from oxydllm_amd._lib import OxqError
from tests import ggufio as G


def _status(exc):
    return exc.value.status


# ------------------------------------------------------------------------------------------ GGUF
def _sample_tensors(rng):
    q4k = synth.gguf_weight(synth.GGUF_Q4_K, 6, 512, seed=1).tobytes()
    q80 = synth.gguf_weight(synth.GGUF_Q8_0, 5, 96, seed=2).tobytes()
    f32 = rng.standard_normal((3, 7)).astype(np.float32)
    f16 = rng.standard_normal((4,)).astype(np.float16)
    bf16 = rng.integers(0, 65536, size=(2, 3, 4), dtype=np.uint16)
    return [("blk.0.attn_q.weight", (6, 512), 12, q4k), ("blk.0.ffn_down.weight", (5, 96), 8, q80),
            ("output_norm.weight", (3, 7), 0, f32.tobytes()), ("a.f16", (4,), 1, f16.tobytes()),
            ("z.bf16", (2, 3, 4), 30, bf16.tobytes())], f32, f16, bf16


META = [("general.architecture", G.STRING, "llama"), ("general.alignment", G.U32, 64),
        ("llama.block_count", G.U32, 32), ("llama.rope.freq_base", G.F32, 500000.0),
        ("llama.attention.head_count", G.U64, 32), ("some.i8", G.I8, -5), ("some.bool", G.BOOL, 1),
        ("some.f64", G.F64, 2.5), ("some.i32", G.I32, 7),
        ("tokenizer.ggml.tokens", G.ARRAY, (G.STRING, ["<s>", "</s>", "héllo", ""])),
        ("tokenizer.ggml.scores", G.ARRAY, (G.F32, [0.0, -1.5, 2.0])),
        ("nested", G.ARRAY, (G.ARRAY, [(G.U16, [1, 2]), (G.U16, [])])),
        ("tokenizer.ggml.eos_token_id", G.U32, 2),
        ("tokenizer.ggml.eos_token_ids", G.ARRAY, (G.U32, [2, 7, 7, 9]))]


@pytest.mark.parametrize("version", [1, 2, 3])
def test_gguf_index_and_metadata(tmp_path, version):
    rng = np.random.default_rng(0)
    tensors, f32, f16, bf16 = _sample_tensors(rng)
    path = str(tmp_path / "m.gguf")
    G.write_gguf(path, META, tensors, version=version, alignment=64)
    with ck.GgufWeights.load(path) as w:
        assert len(w) == 5
        assert w.names() == sorted(t[0] for t in tensors)
        for name, dims, gtype, payload in tensors:
            t = w.get(name)
            assert t.shape == tuple(dims) and t.ggml_type == gtype and t.nbytes == len(payload)
            assert t.numpy().tobytes() == payload
        q = w.get("blk.0.attn_q.weight")
        assert q.file_dtype == ck.FILE_GGML_BLOCK and q.gguf_quant == synth.GGUF_Q4_K
        assert w.get("blk.0.ffn_down.weight").gguf_quant == synth.GGUF_Q8_0
        np.testing.assert_array_equal(w.get("output_norm.weight").numpy(), f32)
        np.testing.assert_array_equal(w.get("a.f16").numpy(), f16)
        np.testing.assert_array_equal(w.get("z.bf16").numpy(), bf16)
        assert w.get("z.bf16").file_dtype == ck.FILE_BF16 and w.get("z.bf16").gguf_quant == -1
        assert w.try_get("missing") is None
        with pytest.raises(KeyError):
            w.get("missing")
        assert w.total_size_bytes() == sum(len(t[3]) for t in tensors)

        assert w.architecture() == "llama"
        assert w.metadata_u32("llama.block_count") == 32
        assert w.metadata_f32("llama.rope.freq_base") == 500000.0
        # the typed getters are strict about the stored type (candle's Value::to_u32 / to_f32)
        with pytest.raises(KeyError):
            w.metadata_u32("llama.attention.head_count")       # stored as u64
        with pytest.raises(KeyError):
            w.metadata_f32("some.f64")
        with pytest.raises(KeyError):
            w.metadata_string("llama.block_count")
        assert w.metadata_u32_or("llama.attention.head_count", 11) == 11
        assert w.metadata_u32_or("llama.block_count", 11) == 32
        assert w.metadata_f32_or("absent", 1.25) == 1.25
        assert w.metadata_number("llama.attention.head_count") == 32
        assert w.metadata_number("some.i8") == -5 and w.metadata_number("some.bool") == 1
        assert w.metadata_number("some.f64") == 2.5 and w.metadata_number("some.i32") == 7
        assert w.metadata_number("general.architecture") is None
        assert w.eos_token_ids() == [2, 7, 9]
        keys = w.metadata_keys()
        assert list(keys) == [m[0] for m in META]
        assert keys["tokenizer.ggml.tokens"] == (ck.GGUF_VAL_ARRAY, ck.GGUF_VAL_STRING, 4)
        assert keys["tokenizer.ggml.scores"] == (ck.GGUF_VAL_ARRAY, ck.GGUF_VAL_F32, 3)
        assert keys["nested"] == (ck.GGUF_VAL_ARRAY, ck.GGUF_VAL_ARRAY, 2)
        assert keys["general.architecture"][0] == ck.GGUF_VAL_STRING
    with pytest.raises(OxqError):
        w.get("a.f16")            # closed


def test_gguf_default_alignment_and_eos_variants(tmp_path):
    payload = np.arange(8, dtype=np.float32).tobytes()
    path = str(tmp_path / "a.gguf")
    G.write_gguf(path, [("tokenizer.ggml.eos_token_ids", G.ARRAY, (G.U32, [5, 6]))], [("t", (8,), 0, payload)])
    with ck.GgufWeights.load(path) as w:
        assert w.get("t").numpy().tobytes() == payload
        assert w.eos_token_ids() == [5, 6]
        with pytest.raises(KeyError):
            w.architecture()
    # an eos id of another integer width is not a u32 and is skipped, as are non-u32 arrays
    G.write_gguf(path, [("tokenizer.ggml.eos_token_id", G.I32, 3),
                        ("tokenizer.ggml.eos_token_ids", G.ARRAY, (G.I32, [5]))], [])
    with ck.GgufWeights.load(path) as w:
        assert w.eos_token_ids() == [] and len(w) == 0


def test_gguf_shards_merge_and_first_metadata(tmp_path):
    a, b = str(tmp_path / "s1.gguf"), str(tmp_path / "s2.gguf")
    pa, pb, pc = (np.full(4, v, np.float32).tobytes() for v in (1, 2, 3))
    G.write_gguf(a, [("general.architecture", G.STRING, "qwen2")], [("x", (4,), 0, pa), ("both", (4,), 0, pa)])
    G.write_gguf(b, [("general.architecture", G.STRING, "other"), ("extra", G.U32, 1)],
                 [("y", (2, 2), 0, pb), ("both", (4,), 0, pc)], version=2)
    with ck.GgufWeights.load_shards([a, b]) as w:
        assert w.names() == ["both", "x", "y"]
        assert w.architecture() == "qwen2"                 # metadata of the first shard only
        assert w.metadata_u32_or("extra", 0) == 0
        assert w.get("both").numpy().tobytes() == pc and w.get("both").shard == 1
        assert w.get("x").shard == 0 and w.get("y").shape == (2, 2)
    with pytest.raises(OxqError) as e:
        ck.GgufWeights.load_shards([])
    assert _status(e) == -1


def test_gguf_rejects_malformed_files(tmp_path):
    path = str(tmp_path / "bad.gguf")
    good = G.write_gguf(path, META, _sample_tensors(np.random.default_rng(0))[0], alignment=64)

    def expect(data, status, text):
        with open(path, "wb") as f:
            f.write(data)
        with pytest.raises(OxqError) as e:
            ck.GgufWeights.load(path)
        assert _status(e) == status, e.value
        assert text in e.value.message, e.value.message

    expect(b"GGML" + good[4:], -13, "not a GGUF file")
    expect(good[:4] + struct.pack("<I", 4) + good[8:], -13, "unsupported GGUF version")
    expect(good[:100], -13, "truncated")
    expect(good[:-64], -13, "out of mmap bounds")               # last payload cut short
    expect(b"", -13, "empty")
    # element count not a multiple of the block size (gguf_weights.rs:320-327)
    G.write_gguf(path, [], [("w", (3, 100), 12, b"\0" * 144)])
    with pytest.raises(OxqError) as e:
        ck.GgufWeights.load(path)
    assert "not divisible by block size 256" in e.value.message
    # unknown ggml type
    G.write_gguf(path, [], [("w", (32,), 2, b"\0" * 18)])
    data = bytearray(open(path, "rb").read())
    i = data.index(b"w") + 1 + 4 + 8                             # name, n_dims, one dim
    data[i:i + 4] = struct.pack("<I", 99)
    expect(bytes(data), -13, "unknown ggml type 99")
    # unknown metadata value type
    G.write_gguf(path, [("k", G.U32, 1)], [])
    data = bytearray(open(path, "rb").read())
    i = data.index(b"k") + 1
    data[i:i + 4] = struct.pack("<I", 13)
    expect(bytes(data), -13, "unknown value type 13")
    # Byte counts that wrap 64 bits: one F32 tensor of 2^62 elements (2^62 * 4 = 0 mod 2^64) and one of
    # 2^31 x 2^31.  Without a check the slice has "0 bytes", lies inside the map and carries dims that do
    # not match it; a caller that sizes a read from the dims would run past the mapping.
    for dims in ((1 << 62,), (1 << 31, 1 << 31)):
        G.write_gguf(path, [], [("w", dims, 0, b"\0" * 32)])
        with pytest.raises(OxqError) as e:
            ck.GgufWeights.load(path)
        assert _status(e) == -13 and "overflows" in e.value.message, e.value.message
    # more tensor / metadata records than the file has bytes for: refused before anything is reserved
    G.write_gguf(path, [], [])
    data = bytearray(open(path, "rb").read())
    data[8:16] = struct.pack("<Q", 1 << 40)
    expect(bytes(data), -13, "cannot fit")
    with pytest.raises(OxqError) as e:
        ck.GgufWeights.load(str(tmp_path / "nope.gguf"))
    assert _status(e) == -12


# ------------------------------------------------------------------------------------ safetensors
def _save(path, tensors, metadata=None):
    from safetensors.numpy import save_file
    save_file(tensors, path, metadata=metadata)


def test_safetensors_index_matches_the_safetensors_package(tmp_path):
    rng = np.random.default_rng(3)
    tensors = {
        "model.layers.0.mlp.up_proj.qweight": rng.integers(-2**31, 2**31, size=(64, 4), dtype=np.int64).astype(np.int32),
        "model.layers.0.mlp.up_proj.qzeros": rng.integers(0, 2**31, size=(1, 4), dtype=np.int64).astype(np.int32),
        "model.layers.0.mlp.up_proj.scales": rng.standard_normal((1, 32)).astype(np.float16),
        "model.norm.weight": rng.standard_normal((8,)).astype(np.float32),
        "bytes": rng.integers(0, 256, size=(2, 3, 5), dtype=np.uint8),
        "i64": np.arange(6, dtype=np.int64).reshape(2, 3),
        "empty": np.zeros((0, 4), np.float32),
        "flag": np.array([True, False]),
    }
    path = str(tmp_path / "model.safetensors")
    _save(path, tensors, metadata={"format": "pt"})
    with ck.ModelWeights.load([path]) as w:
        assert w.names() == sorted(tensors)
        for name, arr in tensors.items():
            t = w.get(name)
            assert t.shape == arr.shape and t.nbytes == arr.nbytes and t.ggml_type == -1 and t.gguf_quant == -1
            got = t.numpy()
            np.testing.assert_array_equal(got.view(arr.dtype) if arr.dtype == np.bool_ else got, arr)
        assert w.get("model.norm.weight").dtype_name == "F32"
        assert w.get("model.layers.0.mlp.up_proj.qweight").dtype_name == "I32"
        assert w.get("flag").dtype_name == "BOOL"
        assert w.runtime_size_bytes() == sum(a.nbytes for a in tensors.values())
        assert w.has_packed_quantized_weights()


def test_safetensors_bf16_and_f8_dtypes_via_torch(tmp_path):
    torch = pytest.importorskip("torch")
    from safetensors.torch import save_file
    bf = torch.randn(4, 6).to(torch.bfloat16)
    f8 = torch.randn(8, 16).to(torch.float8_e4m3fn)
    path = str(tmp_path / "t.safetensors")
    save_file({"w.weight": f8, "w.weight_scale_inv": torch.ones(1, 1), "b": bf}, path)
    with ck.ModelWeights.load([path]) as w:
        assert w.get("b").dtype_name == "BF16" and w.get("w.weight").dtype_name == "F8_E4M3"
        np.testing.assert_array_equal(w.get("b").numpy(), bf.view(torch.uint16).numpy())
        np.testing.assert_array_equal(w.get("w.weight").numpy(), f8.view(torch.uint8).numpy())
        assert w.try_get_scale_inv("w.weight").shape == (1, 1)
        assert w.try_get_scale_inv("b") is None
        assert not w.has_packed_quantized_weights()


def test_runtime_size_bytes_reference_cases(tmp_path):
    """weights.rs:659-697."""
    path = str(tmp_path / "m.safetensors")
    _save(path, {"layer.0.q_proj.qweight": np.zeros((1, 4), np.int32), "layer.0.q_proj.qzeros": np.zeros((1, 4), np.int32),
                 "layer.0.q_proj.scales": np.zeros((1, 32), np.float16), "layer.0.q_proj.bias": np.zeros((32,), np.float16),
                 "layer.0.input_layernorm.weight": np.zeros((8,), np.float16)})
    with ck.ModelWeights.load([path]) as w:
        assert w.runtime_size_bytes() == 16 + 16 + 64 + 64 + 16
    _save(path, {"layer.0.self_attn.q_proj.weight": np.zeros((4, 4), np.float16),
                 "layer.0.input_layernorm.weight": np.zeros((4,), np.float16)})
    with ck.ModelWeights.load([path]) as w:
        assert w.runtime_size_bytes() == 40


def test_safetensors_alias_resolution_and_shards(tmp_path):
    """weights.rs:452-503: canonical names resolve through the multimodal nestings, exact name first."""
    a, b = str(tmp_path / "a.safetensors"), str(tmp_path / "b.safetensors")
    one = lambda v: np.full((2,), v, np.float32)
    _save(a, {"model.language_model.layers.0.w": one(1), "model.layers.1.w": one(2),
              "model.language_model.layers.1.w": one(3), "language_model.model.layers.2.w": one(4),
              "model.language_model.lm_head.weight": one(5)})
    _save(b, {"model.model.layers.3.w": one(6), "language_model.layers.4.w": one(7),
              "model.language_model.model.layers.4.w": one(8), "language_model.lm_head.weight_scale_inv": one(9),
              "other.layers.5.w": one(10)})
    with ck.ModelWeights.load([a, b]) as w:
        val = lambda name: float(w.get(name).numpy()[0])
        assert val("model.layers.0.w") == 1
        assert val("model.layers.1.w") == 2                    # the exact name wins over an alias
        assert val("model.layers.2.w") == 4
        assert val("model.layers.3.w") == 6 and w.get("model.layers.3.w").shard == 1
        assert val("model.layers.4.w") == 8                    # alias order: language_model.model before language_model
        assert val("lm_head.weight") == 5
        assert val("lm_head.weight_scale_inv") == 9
        assert w.try_get("model.layers.5.w") is None
        assert w.try_get("layers.0.w") is None                 # only `model.`-prefixed names are aliased
        assert w.try_get("lm_head.bias") is None


def test_try_get_quant_by_scheme(tmp_path):
    """weights.rs:523-565."""
    path = str(tmp_path / "q.safetensors")
    i32 = lambda *s: np.zeros(s, np.int32)
    f16 = lambda *s: np.zeros(s, np.float16)
    _save(path, {"model.language_model.layers.0.q.qweight": i32(128, 8), "model.language_model.layers.0.q.qzeros": i32(1, 8),
                 "model.language_model.layers.0.q.scales": f16(1, 64),
                 "p.k.qweight": i32(16, 64), "p.k.scales": f16(1, 64),
                 "p.v.qweight": i32(16, 64), "p.v.scales": f16(1, 64), "p.v.qzeros": i32(1, 8),
                 "p.c.weight_packed": i32(64, 16), "p.c.weight_scale": f16(64, 1), "p.c.weight_shape": np.array([64, 128]),
                 "p.partial.qweight": i32(16, 64)})
    with ck.ModelWeights.load([path]) as w:
        assert w.find_quant("model.layers.0.q") is None                         # no scheme attached
        w.with_quant_scheme(ck.QuantScheme.awq(4))
        assert w.quant_scheme() == ck.QuantScheme(ck.SCHEME_AWQ, 4, False)
        qw, qz, sc = w.find_quant("model.layers.0.q")
        assert (qw.shape, qz.shape, sc.shape) == ((128, 8), (1, 8), (1, 64))
        assert qw.name == "model.language_model.layers.0.q.qweight"
        assert w.find_quant("p.k") is None                                      # AWQ needs all three
        assert w.find_quant("absent") is None
        qw, qz, sc = w.find_quant("p.k", ck.QuantScheme.gptq(4, True))          # GPTQ: qzeros optional
        assert qz is None and qw.shape == (16, 64)
        qw, qz, sc = w.find_quant("p.v", ck.QuantScheme.gptq(8, False))
        assert qz is not None and qz.shape == (1, 8)
        assert w.find_quant("p.partial", ck.QuantScheme.gptq(4, True)) is None
        qw, qz, sc = w.find_quant("p.c", ck.QuantScheme.compressed_tensors4())
        assert qw.name == "p.c.weight_packed" and sc.name == "p.c.weight_scale" and qz is None
        assert w.find_quant("p.v", ck.QuantScheme.compressed_tensors4()) is None


def test_safetensors_rejects_malformed_files(tmp_path):
    path = str(tmp_path / "bad.safetensors")

    def expect(data, text):
        with open(path, "wb") as f:
            f.write(data)
        with pytest.raises(OxqError) as e:
            ck.ModelWeights.load([path])
        assert _status(e) == -13 and text in e.value.message, e.value.message

    def file_of(header: dict, data=b""):
        h = json.dumps(header).encode()
        return struct.pack("<Q", len(h)) + h + data

    expect(b"\1\2\3", "too short")
    expect(struct.pack("<Q", 1000) + b"{}", "header length")
    expect(struct.pack("<Q", 2) + b"[]", "not a JSON object")
    expect(struct.pack("<Q", 5) + b'{"a":', "not a JSON object")
    expect(file_of({"t": {"dtype": "F32", "shape": [2], "data_offsets": [0, 8]}}, b"\0" * 4), "data_offsets")
    expect(file_of({"t": {"dtype": "F32", "shape": [3], "data_offsets": [0, 8]}}, b"\0" * 8), "data_offsets")
    expect(file_of({"t": {"dtype": "F33", "shape": [2], "data_offsets": [0, 8]}}, b"\0" * 8), "unknown dtype")
    expect(file_of({"t": {"dtype": "F32", "shape": [-1], "data_offsets": [0, 8]}}, b"\0" * 8), "bad shape")
    expect(file_of({"t": {"dtype": "F32", "shape": [2]}}, b"\0" * 8), "malformed header entry")
    # escapes and unicode in names parse
    h = b'{"a\\u00e9\\n\\"": {"dtype": "U8", "shape": [1], "data_offsets": [0, 1]}, "__metadata__": {"k": "v"}}'
    with open(path, "wb") as f:
        f.write(struct.pack("<Q", len(h)) + h + b"\7")
    with ck.ModelWeights.load([path]) as w:
        assert w.names() == ["aé\n\""] and w.get("aé\n\"").numpy()[0] == 7
    with pytest.raises(OxqError) as e:
        ck.ModelWeights.load([str(tmp_path / "absent.safetensors")])
    assert _status(e) == -12


# ------------------------------------------------------------------- quantization_config rules
CT_OK = {"quant_method": "compressed-tensors", "format": "pack-quantized",
         "config_groups": {"group_0": {"weights": {"num_bits": 4, "symmetric": True, "type": "int", "strategy": "group",
                                                   "group_size": 128, "actorder": None}}}}


def _ct(**changes):
    cfg = json.loads(json.dumps(CT_OK))
    w = cfg["config_groups"]["group_0"]["weights"]
    for k, v in changes.items():
        if k == "format":
            cfg["format"] = v
        elif k == "extra_group":
            cfg["config_groups"]["group_1"] = v
        else:
            w[k] = v
    return cfg


@pytest.mark.parametrize("cfg, want", [
    (None, None),
    ({}, None),
    ({"bits": 4}, None),                                                    # no quant_method
    ({"quant_method": "fp8", "fmt": "e4m3"}, None),                         # hf_parser.rs:765-775
    ({"quant_method": "FP8"}, None),
    ({"quant_method": "mxfp4"}, None),
    ({"quant_method": "awq", "bits": 4, "group_size": 128, "version": "gemm"}, ck.QuantScheme(ck.SCHEME_AWQ, 4, False)),
    ({"quant_method": "AWQ", "bits": 8, "version": "GEMM"}, ck.QuantScheme(ck.SCHEME_AWQ, 8, False)),
    ({"quant_method": "awq", "bits": 4}, ck.QuantScheme(ck.SCHEME_AWQ, 4, False)),           # version defaults to gemm
    ({"quant_method": "gptq", "bits": 4}, ck.QuantScheme(ck.SCHEME_GPTQ, 4, True)),          # sym defaults to true
    ({"quant_method": "gptq", "bits": 8, "sym": False, "desc_act": False, "checkpoint_format": "GPTQ"},
     ck.QuantScheme(ck.SCHEME_GPTQ, 8, False)),
    ({"quant_method": "gptq", "bits": 4, "sym": "no"}, ck.QuantScheme(ck.SCHEME_GPTQ, 4, True)),  # non-bool -> default
    (CT_OK, ck.QuantScheme(ck.SCHEME_COMPRESSED_TENSORS4, 4, True)),
    (_ct(actorder=None), ck.QuantScheme(ck.SCHEME_COMPRESSED_TENSORS4, 4, True)),
])
def test_validate_quantization_config_accepts(cfg, want):
    assert ck.validate_quantization_config(cfg) == want
    assert ck.validate_quantization_config({"model_type": "llama", "quantization_config": cfg}, whole_config=True) == want


@pytest.mark.parametrize("cfg, text", [
    ({"quant_method": "awq"}, "missing required 'bits'"),
    ({"quant_method": "awq", "bits": 4.0}, "missing required 'bits'"),      # a float is not an unsigned integer
    ({"quant_method": "awq", "bits": -4}, "missing required 'bits'"),
    ({"quant_method": "awq", "bits": 3}, "bits=3 not supported"),
    ({"quant_method": "awq", "bits": 4, "version": "gemv"}, "version 'gemv'"),
    ({"quant_method": "gptq"}, "missing required 'bits'"),
    ({"quant_method": "gptq", "bits": 2}, "bits=2 not supported"),
    ({"quant_method": "gptq", "bits": 4, "desc_act": True}, "desc_act=true"),
    ({"quant_method": "gptq", "bits": 4, "checkpoint_format": "gptq_v2"}, "checkpoint_format='gptq_v2'"),
    (_ct(format="int-quantized"), "format 'int-quantized'"),
    (_ct(num_bits=8), "bits=8"),
    (_ct(symmetric=False), "sym=false"),
    (_ct(type="float"), "type='float'"),
    (_ct(strategy="channel"), "strategy='channel'"),
    (_ct(actorder="group"), "actorder=set"),
    (_ct(extra_group={"weights": {}}), "groups=2"),
    ({"quant_method": "compressed-tensors", "format": "pack-quantized"}, "groups=0"),
    ({"quant_method": "bitsandbytes"}, "Unknown quantization method 'bitsandbytes'"),
])
def test_validate_quantization_config_rejects(cfg, text):
    with pytest.raises(OxqError) as e:
        ck.validate_quantization_config(cfg)
    assert _status(e) == -11 and text in e.value.message, e.value.message


def test_validate_quantization_config_json_text():
    assert ck.validate_quantization_config("null") is None
    assert ck.validate_quantization_config('"awq"') is None                 # not an object: no method
    assert ck.validate_quantization_config(' {"quant_method":"awq","bits":4,"bits":8} ').bits == 8   # last key wins
    assert ck.validate_quantization_config('{"a": 1}', whole_config=True) is None
    for bad in ["", "{", '{"a":1,}', '{"a" 1}', "nul", '{"a":"\\x"}', '{"a":1} x', "[1,]", '"\\ud800"']:
        with pytest.raises(OxqError) as e:
            ck.validate_quantization_config(bad)
        assert _status(e) == -13, bad
