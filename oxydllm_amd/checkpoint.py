"""Checkpoint files -> resident layers, named after the reference's loaders
(``src/common/gguf_weights.rs`` GgufWeights, ``src/common/weights.rs`` ModelWeights /
QuantScheme, ``src/models/parsers/hf_parser.rs`` validate_quantization_config).

Parsing, name resolution and the quantization-config rules live behind the C ABI
(``include/oxq_files.h``); this module turns the answers into Python objects and, with
torch as the owner of device memory, uploads payloads and builds the layer objects of
:mod:`oxydllm_amd.ops`.  Indexing and metadata need no GPU.
"""
from __future__ import annotations

import ctypes as C
import json
from dataclasses import dataclass
from typing import Dict, Iterator, List, Optional, Sequence, Tuple, Union

import numpy as np

from . import _lib
from ._lib import OxqError, OxqFileTensor, OxqQuantScheme

(FILE_F32, FILE_F16, FILE_BF16, FILE_F64, FILE_U8, FILE_I8, FILE_U16, FILE_I16, FILE_U32, FILE_I32, FILE_U64,
 FILE_I64, FILE_BOOL, FILE_F8_E4M3, FILE_F8_E5M2, FILE_GGML_BLOCK) = range(16)
FILE_DTYPE_NAMES = ["F32", "F16", "BF16", "F64", "U8", "I8", "U16", "I16", "U32", "I32", "U64", "I64", "BOOL",
                    "F8_E4M3", "F8_E5M2", "GGML_BLOCK"]
# numpy view of a payload: 16-bit floats that numpy lacks and the 8-bit floats stay raw
_NP_VIEW = {FILE_F32: np.float32, FILE_F16: np.float16, FILE_BF16: np.uint16, FILE_F64: np.float64, FILE_U8: np.uint8,
            FILE_I8: np.int8, FILE_U16: np.uint16, FILE_I16: np.int16, FILE_U32: np.uint32, FILE_I32: np.int32,
            FILE_U64: np.uint64, FILE_I64: np.int64, FILE_BOOL: np.uint8, FILE_F8_E4M3: np.uint8,
            FILE_F8_E5M2: np.uint8, FILE_GGML_BLOCK: np.uint8}

SCHEME_NONE, SCHEME_AWQ, SCHEME_GPTQ, SCHEME_COMPRESSED_TENSORS4 = range(4)
(GGUF_VAL_U8, GGUF_VAL_I8, GGUF_VAL_U16, GGUF_VAL_I16, GGUF_VAL_U32, GGUF_VAL_I32, GGUF_VAL_F32, GGUF_VAL_BOOL,
 GGUF_VAL_STRING, GGUF_VAL_ARRAY, GGUF_VAL_U64, GGUF_VAL_I64, GGUF_VAL_F64) = range(13)


@dataclass(frozen=True)
class QuantScheme:
    """weights.rs:22-26."""
    kind: int
    bits: int = 0
    sym: bool = False

    @staticmethod
    def awq(bits: int) -> "QuantScheme":
        return QuantScheme(SCHEME_AWQ, bits, False)

    @staticmethod
    def gptq(bits: int, sym: bool) -> "QuantScheme":
        return QuantScheme(SCHEME_GPTQ, bits, sym)

    @staticmethod
    def compressed_tensors4() -> "QuantScheme":
        return QuantScheme(SCHEME_COMPRESSED_TENSORS4, 4, True)

    def _c(self) -> OxqQuantScheme:
        return OxqQuantScheme(self.kind, self.bits, 1 if self.sym else 0)


def validate_quantization_config(config: Union[None, str, dict], whole_config: bool = False) -> Optional[QuantScheme]:
    """hf_parser.rs:451-585.  ``config`` is the ``quantization_config`` value (dict, JSON text or None), or a
    whole config.json with ``whole_config=True``.  Returns None for dense / FP8 / MXFP4 checkpoints and raises
    :class:`OxqError` (OXQ_ERR_UNSUPPORTED) for a recognised but unsupported combination."""
    text = config if isinstance(config, str) else json.dumps(config)
    out = OxqQuantScheme()
    _lib.check(_lib.load().oxq_validate_quantization_config(text.encode(), 1 if whole_config else 0, C.byref(out)))
    if out.kind == SCHEME_NONE:
        return None
    return QuantScheme(out.kind, out.bits, bool(out.sym))


class FileTensor:
    """One tensor of an open file: metadata plus a pointer into the read-only mapping."""

    def __init__(self, owner: "TensorFile", raw: OxqFileTensor):
        self._owner = owner            # keeps the mapping alive
        self.name: str = raw.name.decode()
        self.file_dtype: int = raw.file_dtype
        self.ggml_type: int = raw.ggml_type
        self.gguf_quant: int = raw.gguf_quant
        self.shape: Tuple[int, ...] = tuple(raw.dims[i] for i in range(raw.rank))
        self.nbytes: int = raw.nbytes
        self.shard: int = raw.shard
        self._addr: int = raw.data or 0

    @property
    def dtype_name(self) -> str:
        return FILE_DTYPE_NAMES[self.file_dtype]

    def numpy(self) -> np.ndarray:
        """A read-only view of the payload (flat bytes for block formats, raw codes for bf16 / f8)."""
        self._owner._check_open()
        if self.nbytes == 0:
            return np.zeros(self.shape if self.file_dtype != FILE_GGML_BLOCK else (0,), _NP_VIEW[self.file_dtype])
        buf = (C.c_uint8 * self.nbytes).from_address(self._addr)
        a = np.frombuffer(buf, dtype=np.uint8)
        a.flags.writeable = False
        if self.file_dtype == FILE_GGML_BLOCK:
            return a
        return a.view(_NP_VIEW[self.file_dtype]).reshape(self.shape)

    def to_device(self, ctx=None):
        """Payload -> a new device tensor (weights.rs:392-404 / gguf_weights.rs:352-358).  Packed words become
        int32, block formats and F8 flat / shaped uint8, floats keep their type."""
        import torch
        from . import ops
        self._owner._check_open()
        ctx = ops._ctx(ctx)
        table = {FILE_F32: torch.float32, FILE_F16: torch.float16, FILE_BF16: torch.bfloat16, FILE_F64: torch.float64,
                 FILE_U8: torch.uint8, FILE_I8: torch.int8, FILE_I16: torch.int16, FILE_U32: torch.int32,
                 FILE_I32: torch.int32, FILE_I64: torch.int64, FILE_BOOL: torch.bool, FILE_F8_E4M3: torch.uint8,
                 FILE_GGML_BLOCK: torch.uint8}
        if self.file_dtype not in table:
            raise OxqError(-2, f"{self.name}: no device type for file dtype {self.dtype_name}")
        shape = (self.nbytes,) if self.file_dtype == FILE_GGML_BLOCK else self.shape
        t = torch.empty(shape, dtype=table[self.file_dtype], device=torch.device("cuda", ctx.device))
        _lib.check(ctx._lib.oxq_upload(ctx.handle, ctx.stream(), t.data_ptr(), self._addr, self.nbytes))
        return t

    def __repr__(self):
        return f"FileTensor({self.name!r}, {self.dtype_name}, shape={self.shape}, nbytes={self.nbytes})"


class TensorFile:
    """An open, memory-mapped set of checkpoint files (one index over all shards)."""

    _opener = None

    def __init__(self, paths: Union[str, Sequence[str]]):
        if isinstance(paths, (str, bytes)):
            paths = [paths]
        self._lib = _lib.load()
        self.paths = [p if isinstance(p, str) else p.decode() for p in paths]
        arr = (C.c_char_p * max(len(self.paths), 1))(*[p.encode() for p in self.paths])
        self.handle = C.c_void_p()
        _lib.check(getattr(self._lib, self._opener)(arr, len(self.paths), C.byref(self.handle)))

    def _check_open(self):
        if not self.handle:
            raise OxqError(-1, "the file has been closed")

    def close(self):
        if self.handle:
            self._lib.oxq_tensor_file_close(self.handle)
            self.handle = C.c_void_p()

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def __len__(self) -> int:
        self._check_open()
        return self._lib.oxq_tensor_file_count(self.handle)

    def tensors(self) -> Iterator[FileTensor]:
        for i in range(len(self)):
            raw = OxqFileTensor()
            _lib.check(self._lib.oxq_tensor_file_at(self.handle, i, C.byref(raw)))
            yield FileTensor(self, raw)

    def names(self) -> List[str]:
        return [t.name for t in self.tensors()]

    def try_get(self, name: str) -> Optional[FileTensor]:
        self._check_open()
        raw, found = OxqFileTensor(), C.c_int()
        _lib.check(self._lib.oxq_tensor_file_find(self.handle, name.encode(), C.byref(raw), C.byref(found)))
        return FileTensor(self, raw) if found.value else None

    def get(self, name: str) -> FileTensor:
        t = self.try_get(name)
        if t is None:
            raise KeyError(f"Tensor not found: {name}")
        return t

    def total_size_bytes(self) -> int:
        self._check_open()
        return self._lib.oxq_tensor_file_total_bytes(self.handle)


class GgufWeights(TensorFile):
    """gguf_weights.rs:23-241.  ``GgufWeights.load(path)`` / ``load_shards(paths)``."""

    _opener = "oxq_gguf_open"

    @classmethod
    def load(cls, path: str) -> "GgufWeights":
        return cls([path])

    @classmethod
    def load_shards(cls, paths: Sequence[str]) -> "GgufWeights":
        return cls(list(paths))

    # ---- metadata (gguf_weights.rs:95-144, 216-240)
    def metadata_keys(self) -> Dict[str, Tuple[int, int, int]]:
        """key -> (value type, element type or -1, element count), in file order."""
        self._check_open()
        out = {}
        for i in range(self._lib.oxq_gguf_metadata_count(self.handle)):
            key, vt, et, n = C.c_char_p(), C.c_int(), C.c_int(), C.c_uint64()
            _lib.check(self._lib.oxq_gguf_metadata_at(self.handle, i, C.byref(key), C.byref(vt), C.byref(et), C.byref(n)))
            out[key.value.decode()] = (vt.value, et.value, n.value)
        return out

    def metadata_u32(self, key: str) -> int:
        self._check_open()
        v, found = C.c_uint32(), C.c_int()
        _lib.check(self._lib.oxq_gguf_metadata_u32(self.handle, key.encode(), C.byref(v), C.byref(found)))
        if not found.value:
            raise KeyError(f"Missing or non-u32 GGUF metadata key: {key}")
        return v.value

    def metadata_f32(self, key: str) -> float:
        self._check_open()
        v, found = C.c_float(), C.c_int()
        _lib.check(self._lib.oxq_gguf_metadata_f32(self.handle, key.encode(), C.byref(v), C.byref(found)))
        if not found.value:
            raise KeyError(f"Missing or non-f32 GGUF metadata key: {key}")
        return v.value

    def metadata_string(self, key: str) -> str:
        self._check_open()
        p, n, found = C.c_void_p(), C.c_uint64(), C.c_int()
        _lib.check(self._lib.oxq_gguf_metadata_string(self.handle, key.encode(), C.byref(p), C.byref(n), C.byref(found)))
        if not found.value:
            raise KeyError(f"Missing or non-string GGUF metadata key: {key}")
        return C.string_at(p.value, n.value).decode("utf-8", "replace")

    def metadata_number(self, key: str) -> Optional[float]:
        self._check_open()
        v, found = C.c_double(), C.c_int()
        _lib.check(self._lib.oxq_gguf_metadata_number(self.handle, key.encode(), C.byref(v), C.byref(found)))
        return v.value if found.value else None

    def metadata_u32_or(self, key: str, default: int) -> int:
        try:
            return self.metadata_u32(key)
        except KeyError:
            return default

    def metadata_f32_or(self, key: str, default: float) -> float:
        try:
            return self.metadata_f32(key)
        except KeyError:
            return default

    def architecture(self) -> str:
        return self.metadata_string("general.architecture")

    def eos_token_ids(self) -> List[int]:
        self._check_open()
        n = C.c_uint64()
        _lib.check(self._lib.oxq_gguf_eos_token_ids(self.handle, None, 0, C.byref(n)))
        ids = (C.c_uint32 * max(n.value, 1))()
        _lib.check(self._lib.oxq_gguf_eos_token_ids(self.handle, ids, n.value, C.byref(n)))
        return list(ids[:n.value])

    # ---- layers
    def qlinear(self, name: str, bias=None, out_dtype=None, depermute: Optional[Tuple[int, int]] = None, ctx=None):
        """The block-quantized [out, in] tensor ``name`` as a resident :class:`ops.QLinear`
        (linear.rs:179-260).  ``depermute=(n_heads, head_dim)`` undoes the converter's q/k row
        interleave on the device first (gguf_weights.rs:255-291)."""
        import torch
        from . import ops
        t = self.get(name)
        if t.gguf_quant < 0:
            raise OxqError(-11, f"{name}: ggml type {t.ggml_type} has no block-quant kernel")
        if len(t.shape) != 2:
            raise OxqError(-3, f"{name}: expected a 2-D [out, in] weight, got {t.shape}")
        out_f, in_f = t.shape
        w = t.to_device(ctx)
        if depermute is not None:
            w = ops.gguf_depermute_qk_rows(w, in_f, out_f, t.gguf_quant, depermute[0], depermute[1], ctx=ctx)
        return ops.QLinear(t.gguf_quant, w, in_f, out_f, bias, out_dtype or torch.bfloat16, ctx=ctx)

    def feed_forward(self, layer_idx: int, intermediate_size: int, activation: Optional[int] = None, out_dtype=None,
                     ctx=None, fuse: bool = True):
        """ffn.rs:307-373 FeedForward::load_gguf: ``blk.{i}.ffn_{gate,up,down}.weight`` kept quantized.
        Separate when ``ffn_gate`` exists, packed when ``ffn_up`` holds gate and up, ungated otherwise.

        With ``fuse`` a gated bf16 layer whose format and shape have the matrix-core copy becomes one projection with
        the activation in its epilogue (separate ``ffn_gate`` / ``ffn_up`` tensors of one format are fused by
        concatenating their bytes): two launches a forward instead of four, the same bits."""
        import torch
        from . import ops
        activation = ops.ACT_GATED_SILU if activation is None else activation
        prefix = f"blk.{layer_idx}"
        up_t = self.get(f"{prefix}.ffn_up.weight")
        down_t = self.get(f"{prefix}.ffn_down.weight")
        up_out = up_t.shape[0]
        if down_t.shape[1] != intermediate_size:
            raise OxqError(-3, f"GGUF ffn_down shape mismatch at {prefix}: expected dim1={intermediate_size}, "
                               f"got {down_t.shape[1]}")
        gate_t = self.try_get(f"{prefix}.ffn_gate.weight")
        mk = lambda part: self.qlinear(f"{prefix}.ffn_{part}.weight", out_dtype=out_dtype, ctx=ctx)
        if gate_t is not None:
            if gate_t.shape[0] != intermediate_size:
                raise OxqError(-3, f"GGUF ffn_gate shape mismatch at {prefix}: expected dim0={intermediate_size}, "
                                   f"got {gate_t.shape[0]}")
            if up_out != intermediate_size:
                raise OxqError(-3, f"GGUF ffn_up shape mismatch at {prefix}: expected dim0={intermediate_size}, "
                                   f"got {up_out}")
            a = None
            if fuse and gate_t.gguf_quant == up_t.gguf_quant and gate_t.shape == up_t.shape:
                both = torch.cat([gate_t.to_device(ctx).reshape(-1), up_t.to_device(ctx).reshape(-1)])
                a = self._fused_gate_up(up_t.gguf_quant, both, up_t.shape[1], 2 * intermediate_size, activation, out_dtype, ctx)
            if a is not None:
                kind, b = ops.GATE_UP_FUSED, None
            else:
                kind, a, b = ops.GATE_UP_SEPARATE, mk("gate"), mk("up")
        elif up_out == 2 * intermediate_size:
            a = self._fused_gate_up(up_t.gguf_quant, up_t.to_device(ctx), up_t.shape[1], up_out, activation, out_dtype,
                                    ctx) if fuse else None
            kind, a, b = ops.GATE_UP_FUSED, a if a is not None else mk("up"), None
        elif up_out == intermediate_size:
            kind, a, b = ops.GATE_UP_SIMPLE, mk("up"), None
        else:
            raise OxqError(-3, f"Unsupported GGUF FFN up-proj shape at {prefix}: dim0={up_out} (expected "
                               f"{intermediate_size} or {2 * intermediate_size})")
        return ops.FeedForward(kind, a, b, mk("down"), intermediate_size, activation, ctx=ctx)


    @staticmethod
    def _fused_gate_up(quant: int, both, in_f: int, out_f: int, activation: int, out_dtype, ctx):
        """The gate|up bytes as one layer with the activation in its epilogue, or None where that layer cannot be
        built (format, shape or dtype without the matrix-core copy)."""
        import torch
        from . import ops
        if quant < 0 or (out_dtype or torch.bfloat16) != torch.bfloat16:
            return None
        try:
            return ops.QLinear(quant, both, in_f, out_f, None, torch.bfloat16, ctx=ctx, gate_up_act=activation)
        except OxqError as e:
            if e.status != -11:  # OXQ_ERR_UNSUPPORTED: take the plain layers
                raise
            return None


@dataclass
class QuantWeight:
    """awq.rs:45-92: the packed tensors of one projection, on the device."""
    bits: int
    pack_dim: int
    sym: bool
    qweight: "object"
    qzeros: Optional["object"]
    scales: "object"


class ModelWeights(TensorFile):
    """weights.rs:36-581, the part that serves packed-quantized projections: an index over the
    safetensors shards with alias-aware names and the scheme-driven ``try_get_quant``.  Unlike the
    reference nothing is cast or uploaded at load; tensors move to the device when asked for."""

    _opener = "oxq_safetensors_open"

    def __init__(self, paths, quant_scheme: Optional[QuantScheme] = None):
        super().__init__(paths)
        self._scheme = quant_scheme

    @classmethod
    def load(cls, paths: Sequence[str]) -> "ModelWeights":
        return cls(list(paths))

    def with_quant_scheme(self, scheme: Optional[QuantScheme]) -> "ModelWeights":
        self._scheme = scheme
        return self

    def quant_scheme(self) -> Optional[QuantScheme]:
        return self._scheme

    def try_get_scale_inv(self, weight_name: str) -> Optional[FileTensor]:
        return self.try_get(f"{weight_name}_scale_inv")

    def has_packed_quantized_weights(self) -> bool:
        self._check_open()
        return bool(self._lib.oxq_tensor_file_has_packed_quantized_weights(self.handle))

    def runtime_size_bytes(self) -> int:
        return self.total_size_bytes()

    def find_quant(self, prefix: str, scheme: Optional[QuantScheme] = None):
        """The (qweight, qzeros or None, scales) file tensors of ``prefix`` under ``scheme``, or None."""
        self._check_open()
        scheme = scheme or self._scheme
        if scheme is None:
            return None
        qw, qz, sc, found = OxqFileTensor(), OxqFileTensor(), OxqFileTensor(), C.c_int()
        c_scheme = scheme._c()
        _lib.check(self._lib.oxq_safetensors_try_get_quant(self.handle, C.byref(c_scheme), prefix.encode(), C.byref(qw),
                                                          C.byref(qz), C.byref(sc), C.byref(found)))
        if not found.value:
            return None
        return FileTensor(self, qw), (FileTensor(self, qz) if qz.data else None), FileTensor(self, sc)

    def try_get_quant(self, prefix: str, scheme: Optional[QuantScheme] = None, ctx=None) -> Optional[QuantWeight]:
        """weights.rs:557-565: the packed weight at ``prefix`` on the device, in the layout the layer takes
        (compressed-tensors converted to AWQ by the device transform, awq.rs:187-254)."""
        from . import ops
        scheme = scheme or self._scheme
        found = self.find_quant(prefix, scheme)
        if found is None:
            return None
        qw, qz, sc = found
        if scheme.kind == SCHEME_COMPRESSED_TENSORS4:
            try:
                q, z, s = ops.compressed_to_awq(qw.to_device(ctx), sc.to_device(ctx), ctx=ctx)
            except OxqError:
                return None          # the reference logs the failed conversion and reports "absent"
            return QuantWeight(4, ops.PACK_OUT, True, q, z, s)
        pack_dim = ops.PACK_OUT if scheme.kind == SCHEME_AWQ else ops.PACK_IN
        return QuantWeight(scheme.bits, pack_dim, scheme.sym and scheme.kind == SCHEME_GPTQ, qw.to_device(ctx),
                           qz.to_device(ctx) if qz is not None else None, sc.to_device(ctx))

    def try_get_awq(self, prefix: str, bits: int, ctx=None) -> Optional[QuantWeight]:
        return self.try_get_quant(prefix, QuantScheme.awq(bits), ctx)

    def try_get_gptq(self, prefix: str, bits: int, sym: bool, ctx=None) -> Optional[QuantWeight]:
        return self.try_get_quant(prefix, QuantScheme.gptq(bits, sym), ctx)

    def try_get_compressed(self, prefix: str, ctx=None) -> Optional[QuantWeight]:
        return self.try_get_quant(prefix, QuantScheme.compressed_tensors4(), ctx)

    def packed_linear(self, prefix: str, dtype=None, bias_name: Optional[str] = None, ctx=None):
        """``prefix`` as a resident :class:`ops.PackedQuantLinear` (linear.rs:416-447); scales are cast to
        the runtime dtype as the constructor there does."""
        import torch
        from . import ops
        dtype = dtype or torch.float16
        raw = self.try_get_quant(prefix, ctx=ctx)
        if raw is None:
            raise KeyError(f"no packed-quantized weight at {prefix}")
        if raw.qzeros is None:
            raise OxqError(-1, "PackedQuantLinear: qzeros missing")
        bias = None
        b = self.try_get(bias_name or f"{prefix}.bias")
        if b is not None:
            bias = b.to_device(ctx).to(dtype)
        return ops.PackedQuantLinear(raw.bits, raw.pack_dim, raw.qweight, raw.qzeros, raw.scales.to(dtype), bias, dtype,
                                     ctx=ctx)

    def feed_forward(self, layer_idx: int, activation: Optional[int] = None, dtype=None, ctx=None):
        """ffn.rs:62-68 + 200-285 FeedForward::load, the packed-quant arm: ``model.layers.{i}.mlp`` with
        down_proj packed.  Separate gate_proj / up_proj tensors whose columns can be joined (out_features a
        multiple of 8) become one fused gate|up projection, as the reference does for AWQ; here GPTQ is
        joined too, its tensors concatenate along the same axis.  The fused projection runs the activation in
        its matmul when the layer qualifies for the tile-major copy; otherwise the activation is a second
        launch."""
        import torch
        from . import ops
        activation = ops.ACT_GATED_SILU if activation is None else activation
        dtype = dtype or torch.float16
        p = f"model.layers.{layer_idx}.mlp"
        down_raw = self.try_get_quant(f"{p}.down_proj", ctx=ctx)
        if down_raw is None:
            raise KeyError(f"no packed-quantized weight at {p}.down_proj")

        def layer(raw, act=None):
            if raw.qzeros is None:
                raise OxqError(-1, "PackedQuantLinear: qzeros missing")
            return ops.PackedQuantLinear(raw.bits, raw.pack_dim, raw.qweight, raw.qzeros, raw.scales.to(dtype), None,
                                         dtype, ctx=ctx, gate_up_act=act)

        def fused(raw):
            try:
                return layer(raw, activation)
            except OxqError as e:
                if e.status != -11:     # only "no tile-major copy for this shape" falls back to two launches
                    raise
                return layer(raw)

        down = layer(down_raw)
        inter = down.in_features
        gate_raw = self.try_get_quant(f"{p}.gate_proj", ctx=ctx)
        up_raw = self.try_get_quant(f"{p}.up_proj", ctx=ctx)
        if gate_raw is not None and up_raw is not None:
            gate_out, up_out = gate_raw.scales.shape[1], up_raw.scales.shape[1]
            if gate_out != inter or up_out != inter:
                raise OxqError(-3, f"Packed-quant FFN shape mismatch at {p}: gate/up out_features must both be "
                                   f"{inter}, got gate={gate_out} up={up_out}")
            if inter % 8 == 0 and gate_raw.qzeros is not None and up_raw.qzeros is not None:
                if gate_raw.pack_dim == ops.PACK_OUT:
                    q, z, sc = ops.concat_awq_along_out([(gate_raw.qweight, gate_raw.qzeros, gate_raw.scales),
                                                         (up_raw.qweight, up_raw.qzeros, up_raw.scales)],
                                                        gate_raw.bits, ctx=ctx)
                else:
                    q, z, sc = (torch.cat([getattr(gate_raw, f), getattr(up_raw, f)], dim=1).contiguous()
                                for f in ("qweight", "qzeros", "scales"))
                both = QuantWeight(gate_raw.bits, gate_raw.pack_dim, gate_raw.sym, q, z, sc)
                return ops.FeedForward(ops.GATE_UP_FUSED, fused(both), None, down, inter, activation, ctx=ctx)
            return ops.FeedForward(ops.GATE_UP_SEPARATE, layer(gate_raw), layer(up_raw), down, inter, activation,
                                   ctx=ctx)
        gate_up_raw = self.try_get_quant(f"{p}.gate_up_proj", ctx=ctx)
        if gate_up_raw is not None:
            packed_out = gate_up_raw.scales.shape[1]
            if packed_out != 2 * inter:
                raise OxqError(-3, f"Packed-quant FFN gate_up out_features {packed_out} != 2*{inter}")
            return ops.FeedForward(ops.GATE_UP_FUSED, fused(gate_up_raw), None, down, inter, activation, ctx=ctx)
        if up_raw is not None:
            if up_raw.scales.shape[1] != inter:
                raise OxqError(-3, f"Packed-quant FFN up_proj out_features {up_raw.scales.shape[1]} != {inter}")
            return ops.FeedForward(ops.GATE_UP_SIMPLE, layer(up_raw), None, down, inter, activation, ctx=ctx)
        raise OxqError(-3, f"Mixed quantization at {p}: down_proj is packed but no gate/up tensors are packed. "
                           "Expected one of: ({gate,up}_proj.qweight) or (gate_up_proj.qweight) or (up_proj.qweight).")

    def mxfp4_experts(self, prefix: str, ctx=None) -> dict:
        """The stacked GPT-OSS expert tensors under ``prefix`` (``…mlp``), checked as moe.rs:397-417 checks
        them: ``*_blocks`` U8 [E, out, K/32, 16], ``*_scales`` U8 [E, out, K/32], ``*_bias`` [E, out].
        Returns device tensors ready for ``ops.mxfp4_moe_matmul`` plus the (out, in) of both projections."""
        out = {}
        for proj in ("gate_up_proj", "down_proj"):
            blocks = self.get(f"{prefix}.experts.{proj}_blocks")
            scales = self.get(f"{prefix}.experts.{proj}_scales")
            bias = self.get(f"{prefix}.experts.{proj}_bias")
            d = blocks.shape
            if len(d) != 4 or d[3] != 16:
                raise OxqError(-3, f"{proj}_blocks shape {d} != [E, out, K/32, 16]")
            if scales.shape != d[:3] or bias.shape != d[:2]:
                raise OxqError(-3, f"{proj}: scales {scales.shape} / bias {bias.shape} do not match blocks {d}")
            out[proj] = {"blocks": blocks.to_device(ctx), "scales": scales.to_device(ctx),
                         "bias": bias.to_device(ctx), "out_features": d[1], "in_features": d[2] * 32}
        out["num_experts"] = self.get(f"{prefix}.experts.gate_up_proj_blocks").shape[0]
        return out
