"""ctypes loader for ``liboxq_hip.so`` (the C ABI declared in ``include/oxq.h`` and ``include/oxq_files.h``).

There is no fallback: if the library is missing the import of any op fails with
an error that says how to build it.
"""
from __future__ import annotations

import ctypes as C
import os

HERE = os.path.dirname(os.path.abspath(__file__))
# OXQ_LIB_PATH names another build of the same library (a tuning variant); the default is the in-tree one
LIB_PATH = os.environ.get("OXQ_LIB_PATH") or os.path.join(HERE, "liboxq_hip.so")

OXQ_MAX_RANK = 4
(F32, F16, BF16, U8, I32, U32, I64) = range(7)
PACK_OUT, PACK_IN = 0, 1
(GGUF_Q4_0, GGUF_Q8_0, GGUF_Q4_K, GGUF_Q6_K, GGUF_Q4_1, GGUF_Q5_0, GGUF_Q5_1, GGUF_Q2_K, GGUF_Q3_K,
 GGUF_Q5_K) = range(10)
DEVICE_HOST = -1
DEVICE_PLAN_ONLY = -1
MFMA_MIN_M = 9

STATUS = {
    0: "OXQ_OK", -1: "OXQ_ERR_ARG", -2: "OXQ_ERR_DTYPE", -3: "OXQ_ERR_SHAPE",
    -4: "OXQ_ERR_CONTIGUOUS", -5: "OXQ_ERR_M_RANGE", -6: "OXQ_ERR_GROUP", -7: "OXQ_ERR_DEVICE",
    -8: "OXQ_ERR_BITS", -9: "OXQ_ERR_RUNTIME", -10: "OXQ_ERR_WORKSPACE", -11: "OXQ_ERR_UNSUPPORTED",
    -12: "OXQ_ERR_IO", -13: "OXQ_ERR_FORMAT",
}


class OxqTensor(C.Structure):
    _fields_ = [("data", C.c_void_p), ("dtype", C.c_int32), ("rank", C.c_int32),
                ("dims", C.c_int64 * OXQ_MAX_RANK), ("contiguous", C.c_int32),
                ("device", C.c_int32)]


class OxqAnyLinear(C.Structure):
    _fields_ = [("kind", C.c_int), ("layer", C.c_void_p)]


class OxqPlan(C.Structure):
    _fields_ = [("kernel", C.c_char * 64), ("grid", C.c_uint32 * 3), ("block", C.c_uint32 * 3),
                ("split_k", C.c_uint32), ("launches", C.c_uint32),
                ("workspace_bytes", C.c_uint64)]


OXQ_FILE_MAX_RANK = 8


class OxqFileTensor(C.Structure):
    """``oxq_file_tensor`` of include/oxq_files.h."""
    _fields_ = [("name", C.c_char_p), ("file_dtype", C.c_int32), ("ggml_type", C.c_int32),
                ("gguf_quant", C.c_int32), ("rank", C.c_int32), ("dims", C.c_int64 * OXQ_FILE_MAX_RANK),
                ("data", C.c_void_p), ("nbytes", C.c_uint64), ("shard", C.c_int32), ("reserved", C.c_int32)]


class OxqQuantScheme(C.Structure):
    _fields_ = [("kind", C.c_int32), ("bits", C.c_uint32), ("sym", C.c_int32)]


class OxqError(RuntimeError):
    def __init__(self, status: int, message: str):
        super().__init__(f"{STATUS.get(status, status)}: {message}")
        self.status = status
        self.message = message


# Every symbol include/*.h declares, with its argument types.
_TP = C.POINTER(OxqTensor)
_VP = C.c_void_p
SIGNATURES = {
    "oxq_ctx_create": (C.c_int, [C.c_int, C.POINTER(_VP)]),
    "oxq_ctx_destroy": (C.c_int, [_VP]),
    "oxq_ctx_device": (C.c_int, [_VP]),
    "oxq_ctx_last_plan": (C.c_int, [_VP, C.POINTER(OxqPlan)]),
    "oxq_last_error": (C.c_char_p, []),
    "oxq_status_name": (C.c_char_p, [C.c_int]),
    "oxq_version": (None, [C.POINTER(C.c_int), C.POINTER(C.c_int)]),
    "oxq_ctx_set_weight_cache": (C.c_int, [_VP, C.c_int64]),
    "oxq_ctx_forget_weights": (C.c_int, [_VP, _VP]),
    "oxq_ctx_weight_cache_bytes": (C.c_int, [_VP, C.POINTER(C.c_int64), C.POINTER(C.c_int64)]),
    "oxq_gguf_block_layout": (C.c_int, [C.c_int, C.POINTER(C.c_int64), C.POINTER(C.c_int64)]),
    "oxq_ctx_set_tuning": (C.c_int, [_VP, C.c_char_p, C.c_int]),
    "oxq_ctx_reset_tuning": (C.c_int, [_VP, C.c_char_p]),
    "oxq_calib_read": (C.c_int, [_VP, _VP, _TP, C.c_int, C.c_int, _TP]),
    "oxq_bench_read_upfront": (C.c_int, [_VP, _VP, _TP, C.c_int, C.c_int, C.c_int, _TP]),
    "oxq_bench_empty_launch": (C.c_int, [_VP, _VP, C.c_int, C.c_int, C.c_int]),
    "oxq_bench_grid_barrier": (C.c_int, [_VP, _VP, C.c_int, C.c_int, _TP, C.c_uint32]),
    "oxq_bench_two_streams": (C.c_int, [_VP, _VP, _TP, _TP, C.c_int, C.c_int, _TP]),
    "oxq_w4a16_matmul": (C.c_int, [_VP, _VP, _TP, _TP, _TP, _TP, _TP]),
    "oxq_w4a16_matmul_static": (C.c_int, [_VP, _VP, _TP, _TP, _TP, _TP, _TP]),
    "oxq_w8a16_matmul": (C.c_int, [_VP, _VP, _TP, _TP, _TP, _TP, _TP]),
    "oxq_gptq_matmul": (C.c_int, [_VP, _VP, _TP, _TP, _TP, _TP, C.c_uint32, _TP]),
    "oxq_dequantize_w4": (C.c_int, [_VP, _VP, _TP, _TP, _TP, _TP]),
    "oxq_dequantize_w8": (C.c_int, [_VP, _VP, _TP, _TP, _TP, _TP]),
    "oxq_dequantize_gptq_packed": (C.c_int, [_VP, _VP, _TP, _TP, _TP, C.c_uint32, _TP]),
    "oxq_mpp_quant_matmul": (C.c_int, [_VP, _VP, _TP, _TP, _TP, _TP, C.c_uint32, C.c_int, _TP]),
    "oxq_maybe_mpp_quant_matmul": (C.c_int, [_VP, _VP, _TP, _TP, _TP, _TP, C.c_uint32, C.c_int,
                                             _TP, C.POINTER(C.c_int)]),
    "oxq_compressed_to_awq": (C.c_int, [_VP, _VP, _TP, _TP, _TP, _TP, _TP]),
    "oxq_concat_awq_along_out": (C.c_int, [_VP, _VP, C.c_int, C.c_int, _TP, _TP, _TP, _TP, _TP, _TP]),
    "oxq_rtn_quantize_awq": (C.c_int, [_VP, _VP, _TP, C.c_int64, _TP, _TP, _TP]),
    "oxq_gguf_depermute_qk_rows": (C.c_int, [_VP, _VP, _TP, C.c_int64, C.c_int64, C.c_int, C.c_int64, C.c_int64, _TP]),
    "oxq_cast_f8e4m3_to_f32": (C.c_int, [_VP, _VP, _TP, _TP]),
    "oxq_f8_block_dequant_bf16": (C.c_int, [_VP, _VP, _TP, _TP, _TP]),
    "oxq_f8_gemv": (C.c_int, [_VP, _VP, _TP, _TP, _TP, _TP]),
    "oxq_f8_matmul": (C.c_int, [_VP, _VP, _TP, _TP, _TP, _TP]),
    "oxq_gguf_quant_matmul": (C.c_int, [_VP, _VP, _TP, _TP, C.c_int64, C.c_int64, C.c_int, _TP]),
    "oxq_gguf_quant_mul_mm": (C.c_int, [_VP, _VP, _TP, _TP, C.c_int64, C.c_int64, C.c_int, _TP]),
    "oxq_gguf_dequantize": (C.c_int, [_VP, _VP, _TP, C.c_int64, C.c_int64, C.c_int, _TP]),
    "oxq_mxfp4_matmul": (C.c_int, [_VP, _VP, _TP, _TP, _TP, C.c_int64, C.c_int64, _TP]),
    "oxq_mxfp4_dequantize": (C.c_int, [_VP, _VP, _TP, _TP, C.c_int64, C.c_int64, _TP]),
    "oxq_mxfp4_moe_matmul": (C.c_int, [_VP, _VP, _TP, _TP, _TP, _TP, _TP, _TP, C.c_int,
                                       C.c_int64, C.c_int64, _TP]),
    "oxq_mxfp4_moe_gate_up_swiglu": (C.c_int, [_VP, _VP, _TP, _TP, _TP, _TP, _TP, _TP, C.c_int,
                                              C.c_int64, C.c_int64, C.c_float, _TP, C.POINTER(C.c_int)]),
    "oxq_mxfp4_experts_new": (C.c_int, [_VP, _TP, _TP, _TP, C.c_int64, C.c_int64, C.c_int64, C.POINTER(_VP)]),
    "oxq_mxfp4_experts_matmul": (C.c_int, [_VP, _VP, _TP, _TP, _TP, C.c_int, _TP]),
    "oxq_mxfp4_experts_gate_up_swiglu": (C.c_int, [_VP, _VP, _TP, _TP, _TP, C.c_int, C.c_float, _TP, C.POINTER(C.c_int)]),
    "oxq_mxfp4_experts_is_resident": (C.c_int, [_VP, C.POINTER(C.c_int)]),
    "oxq_mxfp4_experts_dequantize": (C.c_int, [_VP, _VP, C.c_int64, _TP]),
    "oxq_mxfp4_experts_free": (None, [_VP]),
    "oxq_moe_route": (C.c_int, [_VP, _VP, _TP, C.c_int64, C.c_int, _TP, _TP]),
    "oxq_moe_group": (C.c_int, [_VP, _VP, _TP, _TP, C.c_int64, _TP, _TP, _TP, _TP]),
    "oxq_moe_route_group": (C.c_int, [_VP, _VP, _TP, C.c_int64, C.c_int, _TP, _TP, _TP, _TP, _TP, _TP]),
    "oxq_gated_activation": (C.c_int, [_VP, _VP, _TP, C.c_int, C.c_float, _TP]),
    "oxq_activation_mul": (C.c_int, [_VP, _VP, _TP, _TP, C.c_int, _TP]),
    "oxq_moe_combine": (C.c_int, [_VP, _VP, _TP, _TP, _TP, _TP]),
    "oxq_packed_quant_linear_new": (C.c_int, [_VP, C.c_uint32, C.c_int, _TP, _TP, _TP, _TP,
                                              C.c_int, C.POINTER(_VP)]),
    "oxq_packed_quant_linear_new_gate_up": (C.c_int, [_VP, C.c_uint32, C.c_int, _TP, _TP, _TP, _TP, C.c_int, C.c_int,
                                                      C.POINTER(_VP)]),
    "oxq_packed_quant_linear_forward": (C.c_int, [_VP, _VP, _TP, _TP]),
    "oxq_packed_quant_linear_in_features": (C.c_int, [_VP, C.POINTER(C.c_int64)]),
    "oxq_packed_quant_linear_out_features": (C.c_int, [_VP, C.POINTER(C.c_int64)]),
    "oxq_packed_quant_linear_is_prepacked": (C.c_int, [_VP, C.POINTER(C.c_int)]),
    "oxq_packed_quant_linear_dequantize": (C.c_int, [_VP, _VP, _TP]),
    "oxq_packed_quant_linear_free": (None, [_VP]),
    "oxq_qlinear_new": (C.c_int, [_VP, C.c_int, _TP, C.c_int64, C.c_int64, _TP, C.c_int,
                                  C.POINTER(_VP)]),
    "oxq_qlinear_new_gate_up": (C.c_int, [_VP, C.c_int, _TP, C.c_int64, C.c_int64, _TP, C.c_int, C.c_int,
                                          C.POINTER(_VP)]),
    "oxq_qlinear_forward": (C.c_int, [_VP, _VP, _TP, _TP]),
    "oxq_qlinear_is_resident": (C.c_int, [_VP, C.POINTER(C.c_int)]),
    "oxq_qlinear_dequantize": (C.c_int, [_VP, _VP, _TP]),
    "oxq_qlinear_free": (None, [_VP]),
    "oxq_mxfp4_linear_new": (C.c_int, [_VP, _TP, _TP, _TP, C.c_int64, C.c_int64, C.POINTER(_VP)]),
    "oxq_mxfp4_linear_forward": (C.c_int, [_VP, _VP, _TP, _TP]),
    "oxq_mxfp4_linear_free": (None, [_VP]),
    "oxq_mlp_new": (C.c_int, [_VP, C.c_int, C.POINTER(OxqAnyLinear), C.POINTER(OxqAnyLinear), C.POINTER(OxqAnyLinear),
                              C.c_int64, C.c_int, C.POINTER(_VP)]),
    "oxq_mlp_scratch_elems": (C.c_int, [_VP, C.c_int64, C.POINTER(C.c_int64)]),
    "oxq_mlp_forward": (C.c_int, [_VP, _VP, _TP, _TP, _TP]),
    "oxq_mlp_in_features": (C.c_int, [_VP, C.POINTER(C.c_int64)]),
    "oxq_mlp_out_features": (C.c_int, [_VP, C.POINTER(C.c_int64)]),
    "oxq_mlp_free": (None, [_VP]),
    # include/oxq_files.h
    "oxq_gguf_open": (C.c_int, [C.POINTER(C.c_char_p), C.c_int, C.POINTER(_VP)]),
    "oxq_safetensors_open": (C.c_int, [C.POINTER(C.c_char_p), C.c_int, C.POINTER(_VP)]),
    "oxq_tensor_file_close": (C.c_int, [_VP]),
    "oxq_tensor_file_count": (C.c_int64, [_VP]),
    "oxq_tensor_file_at": (C.c_int, [_VP, C.c_int64, C.POINTER(OxqFileTensor)]),
    "oxq_tensor_file_find": (C.c_int, [_VP, C.c_char_p, C.POINTER(OxqFileTensor), C.POINTER(C.c_int)]),
    "oxq_tensor_file_total_bytes": (C.c_uint64, [_VP]),
    "oxq_tensor_file_has_packed_quantized_weights": (C.c_int, [_VP]),
    "oxq_gguf_metadata_count": (C.c_int64, [_VP]),
    "oxq_gguf_metadata_at": (C.c_int, [_VP, C.c_int64, C.POINTER(C.c_char_p), C.POINTER(C.c_int),
                                       C.POINTER(C.c_int), C.POINTER(C.c_uint64)]),
    "oxq_gguf_metadata_u32": (C.c_int, [_VP, C.c_char_p, C.POINTER(C.c_uint32), C.POINTER(C.c_int)]),
    "oxq_gguf_metadata_f32": (C.c_int, [_VP, C.c_char_p, C.POINTER(C.c_float), C.POINTER(C.c_int)]),
    "oxq_gguf_metadata_string": (C.c_int, [_VP, C.c_char_p, C.POINTER(_VP), C.POINTER(C.c_uint64),
                                           C.POINTER(C.c_int)]),
    "oxq_gguf_metadata_number": (C.c_int, [_VP, C.c_char_p, C.POINTER(C.c_double), C.POINTER(C.c_int)]),
    "oxq_gguf_architecture": (C.c_int, [_VP, C.POINTER(_VP), C.POINTER(C.c_uint64), C.POINTER(C.c_int)]),
    "oxq_gguf_eos_token_ids": (C.c_int, [_VP, C.POINTER(C.c_uint32), C.c_uint64, C.POINTER(C.c_uint64)]),
    "oxq_validate_quantization_config": (C.c_int, [C.c_char_p, C.c_int, C.POINTER(OxqQuantScheme)]),
    "oxq_safetensors_try_get_quant": (C.c_int, [_VP, C.POINTER(OxqQuantScheme), C.c_char_p, C.POINTER(OxqFileTensor),
                                                C.POINTER(OxqFileTensor), C.POINTER(OxqFileTensor), C.POINTER(C.c_int)]),
    "oxq_upload": (C.c_int, [_VP, _VP, _VP, _VP, C.c_uint64]),
}

_lib = None


def load() -> C.CDLL:
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            f"{LIB_PATH} is missing: build it with `python -m oxydllm_amd.build` "
            "(hipcc --offload-arch=gfx950); there is no CPU fallback")
    lib = C.CDLL(LIB_PATH)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)  # AttributeError if the library does not export it
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib


def check(rc: int):
    if rc != 0:
        msg = load().oxq_last_error()
        raise OxqError(rc, msg.decode() if msg else "")
