"""MI355X (gfx950) quantized-weight matmul path of oxydLLM: AWQ / GPTQ int4+int8
GEMV and tile GEMM, GGUF Q4_0 / Q8_0 / Q4_K / Q6_K GEMV, MXFP4 expert GEMV.

The product is ``liboxq_hip.so`` (C ABI in ``include/oxq.h``); ``ops`` is a
thin torch binding over it.  Importing ``oxydllm_amd.ops`` requires the built
library: there is no CPU or PyTorch fallback.
"""
__version__ = "0.1.0"
