"""Compiles the HIP sources into ``oxydllm_amd/liboxq_hip.so`` for gfx950.

hipcc cross-compiles without a GPU.  The library is built in-tree so it
travels with the source snapshot; nothing is JIT-compiled at import time.
"""
from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
INCLUDE = os.path.join(os.path.dirname(HERE), "include")
LIB = os.path.join(HERE, "liboxq_hip.so")
OBJ_DIR = os.path.join(HERE, "csrc", "build")

SOURCES = ["oxq_api.cpp", "wna16_gemv.hip", "wna16_mfma.hip", "wna16_dequant.hip", "awq_transforms.hip", "pk4.hip", "pk4_tile.hip", "pk4_gemm.hip", "gptq_tile.hip",
           "gguf_gemv.hip", "gguf_res.hip", "gguf_mfma.hip", "blockq_mm.hip", "mxfp4_gemv.hip", "mxfp4_gemm.hip", "moe_glue.hip", "f8_block.hip", "calib.hip",
           "checkpoint_files.cpp"]

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = ["--offload-arch=gfx950", "-O3", "-fPIC", "-std=c++17", "-x", "hip",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
         "-Wno-unused-command-line-argument", "-Wno-unknown-attributes",
         f"-I{INCLUDE}", f"-I{CSRC}"]


def _deps():
    return [os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith((".hpp", ".h"))] + \
        [os.path.join(INCLUDE, "oxq.h"), os.path.join(INCLUDE, "oxq_files.h")]


def _compile(src: str, force: bool) -> str:
    obj = os.path.join(OBJ_DIR, os.path.splitext(src)[0] + ".o")
    path = os.path.join(CSRC, src)
    newest = max(os.path.getmtime(p) for p in [path] + _deps())
    if force or not os.path.exists(obj) or os.path.getmtime(obj) < newest:
        cmd = [HIPCC] + FLAGS + ["-c", path, "-o", obj]
        res = subprocess.run(cmd, capture_output=True, text=True)
        err = "\n".join(l for l in res.stderr.splitlines()
                        if "packed-fp32-ops" not in l)
        if res.returncode != 0:
            raise RuntimeError(f"hipcc failed for {src}:\n{err}")
        if err.strip():
            sys.stderr.write(err + "\n")
    return obj


def build(force: bool = False, jobs: int = 6) -> str:
    os.makedirs(OBJ_DIR, exist_ok=True)
    with ThreadPoolExecutor(max_workers=jobs) as ex:
        objs = list(ex.map(lambda s: _compile(s, force), SOURCES))
    newest = max(os.path.getmtime(o) for o in objs)
    if force or not os.path.exists(LIB) or os.path.getmtime(LIB) < newest:
        cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB] + objs
        res = subprocess.run(cmd, capture_output=True, text=True)
        if res.returncode != 0:
            raise RuntimeError(f"link failed:\n{res.stderr}")
    _check_no_missing_kernels(LIB)
    return LIB


def _check_no_missing_kernels(lib: str) -> None:
    """A shared library links with undefined symbols.  One of the library's own (a kernel whose host stub the
    compiler did not emit) would only show at load time on the GPU box: refuse it here."""
    res = subprocess.run(["nm", "-D", "--undefined-only", lib], capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"nm failed on {lib}:\n{res.stderr}")
    own = [l.split()[-1] for l in res.stdout.splitlines() if "_ZN3oxq" in l or " oxq_" in l]
    if own:
        raise RuntimeError(f"{lib} has undefined symbols of its own (first of {len(own)}): {own[0]}")


if __name__ == "__main__":
    print(build(force="--force" in sys.argv))
