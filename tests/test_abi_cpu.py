"""No-GPU tests of the C ABI: the library loads, exports every declared symbol,
and its device-free validation layer rejects what the reference rejects
(metal_ops.rs:1507-1566, 1984-2044, 5357-5431, 6011-6058; awq.rs:1096-1121;
metal_ops.rs:3943-3958) before anything would be launched.
"""
import ctypes as C
import os
import re
import subprocess

import numpy as np
import pytest

from oxydllm_amd import _lib
from tests.helpers import fake

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
F16, BF16, F32, U8, I32, I64 = _lib.F16, _lib.BF16, _lib.F32, _lib.U8, _lib.I32, _lib.I64


@pytest.fixture(scope="module")
def lib():
    return _lib.load()


@pytest.fixture()
def ctx(lib):
    h = C.c_void_p()
    assert lib.oxq_ctx_create(_lib.DEVICE_PLAN_ONLY, C.byref(h)) == 0
    yield h
    lib.oxq_ctx_destroy(h)


def err(lib):
    return lib.oxq_last_error().decode()


def plan(lib, ctx):
    p = _lib.OxqPlan()
    assert lib.oxq_ctx_last_plan(ctx, C.byref(p)) == 0
    return p


def test_library_exports_every_declared_symbol(lib):
    import glob
    headers = sorted(glob.glob(os.path.join(ROOT, "include", "*.h")))
    assert [os.path.basename(h) for h in headers] == ["oxq.h", "oxq_bench.h", "oxq_files.h"]
    header = "".join(open(h).read() for h in headers)
    declared = set(re.findall(r"^(?:int|int64_t|uint64_t|void|const char \*)\s*\*?(oxq_[a-z0-9_]+)\s*\(", header, re.M))
    assert len(declared) >= 30
    missing = [n for n in sorted(declared) if not hasattr(lib, n)]
    assert not missing, f"not exported: {missing}"
    assert declared == set(_lib.SIGNATURES), "binding table out of sync with include/*.h"


def test_version_and_status_names(lib):
    a, b = C.c_int(-1), C.c_int(-1)
    lib.oxq_version(C.byref(a), C.byref(b))
    assert (a.value, b.value) == (0, 1)
    assert lib.oxq_status_name(-5) == b"OXQ_ERR_M_RANGE"
    for code, name in _lib.STATUS.items():
        assert lib.oxq_status_name(code).decode() == name


def test_weight_cache_controls_answer_without_a_gpu(lib, ctx):
    """A plan-only ctx never builds a copy: the controls accept, report an empty cache, and reject
    what cannot be a size."""
    assert lib.oxq_ctx_set_weight_cache(ctx, 1 << 30) == 0
    b, n = C.c_int64(-1), C.c_int64(-1)
    assert lib.oxq_ctx_weight_cache_bytes(ctx, C.byref(b), C.byref(n)) == 0
    assert (b.value, n.value) == (0, 0)
    assert lib.oxq_ctx_forget_weights(ctx, None) == 0
    assert lib.oxq_ctx_forget_weights(ctx, C.c_void_p(0x1000)) == 0
    assert lib.oxq_ctx_set_weight_cache(ctx, -1) == -1 and "negative" in err(lib)
    assert lib.oxq_ctx_set_weight_cache(None, 0) == -1
    assert lib.oxq_ctx_set_weight_cache(ctx, 0) == 0


def test_gguf_block_layout_matches_reference(lib):
    """metal_ops.rs:5228-5241."""
    want = {_lib.GGUF_Q4_0: (32, 18), _lib.GGUF_Q8_0: (32, 34), _lib.GGUF_Q4_K: (256, 144),
            _lib.GGUF_Q6_K: (256, 210), _lib.GGUF_Q4_1: (32, 20), _lib.GGUF_Q5_0: (32, 22),
            _lib.GGUF_Q5_1: (32, 24), _lib.GGUF_Q2_K: (256, 84), _lib.GGUF_Q3_K: (256, 110),
            _lib.GGUF_Q5_K: (256, 176)}
    for q, (e, b) in want.items():
        ee, bb = C.c_int64(), C.c_int64()
        assert lib.oxq_gguf_block_layout(q, C.byref(ee), C.byref(bb)) == 0
        assert (ee.value, bb.value) == (e, b)
    assert lib.oxq_gguf_block_layout(17, None, None) == -1


def _awq(K, N, g, dt=F16, bits=4):
    pf = 32 // bits
    return (fake((K, N // pf), I32), fake((K // g, N // pf), I32), fake((K // g, N), dt))


def test_w4a16_accepts_valid_and_reports_plan(lib, ctx):
    qw, qz, sc = _awq(4096, 14336, 128)
    x, out = fake((1, 4096), F16), fake((1, 14336), F16)
    assert lib.oxq_w4a16_matmul(ctx, None, C.byref(x), C.byref(qw), C.byref(qz), C.byref(sc),
                                C.byref(out)) == 0, err(lib)
    p = plan(lib, ctx)
    assert p.kernel.decode().startswith("awq4_gemv_fast_f16_m1")
    assert p.block[0] % 64 == 0 and p.split_k == p.grid[1] >= 1
    assert p.grid[0] * p.grid[1] >= 128          # enough workgroups for 256 CUs
    assert p.workspace_bytes == (p.split_k * 14336 * 4 if p.split_k > 1 else 0)
    assert p.launches == (2 if p.split_k > 4 else 1)  # many slices -> separate reduce launch
    # odd shape falls to the generic kernel (N not a multiple of 32)
    qw, qz, sc = _awq(192, 104, 64)
    x, out = fake((3, 192), BF16), fake((3, 104), BF16)
    sc.dtype = BF16
    assert lib.oxq_w4a16_matmul(ctx, None, C.byref(x), C.byref(qw), C.byref(qz), C.byref(sc),
                                C.byref(out)) == 0, err(lib)
    assert "awq_gemv_generic_w4_bf16_m4" in plan(lib, ctx).kernel.decode()


def test_w4a16_rejects_host_tensors(lib, ctx):
    """metal_ops.rs:3943-3958 w4a16_matmul_rejects_cpu_tensors."""
    qw, qz, sc = _awq(64, 64, 32)
    x, out = fake((1, 64), F16, device=_lib.DEVICE_HOST), fake((1, 64), F16)
    rc = lib.oxq_w4a16_matmul(ctx, None, C.byref(x), C.byref(qw), C.byref(qz), C.byref(sc), C.byref(out))
    assert rc == -7 and "GPU-resident" in err(lib)


@pytest.mark.parametrize("m", [0, 9, 64])
def test_gemv_m_range(lib, ctx, m):
    qw, qz, sc = _awq(256, 128, 64)
    x, out = fake((m, 256), F16), fake((m, 128), F16)
    rc = lib.oxq_w4a16_matmul(ctx, None, C.byref(x), C.byref(qw), C.byref(qz), C.byref(sc), C.byref(out))
    assert rc == -5 and "m in 1..=8" in err(lib)
    g = (fake((256 // 8, 128), I32), fake((4, 128 // 8), I32), fake((4, 128), F16))
    rc = lib.oxq_gptq_matmul(ctx, None, C.byref(x), C.byref(g[0]), C.byref(g[1]), C.byref(g[2]), 4,
                             C.byref(out))
    assert rc == -5


def test_wna16_validation_errors(lib, ctx):
    K, N, g = 256, 128, 64
    qw, qz, sc = _awq(K, N, g)
    x, out = fake((1, K), F16), fake((1, N), F16)

    def call(x=x, qw=qw, qz=qz, sc=sc, out=out):
        return lib.oxq_w4a16_matmul(ctx, None, C.byref(x), C.byref(qw), C.byref(qz), C.byref(sc),
                                    C.byref(out))

    assert call() == 0
    assert call(x=fake((1, K), F16, contiguous=False)) == -4 and "contiguous" in err(lib)
    assert call(x=fake((K,), F16)) == -3
    assert call(qz=fake((K // g, N // 8 + 1), I32)) == -3 and "qzeros shape" in err(lib)
    assert call(qw=fake((K, N // 8 - 1), I32), qz=fake((K // g, N // 8 - 1), I32)) == -3
    assert "packed_out" in err(lib)
    assert call(x=fake((1, K + 32), F16)) == -3 and "in_features" in err(lib)
    assert call(out=fake((1, N + 8), F16)) == -3 and "output shape" in err(lib)
    assert call(x=fake((1, K), BF16)) == -2 and "must match x dtype" in err(lib)
    assert call(x=fake((1, K), F32), sc=fake((K // g, N), F32), out=fake((1, N), F32)) == -2
    assert "unsupported (bits, dtype) combo" in err(lib)
    assert call(qw=fake((K, N // 8), I64)) == -2
    # 3 groups of 85.33: not divisible
    assert call(qz=fake((3, N // 8), I32), sc=fake((3, N), F16)) == -6 and "not divisible" in err(lib)
    # group size 96 (K=288): not a power of two
    qw2, qz2, sc2 = _awq(288, N, 96)
    assert call(x=fake((1, 288), F16), qw=qw2, qz=qz2, sc=sc2) == -6 and "power of two" in err(lib)
    assert lib.oxq_w4a16_matmul(None, None, C.byref(x), C.byref(qw), C.byref(qz), C.byref(sc),
                                C.byref(out)) == -1
    assert lib.oxq_w4a16_matmul(ctx, None, None, C.byref(qw), C.byref(qz), C.byref(sc), C.byref(out)) == -1


def test_awq_shape_rejection_from_reference(lib, ctx):
    """awq.rs:1096-1121: qweight [8,2], qzeros [2,2], scales [2,8]."""
    qw, qz, sc = fake((8, 2), I32), fake((2, 2), I32), fake((2, 8), F16)
    out = fake((8, 8), F16)
    assert lib.oxq_dequantize_w4(ctx, None, C.byref(qw), C.byref(qz), C.byref(sc), C.byref(out)) == -3


def test_gptq_validation(lib, ctx):
    K, N, g = 5120, 13824, 128
    for bits in (4, 8):
        pf = 32 // bits
        qw, qz, sc = fake((K // pf, N), I32), fake((K // g, N // pf), I32), fake((K // g, N), BF16)
        x, out = fake((8, K), BF16), fake((8, N), BF16)
        assert lib.oxq_gptq_matmul(ctx, None, C.byref(x), C.byref(qw), C.byref(qz), C.byref(sc), bits,
                                   C.byref(out)) == 0, err(lib)
        assert plan(lib, ctx).kernel.decode() == f"gptq{bits}_tile_bf16_mt1"  # the tile kernel on the checkpoint layout
        bad = fake((K // g, N // pf + 1), I32)
        assert lib.oxq_gptq_matmul(ctx, None, C.byref(x), C.byref(qw), C.byref(bad), C.byref(sc),
                                   bits, C.byref(out)) == -3
        w = fake((K, N), BF16)
        assert lib.oxq_dequantize_gptq_packed(ctx, None, C.byref(qw), C.byref(qz), C.byref(sc), bits,
                                              C.byref(w)) == 0
    assert lib.oxq_gptq_matmul(ctx, None, C.byref(x), C.byref(qw), C.byref(qz), C.byref(sc), 3,
                               C.byref(out)) == -8
    assert "bits must be 4 or 8" in err(lib)
    qw_bad = fake((K // 8, N + 8), I32)
    assert lib.oxq_gptq_matmul(ctx, None, C.byref(x), C.byref(qw_bad), C.byref(qz), C.byref(sc), 8,
                               C.byref(out)) == -3 and "qweight dim1" in err(lib)


def test_maybe_mpp_declines_like_reference(lib, ctx):
    """metal_ops.rs:2779-2791: small m, wrong dtype, non-contiguous -> Ok(None)."""
    qw, qz, sc = _awq(4096, 14336, 128)
    taken = C.c_int(7)

    def call(x, out, sc=sc):
        return lib.oxq_maybe_mpp_quant_matmul(ctx, None, C.byref(x), C.byref(qw), C.byref(qz),
                                              C.byref(sc), 4, _lib.PACK_OUT, C.byref(out),
                                              C.byref(taken))

    assert call(fake((4, 4096), F16), fake((4, 14336), F16)) == 0 and taken.value == 0
    assert call(fake((64, 4096), F32), fake((64, 14336), F32)) == 0 and taken.value == 0
    assert call(fake((64, 4096), F16, contiguous=False), fake((64, 14336), F16)) == 0
    assert taken.value == 0
    assert call(fake((64, 4096), F16), fake((64, 14336), F16)) == 0 and taken.value == 1
    p = plan(lib, ctx)
    assert p.kernel.decode() == "awq4_mfma_pipe_f16_mt4" and p.grid[0] == 28 and p.grid[2] == 1
    assert p.launches == 2 and p.workspace_bytes == p.split_k * 64 * 14336 * 4
    assert call(fake((16, 4096), F16), fake((16, 14336), F16)) == 0 and taken.value == 1
    assert plan(lib, ctx).kernel.decode() == "awq4_mfma_pipe_f16_mt1"
    # a real error is still an error
    assert call(fake((64, 4000), F16), fake((64, 14336), F16)) == -3 and taken.value == 0


def test_gguf_validation(lib, ctx):
    K, N = 4096, 4096
    for q, (be, bb) in {_lib.GGUF_Q4_0: (32, 18), _lib.GGUF_Q6_K: (256, 210), _lib.GGUF_Q5_1: (32, 24),
                        _lib.GGUF_Q3_K: (256, 110)}.items():
        w = fake((N * (K // be) * bb,), U8)
        x, out = fake((1, K), BF16), fake((1, N), BF16)

        def call(x=x, w=w, out=out, k=K, n=N, fn=lib.oxq_gguf_quant_matmul):
            return fn(ctx, None, C.byref(x), C.byref(w), k, n, q, C.byref(out))

        assert call() == 0, err(lib)
        assert call(x=fake((1, K), F32), out=fake((1, N), F32)) == 0, err(lib)
        assert call(x=fake((1, K), F16), out=fake((1, N), F16)) == -2 and "BF16" in err(lib)
        assert call(w=fake((N * (K // be) * bb,), I32)) == -2 and "U8" in err(lib)
        assert call(k=K + 8, x=fake((1, K + 8), BF16)) == -3 and "multiple of" in err(lib)
        assert call(x=fake((9, K), BF16), out=fake((9, N), BF16)) == -5 and "out of [1, 8]" in err(lib)
        assert call(x=fake((9, K), BF16), out=fake((9, N), BF16), fn=lib.oxq_gguf_quant_mul_mm) == 0
        assert call(x=fake((1, K), BF16, contiguous=False)) == -4
        assert call(x=fake((1, K - 256), BF16)) == -3 and "x shape" in err(lib)
        assert call(out=fake((1, N - 1), BF16)) == -3 and "output shape" in err(lib)
        assert call(w=fake((N * (K // be) * bb - bb,), U8)) == -3 and "expected" in err(lib)
        assert call(x=fake((1, K), BF16, device=_lib.DEVICE_HOST)) == -7
    # odd N (reference tests n in {1001, 49159}, metal_ops.rs:6471-6536)
    w = fake((1001 * 128 * 18,), U8)
    assert lib.oxq_gguf_quant_matmul(ctx, None, C.byref(fake((1, 4096), BF16)), C.byref(w), 4096,
                                     1001, _lib.GGUF_Q4_0, C.byref(fake((1, 1001), BF16))) == 0


def test_mxfp4_validation(lib, ctx):
    K, N = 2880, 5760
    nb = K // 32
    blocks, scales = fake((N * nb * 16,), U8), fake((N * nb,), U8)
    x, out = fake((8, K), BF16), fake((8, N), BF16)

    def call(x=x, b=blocks, s=scales, out=out, k=K, n=N):
        return lib.oxq_mxfp4_matmul(ctx, None, C.byref(x), C.byref(b), C.byref(s), k, n, C.byref(out))

    assert call() == 0, err(lib)
    assert call(x=fake((33, K), BF16), out=fake((33, N), BF16)) == 0  # any m (mul_mm above 8)
    assert call(x=fake((8, K), F16)) == -2 and "BF16" in err(lib)
    assert call(b=fake((N * nb * 16,), I32)) == -2
    assert call(k=K + 16, x=fake((8, K + 16), BF16)) == -3 and "multiple of 32" in err(lib)
    assert call(b=fake((N * nb * 16 - 16,), U8)) == -3 and "don't match" in err(lib)
    assert call(x=fake((8, K), BF16, contiguous=False)) == -4
    assert call(x=fake((8, K - 32), BF16)) == -3
    assert call(out=fake((7, N), BF16)) == -3 and "output shape" in err(lib)


def test_resident_experts_pick_their_kernel_by_pairs(lib, ctx):
    """oxq_mxfp4_experts_* (moe.rs:366-417, 563-607): below three pairs an expert on average the decode GEMV on the
    copy, above it tiles of an expert's pairs whose rows follow the average; a shape without whole tiles of 16
    weight rows keeps the checkpoint-layout kernels."""
    E, K, N = 32, 2880, 5760
    nb = K // 32
    blocks, scales = fake((E * N * nb * 16,), U8), fake((E * N * nb,), U8)
    h = C.c_void_p()
    assert lib.oxq_mxfp4_experts_new(ctx, C.byref(blocks), C.byref(scales), None, E, K, N, C.byref(h)) == 0, err(lib)
    off = fake((E + 1,), I32)
    for tokens, kern, ytiles in [(8, "mxfp4_experts_gemv_bf16_t4", None), (24, "mxfp4_experts_gemm_bf16_r16x8", 96 // 16 + E),
                                 (96, "mxfp4_experts_gemm_bf16_r16x8", 384 // 16 + E), (128, "mxfp4_experts_gemm_bf16_r32x8", 512 // 32 + E),
                                 (512, "mxfp4_experts_gemm_bf16_r32x8", 2048 // 32 + E), (1024, "mxfp4_experts_gemm_bf16_r64x8", 4096 // 64 + E),
                                 (4096, "mxfp4_experts_gemm_bf16_r128x8", 16384 // 128 + E)]:
        pairs = 4 * tokens
        x, tok = fake((tokens, K), BF16), fake((pairs,), I32)
        assert lib.oxq_mxfp4_experts_matmul(h, None, C.byref(x), C.byref(off), C.byref(tok), 1, C.byref(fake((pairs, N), BF16))) == 0, err(lib)
        pl = plan(lib, ctx)
        assert pl.kernel.decode() == kern and pl.launches == 1, (tokens, pl.kernel)
        if ytiles is not None:
            assert (pl.grid[0], pl.grid[1], pl.block[0]) == (12, ytiles, 512), (tokens, tuple(pl.grid))
        fused = C.c_int(-1)
        assert lib.oxq_mxfp4_experts_gate_up_swiglu(h, None, C.byref(x), C.byref(off), C.byref(tok), 1, 7.0,
                                                    C.byref(fake((pairs, N // 2), BF16)), C.byref(fused)) == 0, err(lib)
        assert fused.value == 1 and plan(lib, ctx).kernel.decode() == kern + "_swiglu"
    x, tok = fake((128, K), BF16), fake((512,), I32)
    assert lib.oxq_mxfp4_experts_matmul(h, None, C.byref(x), C.byref(off), C.byref(tok), 1, C.byref(fake((512, N + 16), BF16))) == -3
    assert lib.oxq_mxfp4_experts_matmul(h, None, C.byref(x), C.byref(off), C.byref(fake((500,), I32)), 1, C.byref(fake((512, N), BF16))) == -3
    assert "token_ids" in err(lib)
    lib.oxq_mxfp4_experts_free(h)


def test_feed_forward_validates_and_plans(lib, ctx):
    """ffn.rs:22-474 at the benchmark's layer size: layouts, shape checks, scratch sizes, launch plans."""
    H, I = 4096, 14336

    def packed(k, n, act=None):
        h = C.c_void_p()
        qw, qz, sc = _awq(k, n, 128, BF16)
        if act is None:
            rc = lib.oxq_packed_quant_linear_new(ctx, 4, 0, C.byref(qw), C.byref(qz), C.byref(sc), None, BF16, C.byref(h))
        else:
            rc = lib.oxq_packed_quant_linear_new_gate_up(ctx, 4, 0, C.byref(qw), C.byref(qz), C.byref(sc), None, act,
                                                         BF16, C.byref(h))
        assert rc == 0, err(lib)
        return h

    def any_(kind, h):
        return C.byref(_lib.OxqAnyLinear(kind, h)) if h is not None else None

    def new(kind, a, b, down, inter=I, act=0, lk=0):
        m = C.c_void_p()
        return lib.oxq_mlp_new(ctx, kind, any_(lk, a), any_(lk, b), any_(lk, down), inter, act, C.byref(m)), m

    gate, up, both, epi, down = packed(H, I), packed(H, I), packed(H, 2 * I), packed(H, 2 * I, 0), packed(I, H)
    x, out = fake((2, 3, H), BF16), fake((2, 3, H), BF16)
    for kind, a, b, per_row in [(1, gate, up, 2 * I), (0, both, None, 3 * I), (0, epi, None, I), (2, up, None, I)]:
        rc, m = new(kind, a, b, down)
        assert rc == 0, err(lib)
        e, k, n = C.c_int64(), C.c_int64(), C.c_int64()
        assert lib.oxq_mlp_scratch_elems(m, 6, C.byref(e)) == 0 and e.value == 6 * per_row
        assert lib.oxq_mlp_in_features(m, C.byref(k)) == 0 and lib.oxq_mlp_out_features(m, C.byref(n)) == 0
        assert (k.value, n.value) == (H, H)
        assert lib.oxq_mlp_forward(m, None, C.byref(x), C.byref(fake((6 * per_row,), BF16)), C.byref(out)) == 0, err(lib)
        assert plan(lib, ctx).kernel.decode().startswith("pk4_mfma_bf16_mt1_gs")       # the last launch: down_proj
        assert lib.oxq_mlp_forward(m, None, C.byref(x), C.byref(fake((6 * per_row - 1,), BF16)), C.byref(out)) == -3
        assert f"at least {6 * per_row} elements" in err(lib)
        assert lib.oxq_mlp_forward(m, None, C.byref(x), C.byref(fake((6 * per_row,), F16)), C.byref(out)) == -3
        assert lib.oxq_mlp_forward(m, None, C.byref(fake((6, H + 1), BF16)), C.byref(fake((6 * per_row,), BF16)),
                                   C.byref(out)) == -3 and "in_features" in err(lib)
        lib.oxq_mlp_free(m)
    # refusals, in the reference's words where it has them
    for args, code, text in [((1, gate, both, down), -3, "gate/up out_features must both be 14336, got 14336 and 28672"),
                             ((0, gate, None, down), -3, "gate_up out_features 14336 != 2*14336"),
                             ((1, gate, up, gate), -3, "down_proj in_features 4096 != intermediate size 14336"),
                             ((0, both, up, down), -1, "second projection"),
                             ((1, gate, None, down), -1, "second projection"),
                             ((2, epi, None, down), -1, "only be the fused gate_up_proj"),
                             ((5, both, None, down), -1, "unknown gate/up layout 5")]:
        rc, _ = new(*args)
        assert rc == code and text in err(lib), (args[0], rc, err(lib))
    rc, _ = new(0, epi, None, down, act=1)
    assert rc == -1 and "another activation" in err(lib)
    rc, _ = new(0, both, None, down, act=2)
    assert rc == -1 and "activation must be" in err(lib)
    rc, _ = new(0, both, None, down, lk=9)
    assert rc == -1 and "unknown layer kind 9" in err(lib)
    assert lib.oxq_mlp_forward(None, None, C.byref(x), C.byref(x), C.byref(out)) == -1
    lib.oxq_mlp_free(None)
    # block-quantized projections (ffn.rs:307-373) with the separate layout
    def gguf(n, k):
        q = C.c_void_p()
        assert lib.oxq_qlinear_new(ctx, _lib.GGUF_Q4_K, C.byref(fake((n * (k // 256) * 144,), U8)), k, n, None, BF16,
                                   C.byref(q)) == 0, err(lib)
        return q
    qg, qu, qd = gguf(I, H), gguf(I, H), gguf(H, I)
    rc, m = new(1, qg, qu, qd, lk=1)
    assert rc == 0, err(lib)
    assert lib.oxq_mlp_forward(m, None, C.byref(fake((1, H), BF16)), C.byref(fake((2 * I,), BF16)),
                               C.byref(fake((1, H), BF16))) == 0, err(lib)
    assert plan(lib, ctx).kernel.decode().startswith("gguf_q4k_mfma_bf16_mt1")  # a bf16 layer: the matrix-core copy
    lib.oxq_mlp_free(m)
    # the fused gate|up projection of a block-quantized FFN with the activation in its epilogue (ffn.rs:307-373 Packed)
    both_bytes = fake((2 * I * (H // 256) * 144,), U8)
    qf = C.c_void_p()
    assert lib.oxq_qlinear_new_gate_up(ctx, _lib.GGUF_Q4_K, C.byref(both_bytes), H, 2 * I, None, 2, BF16, C.byref(qf)) == -1
    assert "activation must be" in err(lib)
    assert lib.oxq_qlinear_new_gate_up(ctx, _lib.GGUF_Q4_K, C.byref(both_bytes), H, 2 * I, None, 0, F32, C.byref(qf)) == -11
    assert "needs a BF16 layer on the matrix-core copy" in err(lib)
    assert lib.oxq_qlinear_new_gate_up(ctx, _lib.GGUF_Q4_K, C.byref(both_bytes), H, 2 * I, None, 0, BF16, C.byref(qf)) == 0, err(lib)
    assert lib.oxq_qlinear_forward(qf, None, C.byref(fake((3, H), BF16)), C.byref(fake((3, 2 * I), BF16))) == -3
    assert lib.oxq_qlinear_forward(qf, None, C.byref(fake((3, H), BF16)), C.byref(fake((3, I), BF16))) == 0, err(lib)
    assert plan(lib, ctx).kernel.decode() == "gguf_q4k_mfma_bf16_mt1_n64_act"
    rc, m = new(0, qf, None, qd, lk=1)
    assert rc == 0, err(lib)
    elems = C.c_int64()
    assert lib.oxq_mlp_scratch_elems(m, 2, C.byref(elems)) == 0 and elems.value == 2 * 3 * I
    for rows, kern in [(2, "gguf_q4k_mfma_bf16_mt1"), (100, "gguf_q4k_mul_mm_bf16")]:  # the down projection ran last
        assert lib.oxq_mlp_forward(m, None, C.byref(fake((rows, H), BF16)), C.byref(fake((rows * 3 * I,), BF16)),
                                   C.byref(fake((rows, H), BF16))) == 0, err(lib)
        assert plan(lib, ctx).kernel.decode().startswith(kern), plan(lib, ctx).kernel
    lib.oxq_mlp_free(m)
    lib.oxq_qlinear_free(qf)
    for h in (qg, qu, qd):
        lib.oxq_qlinear_free(h)
    for h in (gate, up, both, epi, down):
        lib.oxq_packed_quant_linear_free(h)


def test_layers_validate_like_reference(lib, ctx):
    h = C.c_void_p()
    qw, qz, sc = _awq(4096, 14336, 128, BF16)
    # linear.rs:417-419 bits; 420-422 qzeros missing; 431-436 scales mismatch
    assert lib.oxq_packed_quant_linear_new(ctx, 3, 0, C.byref(qw), C.byref(qz), C.byref(sc), None,
                                           BF16, C.byref(h)) == -8
    assert lib.oxq_packed_quant_linear_new(ctx, 4, 0, C.byref(qw), None, C.byref(sc), None, BF16,
                                           C.byref(h)) == -1 and "qzeros missing" in err(lib)
    bad_sc = fake((32, 14336 + 8), BF16)
    assert lib.oxq_packed_quant_linear_new(ctx, 4, 0, C.byref(qw), C.byref(qz), C.byref(bad_sc), None,
                                           BF16, C.byref(h)) == -3 and "derived" in err(lib)
    assert lib.oxq_packed_quant_linear_new(ctx, 4, 0, C.byref(qw), C.byref(qz), C.byref(sc), None,
                                           BF16, C.byref(h)) == 0, err(lib)
    k, n = C.c_int64(), C.c_int64()
    lib.oxq_packed_quant_linear_in_features(h, C.byref(k))
    lib.oxq_packed_quant_linear_out_features(h, C.byref(n))
    assert (k.value, n.value) == (4096, 14336)
    # this layer is tile-aligned, so it is repacked at load and one kernel serves every m
    # (m <= 16: unrounded-weight form, above: tile-GEMM form); leading dims flatten
    flag = C.c_int(-1)
    assert lib.oxq_packed_quant_linear_is_prepacked(h, C.byref(flag)) == 0 and flag.value == 1
    for shape, kern in [((1, 4096), "pk4_mfma_bf16_mt1_gs"), ((2, 3, 4096), "pk4_mfma_bf16_mt1_gs"),
                        ((16, 4096), "pk4_mfma_bf16_mt1_gs"), ((17, 4096), "pk4_mfma_bf16_mt2"),
                        ((4, 16, 4096), "pk4_mfma_bf16_mt4")]:
        x = fake(shape, BF16)
        out = fake(shape[:-1] + (14336,), BF16)
        assert lib.oxq_packed_quant_linear_forward(h, None, C.byref(x), C.byref(out)) == 0, err(lib)
        assert plan(lib, ctx).kernel.decode().startswith(kern), plan(lib, ctx).kernel
    # beyond one row tile: 112 pairs of strips x row tiles of 64 with K split inside the workgroup while 28 groups
    # of eight strips would leave most of the chip idle, then row tiles of 64 or 128 x eight strips, whichever needs
    # the cheaper rounds of 256 workgroups
    for rows, kern, wgs in [(64, "pk4_mfma_bf16_mt4", None), (65, "pk4_gemm_bf16_r64x2k4", 2 * 112),
                            (256, "pk4_gemm_bf16_r64x2k4", 4 * 112), (384, "pk4_gemm_bf16_r64x2k4", 6 * 112), (448, "pk4_gemm_bf16_r64x8", 7 * 28),
                            (512, "pk4_gemm_bf16_r64x8", 4 * 64),
                            (768, "pk4_gemm_bf16_r128x8", 6 * 28), (1000, "pk4_gemm_bf16_r128x8", 4 * 64),
                            (1536, "pk4_gemm_bf16_r64x8", 3 * 4 * 64), (1537, "pk4_gemm_bf16_r64x8", 3 * 4 * 64 + 28),
                            (2100, "pk4_gemm_bf16_r128x8", 2 * 4 * 64 + 28),
                            (4096, "pk4_gemm_bf16_r128x8", 4 * 4 * 64)]:
        x = fake((rows, 4096), BF16)
        assert lib.oxq_packed_quant_linear_forward(h, None, C.byref(x), C.byref(fake((rows, 14336), BF16))) == 0, err(lib)
        pl = plan(lib, ctx)
        assert pl.kernel.decode().startswith(kern), (rows, pl.kernel)
        if wgs is not None:
            assert (pl.grid[0], pl.block[0], pl.launches) == (wgs, 512, 1), (rows, tuple(pl.grid))
    x = fake((1, 4000), BF16)
    assert lib.oxq_packed_quant_linear_forward(h, None, C.byref(x), C.byref(fake((1, 14336), BF16))) == -3
    assert "input last dim 4000 != in_features 4096" in err(lib)
    lib.oxq_packed_quant_linear_free(h)
    # a narrow layer (16-column strips): eight groups of 512 columns fill the chip from 2048 rows on; below, 32 pairs
    # of 64-column groups x row tiles with K split inside the workgroup, from where the split-K tiles need a second
    # round of 256 workgroups
    nqw, nqz, nsc = _awq(4096, 4096, 128, F16)
    assert lib.oxq_packed_quant_linear_new(ctx, 4, 0, C.byref(nqw), C.byref(nqz), C.byref(nsc), None,
                                           F16, C.byref(h)) == 0, err(lib)
    for rows, kern, wgs in [(64, "pk4_mfma_f16_mt4_n16x4", None), (256, "pk4_mfma_f16_mt4_n16x4", None),
                            (384, "pk4_gemm_f16_r64x2k4_n16", 6 * 32), (1024, "pk4_gemm_f16_r64x2k4_n16", 16 * 32),
                            (1536, "pk4_gemm_f16_r64x8_n16", 192), (2048, "pk4_gemm_f16_r64x8_n16", 256), (4096, "pk4_gemm_f16_r128x8_n16", 256),
                            (4100, "pk4_gemm_f16_r64x2k4_n16", 65 * 32)]:  # four rows past two rounds of 128-row workgroups
        assert lib.oxq_packed_quant_linear_forward(h, None, C.byref(fake((rows, 4096), F16)),
                                                   C.byref(fake((rows, 4096), F16))) == 0, err(lib)
        pl = plan(lib, ctx)
        assert pl.kernel.decode().startswith(kern), (rows, pl.kernel)
        if wgs is not None:
            assert (pl.grid[0], pl.block[0], pl.launches) == (wgs, 512, 1), (rows, tuple(pl.grid))
    lib.oxq_packed_quant_linear_free(h)

    # Mxfp4Linear::new (mxfp4.rs:85-105)
    m = C.c_void_p()
    b, s = fake((10 * 2 * 16,), U8), fake((10 * 2,), U8)
    assert lib.oxq_mxfp4_linear_new(ctx, C.byref(b), C.byref(s), None, 64, 10, C.byref(m)) == 0
    assert lib.oxq_mxfp4_linear_forward(m, None, C.byref(fake((3, 64), BF16)),
                                        C.byref(fake((3, 10), BF16))) == 0, err(lib)
    assert lib.oxq_mxfp4_linear_forward(m, None, C.byref(fake((3, 32), BF16)),
                                        C.byref(fake((3, 10), BF16))) == -3
    assert "x last dim 32 != in_features 64" in err(lib)
    lib.oxq_mxfp4_linear_free(m)
    assert lib.oxq_mxfp4_linear_new(ctx, C.byref(b), C.byref(s), None, 48, 10, C.byref(m)) == -3
    assert lib.oxq_mxfp4_linear_new(ctx, C.byref(fake((320,), I32)), C.byref(s), None, 64, 10,
                                    C.byref(m)) == -2
    assert lib.oxq_mxfp4_linear_new(ctx, C.byref(b), C.byref(s), None, 64, 11, C.byref(m)) == -3

    # QLinear / GgufFastPath::build (linear.rs:197-247)
    q = C.c_void_p()
    w = fake((4096 * 16 * 144,), U8)
    assert lib.oxq_qlinear_new(ctx, _lib.GGUF_Q4_K, C.byref(w), 4096, 4096, None, BF16, C.byref(q)) == 0
    # rows 1-4: the GEMV on the layer's strip-major copy; 5-8 the tile matmul with unrounded weights
    for m_rows, kern in [(1, "gguf_q4k_mfma_bf16_mt1"), (2, "gguf_q4k_mfma_bf16_mt1"),
                         (4, "gguf_q4k_mfma_bf16_mt1"), (8, "gguf_q4k_mfma_bf16_mt1"),
                         (16, "gguf_q4k_mfma_bf16_mt1"), (32, "gguf_q4k_mfma_bf16_mt2"), (33, "gguf_q4k_mul_mm_bf16_mt4"),
                         # more rows: the tile matmul on the file layout, then the kernels on the layer's copy - 32
                         # pairs of column groups x row tiles of 64 with K split inside the workgroup, and eight groups
                         # of 512 columns x row tiles once those fill the chip
                         (128, "gguf_q4k_mul_mm_bf16_mt4"), (256, "gguf_q4k_gemm_bf16_r64x2k4"),
                         (1024, "gguf_q4k_gemm_bf16_r64x2k4"), (2048, "gguf_q4k_gemm_bf16_r64x8"),
                         (4096, "gguf_q4k_gemm_bf16_r64x8")]:
        assert lib.oxq_qlinear_forward(q, None, C.byref(fake((m_rows, 4096), BF16)),
                                       C.byref(fake((m_rows, 4096), BF16))) == 0, err(lib)
        p = plan(lib, ctx)
        assert p.kernel.decode().startswith(kern) and p.launches == (2 if p.split_k > 1 else 1)
    res = C.c_int(-1)
    assert lib.oxq_qlinear_is_resident(q, C.byref(res)) == 0 and res.value == 1
    assert lib.oxq_qlinear_dequantize(q, None, C.byref(fake((4096, 4096), F32))) == 0, err(lib)
    assert plan(lib, ctx).kernel.decode() == "gguf_q4k_mfma_dequant"
    assert lib.oxq_qlinear_dequantize(q, None, C.byref(fake((4096, 4095), F32))) == -3
    # a strided view of the right shape would be written past its storage: refused
    assert lib.oxq_qlinear_dequantize(q, None, C.byref(fake((4096, 4096), F32, contiguous=False))) == -4
    lib.oxq_qlinear_free(q)
    # a layer whose rows are not whole strips of 16 keeps the file layout
    w2k = fake((4104 * 16 * 84,), U8)
    assert lib.oxq_qlinear_new(ctx, _lib.GGUF_Q2_K, C.byref(w2k), 4096, 4104, None, BF16, C.byref(q)) == 0
    assert lib.oxq_qlinear_is_resident(q, C.byref(res)) == 0 and res.value == 0
    assert lib.oxq_qlinear_forward(q, None, C.byref(fake((1, 4096), BF16)), C.byref(fake((1, 4104), BF16))) == 0
    assert plan(lib, ctx).kernel.decode().startswith("gguf_q2k_gemv_bf16")
    lib.oxq_qlinear_free(q)
    assert lib.oxq_qlinear_new(ctx, _lib.GGUF_Q4_K, C.byref(w), 4096, 4095, None, BF16, C.byref(q)) == -3


def test_real_context_without_gpu_fails_loudly(lib):
    import torch
    if torch.cuda.is_available():
        pytest.skip("GPU present")
    h = C.c_void_p()
    rc = lib.oxq_ctx_create(0, C.byref(h))
    assert rc == -7 and "no HIP device" in err(lib)


def test_awq_load_time_transforms_validate_like_reference(lib, ctx):
    """awq.rs:188-206 (compressed_to_awq), 257-289 (concat_awq_along_out), 641-654 (rtn_quantize_awq)."""
    F32 = _lib.F32
    # compressed-tensors [out=4096, in/8=512], 32 groups -> AWQ [4096, 512] / [32, 512] / [32, 4096]
    wp, ws = fake((4096, 512), I32), fake((4096, 32), BF16)
    outs = [fake((4096, 512), I32), fake((32, 512), I32), fake((32, 4096), BF16)]

    def ct(wp=wp, ws=ws, outs=outs):
        return lib.oxq_compressed_to_awq(ctx, None, C.byref(wp), C.byref(ws), *[C.byref(o) for o in outs])
    assert ct() == 0, err(lib)
    assert plan(lib, ctx).kernel.decode() == "compressed_to_awq"
    assert ct(ws=fake((4000, 32), BF16)) == -3 and "weight_scale dim0 4000 != weight_packed out_features 4096" in err(lib)
    assert ct(ws=fake((4096, 3), BF16)) == -3 and "not divisible by scale groups" in err(lib)
    assert ct(wp=fake((4100, 512), I32), ws=fake((4100, 32), BF16)) == -3 and "pack factor" in err(lib)
    assert ct(wp=fake((4096, 512), F16)) == -2
    assert ct(outs=[outs[0], outs[1], fake((32, 4096), F16)]) == -2
    assert ct(outs=[fake((4096, 511), I32), outs[1], outs[2]]) == -3

    # concat: q/k/v-like parts of 4096 + 1024 + 1024 columns
    parts = [_awq(4096, n, 128, BF16) for n in (4096, 1024, 1024)]
    arrs = [(_lib.OxqTensor * 3)(*[p[i] for p in parts]) for i in range(3)]
    fo = _awq(4096, 6144, 128, BF16)

    def cat(n=3, arrs=arrs, fo=fo, bits=4):
        return lib.oxq_concat_awq_along_out(ctx, None, bits, n, arrs[0], arrs[1], arrs[2], *[C.byref(o) for o in fo])
    assert cat() == 0, err(lib)
    p = plan(lib, ctx)
    assert p.kernel.decode() == "concat_awq_along_out" and p.launches == 9
    assert cat(n=0) == -1 and "no parts" in err(lib)
    assert cat(bits=3) == -8
    assert cat(fo=_awq(4096, 6152, 128, BF16)) == -3
    bad = [_awq(4096, 4096, 128, BF16), _awq(2048, 1024, 128, BF16), parts[2]]
    barrs = [(_lib.OxqTensor * 3)(*[q[i] for q in bad]) for i in range(3)]
    assert cat(arrs=barrs) == -3 and "in_features mismatch at part 1: expected 4096, got 2048" in err(lib)
    bad = [parts[0], _awq(4096, 1024, 64, BF16), parts[2]]
    barrs = [(_lib.OxqTensor * 3)(*[q[i] for q in bad]) for i in range(3)]
    assert cat(arrs=barrs) == -3 and "group_size mismatch at part 1: expected 128, got 64" in err(lib)

    # rtn: tied lm_head [vocab, hidden]
    w = fake((151936, 4096), BF16)
    ro = [fake((4096, 151936 // 8), I32), fake((32, 151936 // 8), I32), fake((32, 151936), F32)]

    def rtn(w=w, g=128, ro=ro):
        return lib.oxq_rtn_quantize_awq(ctx, None, C.byref(w), g, *[C.byref(o) for o in ro])
    assert rtn() == 0, err(lib)
    p = plan(lib, ctx)
    assert p.kernel.decode() == "rtn_quantize_awq" and p.grid[0] == 151936 // 8 and p.block[0] == 512
    assert rtn(w=fake((151937, 4096), BF16)) == -3 and "must be a multiple of 8" in err(lib)
    assert rtn(g=96) == -6 and "not divisible by group_size (96)" in err(lib)
    assert rtn(g=0) == -6
    assert rtn(w=fake((151936, 4096), I32)) == -2
    assert rtn(ro=[ro[0], ro[1], fake((32, 151936), BF16)]) == -2


def test_f8_ops_validate_like_reference(lib, ctx):
    """metal_ops.rs:5589-5613 (dequant), 5703-5731 (gemv), moe.rs:106-113 (any m)."""
    F32 = _lib.F32
    b, sc = fake((2048, 512), U8), fake((16, 4), F32)
    x2, out2 = fake((2, 512), BF16), fake((2, 2048), BF16)
    assert lib.oxq_f8_gemv(ctx, None, C.byref(x2), C.byref(b), C.byref(sc), C.byref(out2)) == 0, err(lib)
    p = plan(lib, ctx)
    assert p.kernel.decode() == "f8_gemv_bf16" and p.grid[0] == 512 and p.launches == 1
    x, out = fake((4, 512), BF16), fake((4, 2048), BF16)
    assert lib.oxq_f8_gemv(ctx, None, C.byref(x), C.byref(b), C.byref(sc), C.byref(out)) == 0, err(lib)
    assert plan(lib, ctx).kernel.decode() == "f8_mul_mm_bf16_mt1"   # from 3 rows: the tile matmul
    x9, o9 = fake((9, 512), BF16), fake((9, 2048), BF16)
    assert lib.oxq_f8_gemv(ctx, None, C.byref(x9), C.byref(b), C.byref(sc), C.byref(o9)) == -5
    assert "m must be 1..=8" in err(lib)
    assert lib.oxq_f8_matmul(ctx, None, C.byref(x9), C.byref(b), C.byref(sc), C.byref(o9)) == 0, err(lib)
    assert plan(lib, ctx).kernel.decode().startswith("f8_mul_mm_bf16")
    assert lib.oxq_f8_gemv(ctx, None, C.byref(fake((4, 512), F16)), C.byref(b), C.byref(sc), C.byref(out)) == -2
    assert lib.oxq_f8_gemv(ctx, None, C.byref(x), C.byref(b), C.byref(fake((16, 3), F32)), C.byref(out)) == -3
    assert "scale grid [16, 3] does not tile weight [2048, 512]" in err(lib)
    assert lib.oxq_f8_gemv(ctx, None, C.byref(x), C.byref(fake((2048, 512), I32)), C.byref(sc), C.byref(out)) == -2
    dq = fake((2048, 512), BF16)
    assert lib.oxq_f8_block_dequant_bf16(ctx, None, C.byref(b), C.byref(sc), C.byref(dq)) == 0, err(lib)
    assert plan(lib, ctx).kernel.decode() == "f8_block_dequant_bf16"
    assert lib.oxq_f8_block_dequant_bf16(ctx, None, C.byref(b), C.byref(sc), C.byref(fake((2048, 512), F16))) == -3
    assert lib.oxq_cast_f8e4m3_to_f32(ctx, None, C.byref(b), C.byref(fake((2048, 512), F32))) == 0, err(lib)
    assert lib.oxq_cast_f8e4m3_to_f32(ctx, None, C.byref(fake((8,), I32)), C.byref(fake((8,), F32))) == -2
    assert lib.oxq_cast_f8e4m3_to_f32(ctx, None, C.byref(b), C.byref(fake((2048, 511), F32))) == -3


def test_random_descriptors_never_crash_and_always_explain(lib, ctx):
    """Validation reads descriptors only: whatever a caller passes - wrong ranks, negative or huge dims,
    unknown dtypes and enums, host or foreign-device tensors, NULL data - every entry point returns a
    status of the enum and, on failure, a message; nothing is launched (plan-only ctx) and nothing
    crashes.  Half of the cases start from a valid AWQ / GPTQ problem with one field corrupted."""
    rng = np.random.default_rng(20240607)
    DIMS = [0, 1, 2, 3, 7, 8, 16, 31, 32, 33, 64, 100, 128, 256, 1000, 4096, 14336, 2**31 - 1, 2**31, 2**40, 2**62, -1, -5]
    def rt():
        t = _lib.OxqTensor()
        t.data = int(rng.choice([0, 0x1000, 0x1001, 0x7f0000000010]))
        t.dtype = int(rng.integers(-2, 9))
        t.rank = int(rng.choice([0, 1, 2, 2, 2, 3, 4, 5, -1]))
        for i in range(4): t.dims[i] = int(rng.choice(DIMS))
        t.contiguous = int(rng.integers(0, 2))
        t.device = int(rng.choice([0, 0, 0, -1, 1, 7]))
        return t
    def _mk(shape, d):
        t = _lib.OxqTensor(); t.data = 0x1000; t.dtype = d; t.rank = len(shape)
        for i, s in enumerate(shape): t.dims[i] = s
        t.contiguous = 1; t.device = 0
        return t
    names = {}
    def call(name, *args):
        fn = getattr(lib, name)
        rc = fn(*args)
        assert -13 <= rc <= 0, (name, rc)
        names.setdefault(name, [0, 0])[0 if rc == 0 else 1] += 1
        if rc != 0:
            msg = lib.oxq_last_error()
            assert msg and len(msg) > 3, name
    N_IT = 500
    B = C.byref
    for it in range(N_IT):
        ts = [rt() for _ in range(8)]
        # half of the time start from a valid AWQ/GPTQ problem and corrupt one field
        if it % 2 == 0:
            bits = int(rng.choice([4, 8])); pf = 32 // bits
            K = int(rng.choice([128, 256, 4096])); N = int(rng.choice([64, 128, 14336])); g = int(rng.choice([32, 64, 128]))
            m = int(rng.choice([1, 4, 8, 9, 64]))
            dt = int(rng.choice([1, 2]))
            awq = it % 4 == 0
            ts[0] = _mk((m, K), dt)
            ts[1] = _mk((K, N // pf) if awq else (K // pf, N), 4)
            ts[2] = _mk((K // g, N // pf), 4)
            ts[3] = _mk((K // g, N), dt)
            ts[4] = _mk((m, N), dt)
            ts[5] = _mk((K, N), dt)
            v = ts[int(rng.integers(0, 6))]
            f = int(rng.integers(0, 5))
            if f == 0: v.dtype = int(rng.integers(-2, 9))
            elif f == 1: v.rank = int(rng.choice([0, 1, 3, 5]))
            elif f == 2: v.dims[int(rng.integers(0, 2))] = int(rng.choice(DIMS))
            elif f == 3: v.contiguous = 0
            else: v.device = int(rng.choice([-1, 1]))
        bits = int(rng.choice([4, 8, 0, 3, 16, 2**31]))
        pd = int(rng.choice([0, 1, 2, -1]))
        i64 = lambda: int(rng.choice(DIMS))
        q = int(rng.integers(-1, 12))
        taken = C.c_int()
        call("oxq_w4a16_matmul", ctx, None, B(ts[0]), B(ts[1]), B(ts[2]), B(ts[3]), B(ts[4]))
        call("oxq_w8a16_matmul", ctx, None, B(ts[0]), B(ts[1]), B(ts[2]), B(ts[3]), B(ts[4]))
        call("oxq_gptq_matmul", ctx, None, B(ts[0]), B(ts[1]), B(ts[2]), B(ts[3]), bits & 0xFFFFFFFF, B(ts[4]))
        call("oxq_dequantize_w4", ctx, None, B(ts[1]), B(ts[2]), B(ts[3]), B(ts[5]))
        call("oxq_dequantize_w8", ctx, None, B(ts[1]), B(ts[2]), B(ts[3]), B(ts[5]))
        call("oxq_dequantize_gptq_packed", ctx, None, B(ts[1]), B(ts[2]), B(ts[3]), bits & 0xFFFFFFFF, B(ts[5]))
        call("oxq_mpp_quant_matmul", ctx, None, B(ts[0]), B(ts[1]), B(ts[2]), B(ts[3]), bits & 0xFFFFFFFF, pd, B(ts[4]))
        call("oxq_maybe_mpp_quant_matmul", ctx, None, B(ts[0]), B(ts[1]), B(ts[2]), B(ts[3]), bits & 0xFFFFFFFF, pd, B(ts[4]), B(taken))
        call("oxq_compressed_to_awq", ctx, None, B(ts[0]), B(ts[1]), B(ts[2]), B(ts[3]), B(ts[4]))
        arr = (_lib.OxqTensor * 3)(ts[0], ts[1], ts[2])
        call("oxq_concat_awq_along_out", ctx, None, int(rng.choice([4, 8, 3])), int(rng.choice([0, 1, 3, -1])), arr, arr, arr, B(ts[3]), B(ts[4]), B(ts[5]))
        call("oxq_rtn_quantize_awq", ctx, None, B(ts[0]), i64(), B(ts[1]), B(ts[2]), B(ts[3]))
        call("oxq_gguf_depermute_qk_rows", ctx, None, B(ts[0]), i64(), i64(), q, i64(), i64(), B(ts[1]))
        call("oxq_cast_f8e4m3_to_f32", ctx, None, B(ts[0]), B(ts[1]))
        call("oxq_f8_block_dequant_bf16", ctx, None, B(ts[0]), B(ts[1]), B(ts[2]))
        call("oxq_f8_gemv", ctx, None, B(ts[0]), B(ts[1]), B(ts[2]), B(ts[3]))
        call("oxq_f8_matmul", ctx, None, B(ts[0]), B(ts[1]), B(ts[2]), B(ts[3]))
        call("oxq_gguf_quant_matmul", ctx, None, B(ts[0]), B(ts[1]), i64(), i64(), q, B(ts[2]))
        call("oxq_gguf_quant_mul_mm", ctx, None, B(ts[0]), B(ts[1]), i64(), i64(), q, B(ts[2]))
        call("oxq_gguf_dequantize", ctx, None, B(ts[0]), i64(), i64(), q, B(ts[1]))
        call("oxq_mxfp4_matmul", ctx, None, B(ts[0]), B(ts[1]), B(ts[2]), i64(), i64(), B(ts[3]))
        call("oxq_mxfp4_dequantize", ctx, None, B(ts[0]), B(ts[1]), i64(), i64(), B(ts[2]))
        call("oxq_mxfp4_moe_matmul", ctx, None, B(ts[0]), B(ts[1]), B(ts[2]), B(ts[3]), B(ts[4]), B(ts[5]), int(rng.integers(0, 2)), i64(), i64(), B(ts[6]))
        call("oxq_mxfp4_moe_gate_up_swiglu", ctx, None, B(ts[0]), B(ts[1]), B(ts[2]), B(ts[3]), B(ts[4]), B(ts[5]), int(rng.integers(0, 2)), i64(), i64(), C.c_float(7.0), B(ts[6]), B(taken))
        call("oxq_moe_route", ctx, None, B(ts[0]), i64(), 1, B(ts[1]), B(ts[2]))
        call("oxq_moe_group", ctx, None, B(ts[0]), B(ts[1]), i64(), B(ts[2]), B(ts[3]), B(ts[4]), B(ts[5]))
        call("oxq_moe_route_group", ctx, None, B(ts[0]), i64(), 1, B(ts[1]), B(ts[2]), B(ts[3]), B(ts[4]), B(ts[5]), B(ts[6]))
        call("oxq_gated_activation", ctx, None, B(ts[0]), int(rng.integers(-1, 4)), C.c_float(7.0), B(ts[1]))
        call("oxq_activation_mul", ctx, None, B(ts[0]), B(ts[1]), int(rng.integers(-1, 4)), B(ts[2]))
        call("oxq_moe_combine", ctx, None, B(ts[0]), B(ts[1]), B(ts[2]), B(ts[3]))
        # layers
        h = C.c_void_p()
        rc = lib.oxq_packed_quant_linear_new(ctx, bits & 0xFFFFFFFF, pd, B(ts[1]), B(ts[2]), B(ts[3]), None, int(rng.choice([1, 2, 0])), B(h))
        assert -13 <= rc <= 0
        if rc == 0:
            call("oxq_packed_quant_linear_forward", h, None, B(ts[0]), B(ts[4]))
            call("oxq_packed_quant_linear_dequantize", h, None, B(ts[5]))
            lib.oxq_packed_quant_linear_free(h)
        h = C.c_void_p()
        rc = lib.oxq_packed_quant_linear_new_gate_up(ctx, bits & 0xFFFFFFFF, pd, B(ts[1]), B(ts[2]), B(ts[3]), None, int(rng.integers(-1, 4)), int(rng.choice([1, 2])), B(h))
        assert -13 <= rc <= 0
        if rc == 0:
            call("oxq_packed_quant_linear_forward", h, None, B(ts[0]), B(ts[4]))
            lib.oxq_packed_quant_linear_free(h)
        h = C.c_void_p()
        rc = lib.oxq_qlinear_new(ctx, q, B(ts[0]), i64(), i64(), None, int(rng.choice([0, 2, 1])), B(h))
        assert -13 <= rc <= 0
        if rc == 0:
            call("oxq_qlinear_forward", h, None, B(ts[1]), B(ts[2])); lib.oxq_qlinear_free(h)
        h = C.c_void_p()
        rc = lib.oxq_mxfp4_linear_new(ctx, B(ts[0]), B(ts[1]), None, i64(), i64(), B(h))
        assert -13 <= rc <= 0
        if rc == 0:
            call("oxq_mxfp4_linear_forward", h, None, B(ts[2]), B(ts[3])); lib.oxq_mxfp4_linear_free(h)
    assert names['oxq_w4a16_matmul'][0] > 0 and names['oxq_w4a16_matmul'][1] > 0


# ------------------------------------------------------------------ the headers as a C99 consumer sees them
def _c_declarations():
    """(return type, name, [parameter declarations]) of every function include/*.h declares."""
    import glob
    text = "".join(open(h).read() for h in sorted(glob.glob(os.path.join(ROOT, "include", "*.h"))))
    text = re.sub(r"/\*.*?\*/", " ", text, flags=re.S)
    out = []
    for m in re.finditer(r"^(int|int64_t|uint64_t|void|const char \*)\s*(oxq_[a-z0-9_]+)\s*\(([^;{]*)\)\s*;", text, re.M):
        params = [p.strip() for p in re.sub(r"\s+", " ", m.group(3)).split(",")]
        out.append((m.group(1).strip(), m.group(2), [] if params == ["void"] else params))
    return out


def _c_argument(param: str) -> str:
    ptype = re.sub(r"\b[a-z_0-9]+$", "", param).strip()  # drop the parameter name
    if ptype in ("oxq_ctx *", "const oxq_ctx *"):
        return "ctx"
    if ptype == "const oxq_tensor *":
        return "&t"
    if ptype == "const char *":
        return '"x"'
    if "*" in ptype:
        return "NULL"
    if ptype == "float":
        return "1.0f"
    return "1"


def test_headers_compile_as_c99_and_every_entry_point_answers(tmp_path):
    """A C99 translation unit (gcc -std=c99 -pedantic -Wall -Wextra -Werror) includes both headers and calls
    every declared function on a plan-only ctx with a small valid descriptor or NULL per parameter: the
    headers are plain C (what bindgen or a hand-written `extern "C"` block needs), every symbol links, and
    no entry point crashes on arguments it must refuse."""
    decls = _c_declarations()
    assert len(decls) >= 70 and {d[1] for d in decls} == set(_lib.SIGNATURES)
    lines = ['#include <stdio.h>', '#include <string.h>', '#include "oxq.h"', '#include "oxq_bench.h"', '#include "oxq_files.h"', '',
             'int main(void) {', '    oxq_ctx *ctx = NULL;', '    oxq_tensor t;', '    oxq_plan plan;', '    int calls = 0;',
             '    memset(&t, 0, sizeof t);', '    t.dtype = OXQ_F16; t.rank = 2; t.dims[0] = 1; t.dims[1] = 256; t.contiguous = 1;',
             '    if (oxq_ctx_create(OXQ_DEVICE_PLAN_ONLY, &ctx) != OXQ_OK || !ctx) return 2;']
    skip = {"oxq_ctx_create", "oxq_ctx_destroy"}
    for ret, name, params in decls:
        if name in skip:
            continue
        args = ", ".join(_c_argument(p) for p in params)
        lines.append(f"    (void){name}({args}); ++calls;")
    lines += [
        '    {   /* one call that must succeed: the plan of a 4-bit AWQ GEMV */',
        '        oxq_tensor x = t, qw = t, qz = t, sc = t, y = t;',
        '        x.dims[1] = 4096;',
        '        qw.dtype = OXQ_I32; qw.dims[0] = 4096; qw.dims[1] = 512;',
        '        qz.dtype = OXQ_I32; qz.dims[0] = 32; qz.dims[1] = 512;',
        '        sc.dims[0] = 32; sc.dims[1] = 4096;',
        '        y.dims[1] = 4096;',
        '        if (oxq_w4a16_matmul(ctx, NULL, &x, &qw, &qz, &sc, &y) != OXQ_OK) { printf("%s\\n", oxq_last_error()); return 3; }',
        '        if (oxq_ctx_last_plan(ctx, &plan) != OXQ_OK || plan.kernel[0] == 0 || plan.launches < 1) return 4;',
        '        if (oxq_w4a16_matmul_static(ctx, NULL, &x, &qw, &qz, &sc, &y) != OXQ_OK) return 5;',
        '        x.dtype = OXQ_F32;',
        '        if (oxq_w4a16_matmul(ctx, NULL, &x, &qw, &qz, &sc, &y) != OXQ_ERR_DTYPE) return 6;',
        '    }',
        '    if (oxq_ctx_destroy(ctx) != OXQ_OK) return 7;',
        '    printf("%d calls, last kernel %s\\n", calls, plan.kernel);',
        '    return 0;', '}', '']
    src = tmp_path / "abi_c99.c"
    src.write_text("\n".join(lines))
    exe = tmp_path / "abi_c99"
    libdir = os.path.dirname(_lib.LIB_PATH)
    cc = subprocess.run(["gcc", "-std=c99", "-pedantic", "-Wall", "-Wextra", "-Werror", f"-I{os.path.join(ROOT, 'include')}",
                         str(src), "-o", str(exe), f"-L{libdir}", "-loxq_hip", f"-Wl,-rpath,{libdir}",
                         "-Wl,-rpath,/opt/rocm/lib"], capture_output=True, text=True)
    assert cc.returncode == 0, cc.stderr
    run = subprocess.run([str(exe)], capture_output=True, text=True, timeout=120)
    assert run.returncode == 0, (run.returncode, run.stdout, run.stderr)
    assert f"{len(decls) - len(skip)} calls" in run.stdout and "awq4" in run.stdout, run.stdout
