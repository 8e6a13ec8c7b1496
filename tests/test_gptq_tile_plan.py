"""Which stateless GPTQ calls the tile kernel on the checkpoint layout takes (csrc/gptq_tile.hip), asked of
a plan-only ctx: no GPU needed."""
from oxydllm_amd import _lib, ops
from tests.helpers import fake, tune


def test_gptq_tile_routing_and_fallbacks():
    """Wide layers at any row count; layers of few strips from two rows on (8-bit: four), in K slices with a
    second launch; everything above 8 rows; columns that are not whole strips, groups below a block and the switch
    keep the dot-product kernel."""
    lib = _lib.load()
    plan = ops.Context(plan_only=True)

    def kernel(m, K, N, g, bits=4):
        pf = 32 // bits
        args = (fake((m, K), _lib.F16), fake((K // pf, N), _lib.I32), fake((K // g, N // pf), _lib.I32),
                fake((K // g, N), _lib.F16), fake((m, N), _lib.F16))
        refs = [_lib.C.byref(a) for a in args]
        if m <= 8:
            rc = lib.oxq_gptq_matmul(plan.handle, None, *refs[:4], bits, refs[4])
        else:
            rc = lib.oxq_mpp_quant_matmul(plan.handle, None, *refs[:4], bits, 1, refs[4])
        assert rc == 0, lib.oxq_last_error().decode()
        p = plan.last_plan()
        return p["kernel"], p["launches"]

    def split(m, K, N, bits=4):
        kernel(m, K, N, 128, bits)
        p = plan.last_plan()
        return p["split_k"], p["grid"], p["workspace_bytes"]

    assert kernel(1, 5120, 13824, 128) == ("gptq4_tile_f16_mt1", 1)
    assert kernel(1, 5120, 13824, 128, 8) == ("gptq8_tile_f16_mt1", 1)
    assert kernel(1, 4096, 4096, 128)[0].startswith("gptq4_gemv_fast")
    assert kernel(2, 4096, 4096, 128) == ("gptq4_tile_f16_mt1", 2)          # 64 strips: 4 K slices + the sum
    assert split(2, 4096, 4096) == (4, (64, 1, 4), 4 * 2 * 4096 * 4)
    assert kernel(2, 4096, 4096, 128, 8)[0].startswith("gptq8_gemv_fast")
    assert kernel(4, 4096, 4096, 128, 8) == ("gptq8_tile_f16_mt1", 2)
    assert kernel(8, 14336, 4096, 128) == ("gptq4_tile_f16_mt1", 2)
    assert split(16, 14336, 4096) == (4, (64, 1, 4), 4 * 16 * 4096 * 4)
    assert split(64, 8192, 2048) == (8, (32, 1, 8), 8 * 64 * 2048 * 4)
    assert split(100, 14336, 4096) == (2, (64, 2, 2), 2 * 100 * 4096 * 4)   # two row tiles: 128 tiles, 2 slices
    assert kernel(17, 4096, 4096, 128) == ("gptq4_tile_f16_mt2", 2)
    assert kernel(33, 5120, 13824, 128) == ("gptq4_tile_f16_mt4", 1)
    assert kernel(8, 5120, 13824 + 32, 128)[0].startswith("gptq4_gemv_fast")   # 32 columns past the last strip
    assert "tile" not in kernel(8, 5120, 13824, 64)[0]                        # two groups a block
    tune("OXQ_GPTQ_TILE_KS", 1, ctx=plan)
    assert kernel(16, 14336, 4096, 128) == ("gptq4_tile_f16_mt1", 1)
    tune("OXQ_GPTQ_TILE", 0, ctx=plan)
    assert kernel(8, 5120, 13824, 128)[0].startswith("gptq4_gemv_fast")
