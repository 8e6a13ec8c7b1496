"""Which stateless GPTQ calls the tile kernel on the checkpoint layout takes (csrc/gptq_tile.hip), asked of
a plan-only ctx: no GPU needed."""
from oxydllm_amd import _lib, ops
from tests.helpers import fake, tune


def test_gptq_tile_routing_and_fallbacks():
    """Wide layers at any row count, narrow ones from 4 rows (K up to 8192), everything above 8 rows; columns
    that are not whole strips, groups below a block and the switch keep the dot-product kernel."""
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

    assert kernel(1, 5120, 13824, 128) == ("gptq4_tile_f16_mt1", 1)
    assert kernel(1, 5120, 13824, 128, 8) == ("gptq8_tile_f16_mt1", 1)
    assert kernel(1, 4096, 4096, 128)[0].startswith("gptq4_gemv_fast")
    assert kernel(4, 4096, 4096, 128) == ("gptq4_tile_f16_mt1", 1)
    assert kernel(8, 14336, 4096, 128)[0].startswith("gptq4_gemv_fast")
    assert kernel(16, 14336, 4096, 128) == ("gptq4_tile_f16_mt1", 1)
    assert kernel(17, 4096, 4096, 128) == ("gptq4_tile_f16_mt2", 1)
    assert kernel(33, 4096, 4096, 128) == ("gptq4_tile_f16_mt4", 1)
    assert kernel(8, 5120, 13824 + 32, 128)[0].startswith("gptq4_gemv_fast")   # 32 columns past the last strip
    assert "tile" not in kernel(8, 5120, 13824, 64)[0]                        # two groups a block
    tune("OXQ_GPTQ_TILE", 0, ctx=plan)
    assert kernel(8, 5120, 13824, 128)[0].startswith("gptq4_gemv_fast")
