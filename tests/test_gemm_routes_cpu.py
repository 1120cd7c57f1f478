"""Which kernel variant the dispatcher picks is a host-side decision, so it is checked without a GPU: the shapes the
GPU parity tests run (tests/gemm_cases.py) must between them reach every compiled variant, and the full-size benchmark
configurations must only use variants that those tests (or the full-size tests themselves) exercise."""
import pytest

from gemm_cases import (FP8_DECODE_CONFIG, FP8_PREFILL_CONFIG, FP8_REQUIRED_VARIANTS, FP8_ROUTE_SHAPES, INT8_CONFIG,
                        INT8_REQUIRED_VARIANTS, INT8_ROUTE_SHAPES, plan_for, variant_of)


def _reached(kind, shapes):
    return {variant_of(plan_for(kind, *s), s[2]) for s in shapes}


def test_fp8_route_shapes_reach_every_variant():
    missing = FP8_REQUIRED_VARIANTS - _reached("fp8", FP8_ROUTE_SHAPES)
    assert not missing, f"no FP8 test shape reaches {sorted(missing, key=str)}"


def test_int8_route_shapes_reach_every_variant():
    missing = INT8_REQUIRED_VARIANTS - _reached("int8", INT8_ROUTE_SHAPES)
    assert not missing, f"no INT8 test shape reaches {sorted(missing, key=str)}"


def test_benchmark_configurations_use_only_tested_variants():
    for kind, config, routes, required in (("fp8", FP8_DECODE_CONFIG + FP8_PREFILL_CONFIG, FP8_ROUTE_SHAPES, FP8_REQUIRED_VARIANTS),
                                           ("int8", INT8_CONFIG, INT8_ROUTE_SHAPES, INT8_REQUIRED_VARIANTS)):
        tested = _reached(kind, routes)
        for s in config:
            v = variant_of(plan_for(kind, *s), s[2])
            assert v in tested and v in required, f"{kind} {s} runs {v}, which no route shape covers"


def test_every_variant_is_one_the_library_can_name():
    # a variant added to the dispatcher must be added to the required sets, or this fails
    for kind, shapes, required in (("fp8", FP8_ROUTE_SHAPES + FP8_DECODE_CONFIG + FP8_PREFILL_CONFIG, FP8_REQUIRED_VARIANTS),
                                   ("int8", INT8_ROUTE_SHAPES + INT8_CONFIG, INT8_REQUIRED_VARIANTS)):
        extra = _reached(kind, shapes) - required
        assert not extra, f"{kind}: variants reached but not listed as required: {sorted(extra, key=str)}"


def test_plan_query_rejects_bad_arguments():
    import ctypes

    from sglang_amd import _lib

    L = _lib.lib()
    buf = ctypes.create_string_buffer(8)
    assert L.mi355_fp8_blockwise_mm_plan(16, 128, 128, 1, buf, len(buf)) == 1 and b"too small" in L.mi355_last_error()
    assert L.mi355_int8_scaled_mm_plan(0, 128, 128, 1, buf, len(buf)) == 1
    assert L.mi355_fp8_blockwise_mm_plan(16, 128, 128, 1, None, 0) == 1
    p = _lib.gemm_plan("fp8", 1, 36864, 7168)
    assert p["kernel"] == "decode" and p["splits"] >= 1


@pytest.mark.parametrize("kind,M,N,K", [("fp8", 16, 2048, 7168), ("fp8", 128, 36864, 7168), ("int8", 256, 4096, 14336)])
def test_workspace_covers_the_plan(kind, M, N, K):
    from sglang_amd import _lib

    L = _lib.lib()
    p = plan_for(kind, M, N, K)
    ws = (L.mi355_fp8_blockwise_mm_workspace_bytes if kind == "fp8" else L.mi355_int8_scaled_mm_workspace_bytes)(M, N, K)
    assert ws >= (p["splits"] * M * N * 4 if p["splits"] > 1 else 0)
