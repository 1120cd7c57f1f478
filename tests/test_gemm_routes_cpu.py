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


# Tile and split alternatives that a +-10 % change of one time-model constant reaches on a benchmark shape, with the
# median launch time of each in microseconds on MI355X (40 launches after 8 warm-up launches, HIP events around each
# launch, the alternative forced by a build of the dispatcher whose plan is overridden; configuration operands).  The first
# entry of each shape is the dispatcher's own choice.  A boundary is acceptable when both sides of it cost about the same.
RECORDED_BOUNDARIES = {
    ("fp8", (128, 7168, 18432)): {(128, 128, 4): 48.8, (64, 128, 2): 50.0, (128, 192, 6): 52.7},
    ("fp8", (4096, 1536, 7168)): {(128, 192, 1): 63.0, (128, 256, 1): 65.8},
    ("fp8", (4096, 576, 7168)): {(64, 192, 1): 45.7, (128, 128, 1): 47.0},
    ("int8", (256, 4096, 14336)): {(128, 128, 4): 48.9, (64, 256, 4): 49.9, (128, 128, 3): 47.4},
}
BOUNDARY_COST = 1.10  # the slower side of a recorded boundary may cost at most this much more than the dispatcher's choice


def test_benchmark_shapes_hold_their_kernels_when_a_constant_moves():
    """Every measured constant of the dispatcher's time models (sglang_amd/csrc/route_constants.h) is changed by -10 % and
    +10 %, one at a time.  No benchmark shape may move to another kernel.  Within the mid-M kernel a shape may move to
    another tile or split only where both have been timed on the GPU and recorded above, and the recorded times must show
    that the move costs less than BOUNDARY_COST: then the constant's uncertainty (timings spread +-3 %) cannot cost more
    than that.  A new constant, or a changed one, that puts a benchmark shape on an unmeasured boundary fails here."""
    from sglang_amd import _lib

    names = list(_lib.route_constants())
    assert len(names) == _lib.lib().mi355_route_constant_count() and len(set(names)) == len(names)
    tile = lambda p: (p["bm"], p["bn"], p["splits"])
    moved = set()
    for kind, config in (("fp8", FP8_DECODE_CONFIG + FP8_PREFILL_CONFIG), ("int8", INT8_CONFIG)):
        for shape in config:
            base = plan_for(kind, *shape)
            for i, name in enumerate(names):
                for factor in (0.9, 1.1):
                    p = _lib.gemm_plan_perturbed(kind, *shape, i, factor)
                    assert p["kernel"] == base["kernel"], f"{kind} {shape}: {name} x {factor} moves {base['kernel']} -> {p['kernel']}"
                    if tile(p) == tile(base):
                        continue
                    rec = RECORDED_BOUNDARIES.get((kind, shape))
                    assert rec is not None and tile(base) in rec and tile(p) in rec, \
                        f"{kind} {shape}: {name} x {factor} moves tile {tile(base)} -> {tile(p)}: time both and record them"
                    assert next(iter(rec)) == tile(base), f"{kind} {shape}: the recorded choice {next(iter(rec))} is not the plan's {tile(base)}"
                    assert rec[tile(p)] <= BOUNDARY_COST * rec[tile(base)], (kind, shape, name, factor, rec)
                    moved.add((kind, shape, tile(p)))
    # the record holds nothing stale: every recorded alternative is one a perturbation reaches
    for (kind, shape), rec in RECORDED_BOUNDARIES.items():
        for t in list(rec)[1:]:
            assert (kind, shape, t) in moved, f"{kind} {shape}: recorded alternative {t} is no longer reached"


def test_perturbed_plan_query():
    import ctypes

    from sglang_amd import _lib

    L = _lib.lib()
    n = L.mi355_route_constant_count()
    assert n == 53 and L.mi355_route_constant_name(n) is None and L.mi355_route_constant_name(-1) is None
    assert _lib.route_constants()["pp_fp8_us_per_kblock"] == 1.39
    buf = ctypes.create_string_buffer(256)
    assert L.mi355_gemm_plan_perturbed(1, 128, 7168, 18432, 1, n, 1.1, buf, len(buf)) == 1
    assert L.mi355_gemm_plan_perturbed(1, 128, 7168, 18432, 1, 0, 0.0, buf, len(buf)) == 1
    # a factor of one is the plain query, and the perturbed copy does not outlive its call
    for kind, shape in (("fp8", (128, 7168, 18432)), ("int8", (256, 4096, 14336)), ("fp8", (4096, 36864, 7168))):
        assert _lib.gemm_plan_perturbed(kind, *shape, 3, 1.0) == _lib.gemm_plan(kind, *shape)
    far = _lib.gemm_plan_perturbed("fp8", 256, 36864, 7168, 0, 10.0)  # a two-phase kernel ten times slower loses
    assert far["kernel"] == "dma3" and _lib.gemm_plan("fp8", 256, 36864, 7168)["kernel"] == "pingpong"


def test_plan_query_rejects_bad_arguments():
    import ctypes

    from sglang_amd import _lib

    L = _lib.lib()
    buf = ctypes.create_string_buffer(8)
    assert L.mi355_fp8_blockwise_mm_plan(16, 128, 128, 1, buf, len(buf)) == 1 and b"too small" in L.mi355_last_error()
    assert L.mi355_int8_scaled_mm_plan(0, 128, 128, 1, buf, len(buf)) == 1
    assert L.mi355_fp8_blockwise_mm_plan(16, 128, 128, 1, None, 0) == 1
    p = _lib.gemm_plan("fp8", 13, 18432, 7168)
    assert p["kernel"] == "decode" and p["splits"] == 7
    p = _lib.gemm_plan("fp8", 13, 36864, 7168)  # one round of unsplit 64 x 192 tiles beats the split streaming kernel
    assert (p["kernel"], p["bm"], p["bn"], p["splits"]) == ("dma3", 64, 192, 1)
    p = _lib.gemm_plan("fp8", 1, 36864, 7168)
    assert p["kernel"] == "decode_wavesplit" and p["splits"] == 1 and p["bn"] == 16
    p = _lib.gemm_plan("fp8", 3, 36864, 7168)  # two channel tiles per workgroup from three tokens on
    assert p["kernel"] == "decode_wavesplit" and p["bn"] == 32


def test_block_linear_plan():
    """The one-call linear quantizes inside the GEMM kernel - the mid-M kernel's producer waves where one round of unsplit tiles
    fills the chip (and K would make many ranges for the streaming kernel), else the streaming decode kernel's prologue -
    except where a quantizer launch in front of the wave-split kernel was measured faster (long K; short K with more than
    eight tokens) and beyond decode sizes."""
    import ctypes

    from sglang_amd import _lib

    for shape, want in (((1, 36864, 7168), ("fused", "dma3")), ((3, 36864, 7168), ("fused", "dma3")), ((8, 36864, 7168), ("fused", "dma3")),
                        ((1, 28672, 4096), ("fused", "decode")), ((8, 24576, 7168), ("fused", "dma3")),
                        ((16, 2048, 7168), ("fused", "decode")), ((8, 7168, 2048), ("fused", "decode")),
                        ((4, 7168, 18432), ("launch", "decode_wavesplit")), ((16, 7168, 2048), ("launch", "decode_wavesplit")),
                        ((128, 7168, 2048), ("launch", "dma3")), ((4, 1000, 1024), ("launch", "generic"))):
        p = _lib.block_linear_plan(*shape)
        assert (p["quantizer"], p["kernel"]) == want, (shape, p)
        if p["quantizer"] == "launch":
            assert {k: v for k, v in p.items() if k != "quantizer"} == _lib.gemm_plan("fp8", *shape)
    # where the one call multiplies with the GEMM entry point's kernel and tiling (any plan with a quantizer launch, and the
    # fused plans whose kernel the GEMM entry point takes too) the reference-named wrappers equal their two calls bit for bit
    from sglang_amd.fp8_utils import _one_call_takes_the_same_gemm

    for shape, want in (((8, 36864, 7168), True), ((16, 2048, 7168), True), ((4, 7168, 18432), True), ((4100, 1024, 256), True),
                        ((40, 200, 384), True), ((1, 36864, 7168), False), ((8, 24576, 1536), False)):
        assert _one_call_takes_the_same_gemm(*shape) == want, shape
    buf = ctypes.create_string_buffer(256)
    assert _lib.lib().mi355_fp8_block_linear_plan(4, 1024, 1000, buf, len(buf)) == 1  # K not a multiple of 128
    assert _lib.lib().mi355_fp8_block_linear_plan(4, 1024, 1024, buf, 8) == 1 and b"too small" in _lib.lib().mi355_last_error()


@pytest.mark.parametrize("kind,M,N,K", [("fp8", 16, 2048, 7168), ("fp8", 128, 36864, 7168), ("int8", 256, 4096, 14336)])
def test_workspace_covers_the_plan(kind, M, N, K):
    from sglang_amd import _lib

    L = _lib.lib()
    p = plan_for(kind, M, N, K)
    ws = (L.mi355_fp8_blockwise_mm_workspace_bytes if kind == "fp8" else L.mi355_int8_scaled_mm_workspace_bytes)(M, N, K)
    assert ws >= (p["splits"] * M * N * 4 if p["splits"] > 1 else 0)


def test_grouped_plan_bounds_hold_for_any_routing():
    """The grouped GEMM sizes its tile tables and grids on the host from (experts, stacked rows) alone, while the real
    tile counts come from row counts that only exist on the device.  Replay the device rule here (256-row tiles; a rest of
    129..255 rows is one more; a rest of 1..128 rows becomes small tiles of the height the plan names) for random and
    adversarial routings: the host bounds must never be exceeded."""
    import random

    from sglang_amd import _lib

    rnd = random.Random(7)
    cases = []
    for _ in range(300):
        E = rnd.choice([1, 2, 3, 8, 16, 64, 256, 300])
        kind = rnd.choice(["uniform", "skewed", "tiny", "edges"])
        if kind == "uniform":
            sizes = [rnd.randint(0, 600) for _ in range(E)]
        elif kind == "skewed":
            sizes = [rnd.choice([0, 0, 1, 2, 5000]) for _ in range(E)]
        elif kind == "tiny":
            sizes = [rnd.randint(0, 3) for _ in range(E)]
        else:
            sizes = [rnd.choice([1, 63, 64, 65, 127, 128, 129, 255, 256, 257, 384, 385]) for _ in range(E)]
        cases.append(sizes)
    cases += [[128] * 256, [129] * 256, [1] * 256, [64] * 300, [65] * 300, [385] * 16, [0] * 8 + [1]]
    for sizes in cases:
        E, total = len(sizes), sum(sizes)
        if total == 0:
            continue
        plan = _lib.grouped_gemm_plan(E, total, 512, 1024)
        bm = int(plan["small_tile"].split("x")[0])
        big = small = 0
        for rows in sizes:
            b, rest = divmod(rows, 256)
            if rest > 128:
                b += 1
            else:
                small += -(-rest // bm)
            big += b
        assert big <= plan["max_big_tiles"], (sizes[:8], big, plan)
        assert small <= plan["max_small_tiles"], (sizes[:8], small, plan)
        # the re-laid-out scale columns: expert e starts at align4(row0) + 4 e and is read in whole quads
        pitch = (total + 3) // 4 * 4 + 4 * E + 4
        row0 = 0
        for e, rows in enumerate(sizes):
            if rows:
                assert (row0 + 3) // 4 * 4 + 4 * e + (rows + 3) // 4 * 4 <= pitch
            row0 += rows


def test_mid_m_plans_are_consistent():
    """Whatever the time model picks, a split must give every K range some work and the ranges must cover K."""
    from sglang_amd import _lib

    for kind in ("fp8", "int8"):
        for M in (17, 32, 64, 65, 128, 129, 200, 256, 300, 512, 1000, 1024, 1025, 4096):
            for N, K in ((576, 7168), (1536, 7168), (7168, 18432), (36864, 7168), (6144, 4096), (4096, 14336), (256, 128), (512, 16384)):
                p = _lib.gemm_plan(kind, M, N, K)
                kb = -(-K // 128)
                assert p["splits"] >= 1 and p["kb_per_split"] >= 1
                assert p["kb_per_split"] * p["splits"] >= kb and p["kb_per_split"] * (p["splits"] - 1) < kb, (kind, M, N, K, p)
                if p["kernel"] == "dma3":  # the tile shapes that are compiled: 192 channels for FP8 only, splits need N % 4 == 0
                    assert p["bm"] in (64, 128) and p["bn"] in ((128, 192, 256) if kind == "fp8" else (128, 256)), (kind, M, N, K, p)
                    assert p["splits"] == 1 or N % 4 == 0
