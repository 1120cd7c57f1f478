"""GPU parity of the grouped blockwise FP8 GEMM (fp8_blockwise_scaled_grouped_mm, the expert GEMMs of a mixture-of-experts
layer) against the CPU oracle, expert by expert: the oracle's fp8_blockwise_mm on the expert's rows and weight.

Tolerance as for the dense GEMM (tests/test_gpu_fp8_gemm.py): |out - ref| <= 1e-2 * |ref| + 1e-4 * mag, mag = sum |terms|,
plus the rounding of the 16-bit output.  The reference's own acceptance test (sgl-kernel/tests/test_fp8_blockwise_moe.py:
103-216: random expert sizes 1..256, N and K multiples of 128, 1 - cosine-like similarity < 1e-3 against the unquantized
product) is reproduced in test_reference_acceptance_criterion with this package's quantizers in place of its torch helpers.
"""
import pytest
import torch

from fp8_tolerance import check_fp8_gemm
pytestmark = pytest.mark.gpu
FP8 = torch.float8_e4m3fn


def _rand_fp8(shape, g):
    return ((torch.rand(*shape, generator=g) - 0.5) * 2 * 448.0).clamp(-448, 448).to(FP8)


def _call(gpu, a, w, sa, sw, sizes, offsets, out_dtype, out=None, workspace_bytes=0):
    """a [T, K], w [E, N, K] (as stored), sa [T, K/128], sw [E, N/128, K/128]; the reference's argument list and layouts
    (b and scales_b as transposed views)."""
    from sglang_amd.sgl_kernel import fp8_blockwise_scaled_grouped_mm

    E, N, K = w.shape
    T = a.shape[0]
    dev = lambda t: t.to(gpu)
    if out is None:
        out = torch.full((T, N), 7.0, dtype=out_dtype, device=gpu)
    i64 = lambda: torch.empty(E, dtype=torch.int64, device=gpu)
    lay = lambda: torch.zeros(E, 5, dtype=torch.int32, device=gpu)
    a_strides = torch.full((E,), K, dtype=torch.int64, device=gpu)
    c_strides = torch.full((E,), N, dtype=torch.int64, device=gpu)
    problem_sizes = torch.tensor([[m, N, K] for m in sizes], dtype=torch.int32, device=gpu).reshape(E, 3)
    expert_offsets = torch.tensor(offsets, dtype=torch.int32, device=gpu)
    fp8_blockwise_scaled_grouped_mm(
        out, i64(), i64(), i64(), i64(), i64(), dev(a), dev(w).transpose(1, 2), dev(sa), dev(sw).transpose(1, 2),
        a_strides, a_strides, c_strides, lay(), lay(), problem_sizes, expert_offsets,
        torch.empty(workspace_bytes, dtype=torch.uint8, device=gpu))
    return out


def _check_expert(out_rows, ref, mag, what):
    check_fp8_gemm(out_rows, ref, mag, what)


def _problem(sizes, N, K, seed, gap=0):
    g = torch.Generator().manual_seed(seed)
    E = len(sizes)
    offsets, row = [], 0
    for m in sizes:
        offsets.append(row)
        row += m + gap
    T = row
    a, w = _rand_fp8((max(T, 1), K), g)[:T], _rand_fp8((E, N, K), g)
    sa = torch.rand(T, K // 128, generator=g) * 1e-2 + 1e-4
    sw = torch.rand(E, (N + 127) // 128, K // 128, generator=g) * 1e-2 + 1e-4
    return a, w, sa, sw, offsets, T


def _verify(oracle, out, a, w, sa, sw, sizes, offsets, what):
    owned = torch.zeros(a.shape[0], dtype=torch.bool)
    for e, (m, r0) in enumerate(zip(sizes, offsets)):
        if m == 0:
            continue
        ref, mag = oracle.fp8_blockwise_mm(a[r0:r0 + m], w[e], sa[r0:r0 + m], sw[e], torch.float32, want_abs=True)
        _check_expert(out[r0:r0 + m], ref, mag, f"{what} expert {e} rows {m}")
        owned[r0:r0 + m] = True
    # rows that belong to no expert keep what the caller put there
    if (~owned).any():
        assert bool((out.float().cpu()[~owned] == 7.0).all()), f"{what}: rows outside every expert were written"


@pytest.mark.parametrize("num_experts", [8, 16, 32, 64, 128])
@pytest.mark.parametrize("out_dtype", [torch.half, torch.bfloat16])
def test_random_expert_sizes(gpu, oracle, num_experts, out_dtype):
    """The reference test's distribution of problems (sizes 1..256 per expert, N and K random multiples of 128), with N
    and K capped so that the oracle stays fast."""
    import random

    rnd = random.Random(1000 * num_experts + (out_dtype == torch.half))
    N, K = rnd.randint(1, 6) * 128, rnd.randint(1, 8) * 128
    sizes = [rnd.randint(1, 256) for _ in range(num_experts)]
    print(f"case E={num_experts} N={N} K={K} {out_dtype} rows={sum(sizes)}", flush=True)
    a, w, sa, sw, offsets, _ = _problem(sizes, N, K, num_experts)
    out = _call(gpu, a, w, sa, sw, sizes, offsets, out_dtype, workspace_bytes=64 << 20)
    _verify(oracle, out, a, w, sa, sw, sizes, offsets, f"E={num_experts}")


@pytest.mark.parametrize("name,sizes,N,K,tile", [
    ("decode_like", [1, 0, 3, 1, 0, 0, 2, 8, 1, 1, 0, 5, 16, 1, 2, 1], 512, 7168, "64x256"),
    ("one_token", [1], 256, 128, "64x256"),
    ("empty_experts_around_a_big_one", [0, 0, 700, 0, 1, 0], 384, 512, "128x256"),
    ("prefill_like", [130, 257, 128, 64, 511, 129, 300, 200], 768, 1024, "128x256"),
    ("tile_edges", [64, 65, 63, 128, 127, 129, 1, 256], 256, 256, "128x256"),
    ("many_small", [3] * 300, 128, 256, "64x256"),
    ("large_experts", [1000, 513, 384, 2], 512, 512, "128x256"),
    ("ragged_channels", [40, 90, 17], 200, 384, "64x256"),
])
def test_shapes_and_tile_heights(gpu, oracle, name, sizes, N, K, tile):
    from sglang_amd import _lib

    print(f"case {name}", flush=True)
    a, w, sa, sw, offsets, T = _problem(sizes, N, K, len(sizes) + N)
    assert _lib.grouped_gemm_plan(len(sizes), T, N, K)["small_tile"] == tile
    out = _call(gpu, a, w, sa, sw, sizes, offsets, torch.bfloat16)  # no usable workspace given: the wrapper allocates one
    _verify(oracle, out, a, w, sa, sw, sizes, offsets, name)


def test_padded_layout_leaves_gaps_alone(gpu, oracle):
    """Experts laid out with unused rows between them (what a 128-aligned contiguous layout looks like): only the rows
    named by problem_sizes are written."""
    sizes = [5, 100, 0, 33, 64]
    a, w, sa, sw, offsets, _ = _problem(sizes, 256, 512, 9, gap=7)
    out = _call(gpu, a, w, sa, sw, sizes, offsets, torch.float16, workspace_bytes=8 << 20)
    _verify(oracle, out, a, w, sa, sw, sizes, offsets, "gaps")


def test_sizes_are_clamped_into_the_stacked_matrix(gpu, oracle):
    """A last expert that claims more rows than the stacked matrix has gets the rows that exist."""
    sizes = [20, 30, 50]
    a, w, sa, sw, offsets, T = _problem(sizes, 256, 256, 11)
    claimed = [20, 30, 1 << 20]
    out = _call(gpu, a, w, sa, sw, claimed, offsets, torch.bfloat16)
    _verify(oracle, out, a, w, sa, sw, sizes, offsets, "clamped")


def test_token_scales_in_either_layout(gpu, oracle):
    """scales_a column-major (what the dense GEMM's callers pass) gives the same result as row-major."""
    from sglang_amd.sgl_kernel import fp8_blockwise_scaled_grouped_mm  # noqa: F401

    sizes = [70, 9, 140]
    a, w, sa, sw, offsets, T = _problem(sizes, 512, 640, 13)
    out_row = _call(gpu, a, w, sa, sw, sizes, offsets, torch.bfloat16)
    sa_col = sa.t().contiguous().t()
    assert sa_col.stride(0) == 1
    out_col = _call(gpu, a, w, sa_col, sw, sizes, offsets, torch.bfloat16)
    assert torch.equal(out_row, out_col)


def test_expert_specialised_entry_point(gpu, oracle):
    """es_fp8_blockwise_scaled_grouped_mm (sgl-kernel/tests/test_es_fp8_blockwise_moe.py:103-196): same layouts, no
    scratch tensors in the argument list; same result as the other entry point, bit for bit."""
    from sglang_amd.sgl_kernel import es_fp8_blockwise_scaled_grouped_mm

    sizes = [200, 1, 77, 300, 0, 129]
    E, N, K = len(sizes), 384, 768
    a, w, sa, sw, offsets, T = _problem(sizes, N, K, 21)
    out = torch.full((T, N), 7.0, dtype=torch.bfloat16, device=gpu)
    strides = torch.full((E,), K, dtype=torch.int64, device=gpu)
    es_fp8_blockwise_scaled_grouped_mm(
        out, a.to(gpu), w.to(gpu).transpose(1, 2), sa.to(gpu), sw.to(gpu).transpose(1, 2), strides, strides,
        torch.full((E,), N, dtype=torch.int64, device=gpu),
        torch.tensor([[m, N, K] for m in sizes], dtype=torch.int32, device=gpu),
        torch.tensor(offsets, dtype=torch.int32, device=gpu), torch.empty(16 << 20, dtype=torch.uint8, device=gpu))
    _verify(oracle, out, a, w, sa, sw, sizes, offsets, "es")
    assert torch.equal(out, _call(gpu, a, w, sa, sw, sizes, offsets, torch.bfloat16))


def test_reference_acceptance_criterion(gpu):
    """sgl-kernel/tests/test_fp8_blockwise_moe.py:24-29, :205-216: quantize bf16 operands (1 x 128 groups, 128 x 128
    blocks), run the grouped GEMM, compare with the unquantized product: 1 - 2<x,y> / (<x,x> + <y,y>) < 1e-3."""
    from sglang_amd.fp8_kernel import sglang_per_token_group_quant_fp8
    from sglang_amd.fp8_utils import per_block_cast_to_fp8
    from sglang_amd.sgl_kernel import fp8_blockwise_scaled_grouped_mm

    g = torch.Generator().manual_seed(5)
    sizes = [int(v) for v in torch.randint(1, 257, (16,), generator=g)]
    E, N, K, T = len(sizes), 768, 1024, sum(sizes)
    x = torch.randn(T, K, generator=g).to(torch.bfloat16).to(gpu)
    wt = torch.randn(E, N, K, generator=g).to(torch.bfloat16).to(gpu)
    a_q, a_s = sglang_per_token_group_quant_fp8(x, 128)
    w_q = torch.empty(E, N, K, dtype=FP8, device=gpu)
    w_s = torch.empty(E, N // 128, K // 128, dtype=torch.float32, device=gpu)
    for e in range(E):
        w_q[e], w_s[e] = per_block_cast_to_fp8(wt[e])
    offsets = [sum(sizes[:e]) for e in range(E)]
    out = torch.empty(T, N, dtype=torch.bfloat16, device=gpu)
    i64 = lambda: torch.empty(E, dtype=torch.int64, device=gpu)
    lay = lambda: torch.zeros(E, 5, dtype=torch.int32, device=gpu)
    fp8_blockwise_scaled_grouped_mm(
        out, i64(), i64(), i64(), i64(), i64(), a_q, w_q.transpose(1, 2), a_s, w_s.transpose(1, 2), i64(), i64(), i64(),
        lay(), lay(), torch.tensor([[m, N, K] for m in sizes], dtype=torch.int32, device=gpu),
        torch.tensor(offsets, dtype=torch.int32, device=gpu), torch.empty(32 << 20, dtype=torch.uint8, device=gpu))
    for e, (m, r0) in enumerate(zip(sizes, offsets)):
        ref = (x[r0:r0 + m].float() @ wt[e].float().t()).double().cpu()
        got = out[r0:r0 + m].double().cpu()
        diff = 1 - 2 * (ref * got).sum() / ((ref * ref).sum() + (got * got).sum())
        assert float(diff) < 1e-3, (e, float(diff))


def test_argument_checks(gpu):
    from sglang_amd.sgl_kernel import fp8_blockwise_scaled_grouped_mm

    E, N, K, T = 2, 256, 256, 8
    i64 = lambda: torch.empty(E, dtype=torch.int64, device=gpu)
    lay = lambda: torch.zeros(E, 5, dtype=torch.int32, device=gpu)
    args = dict(
        out=torch.empty(T, N, dtype=torch.bfloat16, device=gpu), a=torch.zeros(T, K, device=gpu).to(FP8),
        b=torch.zeros(E, N, K, device=gpu).to(FP8).transpose(1, 2), sa=torch.ones(T, 2, device=gpu),
        sb=torch.ones(E, 2, 2, device=gpu), ps=torch.tensor([[4, N, K]] * 2, dtype=torch.int32, device=gpu),
        eo=torch.tensor([0, 4], dtype=torch.int32, device=gpu))

    def run(**kw):
        v = dict(args, **kw)
        fp8_blockwise_scaled_grouped_mm(v["out"], i64(), i64(), i64(), i64(), i64(), v["a"], v["b"], v["sa"], v["sb"], i64(),
                                        i64(), i64(), lay(), lay(), v["ps"], v["eo"], torch.empty(0, dtype=torch.uint8, device=gpu))

    run()
    with pytest.raises(RuntimeError, match="problem_sizes must be int32"):
        run(ps=args["ps"].to(torch.int64))
    with pytest.raises(RuntimeError, match="output must be bfloat16 or half"):
        run(out=torch.empty(T, N, dtype=torch.float32, device=gpu))
    with pytest.raises(RuntimeError, match="must match expert_offsets"):
        run(eo=torch.tensor([0], dtype=torch.int32, device=gpu))
    with pytest.raises(RuntimeError, match="column-major"):
        run(b=torch.zeros(E, K, N, device=gpu).to(FP8))
