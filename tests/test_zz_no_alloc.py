"""The FP8 GEMM entry point that allocates nothing (mi355_fp8_blockwise_mm_noalloc) against the ordinary entry point.

Both run the same kernels with the same deterministic reduce order, so outputs must be identical bit for bit; the
ordinary entry point is itself held to the oracle elsewhere.  Two calls in a row share the built-in scratch array, the
second with a smaller problem, so stale partial sums of the first call would show.  Called through the C ABI (ctypes)
with preallocated outputs.
"""
import pytest
import torch

from fp8_tolerance import check_fp8_gemm
from sglang_amd.workloads import cdiv

pytestmark = pytest.mark.gpu
FP8 = torch.float8_e4m3fn


def _problem(M, N, K, seed, gpu):
    g = torch.Generator().manual_seed(seed)
    c = torch.randint(0, 256, (M + N, K), generator=g, dtype=torch.uint8)
    c = torch.where((c & 0x7F) == 0x7F, c & 0xF7, c).view(FP8)
    a, w = c[:M].contiguous().to(gpu), c[M:].contiguous().to(gpu)
    As = (torch.rand(M, cdiv(K, 128), generator=g) * 1e-2 + 1e-4).to(gpu)
    Bs = (torch.rand(cdiv(N, 128), cdiv(K, 128), generator=g) * 1e-2 + 1e-4).to(gpu)
    return a, w, As, Bs


def _call(L, _lib, noalloc, a, w, As, Bs, out, ws=None):
    M, K = a.shape
    N = w.shape[0]
    stream = torch.cuda.current_stream().cuda_stream
    head = (a.data_ptr(), w.data_ptr(), As.data_ptr(), Bs.data_ptr(), out.data_ptr(), _lib.BF16, M, N, K,
            a.stride(0), w.stride(0), As.stride(0), As.stride(1), Bs.stride(0), Bs.stride(1), out.stride(0))
    if noalloc:
        return L.mi355_fp8_blockwise_mm_noalloc(*head, stream)
    return L.mi355_fp8_blockwise_mm(*head, ws.data_ptr() if ws is not None else None, ws.numel() if ws is not None else 0, stream)


def test_noalloc_matches_workspace_entry_point_twice_in_a_row(gpu, oracle):
    from sglang_amd import _lib

    L = _lib.lib()
    # split-K decode (18 splits, 2.4 MB of partials), then a smaller split problem, then mid-M split, then one without split
    shapes = [(8, 4096, 18432), (12, 2048, 7168), (48, 7168, 18432), (300, 1024, 512)]
    plans = [_lib.gemm_plan("fp8", *s) for s in shapes]
    assert plans[0]["splits"] > 1 and plans[1]["splits"] > 1 and plans[2]["splits"] > 1 and plans[3]["splits"] == 1
    problems = [_problem(*s, seed=i + 1, gpu=gpu) for i, s in enumerate(shapes)]
    outs_ws, outs_na = [], []
    for (M, N, K), pr in zip(shapes, problems):
        nbytes = L.mi355_fp8_blockwise_mm_workspace_bytes(M, N, K)
        ws = torch.empty(max(nbytes, 16), dtype=torch.uint8, device=gpu)
        o = torch.empty(M, N, dtype=torch.bfloat16, device=gpu)
        _lib.check(_call(L, _lib, False, *pr, o, ws))
        outs_ws.append(o)
    for (M, N, K) in shapes:
        outs_na.append(torch.full((M, N), float("nan"), dtype=torch.bfloat16, device=gpu))
    torch.cuda.synchronize()
    free_before = torch.cuda.mem_get_info()[0]
    for s, pr, o in zip(shapes, problems, outs_na):  # back to back on one stream, sharing the scratch array
        print(f"noalloc M,N,K={s}", flush=True)
        _lib.check(_call(L, _lib, True, *pr, o))
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] >= free_before - (1 << 20), "the no-allocation entry point took device memory"
    for s, x, y in zip(shapes, outs_ws, outs_na):
        assert torch.equal(x.view(torch.int16), y.view(torch.int16)), s
    # and the first (largest) once more after the smaller ones
    o = torch.full_like(outs_na[0], float("nan"))
    _lib.check(_call(L, _lib, True, *problems[0], o))
    assert torch.equal(o.view(torch.int16), outs_ws[0].view(torch.int16))
    # anchored on the oracle as well, for one of them
    a, w, As, Bs = (t.cpu() for t in problems[1])
    ref, mag = oracle.fp8_blockwise_mm(a, w, As, Bs, torch.float32, want_abs=True)
    check_fp8_gemm(outs_na[1], ref, mag, "no-alloc entry")


def test_noalloc_rejects_what_does_not_fit(gpu):
    from sglang_amd import _lib

    L = _lib.lib()
    M, N, K = 255, 4096, 7184  # generic kernel (K not a multiple of 128), 12 splits: 47.8 MiB of partial sums
    plan = _lib.gemm_plan("fp8", M, N, K)
    assert plan["splits"] * M * N * 4 > _lib.NOALLOC_SCRATCH_BYTES
    a, w, As, Bs = _problem(M, N, K, seed=9, gpu=gpu)
    out = torch.zeros(M, N, dtype=torch.bfloat16, device=gpu)
    rc = _call(L, _lib, True, a, w, As, Bs, out)
    assert rc == 4 and b"built-in scratch" in L.mi355_last_error()
    torch.cuda.synchronize()
    assert not bool(out.any()), "a rejected call must not launch anything"
