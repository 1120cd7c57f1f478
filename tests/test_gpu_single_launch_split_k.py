"""Split K in one launch (the last-arriving workgroup adds the partial sums) against the two-launch path.

Both add the partial tiles in ascending K-range order, so outputs must be bit-identical.  What this pins beyond the
ordinary parity tests, which already run through the single-launch path:
  * the arrival counters are back at zero after every call (three calls in a row, shapes of different sizes sharing
    one block of counters),
  * calls on two streams use different counter blocks and may overlap,
  * a captured graph replays correctly several times (its counters belong to the capture, not to the stream),
  * the switch mi355_set_single_launch_split_k really changes the number of kernels (checked through results only:
    both settings must agree with each other and with the oracle).
"""
import pytest
import torch

from sglang_amd.workloads import make_activation, make_fp8_weight, make_int8_weight

pytestmark = pytest.mark.gpu

# (M, N, K): decode plans with more than one K range; 1, 2 and 3+ channel groups per workgroup, short last range
SHAPES = [(1, 512, 7168), (16, 2048, 7168), (1, 16640, 4480), (9, 33280, 2176), (7, 33280, 4096), (3, 256, 2048)]


def _fp8_case(M, N, K, gpu, seed):
    from sglang_amd.fp8_kernel import per_token_group_quant_fp8

    w_q, w_s = make_fp8_weight(N, K, seed=seed)
    x = make_activation(M, K, seed=seed + 1).to(gpu)
    x_q, x_s = per_token_group_quant_fp8(x, 128, column_major_scales=True)
    return x_q, x_s, w_q.to(gpu), w_s.to(gpu)


def _fp8_mm(case):
    from sglang_amd.sgl_kernel import fp8_blockwise_scaled_mm

    x_q, x_s, w_q, w_s = case
    return fp8_blockwise_scaled_mm(x_q, w_q.t(), x_s, w_s.t(), torch.bfloat16)


def _int8_case(M, N, K, gpu, seed):
    from sglang_amd.workloads import make_int8_activation

    a_q, a_s = make_int8_activation(M, K, seed=seed)
    w_q, w_s = make_int8_weight(N, K, seed=seed + 1)
    bias = (torch.randn(N, generator=torch.Generator().manual_seed(seed + 2)) * 0.5).to(torch.bfloat16)
    return a_q.to(gpu), a_s.to(gpu), w_q.to(gpu), w_s.to(gpu), bias.to(gpu)


def _int8_mm(case):
    from sglang_amd.sgl_kernel import int8_scaled_mm

    a_q, a_s, w_q, w_s, bias = case
    return int8_scaled_mm(a_q, w_q.t(), a_s, w_s, torch.bfloat16, bias)


@pytest.fixture
def switch():
    from sglang_amd import _lib

    L = _lib.lib()
    before = L.mi355_set_single_launch_split_k(1)
    yield L.mi355_set_single_launch_split_k
    L.mi355_set_single_launch_split_k(before)


@pytest.mark.parametrize("kind", ["fp8", "int8"])
def test_matches_two_launch_path_call_after_call(gpu, switch, kind):
    from sglang_amd import _lib

    make, run = (_fp8_case, _fp8_mm) if kind == "fp8" else (_int8_case, _int8_mm)
    cases = []
    for i, (M, N, K) in enumerate(SHAPES):
        plan = _lib.gemm_plan(kind, M, N, K)
        assert plan["kernel"] == "decode" and plan["splits"] > 1, (M, N, K, plan)
        cases.append(make(M, N, K, gpu, 50 + 3 * i))
    switch(0)
    want = [run(c) for c in cases]
    torch.cuda.synchronize()
    switch(1)
    for rep in range(3):  # the same counters serve every call on this stream: they must be zero again each time
        for i, c in enumerate(cases):
            print(f"case {kind} rep={rep} shape={SHAPES[i]}", flush=True)
            got = run(c)
            torch.cuda.synchronize()
            assert torch.equal(got, want[i]), (kind, rep, SHAPES[i])


def test_two_streams_overlap(gpu, switch):
    shapes = [(1, 16640, 4480), (16, 2048, 7168)]
    cases = [_fp8_case(M, N, K, gpu, 80 + i) for i, (M, N, K) in enumerate(shapes)]
    switch(0)
    want = [_fp8_mm(c) for c in cases]
    torch.cuda.synchronize()
    switch(1)
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]  # default priority
    outs = [[], []]
    for rep in range(8):
        for k, st in enumerate(streams):
            with torch.cuda.stream(st):
                outs[k].append(_fp8_mm(cases[k]))
    torch.cuda.synchronize()
    for k in range(2):
        for rep, o in enumerate(outs[k]):
            assert torch.equal(o, want[k]), (k, rep)


def test_graph_replays(gpu, switch):
    M, N, K = 8, 2048, 7168
    case = list(_fp8_case(M, N, K, gpu, 90))
    inputs = [_fp8_case(M, N, K, gpu, 91 + i)[:2] for i in range(3)]
    switch(0)
    want = [_fp8_mm((xq, xs, case[2], case[3])).clone() for xq, xs in inputs]
    torch.cuda.synchronize()
    switch(1)
    static_q, static_s = case[0].clone(), case[1].clone()
    stream = torch.cuda.Stream()
    with torch.cuda.stream(stream):
        for _ in range(2):
            _fp8_mm((static_q, static_s, case[2], case[3]))
        stream.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=stream):
            static_out = _fp8_mm((static_q, static_s, case[2], case[3]))
    torch.cuda.synchronize()
    for rep in range(2):
        for i, (xq, xs) in enumerate(inputs):
            static_q.copy_(xq)
            static_s.copy_(xs)
            torch.cuda.synchronize()
            graph.replay()
            torch.cuda.synchronize()
            assert torch.equal(static_out, want[i]), (rep, i)
            eager = _fp8_mm((xq, xs, case[2], case[3]))  # eager work on the default stream between replays
            torch.cuda.synchronize()
            assert torch.equal(eager, want[i]), (rep, i)
