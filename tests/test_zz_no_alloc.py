"""kmc_build_kernel_cut_static (the cut over k with its partial sums in the library's static
device array, for callers that cannot allocate) against the two-call form it is a variant of:
kmc_build_kernel on ranges of k into a caller-supplied buffer + kmc_build_kernel_finish.
Both go through the C ABI; the launches and their arithmetic are the same, so the results
must agree bit for bit -- on two calls in a row, the second with a smaller input, whose
partial sums land on top of what the first call left in the shared array."""
import ctypes

import pytest
import torch

from kermac_amd import _backend
from oracle import oracle
from tests.helpers import assert_close_to_truth

pytestmark = pytest.mark.gpu

COL, ROW = _backend.COL_MAJOR, _backend.ROW_MAJOR


def block(a, b, out, col_major, inner_power, outer_power, kernel_type=0, bandwidth=0.0, regularization=0.0, p=0.0):
    """Parameter block for a [M, K] x b [N, K] -> out_store[N, M] (m contiguous)."""
    M, K = a.shape
    N = b.shape[0]
    params = _backend.BuildKernelParams()
    params.inner_operator, params.inner_power = 0, inner_power
    params.outer_power, params.kernel_type = outer_power, kernel_type
    params.m, params.n, params.k, params.l = M, N, K, 1
    params.a_majorness = params.b_majorness = COL if col_major else ROW
    params.a, params.a_ld = a.data_ptr(), (a.stride(1) if col_major else a.stride(0))
    params.b, params.b_ld = b.data_ptr(), (b.stride(1) if col_major else b.stride(0))
    params.c, params.c_ld = out.data_ptr(), out.stride(0)
    params.p_inner_value, params.p_outer_value = p, (1.0 / p if p else 0.0)
    params.bandwidth_value, params.regularization_value = bandwidth, regularization
    params.regularization_offset_x, params.regularization_offset_y = 2, 0
    params.epsilon = 1e-5
    return params


def two_call_form(params, ranges, device, stream):
    """What the new entry point is a variant of, with a buffer of the caller's."""
    depth = max(16, -(-(-(-params.k // ranges)) // 16) * 16)
    used = -(-params.k // depth)
    ld = -(-params.m // 4) * 4
    plane = ld * params.n
    partial = torch.full((used * plane,), float("nan"), device=device)
    sums = _backend.BuildKernelParams.from_buffer_copy(params)
    sums.outer_power = sums.kernel_type = 0
    sums.k, sums.l, sums.k_total = depth, used, params.k
    sums.a_bs = depth * (params.a_ld if params.a_majorness == COL else 1)
    sums.b_bs = depth * (params.b_ld if params.b_majorness == COL else 1)
    sums.c, sums.c_ld, sums.c_bs = partial.data_ptr(), ld, plane
    _backend.build_kernel(sums, stream)
    _backend.build_kernel_finish(params, partial.data_ptr(), ld, 0, plane, used, stream)
    return used


def operands(M, N, K, col_major, device, generator):
    if col_major:
        return (torch.randn(K, M, generator=generator).to(device).t(), torch.randn(K, N, generator=generator).to(device).t())
    return torch.randn(M, K, generator=generator).to(device), torch.randn(N, K, generator=generator).to(device)


CASES = [
    # (M, N, K, ranges, col-major operands, inner power, outer power, kernel type, p): first call, then a smaller one
    ((300, 200, 4100, 8, True, 1, 0, 1, 0.0), (100, 90, 1000, 3, True, 1, 0, 1, 0.0)),          # Laplace-L1 with a diagonal
    ((257, 129, 2049, 5, False, 2, 3, 0, 0.0), (64, 17, 530, 4, False, 2, 3, 0, 0.0)),          # cdist p = 2, row-major
    ((130, 260, 3000, 16, True, 4, 4, 0, 1.3), (33, 50, 700, 2, False, 4, 4, 0, 1.3)),          # cdist p = 1.3
]


@pytest.mark.parametrize("first,second", CASES)
def test_static_scratch_matches_the_two_call_form_on_consecutive_calls(device, first, second):
    g = torch.Generator().manual_seed(first[0] + first[2])
    stream = torch.cuda.current_stream(device).cuda_stream
    for M, N, K, ranges, col_major, inner_power, outer_power, kernel_type, p in (first, second):
        print(f"kmc_build_kernel_cut_static M={M} N={N} K={K} ranges={ranges} col_major={col_major} "
              f"inner={inner_power} outer={outer_power} kernel={kernel_type}", flush=True)
        a, b = operands(M, N, K, col_major, device, g)
        kw = dict(kernel_type=kernel_type, bandwidth=float(K) if kernel_type else 0.0,   # keeps exp(-d / bw) well conditioned
                  regularization=0.25 if kernel_type else 0.0, p=p)
        expected = torch.full((N, M + 3), -3.0, device=device)
        got = torch.full((N, M + 3), -3.0, device=device)
        used = two_call_form(block(a, b, expected, col_major, inner_power, outer_power, **kw), ranges, device, stream)
        assert 1 < used <= ranges
        _backend.build_kernel_cut_static(block(a, b, got, col_major, inner_power, outer_power, **kw), ranges, stream)
        torch.cuda.synchronize()
        assert torch.equal(got, expected), "static-scratch entry point differs from kmc_build_kernel + kmc_build_kernel_finish"
        assert torch.all(got[:, M:] == -3.0), "columns past m were written"
        # and both are right: float64 oracle at the tolerance of the path
        names = {1: "ABS", 2: "SQUARE", 4: "POW"}[inner_power], {0: "NOOP", 3: "SQRT", 4: "POW"}[outer_power]
        truth = oracle.build_kernel("DIFF", names[0], names[1], {0: "NONE", 1: "LAPLACE"}[kernel_type], a.cpu(), b.cpu(),
                                    p_inner=p or None, p_outer=(1.0 / p) if p else None,
                                    bandwidth=kw["bandwidth"] or None, regularization=kw["regularization"] or None,
                                    regularization_offset_x=2, regularization_offset_y=0)[0]
        assert_close_to_truth(got[:, :M].t(), truth, rtol=1e-4 if p else 1e-5, what=f"static scratch M={M} N={N} K={K}")


def test_static_scratch_rejects_what_does_not_fit_and_what_it_does_not_do(device):
    stream = torch.cuda.current_stream(device).cuda_stream
    a = torch.zeros(16, 8, device=device).t()                      # pointers are checked, never dereferenced here
    out = torch.zeros(8, 8, device=device)
    big = block(a, a, out, True, 1, 0)
    big.m = big.n = 4096                                           # 4096 x 4096 floats = 64 MiB per range
    big.a_ld = big.b_ld = big.c_ld = 4096
    big.k = 64
    with pytest.raises(_backend.BackendError, match="static array holds 64 MiB"):
        _backend.build_kernel_cut_static(big, 2, stream)
    batched = block(a, a, out, True, 1, 0)
    batched.l = 2
    with pytest.raises(_backend.BackendError, match="l = 1"):
        _backend.build_kernel_cut_static(batched, 2, stream)
    gram = block(a, a, out, True, 2, 3)
    gram.flags = _backend.FLAG_L2_GRAM
    with pytest.raises(_backend.BackendError, match="matrix-core"):
        _backend.build_kernel_cut_static(gram, 2, stream)
    with pytest.raises(_backend.BackendError, match="at least 1"):
        _backend.build_kernel_cut_static(block(a, a, out, True, 1, 0), 0, stream)
    jit_only = block(a, a, out, True, 3, 0)                        # DIFF + SQRT is compiled at run time only
    with pytest.raises(_backend.BackendError, match="not compiled ahead of time"):
        _backend.build_kernel_cut_static(jit_only, 2, stream)
    assert _backend.STATIC_SCRATCH_BYTES == 64 << 20
    no_result = block(a, a, out, True, 1, 0)
    no_result.c = 0
    with pytest.raises(_backend.BackendError, match="c: null pointer"):          # before anything is launched
        _backend.build_kernel_cut_static(no_result, 2, stream)
    fixed = block(a, a, out, True, 1, 0)
    fixed.flags = _backend.FLAG_L1_FIXED
    with pytest.raises(_backend.BackendError, match="fixed-point"):
        _backend.build_kernel_cut_static(fixed, 2, stream)


def test_static_scratch_replays_from_a_hip_graph(device):
    """After one eager call (which looks up the array's address on this device) the entry point is captured into a
    HIP graph; every replay, with eager work on the shared array and synchronisation in between, gives the bits of the
    two-call form."""
    g = torch.Generator().manual_seed(77)
    M, N, K, ranges = 260, 190, 3000, 6
    a, b = operands(M, N, K, True, device, g)
    expected = torch.empty(N, M, device=device)
    got = torch.empty(N, M, device=device)
    other = torch.empty(90, 100, device=device)
    a2, b2 = operands(100, 90, 800, True, device, g)
    stream = torch.cuda.current_stream(device).cuda_stream
    two_call_form(block(a, b, expected, True, 1, 0, kernel_type=1, bandwidth=float(K)), ranges, device, stream)
    params = block(a, b, got, True, 1, 0, kernel_type=1, bandwidth=float(K))
    _backend.build_kernel_cut_static(params, ranges, stream)                     # eager: the address is looked up here
    torch.cuda.synchronize()
    assert torch.equal(got, expected)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        _backend.build_kernel_cut_static(params, ranges, torch.cuda.current_stream(device).cuda_stream)
    for replay in range(3):
        got.fill_(float("nan"))
        # eager work in between that overwrites the shared array with another problem's partial sums
        _backend.build_kernel_cut_static(block(a2, b2, other, True, 2, 3), 4, torch.cuda.current_stream(device).cuda_stream)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(got, expected), f"replay {replay} differs from the two-call form"
