"""GPU tests of the limits of the path: outputs with more than 2^31 elements (every
offset inside the kernels is 64-bit) and replays from a HIP graph (no entry point
allocates or synchronises, so launches can be captured).  All calls go through the
public operators and therefore through the C ABI.
"""
import pytest
import torch

import kermac_amd as kermac
from kermac_amd import _backend
from oracle import oracle
from tests.helpers import assert_close_to_truth

pytestmark = pytest.mark.gpu


def free_bytes(device):
    return torch.cuda.mem_get_info(device)[0]


def test_cdist_output_beyond_2_31_elements(device):
    """out_store[N, M] with N * M > 2^31: blocks at the start, across element 2^31 and
    at the end are checked against the oracle; a checksum over the whole matrix is
    checked through sum_mn d1(a_m, b_n) for K = 1 sorted data (closed form below)."""
    M = N = 46500
    K = 8
    assert M * N > 2 ** 31
    if free_bytes(device) < 3 * 4 * M * N:
        pytest.skip("not enough free device memory")
    g = torch.Generator().manual_seed(2031)
    a_store = torch.randn(K, M, generator=g).to(device)
    b_store = torch.randn(K, N, generator=g).to(device)
    out_store = torch.full((N, M), float("nan"), device=device)
    out = kermac.cdist(a_store.t(), b_store.t(), p=1.0, out=out_store.t())
    assert out.shape == (M, N) and out.data_ptr() == out_store.data_ptr()
    n_cross = 2 ** 31 // M                                  # the row of out_store that holds element 2^31
    for ms, ns in ((slice(0, 150), slice(0, 150)),
                   (slice(0, M, 311), slice(n_cross - 2, n_cross + 3)),
                   (slice(M - 260, M), slice(n_cross - 130, n_cross + 130)),
                   (slice(M - 150, M), slice(N - 150, N))):
        truth = oracle.cdist(a_store[:, ms].t().cpu(), b_store[:, ns].t().cpu(), p=1.0)[0]
        assert_close_to_truth(out_store[ns, ms].t(), truth, rtol=1e-5, what=f"large out block {ms} {ns}")
    assert not torch.isnan(out_store).any(), "some element was never written"
    # Column sums of the whole matrix against a float64 matrix-vector identity:
    # sum_n |a_mk - b_nk| summed over k, accumulated slab by slab in float64.
    col_sum = torch.zeros(M, dtype=torch.float64, device=device)
    for n0 in range(0, N, 1500):
        col_sum += out_store[n0:n0 + 1500].double().sum(dim=0)
    truth_sum = torch.zeros(M, dtype=torch.float64, device=device)
    b_sorted, _ = torch.sort(b_store.double(), dim=1)
    prefix = torch.cumsum(b_sorted, dim=1)
    total = prefix[:, -1:]
    for k in range(K):
        # sum_n |x - b_n| = x (2 c - N) - 2 prefix[c] + total, c = #{b_n <= x}
        x = a_store[k].double()
        cnt = torch.searchsorted(b_sorted[k].contiguous(), x.contiguous(), right=True)
        below = torch.where(cnt > 0, prefix[k][(cnt - 1).clamp_min(0)], torch.zeros_like(x))
        truth_sum += x * (2 * cnt - N) - 2 * below + total[k]
    assert_close_to_truth(col_sum, truth_sum, rtol=2e-6, what="column sums of the large matrix")


def test_self_matrix_beyond_2_31_elements(device):
    """A set against itself with more than 2^31 results: the mirrored stores of the
    symmetric shortcut use 64-bit offsets too.  Must equal the full computation."""
    M, K = 46500, 8
    if free_bytes(device) < 3 * 4 * M * M:
        pytest.skip("not enough free device memory")
    g = torch.Generator().manual_seed(2035)
    x_store = torch.randn(K, M, generator=g).to(device)
    out_self = torch.full((M, M), float("nan"), device=device)
    out_full = torch.empty(M, M, device=device)
    kermac.cdist(x_store.t(), x_store.t(), p=2.0, out=out_self.t())
    kermac.cdist(x_store.t(), x_store.clone().t(), p=2.0, out=out_full.t())
    assert torch.equal(out_self, out_full)
    del out_full
    truth = oracle.cdist(x_store[:, -200:].t().cpu(), x_store[:, :200].t().cpu(), p=2.0)[0]
    assert_close_to_truth(out_self[:200, -200:].t(), truth, rtol=1e-5, what="corner of the large self matrix")
    assert_close_to_truth(out_self[-200:, :200], truth, rtol=1e-5, what="mirrored corner of the large self matrix")


def test_cdist_batch_stride_beyond_2_31(device):
    """Three batches of 27000 x 27000: the third batch starts past element 2^31 only
    through the batch stride."""
    L, M, N, K = 3, 27000, 27000, 4
    assert (L - 1) * M * N < 2 ** 31 < L * M * N
    if free_bytes(device) < 2 * 4 * L * M * N:
        pytest.skip("not enough free device memory")
    g = torch.Generator().manual_seed(2032)
    a = torch.randn(L, K, M, generator=g).to(device).transpose(1, 2)
    b = torch.randn(L, K, N, generator=g).to(device).transpose(1, 2)
    out_store = torch.full((L, N, M), float("nan"), device=device)
    kermac.cdist(a, b, p=2.0, out=out_store.transpose(1, 2))
    for l, ms, ns in ((0, slice(0, 130), slice(0, 130)), (2, slice(M - 200, M), slice(N - 200, N)),
                      (2, slice(13000, 13200), slice(25900, 26100))):
        truth = oracle.cdist(a[l, ms].cpu(), b[l, ns].cpu(), p=2.0)[0]
        assert_close_to_truth(out_store[l, ns, ms].t(), truth, rtol=1e-5, what=f"batch {l} block")
    assert not torch.isnan(out_store[2, -1]).any()


def test_gradient_output_beyond_2_31_elements(device):
    """out[O, N, M] of cdist_grad with O * N * M > 2^31 (matrix-core kernel, O = 16)
    and with O = 5 (vector-ALU kernel): first and last blocks against the oracle."""
    for O, NM in ((16, 11700), (5, 20800)):
        M = N = NM
        K = 8
        assert O * N * M > 2 ** 31
        if free_bytes(device) < 2 * 4 * O * N * M:
            pytest.skip("not enough free device memory")
        g = torch.Generator().manual_seed(2033 + O)
        a = torch.rand(K, M, generator=g).to(device)
        b = torch.randn(N, K, generator=g).to(device)
        c = torch.randn(O, K, generator=g).to(device)
        d = torch.randn(N, M, generator=g).to(device)
        out = torch.full((O, N, M), float("nan"), device=device)
        kermac.cdist_grad(a, b, c, d, out=out, p=1.0)
        for ms, ns in ((slice(0, 100), slice(0, 40)), (slice(M - 100, M), slice(N - 40, N))):
            truth = oracle.cdist_grad(a[:, ms].cpu().contiguous(), b[ns].cpu(), c.cpu(), d[ns, ms].cpu().contiguous(),
                                      p=1.0)[0]
            assert_close_to_truth(out[:, ns, ms], truth, rtol=1e-5, atol=1e-5 * float(truth.abs().mean()) * 10,
                                  what=f"large gradient O={O} block {ms} {ns}")
        assert not torch.isnan(out[-1, -1]).any() and not torch.isnan(out[O // 2, N // 2]).any()
        del out


def test_operators_replay_from_a_hip_graph(device):
    """cdist, a Laplace kernel, the fused coefficient product and cdist_grad captured
    into one graph; every replay (with eager work and synchronisation in between, on
    new input values) must equal the eager result bit for bit."""
    g = torch.Generator().manual_seed(2034)
    M, N, K, O = 700, 520, 96, 16
    a_store = torch.randn(K, M, generator=g).to(device)
    b_store = torch.randn(K, N, generator=g).to(device)
    coef = torch.randn(N, O, generator=g).to(device)
    weights = torch.rand(N, M, generator=g).to(device)          # cdist_grad's a[K', M'] = [N, M]
    centres = torch.randn(K, N, generator=g).to(device)         # b[N', K'] = [K, N]
    classes = torch.randn(O, N, generator=g).to(device)         # c[O, K'] = [O, N]
    samples = torch.randn(K, M, generator=g).to(device)         # d[N', M'] = [K, M]
    out_p1 = torch.empty(N, M, device=device)
    out_p13 = torch.empty(N, M, device=device)
    out_lap = torch.empty(N, M, device=device)
    out_fused = torch.empty(1, M, O, device=device)
    out_grad = torch.empty(O, K, M, device=device)

    def run_all():
        kermac.cdist(a_store.t(), b_store.t(), p=1.0, out=out_p1.t())
        kermac.cdist(a_store.t(), b_store.t(), p=1.3, out=out_p13.t())
        kermac.run_kernel(kermac.kernel_descriptor_laplace_l2, a_store.t(), b_store.t(), out=out_lap.t(), bandwidth=4.0)
        kermac.run_kernel(kermac.kernel_descriptor_laplace_l1, a_store.t(), b_store.t(), out=out_fused, bandwidth=9.0,
                          coefficients=coef)
        kermac.cdist_grad(weights, centres, classes, samples, out=out_grad, p=1.0)

    outs = (out_p1, out_p13, out_lap, out_fused, out_grad)
    side = torch.cuda.Stream(device=device)
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        run_all()                                               # warm-up outside capture
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        run_all()
    for replay in range(4):
        a_store.copy_(torch.randn(K, M, generator=g))           # new values, same addresses
        samples.mul_(1.25)
        run_all()
        torch.cuda.synchronize()
        eager = [o.clone() for o in outs]
        for o in outs:
            o.fill_(float("nan"))
        scratch = torch.randn(256, 256, device=device) @ torch.randn(256, 256, device=device)   # eager work between replays
        graph.replay()
        torch.cuda.synchronize()
        del scratch
        for name, e, o in zip(("p1", "p1.3", "laplace", "fused", "grad"), eager, outs):
            assert torch.equal(e, o), f"replay {replay}: {name} differs from the eager result"
    truth = oracle.cdist(a_store.t().cpu(), b_store.t().cpu(), p=1.0)[0]
    assert_close_to_truth(out_p1.t(), truth, rtol=1e-5, what="graph replay vs oracle")


def test_workspace_routes_replay_from_a_hip_graph(device, monkeypatch):
    """The routes that go through a workspace allocated by the Python layer (squared differences on
    the fp16 matrix instruction: centre, row statistics, split, product, repair; the L1 and L2
    gradients on the fp16 matrix instruction) captured into one graph: the workspace comes from the graph's memory
    pool, the decision whether to subtract the centre is taken on the device, and every replay on
    new values equals the eager result bit for bit."""
    monkeypatch.setenv("KERMAC_AMD_WIDE_MIN_TILES", "1")
    monkeypatch.setenv("KERMAC_AMD_GRADIENT_F16_MIN_TERMS", "1")
    monkeypatch.setenv("KERMAC_AMD_GRADIENT_L2_MIN_TERMS", "1")
    monkeypatch.setenv("KERMAC_AMD_COEFFICIENT_PANEL_BYTES", "4096")         # panels of 256 centres: three here
    g = torch.Generator().manual_seed(77)
    M, N, K, O = 600, 520, 96, 16
    a_store = torch.randn(K, M, generator=g).to(device)
    b_store = torch.randn(K, N, generator=g).to(device)
    b_store[:, :100] = a_store[:, :100] + 1e-5 * torch.randn(K, 100, generator=g).to(device)      # twins: repaired parts
    weights = torch.rand(N, M, generator=g).to(device)
    centres = torch.randn(K, N, generator=g).to(device)
    classes = torch.randn(O, N, generator=g).to(device)
    samples = torch.randn(K, M, generator=g).to(device)
    out_p2 = torch.empty(N, M, device=device)
    out_self = torch.empty(M, M, device=device)
    out_grad = torch.empty(O, K, M, device=device)
    out_grad_l2 = torch.empty(O, K, M, device=device)
    coefficients = torch.randn(N, 5, generator=g).to(device)
    out_product = torch.empty(1, M, 5, device=device)

    def run_all():
        with kermac.l2_mode("gram_bf16", min_k=0):
            kermac.cdist(a_store.t(), b_store.t(), p=2.0, out=out_p2.t())
            kermac.cdist(a_store.t(), a_store.t(), p=2.0, out=out_self.t())
            # the kernel matrix x coefficients product panel by panel: panel, workspace and partial products
            kermac.run_kernel(kermac.kernel_descriptor_laplace_l2, a_store.t(), b_store.t(), out=out_product,
                              bandwidth=10.0, coefficients=coefficients)
        kermac.cdist_grad(weights, centres, classes, samples, out=out_grad, p=1.0)
        kermac.cdist_grad(weights, centres, classes, samples, out=out_grad_l2, p=2.0)

    outs = (out_p2, out_self, out_grad, out_product, out_grad_l2)
    side = torch.cuda.Stream(device=device)
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        run_all()                                               # warm-up outside capture
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        run_all()
    for replay in range(4):
        a_store.copy_(torch.randn(K, M, generator=g) + (3.0 if replay % 2 else 0.0))     # with and without a centre that matters
        samples.mul_(1.25)
        run_all()
        torch.cuda.synchronize()
        eager = [o.clone() for o in outs]
        for o in outs:
            o.fill_(float("nan"))
        scratch = torch.randn(256, 256, device=device) @ torch.randn(256, 256, device=device)   # eager work between replays
        graph.replay()
        torch.cuda.synchronize()
        del scratch
        for name, e, o in zip(("p2", "p2 self", "grad", "product in panels", "L2 grad"), eager, outs):
            assert torch.equal(e, o), f"replay {replay}: {name} differs from the eager result"
    truth = oracle.cdist(a_store.t().cpu(), b_store.t().cpu(), p=2.0)[0]
    assert_close_to_truth(out_p2.t(), truth, rtol=1e-5, atol=1e-30, what="graph replay vs oracle")
    truth = oracle.kernel_times_coefficients("DIFF", "SQUARE", "SQRT", "LAPLACE", a_store.t().cpu(), b_store.t().cpu(),
                                             coefficients.cpu(), bandwidth=10.0)
    assert_close_to_truth(out_product, truth, rtol=1e-5, atol=1e-4 * float(truth.abs().mean()), what="product replay vs oracle")


def test_cut_launches_replay_from_a_hip_graph(device):
    """The calls that the Python layer cuts into a batched launch plus a sum of partial results
    (few rows against many centres; few results with a deep contraction) allocate a buffer and
    call a library reduction: captured, every replay must equal the eager result bit for bit."""
    import importlib
    grad_module = importlib.import_module("kermac_amd.cdist_grad")
    from kermac_amd import kernel_coefficients as coef_module
    g = torch.Generator().manual_seed(2035)
    M, N, K, O = 200, 5077, 40, 3
    x = torch.rand(M, K, generator=g).to(device)
    z = torch.rand(N, K, generator=g).to(device)
    coef = torch.randn(N, O, generator=g).to(device)
    out_fused = torch.empty(1, M, O, device=device)
    plan = coef_module._plan_run_kernel_coefficients(kermac.kernel_descriptor_laplace_l1, x, z, coef, None, None, None,
                                                     None, 2.0, None, None, 0, 0)
    assert coef_module._centre_ranges(plan, three_resident=True) > 1
    weights = torch.rand(4100, 150, generator=g).to(device)     # cdist_grad's a[K', M']
    centres = torch.randn(30, 4100, generator=g).to(device)     # b[N', K']
    classes = torch.randn(2, 4100, generator=g).to(device)      # c[O', K']
    samples = torch.randn(30, 150, generator=g).to(device)      # d[N', M']
    out_grad = torch.empty(2, 30, 150, device=device)
    assert grad_module._split_over_contraction(
        grad_module._plan_cdist_grad(weights, centres, classes, samples, None, 1.0)) is not None

    long_a = torch.rand(150, 3000, generator=g).to(device)      # a small distance matrix over a long contraction
    long_b = torch.rand(90, 3000, generator=g).to(device)
    out_long = torch.empty(150, 90, device=device)
    from kermac_amd import build_a_kernel as kernel_module
    planned = kernel_module._plan_run_kernel(kermac.kernel_descriptor_l2_norm, long_a, long_b, out_long, None, None, None, None,
                                             None, None, 0, 0, False).params
    matrix_cores = planned.flags & (_backend.FLAG_L2_GRAM | _backend.FLAG_L2_GRAM_BF16)
    assert matrix_cores and kernel_module._auto_matrix_core_flags(planned, matrix_cores) == 0      # two tiles: the direct path
    planned.flags &= ~matrix_cores
    assert kernel_module._cut_over_contraction(planned) is not None                                # ... which cuts it over k

    def run_all():
        kermac.run_kernel(kermac.kernel_descriptor_laplace_l1, x, z, out=out_fused, bandwidth=2.0, coefficients=coef)
        kermac.cdist_grad(weights, centres, classes, samples, out=out_grad, p=1.0)
        kermac.cdist(long_a, long_b, out=out_long, p=2.0)

    outs = (out_fused, out_grad, out_long)
    side = torch.cuda.Stream(device=device)
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        run_all()                                               # warm-up outside capture
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        run_all()
    for replay in range(4):
        x.copy_(torch.rand(M, K, generator=g))                  # new values, same addresses
        samples.mul_(1.25)
        long_a.mul_(0.9)
        run_all()
        torch.cuda.synchronize()
        eager = [o.clone() for o in outs]
        for o in outs:
            o.fill_(float("nan"))
        scratch = torch.randn(256, 256, device=device) @ torch.randn(256, 256, device=device)   # eager work between replays
        graph.replay()
        torch.cuda.synchronize()
        del scratch
        for name, e, o in zip(("fused", "grad", "long contraction"), eager, outs):
            assert torch.equal(e, o), f"replay {replay}: {name} differs from the eager result"
    truth = oracle.kernel_times_coefficients("DIFF", "ABS", "NOOP", "LAPLACE", x.cpu(), z.cpu(), coef.cpu(), bandwidth=2.0)
    assert_close_to_truth(out_fused, truth, rtol=1e-5, atol=1e-5 * truth.abs().max().item(), what="cut fused replay")


def test_concurrent_host_threads_on_their_own_streams(device):
    """Four host threads, each with its own stream, call the three operators at the same
    time; ctypes releases the interpreter lock during the launches, so this exercises the
    thread-local error state and the absence of shared mutable state on the launch path."""
    import threading
    g = torch.Generator().manual_seed(99)
    problems = []
    for t in range(4):
        M, N, K, O = 200 + 37 * t, 150 + 11 * t, 48 + 5 * t, 3 + t
        a = torch.rand(M, K, generator=g).to(device)
        b = torch.rand(N, K, generator=g).to(device)
        grad = [torch.rand(K, M, generator=g).to(device), torch.randn(N, K, generator=g).to(device),
                torch.randn(O, K, generator=g).to(device), torch.randn(N, M, generator=g).to(device)]
        coef = torch.randn(N, O, generator=g).to(device)
        problems.append((a, b, grad, coef))
    results, errors = [None] * 4, []
    torch.cuda.synchronize()

    def work(t):
        try:
            a, b, grad, coef = problems[t]
            stream = torch.cuda.Stream(device=device)
            with torch.cuda.stream(stream):
                for _ in range(25):
                    d1 = kermac.cdist(a, b, p=1.0)
                    d13 = kermac.cdist(a, b, p=1.3)
                    e = kermac.cdist_grad(*grad, p=1.0)
                    f = kermac.run_kernel(kermac.kernel_descriptor_laplace_l1, a, b, coefficients=coef, bandwidth=2.0)
            stream.synchronize()
            results[t] = (d1, d13, e, f)
        except Exception as exc:       # reported by the main thread
            errors.append((t, exc))

    threads = [threading.Thread(target=work, args=(t,)) for t in range(4)]
    for th in threads:
        th.start()
    for th in threads:
        th.join()
    assert not errors, errors
    for t, (a, b, grad, coef) in enumerate(problems):
        d1, d13, e, f = results[t]
        cpu = [x.cpu() for x in (a, b)]
        assert_close_to_truth(d1, oracle.cdist(*cpu, p=1.0), rtol=1e-5, what=f"thread {t} p=1")
        assert_close_to_truth(d13, oracle.cdist(*cpu, p=1.3), rtol=1e-4, what=f"thread {t} p=1.3")
        truth = oracle.cdist_grad(*[x.cpu() for x in grad], p=1.0)
        assert_close_to_truth(e, truth, rtol=1e-5, atol=1e-5 * truth.abs().max().item(), what=f"thread {t} grad")
        truth = oracle.kernel_times_coefficients("DIFF", "ABS", "NOOP", "LAPLACE", *cpu, coef.cpu(), bandwidth=2.0)
        assert_close_to_truth(f, truth, rtol=1e-5, atol=1e-5 * truth.abs().max().item(), what=f"thread {t} fused")
