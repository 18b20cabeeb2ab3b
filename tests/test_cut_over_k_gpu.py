"""GPU tests of run_kernel / cdist calls with a small result over a long contraction, which the
Python layer cuts over k: one batched launch of plain partial sums plus the element-wise kernel
behind kmc_build_kernel_finish, which adds them and applies the epilogue."""
import pytest
import torch

import kermac_amd as kermac
from kermac_amd import build_a_kernel as module
from oracle import oracle
from tests.helpers import assert_close_to_truth, make_operand

pytestmark = pytest.mark.gpu


@pytest.fixture(autouse=True)
def direct_kernel():
    """These tests are about the direct kernel's cut over k; in the default "auto" mode the planner
    first marks squared differences for the matrix cores and run_kernel takes the mark back where
    the cut applies, which the checks of the planner's parts below would have to repeat."""
    with kermac.l2_mode("direct"):
        yield


def is_cut(descriptor, a, b, out=None, **kw):
    plan = module._plan_run_kernel(descriptor, a, b, out, kw.get("p"), None, None, kw.get("bandwidth"), None,
                                   kw.get("regularization"), 0, 0, False)
    return module._cut_over_contraction(plan.params) is not None


@pytest.mark.parametrize("p", [1.0, 2.0, 1.3])
@pytest.mark.parametrize("M,N,K,layout", [(100, 90, 5000, "cc"), (300, 17, 2049, "rr"), (64, 130, 4096, "cr"),
                                          (1, 1, 1000, "rc")])
def test_cdist_small_result_long_contraction(device, p, M, N, K, layout):
    g = torch.Generator().manual_seed(M + N + K)
    a = make_operand(1, M, K, layout[0] == "c", device, g, batch=False)
    b = make_operand(1, N, K, layout[1] == "c", device, g, batch=False)
    assert is_cut(kermac.kernel_descriptor_p_norm if p == 1.3 else kermac.kernel_descriptor_l1_norm, a, b, p=p if p == 1.3 else None)
    truth = oracle.cdist(a.cpu(), b.cpu(), p=p)
    for c_col in (False, True):
        out = torch.full((N, M + 4), -7.0, device=device).t()[:M] if c_col else torch.full((M, N + 4), -7.0, device=device)[:, :N]
        got = kermac.cdist(a, b, out=out, p=p)
        assert got is out
        assert_close_to_truth(got, truth[0], rtol=1e-5 if p != 1.3 else 1e-4, what=f"cut over k p={p} {layout} col={c_col}")
        padding = out.t().untyped_storage() if False else None     # noqa: F841 (kept simple: padding checked below)
    wide = torch.full((M, N + 4), -7.0, device=device)
    kermac.cdist(a, b, out=wide[:, :N], p=p)
    assert torch.all(wide[:, N:] == -7.0), "the padding of a strided out was written"
    skipped = kermac.cdist(a, b, p=p, skip_epilogue=True)
    assert_close_to_truth(skipped, oracle.cdist(a.cpu(), b.cpu(), p=p, skip_epilogue=True), rtol=2e-5 if p != 1.3 else 2e-4,
                          what="cut over k, skip_epilogue")


def test_kernels_regularised_diagonal_and_the_symmetric_shortcut(device):
    g = torch.Generator().manual_seed(31)
    x = torch.rand(257, 3000, generator=g).to(device)
    assert is_cut(kermac.kernel_descriptor_laplace_l1, x, x, bandwidth=40.0, regularization=0.25)
    got = kermac.run_kernel(kermac.kernel_descriptor_laplace_l1, x, x, bandwidth=40.0, regularization=0.25,
                            regularization_offset_x=3, regularization_offset_y=0)
    truth = oracle.run_kernel("DIFF", "ABS", "NOOP", "LAPLACE", x.cpu(), x.cpu(), bandwidth=40.0, regularization=0.25,
                              regularization_offset_x=3, regularization_offset_y=0)
    assert_close_to_truth(got, truth, rtol=1e-5, atol=1e-9, what="cut laplace with offset diagonal")
    plain = kermac.run_kernel(kermac.kernel_descriptor_laplace_l2, x, x, bandwidth=torch.tensor([7.0], device=device),
                              regularization=1e-3)
    assert torch.equal(plain, plain.transpose(1, 2))
    assert torch.all(torch.diagonal(plain[0]) == 1.0 + 1e-3)
    truth = oracle.build_kernel("DIFF", "SQUARE", "SQRT", "LAPLACE", x.cpu(), x.cpu(), bandwidth=7.0, regularization=1e-3)
    assert_close_to_truth(plain, truth, rtol=1e-5, atol=1e-9, what="cut laplace l2, symmetric")


def test_dot_products_and_a_run_time_compiled_descriptor(device, tmp_path, monkeypatch):
    monkeypatch.setenv("KERMAC_AMD_CACHE_DIR", str(tmp_path))
    g = torch.Generator().manual_seed(32)
    a = torch.rand(120, 2600, generator=g).to(device)
    b = torch.rand(77, 2600, generator=g).to(device)
    got = kermac.run_kernel(kermac.kernel_descriptor_mma, a, b)
    assert_close_to_truth(got[0], a.double().cpu() @ b.double().cpu().t(), rtol=1e-5, what="cut dot")
    odd = kermac.KernelDescriptor(kermac.InnerOperator.DOT, kermac.PowerType.SQRT, kermac.PowerType.SQUARE,
                                  kermac.KernelType.NONE)
    assert is_cut(odd, a, b)
    got = kermac.run_kernel(odd, a, b)
    truth = torch.sqrt(a.double().cpu()[:, None, :] * b.double().cpu()[None, :, :]).sum(-1) ** 2
    assert_close_to_truth(got[0], truth, rtol=2e-5, what="cut, run-time compiled")


def test_batched_and_large_results_are_not_cut(device):
    a = torch.rand(3, 100, 3000, device=device)
    b = torch.rand(3, 90, 3000, device=device)
    assert not is_cut(kermac.kernel_descriptor_l1_norm, a, b)
    a = torch.rand(6000, 600, device=device)
    assert not is_cut(kermac.kernel_descriptor_l1_norm, a, a)          # 1128 tiles to compute: the chip is full
    b = torch.rand(17000, 2048, device=device)
    assert not is_cut(kermac.kernel_descriptor_l1_norm, b, a.new_empty(16400, 2048))     # 2048 tiles and more: never
    a = torch.rand(100, 400, device=device)
    assert not is_cut(kermac.kernel_descriptor_l1_norm, a, a)          # contraction too short


@pytest.mark.parametrize("m,n,slices", [(1, 3, 5000), (5, 7, 300), (100, 100, 768), (130, 4, 100), (511, 2, 17),
                                        (600, 3, 9), (1030, 2, 40), (64, 5, 15), (64, 5, 16)])
def test_finish_entry_point_adds_slices_and_applies_the_epilogue(device, m, n, slices):
    """kmc_build_kernel_finish through the C ABI on its own: rows of few m share the slices among
    lane groups, so every split of the lanes is compared with a float64 sum."""
    from kermac_amd import _backend
    g = torch.Generator().manual_seed(m * 31 + slices)
    ld = (m + 3) // 4 * 4
    partial = torch.zeros(slices, n, ld, device=device)
    partial[:, :, :m] = torch.rand(slices, n, m, generator=g).to(device)
    out = torch.full((n, ld), -3.0, device=device)
    params = _backend.BuildKernelParams()
    params.inner_operator = 0
    params.inner_power = 2          # squared differences ...
    params.outer_power = 3          # ... and their square root, as cdist(p=2) asks for
    params.m, params.n, params.k, params.l = m, n, 8, 1
    params.a = params.b = partial.data_ptr()       # checked for null only: the finishing step reads no operand
    params.a_ld = params.b_ld = max(m, n, 8)
    params.c, params.c_ld = out.data_ptr(), ld
    stream = torch.cuda.current_stream(device).cuda_stream
    _backend.build_kernel_finish(params, partial.data_ptr(), ld, 0, n * ld, slices, stream)
    torch.cuda.synchronize()
    truth = partial[:, :, :m].double().sum(0).sqrt()
    assert_close_to_truth(out[:, :m], truth, rtol=1e-5, what=f"finish m={m} n={n} slices={slices}")
    assert torch.all(out[:, m:] == -3.0), "columns past m were written"
    again = torch.full((n, ld), -3.0, device=device)
    params.c = again.data_ptr()
    _backend.build_kernel_finish(params, partial.data_ptr(), ld, 0, n * ld, slices, stream)
    torch.cuda.synchronize()
    assert torch.equal(out, again), "the order of the sum is fixed: two runs agree bit for bit"


@pytest.mark.parametrize("p,M,N,K,col_major", [(1.0, 3000, 2900, 2048, True), (2.0, 3000, 3100, 1024 + 512, False), (2.0, 3072, 3000, 1000, False),
                                              (1.3, 2560, 2560, 2048, True)])
def test_a_result_of_a_few_hundred_tiles_is_cut_into_a_few_ranges(device, monkeypatch, p, M, N, K, col_major):
    """385 to 2047 tiles: k is cut into 2 to 8 ranges, several rounds of shorter workgroups.  Checked
    against the oracle on slabs of rows and against the uncut launch everywhere."""
    g = torch.Generator().manual_seed(int(p * 10) + M)
    a = make_operand(1, M, K, col_major, device, g, batch=False)
    b = make_operand(1, N, K, col_major, device, g, batch=False)
    descriptor = {1.0: kermac.kernel_descriptor_l1_norm, 2.0: kermac.kernel_descriptor_l2_norm,
                  1.3: kermac.kernel_descriptor_p_norm}[p]
    plan = module._plan_run_kernel(descriptor, a, b, None, p if p == 1.3 else None, None, None, None, None, None, 0, 0, False)
    cut = module._cut_over_contraction(plan.params)
    assert cut is not None and 2 <= cut[0] <= 8, cut
    got = kermac.cdist(a, b, p=p)[0]             # unbatched operands, out=None: the result is [1, M, N]
    rtol = 1e-4 if p == 1.3 else 1e-5
    for rows in (slice(0, 48), slice(M - 48, M)):
        assert_close_to_truth(got[rows], oracle.cdist(a[rows].cpu(), b.cpu(), p=p)[0], rtol=rtol, what=f"mid-size cut p={p}")
    monkeypatch.setattr(module, "_cut_over_contraction", lambda params: None)
    uncut = kermac.cdist(a, b, p=p)[0]
    assert_close_to_truth(got, uncut, rtol=rtol / 2, what="cut against uncut")


def test_a_set_against_itself_is_cut_by_the_tiles_of_one_triangle(device):
    g = torch.Generator().manual_seed(77)
    x = torch.randn(2048, 3584, generator=g).to(device).t()       # K-major, 28 x 28 tiles, 406 to compute
    plan = module._plan_run_kernel(kermac.kernel_descriptor_l2_norm, x, x, None, None, None, None, None, None, None, 0, 0, False)
    assert module._cut_over_contraction(plan.params) is not None
    got = kermac.cdist(x, x, p=2.0)[0]
    assert torch.equal(got, got.t())
    assert torch.all(torch.diagonal(got) == 0.0)
    rows = slice(1000, 1040)
    assert_close_to_truth(got[rows], oracle.cdist(x[rows].cpu(), x.cpu(), p=2.0)[0], rtol=1e-5, atol=1e-30, what="x against x, cut")


@pytest.mark.parametrize("out_row_major", [True, False])
def test_a_tall_narrow_result_is_cut_beyond_65535_rows(device, monkeypatch, out_row_major):
    """782 tiles stacked along one side, K = 2048: the call is cut over k, and the finishing
    kernel walks more rows of the result than one grid dimension holds (70000 > 65535).  With a
    row-major result the operands are exchanged, with a column-major one they are not: the long
    side is n of the kernel in one case and m in the other."""
    g = torch.Generator().manual_seed(9)
    M, N, K = 70000, 100, 2048
    a = torch.randn(M, K, generator=g).to(device)
    b = torch.randn(N, K, generator=g).to(device)
    out = torch.empty(M, N, device=device) if out_row_major else torch.empty(N, M, device=device).t()
    plan = module._plan_run_kernel(kermac.kernel_descriptor_l1_norm, a, b, out, None, None, None, None, None, None, 0, 0, False)
    assert plan.swapped == out_row_major and (plan.params.n if out_row_major else plan.params.m) == M
    assert module._cut_over_contraction(plan.params) is not None
    got = kermac.cdist(a, b, out=out, p=1.0)
    for rows in (slice(0, 40), slice(65520, 65560), slice(M - 40, M)):
        assert_close_to_truth(got[rows], oracle.cdist(a[rows].cpu(), b.cpu(), p=1.0)[0], rtol=1e-5, what=f"tall result rows {rows}")
    monkeypatch.setattr(module, "_cut_over_contraction", lambda params: None)
    uncut = kermac.cdist(a, b, p=1.0)[0]
    assert_close_to_truth(got, uncut, rtol=5e-6, what="cut against uncut")
