"""GPU tests of sums of products (inner operator DOT: linear and polynomial kernels) on the fp16
matrix instruction: in the l2 modes "auto" (large problems) and "gram_bf16", run_kernel offers the
library a workspace and KMC_FLAG_DOT_PIECES, and the 256 x 256 walk of the squared-difference
route multiplies two fp16 pieces per value (include/kermac_amd.h).  Nothing cancels in a product,
so there is no trust check: the error is below 3 * 2^-22 sum_k |a b|, and the tests measure against
that sum (1e-6 of it, the size of an fp32 sum's own rounding).

KERMAC_AMD_WIDE_MIN_TILES=1 sends the small shapes of these tests down the route.
"""
import pytest
import torch

import kermac_amd as kermac
from kermac_amd import _backend, build_a_kernel as module
from oracle import oracle
from tests.helpers import assert_close_to_truth, make_operand

pytestmark = pytest.mark.gpu

DOT = kermac.KernelDescriptor(kermac.InnerOperator.DOT, kermac.PowerType.NOOP, kermac.PowerType.NOOP, kermac.KernelType.NONE)
POLYNOMIAL = kermac.KernelDescriptor(kermac.InnerOperator.DOT, kermac.PowerType.NOOP, kermac.PowerType.POW, kermac.KernelType.NONE)
LAPLACE_OF_DOT = kermac.KernelDescriptor(kermac.InnerOperator.DOT, kermac.PowerType.NOOP, kermac.PowerType.ABS, kermac.KernelType.LAPLACE)


@pytest.fixture
def pieces(monkeypatch):
    monkeypatch.setenv("KERMAC_AMD_WIDE_MIN_TILES", "1")
    kermac.set_l2_mode("gram_bf16", min_k=0)
    yield
    kermac.set_l2_mode(kermac.DEFAULT_L2_MODE)


def plan_of(descriptor, a, b, **kw):
    out = torch.empty(1, a.shape[-2], b.shape[-2], device=a.device)
    return module._plan_run_kernel(descriptor, a, b, out, None, None, kw.get("outer_p"), kw.get("bandwidth"), None, None, 0, 0, False)


def error_of_sum(got, a, b):
    """max |got - a b^T| / sum_k |a b| in float64"""
    truth = torch.matmul(a.double(), b.double().transpose(-1, -2)).cpu()
    scale = torch.matmul(a.abs().double(), b.abs().double().transpose(-1, -2)).cpu()
    return float(((got.cpu().double() - truth).abs() / scale.clamp_min(1e-300)).max())


@pytest.mark.parametrize("M,N,K", [(1, 1, 1), (70, 33, 17), (300, 257, 64), (600, 520, 100), (257, 1000, 33), (256, 256, 16), (513, 255, 1000)])
@pytest.mark.parametrize("layout", ["cc", "rr", "cr"])
def test_products_of_all_layouts(device, pieces, M, N, K, layout):
    g = torch.Generator().manual_seed(M + N + K)
    a = make_operand(1, M, K, layout[0] == "c", device, g, batch=False)
    b = make_operand(1, N, K, layout[1] == "c", device, g, batch=False)
    plan = plan_of(DOT, a, b)
    assert plan.params.flags & _backend.FLAG_DOT_PIECES and _backend.gram_workspace_bytes(plan.params) > 0
    got = kermac.run_kernel(DOT, a, b)
    assert got.shape == (1, M, N)
    assert error_of_sum(got[0], a, b) < 1e-6
    truth = oracle.run_kernel("DOT", "NOOP", "NOOP", "NONE", a.cpu().contiguous(), b.cpu().contiguous())
    assert_close_to_truth(got, truth, rtol=1e-5, atol=1e-6 * float(a.abs().cpu().double().max() * b.abs().cpu().double().max()) * K,
                          what=f"dot {layout}")
    column_major = torch.empty(1, N, M, device=device).transpose(1, 2)
    # the other layout of the result exchanges the roles of the operands, and with them the order of the piece products
    assert error_of_sum(kermac.run_kernel(DOT, a, b, out=column_major)[0], a, b) < 1e-6


def test_kernel_functions_of_a_product_batches_and_the_diagonal(device, pieces):
    g = torch.Generator().manual_seed(41)
    L, M, N, K = 3, 300, 280, 48
    a = make_operand(L, M, K, True, device, g)
    b = make_operand(1, N, K, False, device, g, batch=False)                  # shared by the batch
    got = kermac.run_kernel(POLYNOMIAL, a, b, outer_p=3.0)
    truth = oracle.run_kernel("DOT", "NOOP", "POW", "NONE", a.cpu().contiguous(), b.cpu().contiguous(), p_outer=3.0)
    # the outer power of the reference's epilogue is |x|^p; a product's relative error is that of the sum over |sum|
    assert_close_to_truth(got, truth, rtol=1e-4, atol=1e-4 * float(truth.abs().mean()), what="polynomial kernel")
    bandwidth = torch.tensor([20.0, 30.0, 50.0], device=device)
    kw = dict(bandwidth=bandwidth, regularization=0.25, regularization_offset_x=3, regularization_offset_y=1)
    got = kermac.run_kernel(LAPLACE_OF_DOT, a, b, **kw)
    truth = oracle.run_kernel("DOT", "NOOP", "ABS", "LAPLACE", a.cpu().contiguous(), b.cpu().contiguous(), bandwidth=bandwidth.cpu(),
                              regularization=0.25, regularization_offset_x=3, regularization_offset_y=1)
    assert_close_to_truth(got, truth, rtol=1e-5, atol=1e-6, what="laplace of a product, regularised")
    assert float((got == 1.25).sum()) == L * min(M - 2, N), "the regularised elements"


def test_a_panel_against_itself_is_symmetric_bit_for_bit(device, pieces):
    g = torch.Generator().manual_seed(42)
    a = torch.randn(700, 96, generator=g).to(device)
    got = kermac.run_kernel(DOT, a, a)[0]
    assert torch.equal(got, got.t())
    assert error_of_sum(got, a, a) < 1e-6
    other = kermac.run_kernel(DOT, a, a.clone())[0]                           # two panels: every tile computed
    assert error_of_sum(other, a, a) < 1e-6 and torch.allclose(other, got, rtol=1e-5, atol=1e-4)


def test_rows_of_very_different_magnitude(device, pieces):
    """The scale of the pieces is per row, so a row of values around 1e-6 beside rows around 1e+5 keeps its digits."""
    g = torch.Generator().manual_seed(43)
    M, N, K = 300, 270, 80
    a = torch.randn(M, K, generator=g) * torch.pow(10.0, (torch.arange(M) % 12 - 6).float())[:, None]
    b = torch.randn(N, K, generator=g) * torch.pow(10.0, (torch.arange(N) % 7 - 3).float())[:, None]
    got = kermac.run_kernel(DOT, a.to(device), b.to(device))[0]
    assert error_of_sum(got, a, b) < 1e-6


def test_which_calls_take_the_route(device, monkeypatch):
    a = torch.empty(8192, 512, device=device)
    b = torch.empty(4096, 512, device=device)

    def bytes_wanted(descriptor=DOT, **kw):
        plan = plan_of(descriptor, a, b, **kw)
        return _backend.gram_workspace_bytes(plan.params) if plan.params.flags & _backend.FLAG_DOT_PIECES else 0

    assert kermac.get_l2_mode() == "auto"
    assert bytes_wanted() > 0                                                 # 32 x 16 tiles, 1.7e10 terms
    assert bytes_wanted(POLYNOMIAL, outer_p=2.0) > 0
    assert bytes_wanted(kermac.KernelDescriptor(kermac.InnerOperator.DOT, kermac.PowerType.SQUARE, kermac.PowerType.NOOP,
                                                kermac.KernelType.NONE)) == 0     # the products themselves are squared: not a product of sums
    for mode, expected in (("direct", False), ("gram", False), ("gram_bf16", True)):
        with kermac.l2_mode(mode):
            assert (bytes_wanted() > 0) == expected, mode
    small = plan_of(DOT, a[:300], b[:300])                                    # 4 tiles: the direct kernel
    assert module._auto_matrix_core_flags(small.params, small.params.flags & _backend.FLAG_DOT_PIECES) == 0


def test_without_a_workspace_the_direct_kernel_runs(device, pieces):
    g = torch.Generator().manual_seed(44)
    a = torch.randn(300, 40, generator=g).to(device)
    b = torch.randn(260, 40, generator=g).to(device)
    with kermac.l2_mode("direct"):
        reference = kermac.run_kernel(DOT, a, b)
    plan = plan_of(DOT, a, b)
    stream = torch.cuda.current_stream(device).cuda_stream
    needed = _backend.gram_workspace_bytes(plan.params)
    workspace = torch.empty(needed, dtype=torch.uint8, device=device)
    for pointer, size in ((0, 0), (workspace.data_ptr(), needed - 1), (workspace.data_ptr() + 16, needed)):
        plan.out.fill_(-1.0)
        plan.params.gram_workspace, plan.params.gram_workspace_bytes = pointer, size
        _backend.build_kernel(plan.params, stream)
        assert torch.equal(plan.out, reference), "null, short or misaligned workspace: expected the direct kernel's bits"
    wrong = plan_of(kermac.kernel_descriptor_l1_norm, a, b)
    wrong.params.flags |= _backend.FLAG_DOT_PIECES
    with pytest.raises(_backend.BackendError):
        _backend.build_kernel(wrong.params, stream)


def test_products_times_coefficients_go_in_panels(device, pieces, monkeypatch, capsys):
    """run_kernel(..., coefficients=...) of a sum of products: the matrix panel by panel through the
    same route, each panel contracted by kmc_matrix_times_coefficients."""
    monkeypatch.setenv("KERMAC_AMD_COEFFICIENT_PANEL_BYTES", "4096")          # panels of 256 centres
    g = torch.Generator().manual_seed(45)
    L, M, N, K, O = 2, 300, 700, 40, 5
    a = make_operand(L, M, K, True, device, g)
    b = make_operand(1, N, K, False, device, g, batch=False)
    coef = torch.randn(L, N, O, generator=g).to(device)
    for descriptor, names, kw, okw in ((DOT, ("DOT", "NOOP", "NOOP", "NONE"), {}, {}),
                                       (POLYNOMIAL, ("DOT", "NOOP", "POW", "NONE"), {"outer_p": 2.0}, {"p_outer": 2.0})):
        got = kermac.run_kernel(descriptor, a, b, coefficients=coef, debug=True, **kw)
        assert "(Kermac Debug) Kernel matrix x coefficients in 3 panels of 256 centres" in capsys.readouterr().out
        truth = oracle.run_kernel_coefficients(*names, a.cpu().contiguous(), b.cpu().contiguous(), coef.cpu(), **okw)
        assert_close_to_truth(got, truth, rtol=1e-5, atol=1e-4 * float(truth.abs().mean()), what=f"{names} x coefficients")
    with kermac.l2_mode("direct"):
        kermac.run_kernel(DOT, a, b, coefficients=coef, debug=True)
        assert "panels" not in capsys.readouterr().out
