"""GPU tests of the direct kernel's variant that keeps the b operand in scalar registers (csrc/kernels/
build_kernel_scalar_b.hpp): absolute and squared differences of operands whose rows are contiguous, K and N
multiples of 16.  By its own rule the library launches it from 1800 tiles of 256 x 64 per batch entry and K = 64 on;
KERMAC_AMD_SCALAR_B_MIN_TILES=1 sends the small shapes of these tests to it.  It sums the terms of every element in
the order of the ordinary kernel (include/build_a_kernel.cuh:339-370 has one kernel for all shapes), so beside the
oracle the tests ask for that kernel's bits.
"""
import pytest
import torch

import kermac_amd as kermac
from oracle import oracle
from tests.helpers import assert_close_to_truth, l1_distances_float64

pytestmark = pytest.mark.gpu


@pytest.fixture
def scalar_b(monkeypatch):
    monkeypatch.setenv("KERMAC_AMD_SCALAR_B_MIN_TILES", "1")
    kermac.set_l2_mode("direct")
    yield monkeypatch
    kermac.set_l2_mode(kermac.DEFAULT_L2_MODE)


def panels(M, N, K, device, seed, L=None):
    g = torch.Generator().manual_seed(seed)
    shape = (lambda rows: (K, rows)) if L is None else (lambda rows: (L, K, rows))
    a = torch.randn(shape(M), generator=g).to(device).transpose(-1, -2)
    b = torch.randn(shape(N), generator=g).to(device).transpose(-1, -2)
    return a, b


def ordinary(monkeypatch, call):
    monkeypatch.delenv("KERMAC_AMD_SCALAR_B_MIN_TILES")
    try:
        return call()
    finally:
        monkeypatch.setenv("KERMAC_AMD_SCALAR_B_MIN_TILES", "1")


@pytest.mark.parametrize("M,N,K", [(256, 64, 16), (300, 80, 32), (1000, 912, 64), (257, 16, 48), (3, 160, 16), (1, 16, 1024),
                                   (515, 1040, 208), (1024, 1024, 256), (2047, 2000, 1040)])
@pytest.mark.parametrize("p", [1.0, 2.0])
def test_matches_truth_and_the_ordinary_kernel(device, scalar_b, M, N, K, p):
    a, b = panels(M, N, K, device, 7 * M + N + K)
    out = torch.empty(N, M, device=device).t()
    got = kermac.cdist(a, b, out=out, p=p)
    truth = l1_distances_float64(a, b) if p == 1.0 else torch.cdist(a.double(), b.double(), p=2.0, compute_mode="donot_use_mm_for_euclid_dist")
    assert_close_to_truth(got, truth, rtol=1e-5, atol=1e-30, what=f"p={p} {M}x{N}x{K}")
    plain = ordinary(scalar_b, lambda: kermac.cdist(a, b, p=p))
    assert torch.equal(got, plain.reshape(got.shape)), "not the ordinary kernel's bits"


@pytest.mark.parametrize("M,N,K", [(300, 80, 32), (1000, 912, 64), (515, 1040, 208)])
@pytest.mark.parametrize("p", [3.0, 4.0])
def test_cubes_and_fourth_powers(device, scalar_b, M, N, K, p):
    """The scalar exponents 3 and 4, which the library evaluates as |t| (t t) and (t t)(t t): against float64, and the
    ordinary kernel's bits."""
    a, b = panels(M, N, K, device, M + N + K)
    got = kermac.cdist(a, b, p=p)
    truth = torch.cdist(a.double(), b.double(), p=p)
    assert_close_to_truth(got[0], truth, rtol=1e-5, atol=1e-30, what=f"p={p} {M}x{N}x{K}")
    assert torch.equal(got, ordinary(scalar_b, lambda: kermac.cdist(a, b, p=p))), "not the ordinary kernel's bits"
    raw = kermac.cdist(a, b, p=p, skip_epilogue=True)
    assert torch.equal(raw, ordinary(scalar_b, lambda: kermac.cdist(a, b, p=p, skip_epilogue=True)))


@pytest.mark.parametrize("M,N,K,L", [(256 * 15 + 9, 320, 16, None), (256 * 16, 336, 32, None), (256 * 17 + 100, 64 * 7 + 16, 16, None),
                                     (256 * 35 + 1, 208, 16, None), (256 * 33, 64 * 3, 32, 3), (256 * 18 + 77, 64 * 5 + 48, 16, 5)])
def test_every_tile_of_the_band_order_is_walked_once(device, scalar_b, M, N, K, L):
    """Row blocks of a in bands of 16 (two per XCD) and the row blocks that fill no band, with and without a batch
    whose grid width shifts the XCD of a workgroup from entry to entry: the result is filled with NaN first, and every
    element is the ordinary kernel's."""
    a, b = panels(M, N, K, device, M + N + K, L=L)
    shape = (N, M) if L is None else (L, N, M)
    out = torch.full(shape, float("nan"), device=device).transpose(-1, -2)
    got = kermac.cdist(a, b, out=out, p=1.0)
    assert not torch.isnan(got).any(), "tiles left out"
    plain = ordinary(scalar_b, lambda: kermac.cdist(a, b, p=1.0))
    assert torch.equal(got, plain.reshape(got.shape)), "not the ordinary kernel's bits"
    sample = slice(0, M, 97)
    if L is None:
        truth = l1_distances_float64(a[sample], b)
    else:
        truth = torch.stack([l1_distances_float64(a[entry, sample], b[entry]) for entry in range(L)])
    assert_close_to_truth(got[..., sample, :], truth, rtol=1e-5, atol=1e-30, what=f"{M}x{N}x{K}x{L}")


@pytest.mark.parametrize("M,K,L", [(16, 16, None), (48, 32, None), (256, 16, None), (272, 48, None), (1024, 64, None), (1040, 16, None),
                                   (2000, 32, None), (4112, 16, None), (784, 32, 3)])
@pytest.mark.parametrize("p", [1.0, 2.0])
def test_a_panel_against_itself(device, scalar_b, M, K, L, p):
    """The tiles that reach the diagonal or lie below it, each stored twice: every element is written (the result starts
    as NaN), the matrix is symmetric bit for bit with a zero diagonal, and it is the ordinary kernels' result."""
    a, _ = panels(M, 16, K, device, M + K, L=L)
    shape = (M, M) if L is None else (L, M, M)
    out = torch.full(shape, float("nan"), device=device).transpose(-1, -2)
    got = kermac.cdist(a, a, out=out, p=p)
    assert not torch.isnan(got).any(), "elements left out"
    assert torch.equal(got, got.transpose(-1, -2)) and (torch.diagonal(got, dim1=-2, dim2=-1) == 0).all()
    plain = ordinary(scalar_b, lambda: kermac.cdist(a, a, p=p))
    assert torch.equal(got, plain.reshape(got.shape)), "not the ordinary kernel's bits"
    rows = slice(0, M, 7)
    if L is None:
        truth = l1_distances_float64(a[rows], a) if p == 1.0 else torch.cdist(a[rows].double(), a.double(), p=2.0, compute_mode="donot_use_mm_for_euclid_dist")
        assert_close_to_truth(got[rows], truth, rtol=1e-5, atol=1e-5, what=f"a against a, p={p} {M}x{K}")


def test_a_panel_against_itself_with_a_kernel_function_and_odd_results(device, scalar_b):
    """Laplace kernel with a regularised diagonal; a result whose rows are padded, and one that is off a 16-byte
    boundary (32-bit stores on both sides of the diagonal)."""
    M, K = 600 + 8, 48
    a, _ = panels(M, 16, K, device, 21)
    call = lambda **kw: kermac.run_kernel(kermac.kernel_descriptor_laplace_l1, a, a, bandwidth=5.0, regularization=0.5, **kw)
    plain = ordinary(scalar_b, call)[0]
    assert (torch.diagonal(plain) == 1.5).all()
    store = torch.full((M, M + 4), float("nan"), device=device)
    assert torch.equal(call(out=store[:, :M].t()), plain)
    odd = torch.full((M * M + 1,), float("nan"), device=device)[1:].view(M, M).t()
    assert torch.equal(call(out=odd), plain)
    truth = oracle.run_kernel("DIFF", "ABS", "NOOP", "LAPLACE", a.cpu(), a.cpu(), bandwidth=5.0, regularization=0.5)
    assert_close_to_truth(plain, truth.reshape(plain.shape), rtol=1e-5, atol=1e-7, what="laplace, a against a")


def test_it_is_the_kernel_that_ran(device, scalar_b):
    """Shapes the kernel cannot take (N or K not a multiple of 16, rows not contiguous) run the ordinary kernels and give
    the same numbers; a misaligned operand does too."""
    for M, N, K in ((300, 81, 32), (300, 80, 40), (128, 128, 24)):
        a, b = panels(M, N, K, device, M + N + K)
        truth = l1_distances_float64(a, b)
        assert_close_to_truth(kermac.cdist(a, b, p=1.0)[0], truth, rtol=1e-5, what=f"{M}x{N}x{K}")
    a, b = panels(400, 400, 64, device, 3)
    assert_close_to_truth(kermac.cdist(a, a, p=1.0)[0], l1_distances_float64(a, a), rtol=1e-5, atol=1e-30, what="a against itself")
    rows = a.contiguous()
    assert_close_to_truth(kermac.cdist(rows, b, p=1.0)[0], l1_distances_float64(a, b), rtol=1e-5, what="k contiguous")
    store = torch.randn(64 * 404 + 1, device=device)[1:].view(64, 404)
    odd = store[:, :400].t()
    assert_close_to_truth(kermac.cdist(odd, b, p=1.0)[0], l1_distances_float64(odd, b), rtol=1e-5, what="misaligned a")


def test_kernel_functions_batches_and_offsets(device, scalar_b):
    """Laplace and Gaussian kernels with a regularised off-diagonal, a batch with a broadcast operand and per-entry
    bandwidths, a result with padded rows; against the oracle and the ordinary kernel."""
    L, M, N, K = 3, 520, 336, 48
    a, _ = panels(M, N, K, device, 11, L=L)
    _, b = panels(M, N, K, device, 12)
    bandwidth = torch.tensor([3.0, 7.0, 1.5], device=device)
    store = torch.empty(L, N, M + 4, device=device)
    out = store[:, :, :M].transpose(1, 2)
    for descriptor, names in ((kermac.kernel_descriptor_laplace_l1, ("DIFF", "ABS", "NOOP", "LAPLACE")),
                              (kermac.kernel_descriptor_laplace_l2, ("DIFF", "SQUARE", "SQRT", "LAPLACE"))):
        got = kermac.run_kernel(descriptor, a, b, out=out, bandwidth=bandwidth, regularization=0.25,
                                regularization_offset_x=3, regularization_offset_y=1)
        truth = oracle.run_kernel(*names, a.cpu(), b.cpu(), bandwidth=bandwidth.cpu(), regularization=0.25,
                                  regularization_offset_x=3, regularization_offset_y=1)
        assert_close_to_truth(got, truth, rtol=1e-5, atol=1e-7, what=str(descriptor))
        plain = ordinary(scalar_b, lambda: kermac.run_kernel(descriptor, a, b, bandwidth=bandwidth, regularization=0.25,
                                                             regularization_offset_x=3, regularization_offset_y=1))
        assert torch.equal(got, plain)
    gaussian = kermac.KernelDescriptor(kermac.InnerOperator.DIFF, kermac.PowerType.SQUARE, kermac.PowerType.NOOP, kermac.KernelType.GAUSSIAN)
    got = kermac.run_kernel(gaussian, a[0], b, bandwidth=4.0)
    plain = ordinary(scalar_b, lambda: kermac.run_kernel(gaussian, a[0], b, bandwidth=4.0))
    assert torch.equal(got, plain)


def test_a_large_problem_takes_the_kernel_by_itself(device):
    """16384 x 16384 x 256 is 16384 tiles of 256 x 64: the library's own rule.  Float64 slabs, and the rows and columns at
    the edges of a ragged problem of the same size."""
    with kermac.l2_mode("direct"):
        for M, N in ((16384, 16384), (16000 + 37, 16000)):
            a, b = panels(M, N, 256, device, 5)
            out = torch.empty(N, M, device=device).t()
            for p in (1.0, 2.0):
                kermac.cdist(a, b, out=out, p=p)
                rows = torch.cat([torch.arange(0, 96), torch.arange(M - 64, M)]).to(device)
                columns = torch.cat([torch.arange(0, 64), torch.arange(N - 80, N)]).to(device)
                x, y = a[rows], b[columns]
                truth = l1_distances_float64(x, y) if p == 1.0 else torch.cdist(x.double(), y.double(), p=2.0, compute_mode="donot_use_mm_for_euclid_dist")
                assert_close_to_truth(out[rows][:, columns], truth, rtol=1e-5, what=f"p={p} {M}x{N}")
