"""GPU tests of the fused kernel-matrix x coefficients product with the kernel
values produced on the matrix cores (``set_l2_mode("gram")`` together with
``run_kernel(..., coefficients=...)`` for the squared-difference descriptors).

Stated tolerance: the same as the direct fused kernel, rtol 1e-5 against the
float64 oracle with an absolute floor proportional to the typical magnitude of the
signed sum over n.  Tiles whose squared distances are small against the norms are
recomputed inside the kernel with the direct arithmetic; when that happens to every
tile the result must equal the direct fused kernel bit for bit.
"""
import pytest
import torch

import kermac_amd as kermac
from oracle import oracle
from tests.helpers import assert_close_to_truth, make_operand

pytestmark = pytest.mark.gpu

GAUSSIAN = kermac.KernelDescriptor(kermac.InnerOperator.DIFF, kermac.PowerType.SQUARE, kermac.PowerType.NOOP,
                                   kermac.KernelType.GAUSSIAN)
CASES = (
    (kermac.kernel_descriptor_laplace_l2, ("DIFF", "SQUARE", "SQRT", "LAPLACE"), {"bandwidth": 6.0}),
    (GAUSSIAN, ("DIFF", "SQUARE", "NOOP", "GAUSSIAN"), {"bandwidth": 5.0}),
    (kermac.kernel_descriptor_l2_norm, ("DIFF", "SQUARE", "SQRT", "NONE"), {}),
)


@pytest.fixture
def gram_mode():
    kermac.set_l2_mode("gram", min_k=0)
    yield
    kermac.set_l2_mode(kermac.DEFAULT_L2_MODE)


def atol_for(truth, rtol):
    return rtol * float(truth.abs().mean()) * 10


@pytest.mark.parametrize("M,N,K,O", [(1, 1, 1, 1), (130, 200, 17, 5), (128, 128, 16, 32), (257, 129, 40, 33),
                                     (90, 300, 6, 70), (300, 700, 64, 16)])
@pytest.mark.parametrize("layout", ["cc", "rr", "cr"])
def test_shapes_and_layouts(device, gram_mode, M, N, K, O, layout):
    g = torch.Generator().manual_seed(M + N + K + O)
    a = make_operand(1, M, K, layout[0] == "c", device, g, batch=False)
    b = make_operand(1, N, K, layout[1] == "c", device, g, batch=False)
    coef = torch.randn(N, O, generator=g).to(device)
    for descriptor, names, kw in CASES:
        got = kermac.run_kernel(descriptor, a, b, coefficients=coef, **kw)
        assert got.shape == (1, M, O)
        truth = oracle.kernel_times_coefficients(*names, a.cpu(), b.cpu(), coef.cpu(), **kw)
        assert_close_to_truth(got, truth, rtol=1e-5, atol=atol_for(truth, 1e-5), what=f"{names} {layout}")


def test_batches_regularisation_and_unfused_composition(device, gram_mode):
    g = torch.Generator().manual_seed(71)
    L, M, N, K, O = 3, 200, 260, 24, 12
    x = make_operand(L, M, K, True, device, g)
    z = make_operand(1, N, K, True, device, g, batch=False)                  # broadcast centres
    coef = torch.randn(L, N, O + 3, generator=g).to(device)[:, :, :O]         # padded rows
    bw = torch.tensor([4.0, 6.0, 9.0], device=device)
    out = torch.full((L, M, O + 1), 5.0, device=device)
    kw = dict(bandwidth=bw, regularization=0.5, regularization_offset_x=2, regularization_offset_y=0)
    got = kermac.run_kernel(kermac.kernel_descriptor_laplace_l2, x, z, out=out[..., :O], coefficients=coef, **kw)
    full = kermac.run_kernel(kermac.kernel_descriptor_laplace_l2, x, z, **kw)
    composed = torch.bmm(full.double(), coef.double())
    assert_close_to_truth(got, composed, rtol=1e-5, atol=atol_for(composed, 1e-5), what="fused vs unfused")
    assert torch.all(out[..., O] == 5.0), "wrote outside the out view"
    truth = oracle.run_kernel_coefficients("DIFF", "SQUARE", "SQRT", "LAPLACE", x.cpu().contiguous(),
                                           z.cpu().contiguous(), coef.cpu().contiguous(), bandwidth=bw.cpu(),
                                           regularization=0.5, regularization_offset_x=2, regularization_offset_y=0)
    assert_close_to_truth(got, truth, rtol=1e-5, atol=atol_for(truth, 1e-5), what="fused vs oracle")


def test_distrusted_tiles_take_the_direct_arithmetic(device):
    g = torch.Generator().manual_seed(72)
    # every row of z is a tiny perturbation of a row of x with the same index modulo 50, and all points sit
    # far from the origin: every 128 x 128 tile contains a pair whose distance is tiny against the norms
    base = torch.randn(50, 32, generator=g) + 40.0
    x = (base.repeat(6, 1) + 1e-3 * torch.randn(300, 32, generator=g)).to(device)
    z = (base.repeat(8, 1) + 1e-3 * torch.randn(400, 32, generator=g)).to(device)
    coef = torch.randn(400, 20, generator=g).to(device)
    kermac.set_l2_mode("direct")
    direct = kermac.run_kernel(kermac.kernel_descriptor_laplace_l2, x, z, bandwidth=3.0, coefficients=coef)
    kermac.set_l2_mode("gram", min_k=0)
    try:
        gram = kermac.run_kernel(kermac.kernel_descriptor_laplace_l2, x, z, bandwidth=3.0, coefficients=coef)
    finally:
        kermac.set_l2_mode(kermac.DEFAULT_L2_MODE)
    assert torch.equal(gram, direct)
    truth = oracle.kernel_times_coefficients("DIFF", "SQUARE", "SQRT", "LAPLACE", x.cpu(), z.cpu(), coef.cpu(),
                                             bandwidth=3.0)
    assert_close_to_truth(gram, truth, rtol=1e-5, atol=atol_for(truth, 1e-5), what="all tiles distrusted")
    # a mix: only the first 128 centres are near-duplicates of samples
    z2 = torch.randn(400, 32, generator=g).to(device) + 40.0
    z2[:100] = x[:100] + 1e-4
    kermac.set_l2_mode("gram", min_k=0)
    try:
        mixed = kermac.run_kernel(GAUSSIAN, x, z2, bandwidth=4.0, coefficients=coef)
    finally:
        kermac.set_l2_mode(kermac.DEFAULT_L2_MODE)
    truth = oracle.kernel_times_coefficients("DIFF", "SQUARE", "NOOP", "GAUSSIAN", x.cpu(), z2.cpu(), coef.cpu(),
                                             bandwidth=4.0)
    assert_close_to_truth(mixed, truth, rtol=1e-5, atol=atol_for(truth, 1e-5), what="some tiles distrusted")


def test_headline_shape_gaussian(device, gram_mode):
    """The fused benchmark shape (batch 4, 16384 x 16384, K = 256, O = 32) with a
    Gaussian kernel: float64 slabs of the result."""
    torch.manual_seed(5)
    L, K, NX, MZ, O = 4, 256, 16384, 16384, 32
    x = torch.rand(L, K, NX, device=device) * 2 - 1
    z = torch.rand(K, MZ, device=device) * 2 - 1
    coef = torch.randn(L, MZ, O, device=device)
    out = torch.empty(L, NX, O, device=device)
    kermac.run_kernel(GAUSSIAN, x.transpose(1, 2), z.t(), out=out, bandwidth=9.0, coefficients=coef)
    for l, rows in ((0, slice(0, 96)), (3, slice(16300, 16384))):
        d2 = torch.cdist(x[l, :, rows].t().double(), z.t().double(), p=2.0) ** 2
        truth = torch.exp(-d2 / (2 * 9.0 ** 2)) @ coef[l].double()
        assert_close_to_truth(out[l, rows], truth, rtol=1e-5, atol=atol_for(truth, 1e-5), what=f"gaussian slab batch {l}")
