"""GPU parity tests of cdist_grad against the CPU oracle (float64 mode), the golden
vectors and the einsum identity of the reference's own test.  All calls go through
the public operator and therefore through the C ABI.

Tolerance: the result is a signed sum of K products, so errors are measured against
the magnitude of the sum of absolute terms: |got - truth| <= rtol * |truth| + atol
with atol = rtol * (typical magnitude), rtol = 1e-5 (p = 1, 2) or 1e-4 (fractional p).
"""
from pathlib import Path

import numpy as np
import pytest
import torch

import kermac_amd as kermac
from oracle import oracle
from tests.helpers import assert_close_to_truth

pytestmark = pytest.mark.gpu

GOLDEN = np.load(Path(__file__).resolve().parent / "golden" / "hot_path_vectors.npz")


def tolerances(p, truth):
    rtol = 1e-5 if p in (1.0, 2.0) else 1e-4
    return rtol, rtol * float(truth.abs().mean()) * 10


@pytest.mark.parametrize("p", [1.0, 1.3, 2.0, 3.0])
def test_gradient_golden_vectors(device, p):
    a, b, c, d = (torch.from_numpy(GOLDEN[k]).to(device) for k in ("grad_a", "grad_b", "grad_c", "grad_d"))
    got = kermac.cdist_grad(a, b, c, d, p=p)
    truth = torch.from_numpy(GOLDEN[f"grad_p{p}"])
    rtol, atol = tolerances(p, truth)
    assert_close_to_truth(got, truth, rtol=rtol, atol=atol, what=f"grad golden p={p}")


def test_gradient_reference_test_case(device):
    """tests/test_cdist_grad.py of the reference: L=4, M=N=1000, O=16, K=64, p=2,
    out supplied, compared with the two-einsum identity at RMSE / max-abs < 1e-4."""
    torch.manual_seed(7)
    L, M, N, O, K = 4, 1000, 1000, 16, 64
    a = torch.randn(L, K, M, device=device)
    b = torch.randn(L, N, K, device=device)
    c = torch.randn(L, O, K, device=device)
    d = torch.randn(L, N, M, device=device)
    e = torch.randn(L, O, N, M, device=device)
    out = kermac.cdist_grad(a=a, b=b, c=c, d=d, out=e, p=2.0)
    assert out is e
    x, z = b.permute(0, 2, 1), d.permute(0, 2, 1)
    left = torch.einsum("bli,bij,bjd->bljd", c.double(), a.double(), z.double())
    right = torch.einsum("bli,bij,bid->bljd", c.double(), a.double(), x.double())
    truth = (left - right).permute(0, 1, 3, 2)
    diff = out.double() - truth
    assert torch.sqrt(torch.mean(diff ** 2)).item() < 1e-4
    assert diff.abs().max().item() < 1e-4


@pytest.mark.parametrize("p", [1.0, 2.0, 1.3, 0.7])
@pytest.mark.parametrize("M,N,O,K", [(1, 1, 1, 1), (70, 33, 3, 17), (64, 32, 16, 16), (65, 31, 5, 50), (200, 40, 20, 35),
                                     (130, 64, 8, 100), (129, 66, 1, 48), (256, 64, 2, 64), (67, 35, 2, 19), (128, 64, 7, 32), (90, 40, 6, 21),
                                     # output counts that are cut into runs for kernels of different width
                                     (96, 24, 17, 20), (80, 20, 33, 33), (70, 18, 49, 16), (66, 17, 57, 21), (64, 16, 90, 16)])
def test_gradient_ragged_shapes(device, p, M, N, O, K):
    g = torch.Generator().manual_seed(M + 2 * N + 3 * O + 5 * K)
    a = torch.rand(K, M, generator=g).to(device)
    b = torch.randn(N, K, generator=g).to(device)
    c = torch.randn(O, K, generator=g).to(device)
    d = torch.randn(N, M, generator=g).to(device)
    got = kermac.cdist_grad(a, b, c, d, p=p)
    assert got.shape == (1, O, N, M)
    truth = oracle.cdist_grad(a.cpu(), b.cpu(), c.cpu(), d.cpu(), p=p)
    rtol, atol = tolerances(p, truth)
    assert_close_to_truth(got, truth, rtol=rtol, atol=atol, what=f"grad {M}x{N}x{O}x{K} p={p}")


def test_gradient_batches_broadcast_views_and_p_tensor(device):
    g = torch.Generator().manual_seed(91)
    L, M, N, O, K = 3, 90, 20, 6, 45
    a = torch.rand(L, K, M + 3, generator=g).to(device)[:, :, 1:M + 1]   # padded, misaligned rows
    b = torch.randn(N, K, generator=g).to(device)                        # broadcast over the batch
    c = torch.randn(L, O, K + 1, generator=g).to(device)[:, :, :K]       # padded rows
    d = torch.randn(L, N, M, generator=g).to(device)
    p = torch.tensor([1.5, 2.0, 3.0], device=device)
    out = torch.full((L, O, N, M + 2), -7.0, device=device)
    got = kermac.cdist_grad(a, b, c, d, out=out[..., :M], p=p)
    truth = oracle.cdist_grad(a.cpu(), b.cpu(), c.cpu().contiguous(), d.cpu(), p=p.cpu())
    rtol, atol = tolerances(1.5, truth)
    assert_close_to_truth(got, truth, rtol=rtol, atol=atol, what="batched gradient")
    assert torch.all(out[..., M:] == -7.0), "wrote outside the out view"
    # a one-element p tensor selects the L1 / L2 kernels like a float does
    one = kermac.cdist_grad(a, b, c, d, p=torch.tensor(1.0, device=device))
    assert torch.equal(one, kermac.cdist_grad(a, b, c, d, p=1.0))


def test_gradient_sign_convention_and_linearity(device):
    # x identical to a centre: diff = +0 -> copysign gives +1 for p = 1
    a = torch.tensor([[2.0]], device=device)
    b = torch.tensor([[0.5]], device=device)
    c = torch.tensor([[3.0]], device=device)
    d = torch.tensor([[0.5]], device=device)
    assert kermac.cdist_grad(a, b, c, d, p=1.0).item() == 6.0
    assert kermac.cdist_grad(a, b, c, d, p=2.0).item() == 0.0
    g = torch.Generator().manual_seed(92)
    a = torch.rand(40, 70, generator=g).to(device); b = torch.randn(9, 40, generator=g).to(device)
    c1 = torch.randn(4, 40, generator=g).to(device); c2 = torch.randn(4, 40, generator=g).to(device)
    d = torch.randn(9, 70, generator=g).to(device)
    f = lambda c_: kermac.cdist_grad(a, b, c_, d, p=1.3).double()
    assert_close_to_truth(f(c1 + c2), f(c1) + f(c2), rtol=1e-4, atol=1e-4, what="linearity in c")


@pytest.mark.parametrize("O", [1, 2, 8, 16, 32])
@pytest.mark.parametrize("K", [3, 16, 35])
def test_gradient_l1_sign_of_zero_differences(device, O, K):
    """copysign(1, d - b) for the four combinations of signed zeros, equal non-zero
    values, denormals and ordinary values, in every kernel variant (vector-ALU and
    matrix-core, with and without a partial K slice): d - b is -0 only for
    (d, b) = (-0, +0); the result must equal the oracle bit for bit because every
    product c * a below is a small integer."""
    g = torch.Generator().manual_seed(93 + O + K)
    specials = torch.tensor([0.0, -0.0, 1.5, -1.5, 1e-45, -1e-45, 3e-39, -3e-39, float(2 ** -126), 7.0])
    M, N = 70, 2 * len(specials)
    d = specials[torch.randint(len(specials), (N, M), generator=g)]
    b = specials[torch.randint(len(specials), (N, K), generator=g)]
    a = torch.randint(-3, 4, (K, M), generator=g).float()
    c = torch.randint(-2, 3, (O, K), generator=g).float()
    got = kermac.cdist_grad(a.to(device), b.to(device), c.to(device), d.to(device), p=1.0)
    truth = oracle.cdist_grad(a, b, c, d, p=1.0)
    assert torch.equal(got.cpu().double(), truth.double())
    # and the rule itself, independent of the oracle
    diff = d[:, :, None] - b[:, None, :]                                    # [n, m, k], IEEE fp32
    sign = torch.where(torch.signbit(diff), -1.0, 1.0)
    expected = torch.einsum("ok,km,nmk->onm", c, a, sign)
    assert torch.equal(got[0].cpu(), expected)


def test_gradient_rfm_shape_against_slab_truth(device):
    """The Laplace-kernel RFM gradient configuration (x[512,8192], centres
    z[512,8192], 16 classes, 8192 centres) at p = 1: check float64 slabs."""
    torch.manual_seed(3)
    K_ref, M_ref, N_ref, O = 8192, 8192, 512, 16
    a = torch.rand(K_ref, M_ref, device=device)                      # kernel-gradient weights
    b = torch.randn(N_ref, K_ref, device=device) / 512 ** 0.5        # centres
    c = torch.randn(O, K_ref, device=device)
    d = torch.randn(N_ref, M_ref, device=device) / 512 ** 0.5        # samples
    out = kermac.cdist_grad(a, b, c, d, p=1.0)[0]
    for ms, ns in ((slice(0, 40), slice(0, 24)), (slice(8150, 8192), slice(500, 512))):
        diff = d[ns, ms].double()[:, :, None] - b[ns].double()[:, None, :]          # n m k
        sign = torch.where(torch.signbit(diff), -1.0, 1.0).double()
        truth = torch.einsum("ok,km,nmk->onm", c.double(), a[:, ms].double(), sign)
        assert_close_to_truth(out[:, ns, ms], truth, rtol=1e-5, atol=1e-5 * float(truth.abs().mean()) * 10,
                              what="RFM slab")


def test_gradient_empty_contraction_writes_zeros(device):
    """K = 0: the result buffer is allocated uninitialised, the kernel must still write
    every element (an empty sum)."""
    junk = torch.full((1, 5, 9, 70), float("nan"), device=device)      # make a recycled allocation visible
    del junk
    got = kermac.cdist_grad(torch.zeros(0, 70, device=device), torch.zeros(9, 0, device=device),
                            torch.zeros(5, 0, device=device), torch.randn(9, 70, device=device), p=1.0)
    assert got.shape == (1, 5, 9, 70) and torch.all(got == 0)


@pytest.mark.parametrize("p", [1.0, 2.0, 1.3])
@pytest.mark.parametrize("M,N,O,K", [(200, 40, 1, 4100), (130, 10, 3, 2048), (64, 100, 16, 5000),
                                     (2048, 128, 16, 1100), (4100, 250, 2, 2100)])      # 256 and 520 workgroups
def test_few_results_deep_contraction_is_cut_over_k(device, p, M, N, O, K):
    """Few (m, n) results against a long contraction: one batched launch over slices of k plus a
    fixed-order sum of the partial results (kermac_amd/cdist_grad.py); same values as one walk."""
    import importlib
    module = importlib.import_module("kermac_amd.cdist_grad")    # the package attribute of that name is the function
    g = torch.Generator().manual_seed(M + N + O + K)
    a = torch.rand(K, M, generator=g).to(device)
    b = torch.randn(N, K, generator=g).to(device)
    c = torch.randn(O, K, generator=g).to(device)
    d = torch.randn(N, M, generator=g).to(device)
    assert module._split_over_contraction(module._plan_cdist_grad(a, b, c, d, None, p)) is not None
    got = kermac.cdist_grad(a, b, c, d, p=p)
    assert got.shape == (1, O, N, M)
    truth = oracle.cdist_grad(a.cpu(), b.cpu(), c.cpu(), d.cpu(), p=p)
    rtol, atol = tolerances(p, truth)
    assert_close_to_truth(got, truth, rtol=rtol, atol=atol, what=f"grad cut over k {M}x{N}x{O}x{K} p={p}")
    wide = torch.full((O, N, M + 4), -7.0, device=device)
    out = wide[:, :, :M]
    assert kermac.cdist_grad(a, b, c, d, out=out, p=p) is out
    assert torch.equal(out, got[0]) and torch.all(wide[:, :, M:] == -7.0)
