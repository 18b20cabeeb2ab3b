"""GPU tests of the route that large L2 gradients take when the caller brings a workspace
(include/kermac_amd.h, kmc_norm_gradient_params::workspace):
e = (d - s) g - p a with g = c a, p = c (b - s) and s the row means of b, the product p a on the fp16
matrix instruction from two fp16 pieces per value.  Tolerance as for the other gradient kernels: the
result is a signed sum of K products, |got - truth| <= 1e-5 |truth| + 1e-4 mean |truth|.

KERMAC_AMD_GRADIENT_L2_MIN_TERMS=1 sends the small shapes of these tests down the route, which by
itself only takes problems that fill a few hundred tiles of 256 x 256 over a contraction of 512 or more.
"""
import importlib

import pytest
import torch

import kermac_amd as kermac
from kermac_amd import _backend

module = importlib.import_module("kermac_amd.cdist_grad")       # the package attribute of that name is the operator
from oracle import oracle
from tests.helpers import assert_close_to_truth

pytestmark = pytest.mark.gpu


@pytest.fixture
def l2_route(monkeypatch):
    monkeypatch.setenv("KERMAC_AMD_GRADIENT_L2_MIN_TERMS", "1")


def tolerances(truth):
    return 1e-5, 1e-5 * float(truth.abs().mean()) * 10


def workspace_bytes(a, b, c, d, p=2.0, out=None):
    plan = module._plan_cdist_grad(a, b, c, d, out, p)
    return _backend.norm_gradient_workspace_bytes(plan.params)


@pytest.mark.parametrize("M,N,O,K", [(1, 1, 1, 1), (70, 33, 3, 17), (64, 32, 16, 32), (65, 31, 5, 50), (200, 40, 20, 35),
                                     (130, 64, 8, 100), (129, 66, 1, 48), (256, 64, 16, 64), (67, 35, 2, 19), (96, 24, 17, 20),
                                     (80, 20, 33, 33), (64, 16, 90, 16), (300, 70, 16, 1000), (257, 300, 3, 40), (600, 257, 2, 24)])
def test_gradient_shapes(device, l2_route, M, N, O, K):
    g = torch.Generator().manual_seed(M + 2 * N + 3 * O + 5 * K)
    a = (torch.rand(K, M, generator=g) - 0.3).to(device)        # weights of both signs
    b = torch.randn(N, K, generator=g).to(device)
    c = torch.randn(O, K, generator=g).to(device)
    d = torch.randn(N, M, generator=g).to(device)
    assert workspace_bytes(a, b, c, d) > 0
    got = kermac.cdist_grad(a, b, c, d, p=2.0)
    assert got.shape == (1, O, N, M)
    truth = oracle.cdist_grad(a.cpu(), b.cpu(), c.cpu(), d.cpu(), p=2.0)
    rtol, atol = tolerances(truth)
    assert_close_to_truth(got, truth, rtol=rtol, atol=atol, what=f"L2 grad {M}x{N}x{O}x{K}")
    assert torch.equal(got, kermac.cdist_grad(a, b, c, d, p=2.0)), "two runs differ"


def test_when_the_route_applies(device):
    a = torch.empty(2048, 4096, device=device)
    b = torch.empty(512, 2048, device=device)
    c = torch.empty(16, 2048, device=device)
    d = torch.empty(512, 4096, device=device)
    needed = workspace_bytes(a, b, c, d)                                     # 16 x 32 tiles over k = 2048
    assert needed > 0
    operands = 4 * (a.numel() + 16 * b.numel())                              # a, and c b for every output
    assert 1.5 * operands <= needed <= 2 * operands                          # the products in fp32 and in pieces, the pieces of a
    assert workspace_bytes(a, b, c, d, p=1.3) == 0
    assert workspace_bytes(a[:256], b[:, :256], c[:, :256], d) == 0          # k = 256: the walk is too short
    assert workspace_bytes(a, b[:8], c, d[:8]) == 0                          # 16 x 1 tiles
    assert workspace_bytes(a[:, :256], b, c, d[:, :256]) == 0                # 1 x 32 tiles
    assert workspace_bytes(a, b, c[:4], d) > 0                               # four outputs: 16 x 8 tiles
    # planes of the result that are not one matrix of (o n) rows: the fp32 kernels
    padded = torch.empty(1, 16, 513, 4096, device=device)[:, :, :512]
    assert workspace_bytes(a, b, c, d, out=padded) == 0


def test_a_common_offset_of_d_and_b_and_rows_of_different_magnitude(device, l2_route):
    """d - b does not see an offset that d and b share; the route multiplies d and b out, after
    shifting both by the row means of b.  Rows of a and of c spread over many binades keep the
    tolerance (the scales of the pieces are per row)."""
    g = torch.Generator().manual_seed(5)
    M, N, O, K = 150, 40, 16, 96
    a = torch.randn(K, M, generator=g) * torch.pow(2.0, (torch.arange(M) % 31 - 15).float())[None, :]
    c = torch.randn(O, K, generator=g) * torch.pow(2.0, (torch.arange(O) % 9 - 4).float())[:, None]
    offset = torch.linspace(-1000.0, 1000.0, N)[:, None]
    b = torch.randn(N, K, generator=g) + offset
    d = torch.randn(N, M, generator=g) + offset
    a, b, c, d = a.to(device), b.to(device), c.to(device), d.to(device)
    got = kermac.cdist_grad(a, b, c, d, p=2.0)
    truth = oracle.cdist_grad(a.cpu(), b.cpu(), c.cpu(), d.cpu(), p=2.0)
    # per (o, n, m): the terms are c a (d - b)
    difference = (d.cpu().double()[:, None, :] - b.cpu().double()[:, :, None]).abs()              # [N, K, M]
    scale = torch.einsum("ok,km,nkm->onm", c.abs().cpu().double(), a.abs().cpu().double(), difference)
    error = (got[0].cpu().double() - truth[0].double()).abs() / scale
    assert error.max().item() < 2e-6, f"error {error.max().item():.2e} of the sum of absolute terms"


def test_batches_broadcast_and_views(device, l2_route):
    g = torch.Generator().manual_seed(91)
    L, M, N, O, K = 3, 90, 20, 6, 45
    a = torch.rand(L, K, M + 3, generator=g).to(device)[:, :, 1:M + 1]       # padded, misaligned rows
    b = torch.randn(N, K + 2, generator=g).to(device)[:, 1:K + 1]            # shared by the batch
    c = torch.randn(L, O, K, generator=g).to(device)
    d = torch.randn(L, N, M, generator=g).to(device)
    out = torch.full((L, O, N, M + 1), float("nan"), device=device)[..., :M]
    assert workspace_bytes(a, b, c, d, out=out) > 0
    got = kermac.cdist_grad(a, b, c, d, out=out, p=2.0)
    assert got is out
    truth = oracle.cdist_grad(a.cpu(), b.cpu(), c.cpu(), d.cpu(), p=2.0)
    rtol, atol = tolerances(truth)
    assert_close_to_truth(got, truth, rtol=rtol, atol=atol, what="L2 grad batched")
    shared = kermac.cdist_grad(a[0], b, c, d, p=2.0)                         # a for every batch entry
    truth = oracle.cdist_grad(a[0].cpu(), b.cpu(), c.cpu(), d.cpu(), p=2.0)
    assert_close_to_truth(shared, truth, rtol=rtol, atol=atol, what="L2 grad, a shared")
    one_d = kermac.cdist_grad(a, b, c, d[1], p=2.0)                          # d for every batch entry
    truth = oracle.cdist_grad(a.cpu(), b.cpu(), c.cpu(), d[1].cpu(), p=2.0)
    assert_close_to_truth(one_d, truth, rtol=rtol, atol=atol, what="L2 grad, d shared")


def test_without_a_workspace_the_fp32_kernels_run(device, l2_route, monkeypatch):
    g = torch.Generator().manual_seed(2)
    M, N, O, K = 128, 32, 16, 64
    a = torch.rand(K, M, generator=g).to(device)
    b = torch.randn(N, K, generator=g).to(device)
    c = torch.randn(O, K, generator=g).to(device)
    d = torch.randn(N, M, generator=g).to(device)
    monkeypatch.setenv("KERMAC_AMD_GRADIENT_WORKSPACE", "0")
    reference = kermac.cdist_grad(a, b, c, d, p=2.0)
    plan = module._plan_cdist_grad(a, b, c, d, None, 2.0)
    stream = torch.cuda.current_stream(device).cuda_stream
    needed = _backend.norm_gradient_workspace_bytes(plan.params)
    workspace = torch.empty(needed, dtype=torch.uint8, device=device)
    for pointer, size in ((0, 0), (workspace.data_ptr(), needed - 1), (workspace.data_ptr() + 16, needed)):
        plan.out.fill_(-1.0)
        plan.params.workspace, plan.params.workspace_bytes = pointer, size
        _backend.norm_kernel_gradient(plan.params, stream)
        assert torch.equal(plan.out, reference), "null, short or misaligned workspace: expected the fp32 kernel's bits"
    plan.params.workspace, plan.params.workspace_bytes = workspace.data_ptr(), needed
    _backend.norm_kernel_gradient(plan.params, stream)
    assert not torch.equal(plan.out, reference) and torch.allclose(plan.out, reference, rtol=1e-3, atol=1e-4)


def test_rfm_shape_against_float64_rows(device):
    """8192 x 512 x 16 x 8192 by the route's own rule: rows n of the result against float64."""
    torch.manual_seed(3)
    K, M, N, O = 8192, 8192, 512, 16
    a = torch.rand(K, M, device=device)
    b = torch.randn(N, K, device=device) / 512 ** 0.5 + 3.0
    c = torch.randn(O, K, device=device)
    d = torch.randn(N, M, device=device) / 512 ** 0.5 + 3.0
    assert workspace_bytes(a, b, c, d) > 0
    got = kermac.cdist_grad(a, b, c, d, p=2.0)
    rows = [0, 1, N // 2, N - 1]
    ad, cd = a.double(), c.double()
    g = cd @ ad
    truth = torch.stack([d[n].double()[None, :] * g - (cd * b[n].double()[None, :]) @ ad for n in rows], dim=1)
    error = (got[0][:, rows, :].double() - truth).abs().max().item() / truth.abs().mean().item()
    assert error < 1e-4, f"max abs err / mean |truth| = {error:.2e}"
