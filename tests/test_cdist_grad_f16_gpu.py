"""GPU tests of the route that large L1 gradients take when the caller brings a workspace
(include/kermac_amd.h, kmc_norm_gradient_params::workspace): a and c split once into two fp16
pieces per value with a power-of-two scale per row, the sign of d - b put on the pieces of a, the
contraction on the fp16 matrix instruction.  Tolerance as for the other gradient kernels: the
result is a signed sum of K products, |got - truth| <= 1e-5 |truth| + 1e-4 mean |truth|.

KERMAC_AMD_GRADIENT_F16_MIN_TERMS=1 sends the small shapes of these tests down the route, which by
itself only takes problems of at least 4e8 terms and 3 outputs.
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
def f16_route(monkeypatch):
    monkeypatch.setenv("KERMAC_AMD_GRADIENT_F16_MIN_TERMS", "1")


def tolerances(truth):
    return 1e-5, 1e-5 * float(truth.abs().mean()) * 10


def workspace_bytes(a, b, c, d, p=1.0):
    plan = module._plan_cdist_grad(a, b, c, d, None, p)
    return _backend.norm_gradient_workspace_bytes(plan.params)


@pytest.mark.parametrize("M,N,O,K", [(1, 1, 1, 1), (70, 33, 3, 17), (64, 32, 16, 32), (65, 31, 5, 50), (200, 40, 20, 35),
                                     (130, 64, 8, 100), (129, 66, 1, 48), (256, 64, 16, 64), (67, 35, 2, 19), (96, 24, 17, 20),
                                     (80, 20, 33, 33), (64, 16, 90, 16), (300, 70, 16, 1000),
                                     # 17 and more outputs: tiles of 16 n x 32 o and 8 n x 64 o, what is left beyond whole
                                     # tiles of 64 on the narrower ones
                                     (70, 40, 32, 40), (130, 20, 40, 64), (64, 33, 64, 32), (50, 17, 49, 20), (200, 15, 24, 70),
                                     (65, 31, 25, 200), (60, 12, 70, 40), (40, 9, 130, 33), (33, 7, 90, 64)])
def test_gradient_shapes(device, f16_route, M, N, O, K):
    g = torch.Generator().manual_seed(M + 2 * N + 3 * O + 5 * K)
    a = (torch.rand(K, M, generator=g) - 0.3).to(device)        # weights of both signs
    b = torch.randn(N, K, generator=g).to(device)
    c = torch.randn(O, K, generator=g).to(device)
    d = torch.randn(N, M, generator=g).to(device)
    assert workspace_bytes(a, b, c, d) > 0
    got = kermac.cdist_grad(a, b, c, d, p=1.0)
    assert got.shape == (1, O, N, M)
    truth = oracle.cdist_grad(a.cpu(), b.cpu(), c.cpu(), d.cpu(), p=1.0)
    rtol, atol = tolerances(truth)
    assert_close_to_truth(got, truth, rtol=rtol, atol=atol, what=f"f16 grad {M}x{N}x{O}x{K}")


def test_when_the_route_applies(device, monkeypatch):
    a = torch.empty(2048, 4096, device=device)
    b = torch.empty(512, 2048, device=device)
    c = torch.empty(16, 2048, device=device)
    d = torch.empty(512, 4096, device=device)
    assert workspace_bytes(a, b, c, d) > 0                                   # 4.3e9 terms
    assert workspace_bytes(a, b, c, d, p=1.3) == 0
    assert workspace_bytes(a, b, c, d, p=2.0) not in (0, workspace_bytes(a, b, c, d))         # the L2 norm has a route of its own
    assert workspace_bytes(a[:, :256], b[:64], c, d[:64, :256]) == 0         # 3.4e7 terms
    assert workspace_bytes(a, b, c[:2], d) == 0                              # two outputs: the vector kernel
    needed = workspace_bytes(a, b, c, d)
    operands = 4 * (a.numel() + b.numel() + c.numel())
    assert operands <= needed <= 2 * operands


def test_signs_at_zero_and_rows_of_different_magnitude(device, f16_route):
    """copysign(1, d - b): +1 where d equals b, and for signed zeros the sign of the difference;
    rows of a and of c spread over many binades keep the tolerance (the scale is per row)."""
    g = torch.Generator().manual_seed(5)
    M, N, O, K = 150, 40, 16, 96
    a = torch.randn(K, M, generator=g) * torch.pow(2.0, (torch.arange(M) % 31 - 15).float())[None, :]
    a[:, 0] *= 2.0 ** -100                 # rows far out: the scale is a power of two per row
    a[:, 1] *= 2.0 ** 100
    c = torch.randn(O, K, generator=g) * torch.pow(2.0, (torch.arange(O) % 9 - 4).float())[:, None]
    b = torch.randn(N, K, generator=g)
    d = torch.randn(N, M, generator=g)
    d[3, :] = b[3, 7]                      # exact ties on one row of d
    b[5, 10] = 0.0
    d[5, 20] = -0.0                        # -0 - +0 = -0: the weight is -1
    a, b, c, d = a.to(device), b.to(device), c.to(device), d.to(device)
    got = kermac.cdist_grad(a, b, c, d, p=1.0)
    truth = oracle.cdist_grad(a.cpu(), b.cpu(), c.cpu(), d.cpu(), p=1.0)
    # per (o, m): the terms scale with |c_o| |a_m|
    scale = (c.abs().cpu().double() @ a.abs().cpu().double())[:, None, :]       # [O, 1, M]
    error = (got[0].cpu().double() - truth[0].double()).abs() / scale
    assert error.max().item() < 1e-6, f"error {error.max().item():.2e} of the sum of absolute terms"


@pytest.mark.parametrize("O", [6, 20, 37])                      # one tile shape, the other, both
def test_batches_broadcast_and_views(device, f16_route, O):
    g = torch.Generator().manual_seed(91)
    L, M, N, K = 3, 90, 20, 45
    a = torch.rand(L, K, M + 3, generator=g).to(device)[:, :, 1:M + 1]       # padded, misaligned rows
    b = torch.randn(N, K + 2, generator=g).to(device)[:, 1:K + 1]            # shared by the batch
    c = torch.randn(L, O, K, generator=g).to(device)
    d = torch.randn(L, N, M, generator=g).to(device)
    out = torch.full((L, O, N, M + 1), float("nan"), device=device)[..., :M]
    got = kermac.cdist_grad(a, b, c, d, out=out, p=1.0)
    assert got is out
    truth = oracle.cdist_grad(a.cpu(), b.cpu(), c.cpu(), d.cpu(), p=1.0)
    rtol, atol = tolerances(truth)
    assert_close_to_truth(got, truth, rtol=rtol, atol=atol, what="f16 grad batched")
    shared = kermac.cdist_grad(a[0], b, c, d, p=1.0)                         # a for every batch entry
    truth = oracle.cdist_grad(a[0].cpu(), b.cpu(), c.cpu(), d.cpu(), p=1.0)
    assert_close_to_truth(shared, truth, rtol=rtol, atol=atol, what="f16 grad, a shared")


def test_without_a_workspace_the_fp32_kernels_run(device, f16_route, monkeypatch):
    g = torch.Generator().manual_seed(2)
    M, N, O, K = 128, 32, 16, 64
    a = torch.rand(K, M, generator=g).to(device)
    b = torch.randn(N, K, generator=g).to(device)
    c = torch.randn(O, K, generator=g).to(device)
    d = torch.randn(N, M, generator=g).to(device)
    monkeypatch.setenv("KERMAC_AMD_GRADIENT_WORKSPACE", "0")
    reference = kermac.cdist_grad(a, b, c, d, p=1.0)
    plan = module._plan_cdist_grad(a, b, c, d, None, 1.0)
    stream = torch.cuda.current_stream(device).cuda_stream
    needed = _backend.norm_gradient_workspace_bytes(plan.params)
    workspace = torch.empty(needed, dtype=torch.uint8, device=device)
    for pointer, size in ((0, 0), (workspace.data_ptr(), needed - 1), (workspace.data_ptr() + 16, needed)):
        plan.out.fill_(-1.0)
        plan.params.workspace, plan.params.workspace_bytes = pointer, size
        _backend.norm_kernel_gradient(plan.params, stream)
        assert torch.equal(plan.out, reference), "null, short or misaligned workspace: expected the fp32 kernel's bits"
