"""Pins the CPU oracle (oracle/kermac_oracle.c) before anything is compared with it.

Each check uses an independent source of truth: torch.cdist / torch.linalg in
float64 (library routines), the committed golden vectors, closed forms, numpy
brute force on tiny inputs, and the einsum identity of the reference's own
gradient test.  A dropped term, a wrong sign, a transposed operand or a
swapped stride in the oracle fails at least one of them.
"""
from pathlib import Path

import numpy as np
import pytest
import torch

from oracle import oracle
from tests.helpers import assert_close_to_truth

GOLDEN = np.load(Path(__file__).resolve().parent / "golden" / "hot_path_vectors.npz")


def T(name):
    return torch.from_numpy(GOLDEN[name])


# --------------------------------------------------------------------------- cdist

@pytest.mark.parametrize("p", [1.0, 1.3, 2.0, 0.5, 3.0])
@pytest.mark.parametrize("skip", [False, True])
def test_cdist_golden(p, skip):
    got = oracle.cdist(T("a"), T("b"), p=p, skip_epilogue=skip)
    truth = T(f"cdist_p{p}" + ("_skip" if skip else ""))
    assert_close_to_truth(got, truth, rtol=2e-7, what=f"oracle cdist p={p} skip={skip}")


@pytest.mark.parametrize("p", [1.0, 1.3, 2.0])
def test_cdist_fp32_mode_close_to_truth(p):
    # The fp32 mode follows the reference's operation order; it must stay within
    # fp32 rounding of the float64 truth.
    got = oracle.cdist(T("a"), T("b"), p=p, wide=False)
    assert_close_to_truth(got, T(f"cdist_p{p}"), rtol=5e-6, what=f"oracle fp32 cdist p={p}")


@pytest.mark.parametrize("p", [1.0, 1.7, 2.0])
def test_cdist_against_torch_on_strided_views(p):
    # Column-major (K-major panel) views, a broadcast operand and a ragged shape:
    # catches a transposed operand or a wrong stride in the oracle's indexing.
    g = torch.Generator().manual_seed(5)
    a_store = torch.randn(3, 7, 13, generator=g)          # [L, K, M]
    b_store = torch.randn(7, 10, generator=g)             # [K, N], no batch
    a, b = a_store.transpose(1, 2), b_store.t()
    got = oracle.cdist(a, b, p=p)
    truth = torch.cdist(a.double(), b.double().expand(3, -1, -1), p=p)
    assert got.shape == (3, 13, 10)
    assert_close_to_truth(got, truth, rtol=2e-7, what="strided cdist")


def test_cdist_closed_forms():
    g = torch.Generator().manual_seed(1)
    x = torch.randn(6, 9, generator=g)
    for p in (1.0, 1.3, 2.0):
        # identical points: zero distance on the diagonal, symmetric matrix
        d = oracle.cdist(x, x, p=p)[0]
        assert torch.all(torch.diagonal(d) == 0)
        assert torch.equal(d, d.t())
        # a = 0: distances are the p-norms of b's rows
        z = torch.zeros(4, 9)
        d0 = oracle.cdist(z, x, p=p)[0]
        norms = torch.linalg.vector_norm(x.double(), ord=p, dim=1)
        assert_close_to_truth(d0, norms.expand(4, -1), rtol=2e-7, what=f"zero operand p={p}")
    # K = 1: |b - a| for every p
    a1, b1 = torch.randn(5, 1, generator=g), torch.randn(4, 1, generator=g)
    for p in (1.0, 1.3, 2.0):
        d = oracle.cdist(a1, b1, p=p)[0]
        assert_close_to_truth(d, (b1.double().t() - a1.double()).abs(), rtol=3e-7, what=f"K=1 p={p}")


def test_cdist_brute_force_tiny():
    a = torch.tensor([[0.0, 1.0, -2.0], [3.0, 0.5, 0.25]])
    b = torch.tensor([[1.0, 1.0, 1.0], [-1.0, 0.0, 2.0], [0.0, 1.0, -2.0]])
    for p in (1.0, 2.0, 1.3):
        got = oracle.cdist(a, b, p=p)[0].double().numpy()
        for m in range(2):
            for n in range(3):
                s = sum(abs(float(b[n, k]) - float(a[m, k])) ** p for k in range(3))
                assert got[m, n] == pytest.approx(s ** (1.0 / p), rel=2e-7, abs=1e-12)


# ------------------------------------------------------------- kernel functions

def test_kernel_functions_golden():
    a, b = T("a"), T("b")
    bw = 3.0
    got = oracle.build_kernel("DIFF", "ABS", "NOOP", "LAPLACE", a, b, bandwidth=bw)
    assert_close_to_truth(got, T("laplace_l1_bw3"), rtol=3e-7, what="laplace l1")
    got = oracle.build_kernel("DIFF", "SQUARE", "SQRT", "LAPLACE", a, b, bandwidth=bw)
    assert_close_to_truth(got, T("laplace_l2_bw3"), rtol=3e-7, what="laplace l2")
    got = oracle.build_kernel("DIFF", "SQUARE", "NOOP", "GAUSSIAN", a, b, bandwidth=bw)
    assert_close_to_truth(got, T("gaussian_sq_bw3"), rtol=3e-7, what="gaussian")
    got = oracle.build_kernel("DOT", "NOOP", "NOOP", "NONE", a, b)
    assert_close_to_truth(got, T("dot"), rtol=1e-6, atol=1e-6, what="dot")


def test_regularisation_and_epsilon_golden():
    x = T("a")[0]
    got = oracle.build_kernel("DIFF", "ABS", "NOOP", "LAPLACE", x, x, bandwidth=3.0, regularization=0.25)[0]
    assert_close_to_truth(got, T("laplace_l1_self_bw3_reg0.25"), rtol=3e-7, what="regularised diagonal")
    got = oracle.build_kernel("DIFF", "ABS", "NOOP", "LAPLACE", x, x, bandwidth=3.0, regularization=0.25,
                              regularization_offset_x=3, regularization_offset_y=1)[0]
    assert_close_to_truth(got, T("laplace_l1_self_bw3_reg0.25_off3_1"), rtol=3e-7, what="offset diagonal")
    # epsilon mask: a distance below epsilon is treated as 0 -> kernel value exactly 1
    a = torch.tensor([[0.0, 0.0]])
    b = torch.tensor([[1e-6, 0.0], [1.0, 0.0]])
    got = oracle.build_kernel("DIFF", "ABS", "NOOP", "LAPLACE", a, b, bandwidth=1.0, epsilon=1e-5)[0]
    assert got[0, 0] == 1.0
    assert got[0, 1] == pytest.approx(np.exp(-1.0), rel=1e-6)
    # regularisation == 0 leaves the diagonal alone
    got = oracle.build_kernel("DIFF", "ABS", "NOOP", "LAPLACE", x, x, bandwidth=3.0, regularization=0.0)[0]
    assert torch.all(torch.diagonal(got) == 1.0)


def test_per_batch_hyper_parameters():
    a, b = T("a"), T("b")
    bw = torch.tensor([2.0, 5.0])
    got = oracle.build_kernel("DIFF", "ABS", "NOOP", "LAPLACE", a, b, bandwidth=bw)
    d1 = torch.cdist(a.double(), b.double(), p=1.0)
    truth = torch.exp(-d1 / bw.double()[:, None, None])
    assert_close_to_truth(got, truth, rtol=3e-7, what="per-batch bandwidth")
    p = torch.tensor([1.5, 3.0])
    got = oracle.build_kernel("DIFF", "POW", "POW", "NONE", a, b, p_inner=p, p_outer=1.0 / p)
    truth = torch.stack([torch.cdist(a[i].double(), b[i].double(), p=float(p[i])) for i in range(2)])
    assert_close_to_truth(got, truth, rtol=5e-7, what="per-batch p")


# ---------------------------------------------------------------------- gradient

@pytest.mark.parametrize("p", [1.0, 1.3, 2.0, 3.0])
def test_gradient_golden(p):
    got = oracle.cdist_grad(T("grad_a"), T("grad_b"), T("grad_c"), T("grad_d"), p=p)
    assert_close_to_truth(got, T(f"grad_p{p}"), rtol=1e-6, atol=1e-6, what=f"oracle grad p={p}")


def test_gradient_p2_reference_einsum_identity():
    # tests/test_cdist_grad.py:43-49 of the reference, in its own index names.
    g = torch.Generator().manual_seed(3)
    L, M, N, O, K = 2, 9, 6, 3, 8
    a = torch.randn(L, K, M, generator=g)
    b = torch.randn(L, N, K, generator=g)
    c = torch.randn(L, O, K, generator=g)
    d = torch.randn(L, N, M, generator=g)
    got = oracle.cdist_grad(a, b, c, d, p=2.0).permute(0, 1, 3, 2)
    x, z = b.permute(0, 2, 1).double(), d.permute(0, 2, 1).double()
    left = torch.einsum("bli,bij,bjd->bljd", c.double(), a.double(), z)
    right = torch.einsum("bli,bij,bid->bljd", c.double(), a.double(), x)
    assert_close_to_truth(got, left - right, rtol=1e-6, atol=1e-6, what="grad p=2 einsum identity")


def test_gradient_sign_of_zero_is_plus_one():
    # copysign(1, +0) = +1: a training point compared with itself contributes c*a, not 0.
    a = torch.tensor([[2.0]])        # [K=1, M=1]
    b = torch.tensor([[0.5]])        # [N=1, K=1]
    c = torch.tensor([[3.0]])        # [O=1, K=1]
    d = torch.tensor([[0.5]])        # [N=1, M=1] -> diff = +0
    assert oracle.cdist_grad(a, b, c, d, p=1.0).item() == 6.0
    # p = 2 uses the plain difference: 0
    assert oracle.cdist_grad(a, b, c, d, p=2.0).item() == 0.0


def test_gradient_is_linear_in_coefficients_and_kernel_matrix():
    g = torch.Generator().manual_seed(4)
    a = torch.rand(7, 5, generator=g); b = torch.randn(4, 7, generator=g)
    c1 = torch.randn(3, 7, generator=g); c2 = torch.randn(3, 7, generator=g); d = torch.randn(4, 5, generator=g)
    f = lambda a_, c_: oracle.cdist_grad(a_, b, c_, d, p=1.3).double()
    assert_close_to_truth(f(a, c1 + c2), f(a, c1) + f(a, c2), rtol=1e-5, atol=1e-5, what="linear in c")
    assert_close_to_truth(f(2 * a, c1), 2 * f(a, c1), rtol=1e-6, atol=1e-6, what="linear in a")


# ------------------------------------------------- kernel matrix x coefficients

def test_kernel_times_coefficients_golden_and_composition():
    a, b, coef = T("a"), T("b"), T("coef")
    got = oracle.kernel_times_coefficients("DIFF", "ABS", "NOOP", "LAPLACE", a, b, coef, bandwidth=3.0)
    assert_close_to_truth(got, T("laplace_l1_bw3_times_coef"), rtol=1e-6, atol=1e-6, what="kernel x coef")
    # must equal its own build_kernel followed by a matmul, for another descriptor too
    km = oracle.build_kernel("DIFF", "SQUARE", "NOOP", "GAUSSIAN", a, b, bandwidth=2.0).double()
    got = oracle.kernel_times_coefficients("DIFF", "SQUARE", "NOOP", "GAUSSIAN", a, b, coef, bandwidth=2.0)
    assert_close_to_truth(got, km @ coef.double(), rtol=1e-5, atol=1e-6, what="composition")


def test_run_kernel_wrapper_is_the_references_default_layout_result():
    """oracle.run_kernel = the reference's run_kernel for out=None: operands exchanged in
    front of the kernel, offsets and sign left alone (src/kermac/build_a_kernel.py:259,323-336).
    Its examples/broadcast_kernel.py passes offsets (3, 1): 1 + regularization lands where
    3 + n == 1 + m, at [n + 2, n]; a signed inner term reads a[m] - b[n]."""
    g = torch.Generator().manual_seed(4)
    a, b = torch.randn(9, 5, generator=g), torch.randn(7, 5, generator=g)
    got = oracle.run_kernel("DIFF", "NOOP", "NOOP", "NONE", a, b)[0]
    truth = (a.double()[:, None, :] - b.double()[None, :, :]).sum(-1)
    assert_close_to_truth(got, truth, rtol=1e-6, atol=1e-9, what="signed difference a - b")
    got = oracle.run_kernel("DIFF", "ABS", "NOOP", "LAPLACE", a, b, bandwidth=2.0, regularization=0.25,
                            regularization_offset_x=3, regularization_offset_y=1)[0]
    truth = torch.exp(-torch.cdist(a.double(), b.double(), p=1.0) / 2.0)
    for n in range(7):
        if n + 2 < 9:
            truth[n + 2, n] = 1.25
    assert_close_to_truth(got, truth, rtol=3e-7, what="offset diagonal of the default layout")
    coef = torch.randn(7, 3, generator=g)
    fused = oracle.run_kernel_coefficients("DIFF", "ABS", "NOOP", "LAPLACE", a, b, coef, bandwidth=2.0,
                                           regularization=0.25, regularization_offset_x=3, regularization_offset_y=1)[0]
    assert_close_to_truth(fused, truth @ coef.double(), rtol=1e-6, atol=1e-6, what="fused product, same convention")
