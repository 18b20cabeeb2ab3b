"""A seeded sweep of mid-size calls in the default l2 mode, no route forced: sizes from a few
hundred to twenty thousand rows, contractions from 64 to 3200, 1 to 130 coefficient columns, both
storage orders, padded rows, operands shared by the batch.  Every call takes whatever the rules
pick for it (direct kernel, one-step matrix-core kernels, the route through a workspace, the cut
over k, the fused coefficient kernel in either variant, panels of either kind), and the result is checked
against float64 arithmetic on the device (torch.cdist and matmul in float64; the CPU oracle would
take minutes at these sizes).  Tolerance as everywhere: rtol 1e-5, for sums with coefficients
plus an absolute floor proportional to the typical magnitude of the sum.
"""
import random

import pytest
import torch

import kermac_amd as kermac

pytestmark = pytest.mark.gpu

GAUSSIAN = kermac.KernelDescriptor(kermac.InnerOperator.DIFF, kermac.PowerType.SQUARE, kermac.PowerType.NOOP,
                                   kermac.KernelType.GAUSSIAN)
PRODUCTS = kermac.KernelDescriptor(kermac.InnerOperator.DOT, kermac.PowerType.NOOP, kermac.PowerType.NOOP,
                                   kermac.KernelType.NONE)


def operand(rng, device, L, rows, K, col_major, shared):
    shape = (K, rows) if col_major else (rows, K)
    if not shared:
        shape = (L,) + shape
    pad = rng.choice((0, 0, 4, 3))
    t = torch.randn(shape[:-1] + (shape[-1] + pad,), device=device)[..., :shape[-1]]
    return t.transpose(-1, -2) if col_major else t


def test_mid_size_calls_as_the_rules_route_them(device):
    assert kermac.get_l2_mode() == "auto"
    rng = random.Random(11)
    torch.manual_seed(11)
    done = 0
    while done < 72:
        L = rng.choice((1, 1, 1, 2, 3))
        M = rng.choice((rng.randint(60, 300), rng.randint(300, 1500), rng.randint(1500, 5000)))
        N = rng.choice((rng.randint(100, 600), rng.randint(600, 3000), rng.randint(3000, 20000)))
        K = rng.choice((rng.randint(64, 200), rng.randint(200, 400), rng.randint(700, 900), rng.randint(1500, 3200)))
        O = rng.choice((1, 7, 32, 40, 70, 130))
        if L * M * N * K > 3e10 or L * M * N > 6e7:
            continue
        done += 1
        col_major = rng.random() < 0.4
        kind = rng.choice(("distances", "gaussian x coefficients", "gaussian x coefficients", "laplace x coefficients", "products",
                           "laplace on L1 x coefficients"))
        a = operand(rng, device, L, M, K, col_major, rng.random() < 0.2)
        b = operand(rng, device, L, N, K, col_major if rng.random() < 0.8 else not col_major, rng.random() < 0.2)
        what = f"case {done}: {kind}, L={L} M={M} N={N} K={K} O={O}, a {tuple(a.shape)} {a.stride()}, b {tuple(b.shape)} {b.stride()}"
        print(what, flush=True)
        with_coefficients = kind.endswith("coefficients")
        batch = L if with_coefficients or a.dim() == 3 or b.dim() == 3 else 1         # two shared operands: one matrix
        a64 = (a if a.dim() == 3 else a.unsqueeze(0).expand(batch, -1, -1)).double()
        b64 = (b if b.dim() == 3 else b.unsqueeze(0).expand(batch, -1, -1)).double()
        bandwidth = float(K) ** 0.5
        if kind == "distances":
            got, truth, atol = kermac.cdist(a, b, p=2.0), torch.cdist(a64, b64, p=2.0), 0.0
        elif kind == "products":
            got, truth = kermac.run_kernel(PRODUCTS, a, b), a64 @ b64.transpose(1, 2)
            atol = 1e-5 * float((a64.abs() @ b64.abs().transpose(1, 2)).mean())
        else:
            coef = torch.randn(L, N, O + 1, device=device)[..., :O] / N ** 0.5
            if kind == "gaussian x coefficients":
                got = kermac.run_kernel(GAUSSIAN, a, b, coefficients=coef, bandwidth=bandwidth)
                matrix = torch.exp(-torch.cdist(a64, b64, p=2.0) ** 2 / (2 * bandwidth ** 2))
            elif kind == "laplace on L1 x coefficients":
                got = kermac.run_kernel(kermac.kernel_descriptor_laplace_l1, a, b, coefficients=coef, bandwidth=4 * bandwidth)
                # blocks of rows, explicitly: torch.cdist with p = 1 in float64 returns wrong rows on the device at some sizes
                l1 = torch.stack([torch.cat([(a64[l, i:i + 32, None, :] - b64[l][None]).abs().sum(-1) for i in range(0, M, 32)])
                                  for l in range(batch)])
                matrix = torch.exp(-l1 / (4 * bandwidth))
            else:
                got = kermac.run_kernel(kermac.kernel_descriptor_laplace_l2, a, b, coefficients=coef, bandwidth=bandwidth,
                                        regularization=0.25, regularization_offset_x=3, regularization_offset_y=1)
                matrix = torch.exp(-torch.cdist(a64, b64, p=2.0) / bandwidth)
                m = torch.arange(M, device=device)
                n = m - 2                                      # the elements with offset_x + n == offset_y + m
                keep = (n >= 0) & (n < N)
                matrix[:, m[keep], n[keep]] = 1.25
            truth = matrix @ coef.double()
            atol = 1e-5 * float(truth.abs().mean()) * 10
        assert got.shape == truth.shape, what
        excess = (got.double() - truth).abs() - (1e-5 * truth.abs() + atol)       # compared on the device: up to 6e7 elements
        assert bool(torch.isfinite(got).all()) and float(excess.max()) <= 0.0, f"{what}: {float(excess.max()):.3e} beyond the tolerance"


def test_mid_size_gradients_as_the_rules_route_them(device):
    """cdist_grad for p = 1 and p = 2 at sizes on both sides of the rules that send a gradient to
    the fp16 matrix instruction: e[o, n, m] = sum_k c[o, k] a[k, m] w(d[n, m] - b[n, k]), with
    w = sign for p = 1 and the identity for p = 2, in float64 on the device.  Tolerance of the
    gradient tests: |got - truth| <= 1e-5 |truth| + 1e-4 mean |truth| (a signed sum of K terms)."""
    rng = random.Random(12)
    torch.manual_seed(12)
    done = 0
    while done < 24:
        L = rng.choice((1, 1, 2))
        M = rng.choice((rng.randint(100, 700), rng.randint(700, 3000), rng.randint(3000, 9000)))
        N = rng.choice((rng.randint(8, 40), rng.randint(40, 200), rng.randint(200, 600)))
        O = rng.choice((1, 2, 3, 10, 16, 24, 40))
        K = rng.choice((rng.randint(64, 300), rng.randint(300, 1500), rng.randint(1500, 9000)))
        p = rng.choice((1.0, 2.0))
        if L * M * N * O * K > 6e11 or L * M * N * O > 1.5e8:
            continue
        done += 1
        a = torch.rand(L, K, M, device=device) - 0.3
        b = torch.randn(L, N, K, device=device)
        c = torch.randn(L, O, K, device=device)
        d = torch.randn(L, N, M, device=device)
        what = f"gradient case {done}: p={p} L={L} M={M} N={N} O={O} K={K}"
        print(what, flush=True)
        got = kermac.cdist_grad(a, b, c, d, p=p)
        assert got.shape == (L, O, N, M), what
        a64, b64, c64, d64 = a.double(), b.double(), c.double(), d.double()
        if p == 2.0:
            truth = d64[:, None] * (c64 @ a64)[:, :, None, :] - torch.einsum("lok,lnk,lkm->lonm", c64, b64, a64)
        else:
            truth = torch.empty(L, O, N, M, dtype=torch.float64, device=device)
            for n in range(N):
                sign = torch.copysign(torch.ones((), dtype=torch.float64, device=device), d64[:, n, None, :] - b64[:, n, :, None])
                truth[:, :, n, :] = c64 @ (a64 * sign)           # [L, O, K] @ [L, K, M]
        excess = (got.double() - truth).abs() - (1e-5 * truth.abs() + 1e-4 * float(truth.abs().mean()))
        assert bool(torch.isfinite(got).all()) and float(excess.max()) <= 0.0, f"{what}: {float(excess.max()):.3e} beyond the tolerance"
