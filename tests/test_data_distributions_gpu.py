"""GPU tests of the routes that judge the data before they trust their own result -- squared differences on the
matrix cores (the default for a problem of this size: pair sample, trust rule per 128 x 128 part, repair launch) and
absolute differences on fixed point (opt-in: tile sample, trust rule per tile, repair launch) -- on operands that
are not the i.i.d. normal values of the other tests: offsets, extreme scales, heavy tails, sparsity, integers,
features and rows of different magnitude, constant features, low rank.  Whatever each route decides for such data,
the result must keep rtol 1e-5 against float64, which is what the reference's fp32 kernel is held to
(include/build_a_kernel.cuh:339-370 summed in float64 here).

The shape is the smallest at which both routes apply by their own rules and both take their samples:
8192 x 8192 x 1024 is 1024 tiles of 256 x 256 with 64 slices (squared differences) and 4096 tiles of 128 x 128
(absolute differences).
"""
import math

import pytest
import torch

import kermac_amd as kermac
from tests.helpers import assert_close_to_truth, l1_distances_float64

pytestmark = pytest.mark.gpu

M = N = 8192
K = 1024


def operand(kind, rows, device, g):
    def randn(*shape):
        return torch.randn(*shape, device=device, generator=g)

    def rand(*shape):
        return torch.rand(*shape, device=device, generator=g)

    if kind == "uniform in [0, 1)":
        return rand(K, rows)
    if kind == "offset of 1e4":
        return 1e4 + randn(K, rows)
    if kind == "scale 1e-20":
        return 1e-20 * randn(K, rows)
    if kind == "scale 1e15":
        return 1e15 * randn(K, rows)
    if kind == "student t, 2 degrees":
        return randn(K, rows) / (rand(K, rows) + 1e-3).sqrt()
    if kind == "cauchy":
        return torch.tan(math.pi * (rand(K, rows) - 0.5))
    if kind == "80 % zeros":
        return rand(K, rows) * (rand(K, rows) > 0.8)
    if kind == "99 % zeros":
        return rand(K, rows) * (rand(K, rows) > 0.99)
    if kind == "zeros and ones":
        return (rand(K, rows) > 0.5).float()
    if kind == "integers below 256":
        return torch.randint(0, 256, (K, rows), device=device, generator=g).float()
    if kind == "features over six decades":
        return randn(K, rows) * (10.0 ** (torch.arange(K, device=device) % 6).float())[:, None]
    if kind == "rows over six decades":
        return randn(K, rows) * (10.0 ** (torch.arange(rows, device=device) % 6).float())[None, :]
    if kind == "one row a million times larger":
        x = randn(K, rows)
        x[:, 7] *= 1e6
        return x
    if kind == "every other feature constant":
        x = randn(K, rows)
        x[::2] = 3.0
        return x
    if kind == "rank 8 plus noise":
        return randn(K, 8) @ randn(8, rows) + 1e-2 * randn(K, rows)
    raise ValueError(kind)


KINDS = ["uniform in [0, 1)", "offset of 1e4", "scale 1e-20", "scale 1e15", "student t, 2 degrees", "cauchy", "80 % zeros",
         "99 % zeros", "zeros and ones", "integers below 256", "features over six decades", "rows over six decades",
         "one row a million times larger", "every other feature constant", "rank 8 plus noise"]


@pytest.mark.parametrize("kind", KINDS)
def test_both_routes_keep_their_tolerance_whatever_the_data(device, kind):
    g = torch.Generator(device=device).manual_seed(KINDS.index(kind) + 100)
    a, b = operand(kind, M, device, g).t(), operand(kind, N, device, g).t()     # rows contiguous: the benchmark's storage
    out = torch.empty(N, M, device=device).t()
    rows = torch.cat([torch.arange(0, 200), torch.arange(M - 56, M)]).to(device)      # includes row 7 and the last tiles
    columns = slice(N - 384, N)

    assert kermac.get_l2_mode() == "auto"
    kermac.cdist(a, b, out=out, p=2.0)
    truth = torch.cdist(a[rows].double(), b[columns].double(), p=2.0, compute_mode="donot_use_mm_for_euclid_dist")
    assert_close_to_truth(out[rows][:, columns], truth, rtol=1e-5, atol=1e-300, what=f"squared differences, {kind}")

    truth = l1_distances_float64(a[rows], b[columns])
    with kermac.l1_mode("fixed"):
        kermac.cdist(a, b, out=out, p=1.0)
    assert_close_to_truth(out[rows][:, columns], truth, rtol=1e-5, atol=1e-300, what=f"absolute differences on fixed point, {kind}")
