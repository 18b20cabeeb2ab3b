"""GPU parity tests of the fused kernel-matrix x coefficients path
(``run_kernel(..., coefficients=...)``) against the CPU oracle, the golden vector
and the unfused composition run_kernel(...) @ coefficients on the GPU."""
from pathlib import Path

import numpy as np
import pytest
import torch

import kermac_amd as kermac
from oracle import oracle
from tests.helpers import assert_close_to_truth, l1_distances_float64, make_operand

pytestmark = pytest.mark.gpu

GOLDEN = np.load(Path(__file__).resolve().parent / "golden" / "hot_path_vectors.npz")


def atol_for(truth, rtol):
    # a signed sum over n: measure against the typical magnitude of the result
    return rtol * float(truth.abs().mean()) * 10


def test_golden_vector(device):
    a, b, coef = (torch.from_numpy(GOLDEN[k]).to(device) for k in ("a", "b", "coef"))
    got = kermac.run_kernel(kermac.kernel_descriptor_laplace_l1, a, b, bandwidth=3.0, coefficients=coef)
    truth = torch.from_numpy(GOLDEN["laplace_l1_bw3_times_coef"])
    assert_close_to_truth(got, truth, rtol=1e-5, atol=atol_for(truth, 1e-5), what="golden kernel x coef")


@pytest.mark.parametrize("M,N,K,O", [(1, 1, 1, 1), (130, 200, 17, 5), (128, 128, 16, 32), (257, 129, 40, 33),
                                     (90, 300, 6, 70), (64, 31, 33, 16), (200, 150, 24, 64), (140, 260, 19, 129)])
@pytest.mark.parametrize("layout", ["cc", "rr", "cr"])
def test_shapes_and_layouts(device, M, N, K, O, layout):
    g = torch.Generator().manual_seed(M + N + K + O)
    a = make_operand(1, M, K, layout[0] == "c", device, g, batch=False, dist="rand")
    b = make_operand(1, N, K, layout[1] == "c", device, g, batch=False, dist="rand")
    coef = torch.randn(N, O, generator=g).to(device)
    for desc, names, kw in (
        (kermac.kernel_descriptor_laplace_l1, ("DIFF", "ABS", "NOOP", "LAPLACE"), {"bandwidth": 2.0}),
        (kermac.kernel_descriptor_laplace_l2, ("DIFF", "SQUARE", "SQRT", "LAPLACE"), {"bandwidth": 1.5}),
        (kermac.kernel_descriptor_l2_norm, ("DIFF", "SQUARE", "SQRT", "NONE"), {}),
    ):
        got = kermac.run_kernel(desc, a, b, coefficients=coef, **kw)
        assert got.shape == (1, M, O)
        truth = oracle.kernel_times_coefficients(*names, a.cpu(), b.cpu(), coef.cpu(), **kw)
        assert_close_to_truth(got, truth, rtol=1e-5, atol=atol_for(truth, 1e-5), what=f"{names} {layout}")


def test_matches_unfused_composition_with_batches_and_regularisation(device):
    g = torch.Generator().manual_seed(61)
    L, M, N, K, O = 3, 200, 260, 24, 12
    x = make_operand(L, M, K, True, device, g, dist="rand")
    z = make_operand(1, N, K, True, device, g, batch=False, dist="rand")     # broadcast centres
    coef = torch.randn(L, N, O + 3, generator=g).to(device)[:, :, :O]         # padded rows
    bw = torch.tensor([1.0, 2.0, 3.0], device=device)
    out = torch.full((L, M, O + 1), 5.0, device=device)
    kw = dict(bandwidth=bw, regularization=0.5, regularization_offset_x=2, regularization_offset_y=0)
    got = kermac.run_kernel(kermac.kernel_descriptor_laplace_l1, x, z, out=out[..., :O], coefficients=coef, **kw)
    full = kermac.run_kernel(kermac.kernel_descriptor_laplace_l1, x, z, **kw)
    truth = full.double() @ coef.double()
    assert_close_to_truth(got, truth, rtol=1e-5, atol=atol_for(truth, 1e-5), what="fused vs unfused")
    assert torch.all(out[..., O] == 5.0), "wrote outside the out view"
    # fractional p descriptor with per-batch p (ahead-of-time POW variant)
    desc = kermac.KernelDescriptor(kermac.InnerOperator.DIFF, kermac.PowerType.POW, kermac.PowerType.POW,
                                   kermac.KernelType.GAUSSIAN)
    p = torch.tensor([1.3, 1.6, 0.8], device=device)
    got = kermac.run_kernel(desc, x, z, p=p, bandwidth=2.0, coefficients=coef)
    truth = kermac.run_kernel(desc, x, z, p=p, bandwidth=2.0).double() @ coef.double()
    assert_close_to_truth(got, truth, rtol=1e-4, atol=atol_for(truth, 1e-4), what="fused fractional p")


def test_jit_variant_of_fused_kernel(device, tmp_path, monkeypatch):
    from kermac_amd.module_cache import module_cache as mc
    monkeypatch.setenv("KERMAC_AMD_CACHE_DIR", str(tmp_path))
    mc.Singleton._instances.pop(mc.ModuleCache, None)
    try:
        g = torch.Generator().manual_seed(62)
        a = torch.randn(140, 20, generator=g).to(device)
        b = torch.randn(150, 20, generator=g).to(device)
        coef = torch.randn(150, 7, generator=g).to(device)
        got = kermac.run_kernel(kermac.kernel_descriptor_mma, a, b, coefficients=coef)     # DOT: not ahead of time
        truth = (a.double() @ b.double().t()) @ coef.double()
        assert_close_to_truth(got[0], truth, rtol=1e-5, atol=atol_for(truth, 1e-5), what="jit fused dot")
    finally:
        mc.Singleton._instances.pop(mc.ModuleCache, None)


def test_laplace_times_coefficients_headline_shape(device):
    """batch 4, x[4,K=256,N=16384], centres z[K=256,M=16384] broadcast, U(-1,1),
    exp(-||x - z||_1 / 10) contracted with coeffs[4,16384,32]: float64 slabs."""
    torch.manual_seed(5)
    L, K, NX, MZ, O = 4, 256, 16384, 16384, 32
    x_store = torch.rand(L, K, NX, device=device) * 2 - 1
    z_store = torch.rand(K, MZ, device=device) * 2 - 1
    coef = torch.randn(L, MZ, O, device=device)
    out = kermac.run_kernel(kermac.kernel_descriptor_laplace_l1, x_store.transpose(1, 2), z_store.t(), bandwidth=10.0,
                            coefficients=coef)
    assert out.shape == (L, NX, O)
    for l, rows in ((0, slice(0, 96)), (3, slice(16300, 16384))):
        d = l1_distances_float64(x_store[l, :, rows].t(), z_store.t())
        truth = torch.exp(-d / 10.0) @ coef[l].double()
        assert_close_to_truth(out[l, rows], truth, rtol=1e-5, atol=atol_for(truth, 1e-5), what=f"slab batch {l}")


def test_no_centres_gives_zeros(device):
    """N = 0: the result buffer is allocated uninitialised, the kernel must still write
    every element (an empty sum)."""
    junk = torch.full((1, 200, 7), float("nan"), device=device)         # make a recycled allocation visible
    del junk
    a = torch.randn(200, 6, device=device)
    got = kermac.run_kernel(kermac.kernel_descriptor_laplace_l1, a, torch.zeros(0, 6, device=device), bandwidth=2.0,
                            coefficients=torch.zeros(0, 7, device=device))
    assert got.shape == (1, 200, 7) and torch.all(got == 0)


@pytest.mark.parametrize("M,N,K,O,layout", [(130, 5077, 24, 3, "cc"), (1000, 20000, 16, 1, "rr"), (64, 4096, 33, 70, "cr"),
                                            (300, 1024, 8, 5, "rc")])
def test_few_rows_many_centres_are_cut_over_the_centres(device, monkeypatch, M, N, K, O, layout):
    """Few rows against many centres: the launch takes the centres in ranges (n_ranges of the C
    parameter block), each with workgroups and a partial product of its own, and the partial
    products are added in range order (kermac_amd/kernel_coefficients.py); same values as the
    composition, with a regularised diagonal and into a caller's strided out as well."""
    from kermac_amd import kernel_coefficients as kc
    g = torch.Generator().manual_seed(M + N + K + O)
    a = make_operand(1, M, K, layout[0] == "c", device, g, batch=False, dist="rand")
    b = make_operand(1, N, K, layout[1] == "c", device, g, batch=False, dist="rand")
    coef = torch.randn(N, O, generator=g).to(device)
    plan = kc._plan_run_kernel_coefficients(kermac.kernel_descriptor_laplace_l1, a, b, coef, None, None, None, None, 2.0,
                                            None, None, 0, 0)
    assert kc._centre_ranges(plan, three_resident=O <= 32) > 1
    got = kermac.run_kernel(kermac.kernel_descriptor_laplace_l1, a, b, coefficients=coef, bandwidth=2.0)
    assert got.shape == (1, M, O)
    truth = oracle.kernel_times_coefficients("DIFF", "ABS", "NOOP", "LAPLACE", a.cpu(), b.cpu(), coef.cpu(), bandwidth=2.0)
    assert_close_to_truth(got, truth, rtol=1e-5, atol=atol_for(truth, 1e-5), what="split over centres")
    monkeypatch.setattr(kc, "_centre_ranges", lambda plan, three_resident: 1)
    unsplit = kermac.run_kernel(kermac.kernel_descriptor_laplace_l1, a, b, coefficients=coef, bandwidth=2.0)
    monkeypatch.undo()
    torch.testing.assert_close(got, unsplit, rtol=1e-5, atol=atol_for(truth, 1e-5))
    # the regularised diagonal is addressed by the global centre index, whatever the range
    kw = dict(bandwidth=2.0, regularization=0.5, regularization_offset_x=0, regularization_offset_y=N - M)   # n = m + N - M: the last centres
    got_reg = kermac.run_kernel(kermac.kernel_descriptor_laplace_l1, a, b, coefficients=coef, **kw)
    truth_reg = oracle.run_kernel_coefficients("DIFF", "ABS", "NOOP", "LAPLACE", a.cpu(), b.cpu(), coef.cpu(), **kw)
    assert (truth_reg - truth).abs().max() > 0, "the diagonal must fall inside the matrix for this check to mean anything"
    assert_close_to_truth(got_reg, truth_reg, rtol=1e-5, atol=atol_for(truth, 1e-5), what="ranges of centres, regularised diagonal")
    wide = torch.full((M, O + 3), -7.0, device=device)
    out = wide[:, :O]
    assert kermac.run_kernel(kermac.kernel_descriptor_laplace_l1, a, b, coefficients=coef, bandwidth=2.0, out=out) is out
    assert torch.equal(out, got[0]) and torch.all(wide[:, O:] == -7.0)


def test_batched_calls_take_the_centres_in_ranges(device, monkeypatch):
    """A batch with broadcast centres and per-batch bandwidths, cut into ranges of centres with a
    ragged last range; same values as the uncut launch and as the oracle, and the n_ranges field
    of the C parameter block on its own with a range count that leaves ranges empty."""
    from kermac_amd import kernel_coefficients as kc
    g = torch.Generator().manual_seed(99)
    L, M, N, K, O = 3, 200, 1100, 20, 12
    x = make_operand(L, M, K, True, device, g, dist="rand")
    z = make_operand(1, N, K, True, device, g, batch=False, dist="rand")
    coef = torch.randn(L, N, O, generator=g).to(device)
    bw = torch.tensor([1.0, 2.0, 3.0], device=device)
    truth = oracle.kernel_times_coefficients("DIFF", "ABS", "NOOP", "LAPLACE", x.cpu().contiguous(), z.cpu().contiguous(),
                                             coef.cpu(), bandwidth=bw.cpu())
    for ranges in (1, 2, 4, 9, 13):                     # 9 tiles of centres: 13 leaves four ranges empty
        monkeypatch.setattr(kc, "_centre_ranges", lambda plan, three_resident, r=ranges: r)
        got = kermac.run_kernel(kermac.kernel_descriptor_laplace_l1, x, z, coefficients=coef, bandwidth=bw)
        assert_close_to_truth(got, truth, rtol=1e-5, atol=atol_for(truth, 1e-5), what=f"{ranges} ranges of centres")
