"""GPU tests of the kernel matrix x coefficients product taken panel by panel: for squared
differences in the l2 modes "auto" and "gram_bf16", ``run_kernel(..., coefficients=...)`` builds the
kernel matrix of all rows against a few thousand centres at a time with kmc_build_kernel's
workspace route and contracts each panel with kmc_matrix_times_coefficients.  Same stated
tolerance as the fused kernel: rtol 1e-5 against the float64 oracle with an absolute floor
proportional to the typical magnitude of the signed sum over n.

KERMAC_AMD_WIDE_MIN_TILES=1 and a small KERMAC_AMD_COEFFICIENT_PANEL_BYTES send the small shapes of
these tests down the route, in several panels.
"""
import pytest
import torch

import kermac_amd as kermac
from kermac_amd import _backend
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
PANELS = "(Kermac Debug) Kernel matrix x coefficients in"


@pytest.fixture
def panels(monkeypatch):
    monkeypatch.setenv("KERMAC_AMD_WIDE_MIN_TILES", "1")
    monkeypatch.setenv("KERMAC_AMD_COEFFICIENT_PANEL_BYTES", "4096")      # the smallest panels: 256 centres
    kermac.set_l2_mode("gram_bf16", min_k=0)
    yield
    kermac.set_l2_mode(kermac.DEFAULT_L2_MODE)


def atol_for(truth, rtol):
    return rtol * float(truth.abs().mean()) * 10


def contraction(matrix, coef, out, accumulate=0, splits=1):
    """kmc_matrix_times_coefficients on matrix [L, N, M] (m contiguous), coef [L, N, O], out [S?, L, M, O]."""
    L, N, M = matrix.shape
    params = _backend.MatrixCoefficientsParams()
    params.m, params.n, params.o, params.l = M, N, coef.shape[-1], L
    params.matrix, params.matrix_ld, params.matrix_bs = matrix.data_ptr(), matrix.stride(1), matrix.stride(0)
    params.coef, params.coef_ld, params.coef_bs = coef.data_ptr(), coef.stride(1), coef.stride(0)
    params.out, params.out_ld, params.out_bs = out.data_ptr(), out.stride(-2), out.stride(-3)
    params.accumulate = accumulate
    if splits > 1:
        params.n_splits, params.out_split_stride = splits, out.stride(0)
    _backend.matrix_times_coefficients(params, torch.cuda.current_stream().cuda_stream)


@pytest.mark.parametrize("L,N,M,O", [(1, 1, 1, 1), (2, 77, 130, 5), (3, 1000, 65, 33), (1, 513, 64, 32), (2, 64, 300, 48),
                                     (1, 9, 7, 17), (1, 4097, 100, 8), (1, 300, 1029, 4), (1, 100, 50, 31), (1, 2100, 600, 12)])
@pytest.mark.parametrize("padded", [False, True])
def test_contraction_of_a_stored_panel(device, L, N, M, O, padded):
    """Both kernels (rows read 4 or 16 bytes per lane), whole and in ranges of n, stored and added,
    with padded rows of every operand; elements beside the result stay as they were."""
    g = torch.Generator().manual_seed(L + N + M + O)
    ld = (M + 3) // 4 * 4 if padded else M
    matrix = torch.randn(L, N, ld, generator=g).to(device)[:, :, :M]
    coef = torch.randn(L, N, O + 2, generator=g).to(device)[:, :, :O]
    truth = torch.bmm(matrix.double().transpose(1, 2), coef.double())
    scale = torch.bmm(matrix.double().abs().transpose(1, 2), coef.double().abs())
    store = torch.full((L, M, O + 3), 7.0, device=device)
    out = store[:, :, :O]
    contraction(matrix, coef, out)
    assert float(((out.double() - truth).abs() / scale).max()) < 1e-6
    again = torch.full_like(store, 7.0)
    contraction(matrix, coef, again[:, :, :O])
    assert torch.equal(again, store), "two runs differ"
    contraction(matrix, coef, out, accumulate=1)
    assert float(((out.double() - 2 * truth).abs() / scale).max()) < 2e-6
    assert torch.all(store[:, :, O:] == 7.0), "wrote outside the out view"
    for splits in (2, 5):
        partial = torch.full((splits, L, M, O), float("nan"), device=device)
        contraction(matrix, coef, partial, splits=splits)
        assert float(((partial.double().sum(0) - truth).abs() / scale).max()) < 1e-6, f"{splits} ranges"


def test_contraction_without_rows_stores_zeros(device):
    matrix = torch.empty(2, 0, 64, device=device)
    coef = torch.empty(2, 0, 5, device=device)
    out = torch.full((2, 64, 5), 3.0, device=device)
    contraction(matrix, coef, out, accumulate=1)
    assert torch.all(out == 3.0)
    contraction(matrix, coef, out)
    assert torch.all(out == 0.0)


@pytest.mark.parametrize("M,N,K,O", [(130, 700, 17, 5), (257, 1029, 40, 33), (300, 512, 64, 70), (64, 300, 33, 1), (1000, 260, 24, 16)])
@pytest.mark.parametrize("layout", ["cc", "rr", "cr"])
def test_shapes_and_layouts(device, panels, capsys, M, N, K, O, layout):
    g = torch.Generator().manual_seed(M + N + K + O)
    a = make_operand(1, M, K, layout[0] == "c", device, g, batch=False)
    b = make_operand(1, N, K, layout[1] == "c", device, g, batch=False)
    coef = torch.randn(N, O, generator=g).to(device)
    for descriptor, names, kw in CASES:
        got = kermac.run_kernel(descriptor, a, b, coefficients=coef, debug=True, **kw)
        assert f"{PANELS} {-(-N // 256)} panels of 256 centres" in capsys.readouterr().out
        assert got.shape == (1, M, O)
        truth = oracle.kernel_times_coefficients(*names, a.cpu(), b.cpu(), coef.cpu(), **kw)
        assert_close_to_truth(got, truth, rtol=1e-5, atol=atol_for(truth, 1e-5), what=f"{names} {layout}")
        assert torch.equal(got, kermac.run_kernel(descriptor, a, b, coefficients=coef, **kw)), "two runs differ"


def test_batches_and_a_regularised_diagonal_across_panels(device, panels, capsys):
    g = torch.Generator().manual_seed(81)
    L, M, N, K, O = 3, 700, 900, 24, 12
    x = make_operand(L, M, K, True, device, g)
    z = make_operand(1, N, K, True, device, g, batch=False)                  # broadcast centres
    coef = torch.randn(L, N, O + 3, generator=g).to(device)[:, :, :O]         # padded rows
    bw = torch.tensor([4.0, 6.0, 9.0], device=device)
    out = torch.full((L, M, O + 1), 5.0, device=device)
    # the elements with 2 + n == m get 1 + regularization: they lie in each of the four panels
    kw = dict(bandwidth=bw, regularization=0.5, regularization_offset_x=2, regularization_offset_y=0)
    got = kermac.run_kernel(kermac.kernel_descriptor_laplace_l2, x, z, out=out[..., :O], coefficients=coef, debug=True, **kw)
    assert f"{PANELS} 4 panels" in capsys.readouterr().out
    assert torch.all(out[..., O] == 5.0), "wrote outside the out view"
    truth = oracle.run_kernel_coefficients("DIFF", "SQUARE", "SQRT", "LAPLACE", x.cpu().contiguous(),
                                           z.cpu().contiguous(), coef.cpu().contiguous(), bandwidth=bw.cpu(),
                                           regularization=0.5, regularization_offset_x=2, regularization_offset_y=0)
    assert_close_to_truth(got, truth, rtol=1e-5, atol=atol_for(truth, 1e-5), what="panels vs oracle")
    # without the diagonal the result differs: the test above does see it
    plain = kermac.run_kernel(kermac.kernel_descriptor_laplace_l2, x, z, coefficients=coef, bandwidth=bw)
    assert not torch.allclose(plain, got, rtol=1e-3, atol=0.0)
    # rows broadcast over the batch, centres per batch entry, a row-major result view
    x1 = make_operand(1, M, K, False, device, g, batch=False)
    zl = make_operand(L, N, K, False, device, g)
    got = kermac.run_kernel(GAUSSIAN, x1, zl, coefficients=coef, bandwidth=5.0)
    truth = oracle.run_kernel_coefficients("DIFF", "SQUARE", "NOOP", "GAUSSIAN", x1.cpu().contiguous(),
                                           zl.cpu().contiguous(), coef.cpu().contiguous(), bandwidth=5.0)
    assert_close_to_truth(got, truth, rtol=1e-5, atol=atol_for(truth, 1e-5), what="broadcast rows")


def test_one_panel_goes_straight_into_a_strided_result(device, panels, capsys):
    """Many rows against one panel of centres: no partial products, the contraction writes the
    caller's result, here a view with padded rows and shared coefficients."""
    g = torch.Generator().manual_seed(84)
    L, M, N, K, O = 8, 4096, 200, 16, 4
    x = make_operand(L, M, K, True, device, g)
    z = make_operand(L, N, K, False, device, g)
    coef = torch.randn(N, O, generator=g).to(device)                          # one set of coefficients for the batch
    store = torch.full((L, M, O + 2), 5.0, device=device)
    got = kermac.run_kernel(GAUSSIAN, x, z, out=store[..., :O], coefficients=coef, bandwidth=3.0, debug=True)
    assert f"{PANELS} 1 panels of 200 centres, 1 partial products each" in capsys.readouterr().out
    assert torch.all(store[..., O:] == 5.0), "wrote outside the out view"
    truth = oracle.run_kernel_coefficients("DIFF", "SQUARE", "NOOP", "GAUSSIAN", x.cpu().contiguous(), z.cpu().contiguous(),
                                           coef.cpu().expand(L, N, O).contiguous(), bandwidth=3.0)
    assert_close_to_truth(got, truth, rtol=1e-5, atol=atol_for(truth, 1e-5), what="one panel")


def test_near_duplicates_far_from_the_origin(device, panels):
    """Parts of the panels whose squared distances cancel are recomputed by the direct kernel
    before the contraction reads them."""
    g = torch.Generator().manual_seed(82)
    base = torch.randn(50, 32, generator=g) + 40.0
    x = (base.repeat(6, 1) + 1e-3 * torch.randn(300, 32, generator=g)).to(device)
    z = (base.repeat(12, 1) + 1e-3 * torch.randn(600, 32, generator=g)).to(device)
    coef = torch.randn(600, 20, generator=g).to(device)
    for descriptor, names, kw in CASES[:2]:
        got = kermac.run_kernel(descriptor, x, z, coefficients=coef, **kw)
        truth = oracle.kernel_times_coefficients(*names, x.cpu(), z.cpu(), coef.cpu(), **kw)
        assert_close_to_truth(got, truth, rtol=1e-5, atol=atol_for(truth, 1e-5), what=f"{names} near duplicates")


def test_which_calls_go_in_panels(device, monkeypatch, capsys):
    """Squared differences in the modes "auto" and "gram_bf16" only, only when the panels are large
    enough for the workspace route, and not with KERMAC_AMD_COEFFICIENT_PANEL_BYTES=0."""
    g = torch.Generator().manual_seed(83)
    a = torch.randn(2048, 1024, generator=g).to(device)
    b = torch.randn(8192, 1024, generator=g).to(device)
    coef = torch.randn(8192, 8, generator=g).to(device)

    def in_panels(descriptor=GAUSSIAN, rows=a, **kw):
        capsys.readouterr()
        kw.setdefault("bandwidth", 32.0)
        kermac.run_kernel(descriptor, rows, b, coefficients=coef, debug=True, **kw)
        return PANELS in capsys.readouterr().out

    assert kermac.get_l2_mode() == "auto"
    assert in_panels()                                               # 8 x 32 tiles, 1.7e10 terms
    assert in_panels(kermac.kernel_descriptor_laplace_l2)
    assert not in_panels(kermac.kernel_descriptor_laplace_l1)
    assert not in_panels(rows=a[:256])                               # 1 x 32 tiles: the split is not earned back
    monkeypatch.setenv("KERMAC_AMD_COEFFICIENT_PANEL_BYTES", "0")
    assert not in_panels()
    monkeypatch.delenv("KERMAC_AMD_COEFFICIENT_PANEL_BYTES")
    monkeypatch.setenv("KERMAC_AMD_L2_WORKSPACE", "0")
    assert not in_panels()
    monkeypatch.delenv("KERMAC_AMD_L2_WORKSPACE")
    for mode, expected in (("gram", False), ("direct", False), ("gram_bf16", True)):
        with kermac.l2_mode(mode):
            assert in_panels() == expected, mode
    with kermac.l2_mode("direct"):
        direct = kermac.run_kernel(GAUSSIAN, a, b, coefficients=coef, bandwidth=32.0)
    got = kermac.run_kernel(GAUSSIAN, a, b, coefficients=coef, bandwidth=32.0)
    assert_close_to_truth(got, direct.double(), rtol=1e-5, atol=atol_for(direct, 1e-5), what="panels vs direct fused kernel")


def test_headline_shape_gaussian(device, capsys):
    """The fused benchmark shape (batch 4, 16384 x 16384, K = 256, O = 32) with a Gaussian kernel in
    the default mode: four panels of 4096 centres; float64 slabs of the result."""
    torch.manual_seed(5)
    L, K, NX, MZ, O = 4, 256, 16384, 16384, 32
    x = torch.rand(L, K, NX, device=device) * 2 - 1
    z = torch.rand(K, MZ, device=device) * 2 - 1
    coef = torch.randn(L, MZ, O, device=device)
    out = torch.empty(L, NX, O, device=device)
    kermac.run_kernel(GAUSSIAN, x.transpose(1, 2), z.t(), out=out, bandwidth=9.0, coefficients=coef, debug=True)
    assert f"{PANELS} 4 panels of 4096 centres" in capsys.readouterr().out
    for l, rows in ((0, slice(0, 96)), (3, slice(16300, 16384))):
        d2 = torch.cdist(x[l, :, rows].t().double(), z.t().double(), p=2.0) ** 2
        truth = torch.exp(-d2 / (2 * 9.0 ** 2)) @ coef[l].double()
        assert_close_to_truth(out[l, rows], truth, rtol=1e-5, atol=atol_for(truth, 1e-5), what=f"gaussian slab batch {l}")


@pytest.mark.parametrize("M,N,K,O,k_contiguous", [(500, 480, 1600, 5, True), (500, 480, 1600, 5, False),      # a long contraction, 4 tiles
                                                  (100, 16500, 800, 40, True),                               # 65 tiles, more than 32 columns
                                                  (2100, 6000, 256, 3, False)])                              # 216 tiles
def test_auto_mode_takes_panels_where_the_fused_kernel_is_the_slower_one(device, capsys, M, N, K, O, k_contiguous):
    """The default mode asks for the route through a workspace (KMC_FLAG_GRAM_WORKSPACE_ANY_SIZE) for
    products that the library's own rule, made for stored matrices, leaves to the one-step kernels."""
    assert kermac.get_l2_mode() == "auto"
    g = torch.Generator().manual_seed(M + N + K + O)
    a = make_operand(1, M, K, not k_contiguous, device, g, batch=False)
    b = make_operand(1, N, K, not k_contiguous, device, g, batch=False)
    coef = torch.randn(N, O, generator=g).to(device)
    bandwidth = float(K) ** 0.5
    got = kermac.run_kernel(GAUSSIAN, a, b, coefficients=coef, bandwidth=bandwidth, debug=True)
    assert PANELS in capsys.readouterr().out
    squared = torch.cdist(a.double(), b.double(), p=2.0) ** 2                 # float64 on the device: the larger cases take the CPU oracle too long
    truth = torch.exp(-squared / (2 * bandwidth ** 2)) @ coef.double()
    assert_close_to_truth(got[0], truth, rtol=1e-5, atol=atol_for(truth, 1e-5), what=f"auto panels {M}x{N}x{K}x{O}")
    with kermac.l2_mode("gram_bf16"):           # the explicit mode follows the library's rule: the fused kernel
        kermac.run_kernel(GAUSSIAN, a, b, coefficients=coef, bandwidth=bandwidth, debug=True)
        assert PANELS not in capsys.readouterr().out


@pytest.mark.parametrize("descriptor,names,kw", [
    (kermac.kernel_descriptor_laplace_l1, ("DIFF", "ABS", "NOOP", "LAPLACE"), {"bandwidth": 7.0}),
    (kermac.kernel_descriptor_p_norm, ("DIFF", "POW", "POW", "NONE"), {"p": 1.3}),
    (kermac.kernel_descriptor_laplace_l2, ("DIFF", "SQUARE", "SQRT", "LAPLACE"), {"bandwidth": 5.0}),
])
def test_more_than_64_columns_go_in_panels_for_every_descriptor(device, monkeypatch, capsys, descriptor, names, kw):
    """The fused kernel holds 64 coefficient columns per walk of the kernel matrix; with more, the
    matrix is built once per panel by kmc_build_kernel (whatever kernel the descriptor launches)
    and contracted with all columns.  Same tolerance as the fused kernel; a regularised diagonal
    across panels; partial products, and panels added one after the other when the partial
    products would take too much memory."""
    from kermac_amd import kernel_coefficients as module
    g = torch.Generator().manual_seed(87)
    L, M, N, K, O = 2, 700, 1800, 24, 70
    a = make_operand(L, M, K, False, device, g)
    b = make_operand(L, N, K, True, device, g)
    coef = torch.randn(L, N, O, generator=g).to(device)
    extra = dict(kw)
    if "bandwidth" in kw:
        extra.update(regularization=0.5, regularization_offset_x=1, regularization_offset_y=4)
    oracle_kw = dict(kw)
    if "p" in oracle_kw:
        oracle_kw = {"p_inner": kw["p"], "p_outer": 1.0 / kw["p"]}
    if "bandwidth" in kw:
        oracle_kw.update(regularization=0.5, regularization_offset_x=1, regularization_offset_y=4)
    truth = oracle.run_kernel_coefficients(*names, a.cpu().contiguous(), b.cpu().contiguous(), coef.cpu(), **oracle_kw)
    rtol = 1e-4 if "p" in kw else 1e-5
    monkeypatch.setenv("KERMAC_AMD_COEFFICIENT_PANEL_BYTES", str(4 * L * 700 * 512))           # panels of 512 centres
    for cap, said in ((module._PANEL_MAX_PARTIAL_BYTES, "partial products each"), (1024, "added to the result one after the other")):
        monkeypatch.setattr(module, "_PANEL_MAX_PARTIAL_BYTES", cap)
        out = torch.full((L, M, O + 2), 3.0, device=device)
        got = kermac.run_kernel(descriptor, a, b, out=out[..., :O], coefficients=coef, debug=True, **extra)
        printed = capsys.readouterr().out
        assert f"{PANELS} 4 panels of 512 centres" in printed and said in printed, printed
        assert_close_to_truth(got, truth, rtol=rtol, atol=atol_for(truth, rtol), what=f"{names}, {said}")
        assert torch.all(out[..., O:] == 3.0), "wrote outside the out view"
    kermac.run_kernel(descriptor, a, b, coefficients=coef[..., :64], debug=True, **extra)      # 64 columns: one walk, fused
    assert PANELS not in capsys.readouterr().out
    kermac.run_kernel(descriptor, a[:, :300], b[:, :300], coefficients=coef[:, :300], debug=True, **extra)     # a small problem: fused
    assert PANELS not in capsys.readouterr().out


def test_more_than_64_columns_of_a_run_time_compiled_descriptor(device, monkeypatch, capsys):
    """sum_k sqrt(a b), squared: not built ahead of time; its panels come from the run-time compiled
    kernel of run_kernel, the contraction is the same."""
    g = torch.Generator().manual_seed(88)
    desc = kermac.KernelDescriptor(kermac.InnerOperator.DOT, kermac.PowerType.SQRT, kermac.PowerType.SQUARE, kermac.KernelType.NONE)
    M, N, K, O = 900, 1300, 20, 66
    a = torch.rand(M, K, generator=g).to(device)
    b = torch.rand(K, N, generator=g).to(device).t()
    coef = torch.randn(N, O, generator=g).to(device)
    monkeypatch.setenv("KERMAC_AMD_COEFFICIENT_PANEL_BYTES", str(4 * 900 * 512))
    got = kermac.run_kernel(desc, a, b, coefficients=coef, debug=True)
    assert f"{PANELS} 3 panels of 512 centres" in capsys.readouterr().out
    truth = oracle.run_kernel_coefficients("DOT", "SQRT", "SQUARE", "NONE", a.cpu(), b.cpu().contiguous(), coef.cpu())
    assert_close_to_truth(got, truth, rtol=1e-5, atol=atol_for(truth, 1e-5), what="run-time compiled descriptor in panels")
    monkeypatch.setenv("KERMAC_AMD_COEFFICIENT_PANEL_BYTES", "0")
    fused = kermac.run_kernel(desc, a, b, coefficients=coef)
    assert_close_to_truth(fused, truth, rtol=1e-5, atol=atol_for(truth, 1e-5), what="the same on the fused kernel")


@pytest.mark.parametrize("M,N,K,O,L", [(300, 1100, 24, 70, 2), (130, 700, 40, 5, 1), (257, 520, 17, 33, 3)])
def test_contraction_from_fp16_pieces(device, monkeypatch, capsys, M, N, K, O, L):
    """Hundreds of columns on many rows contract their panels as a product of fp16 pieces
    (kmc_build_kernel's route for sums of products) instead of kmc_matrix_times_coefficients;
    KERMAC_AMD_COEFFICIENT_PIECES_MIN_COLUMNS=1 sends these small shapes that way.  Several panels
    (the first is stored, the others are added), padded and misaligned coefficients, a padded result."""
    from kermac_amd import kernel_coefficients as module
    g = torch.Generator().manual_seed(M + N + K + O)
    monkeypatch.setenv("KERMAC_AMD_COEFFICIENT_PIECES_MIN_COLUMNS", "1")
    monkeypatch.setenv("KERMAC_AMD_COEFFICIENT_PANEL_BYTES", str(4 * L * 512 * (-(-M // 4) * 4)))       # panels of 512 centres
    monkeypatch.setattr(module, "_FUSED_COLUMNS_PER_WALK", 0)                # any number of columns in plain panels
    monkeypatch.setattr(module, "_MANY_COLUMNS_MIN_ELEMENTS", 0.0)
    a = make_operand(L, M, K, False, device, g)
    b = make_operand(L, N, K, True, device, g)
    coef = torch.randn(L, N, O + 3, generator=g).to(device)[..., 1:O + 1]    # rows neither aligned nor a multiple of 4 long
    out = torch.full((L, M, O + 1), 9.0, device=device)
    for descriptor, names, kw in ((kermac.kernel_descriptor_laplace_l1, ("DIFF", "ABS", "NOOP", "LAPLACE"), {"bandwidth": 9.0}),
                                  (GAUSSIAN, ("DIFF", "SQUARE", "NOOP", "GAUSSIAN"), {"bandwidth": 5.0})):
        got = kermac.run_kernel(descriptor, a, b, out=out[..., :O], coefficients=coef, debug=True, **kw)
        printed = capsys.readouterr().out
        assert f"{PANELS} {-(-N // 512)} panels of 512 centres, contracted from fp16 pieces" in printed, printed
        truth = oracle.run_kernel_coefficients(*names, a.cpu().contiguous(), b.cpu().contiguous(), coef.cpu().contiguous(), **kw)
        assert_close_to_truth(got, truth, rtol=1e-5, atol=atol_for(truth, 1e-5), what=f"{names} contracted from pieces")
        assert torch.all(out[..., O] == 9.0), "wrote outside the out view"
        assert torch.equal(got, kermac.run_kernel(descriptor, a, b, coefficients=coef, **kw)), "two runs differ"



def test_headline_shape_with_256_columns(device, capsys):
    """The fused benchmark shape with 256 coefficient columns, by the rules alone: panels on the
    fp16 matrix instruction, each contracted as a product of fp16 pieces; float64 slabs."""
    torch.manual_seed(6)
    L, K, NX, MZ, O = 4, 256, 16384, 16384, 256
    x = torch.rand(L, K, NX, device=device) * 2 - 1
    z = torch.rand(K, MZ, device=device) * 2 - 1
    coef = torch.randn(L, MZ, O, device=device)
    out = torch.empty(L, NX, O, device=device)
    kermac.run_kernel(GAUSSIAN, x.transpose(1, 2), z.t(), out=out, bandwidth=9.0, coefficients=coef, debug=True)
    assert f"{PANELS} 4 panels of 4096 centres, contracted from fp16 pieces" in capsys.readouterr().out
    for l, rows in ((0, slice(0, 96)), (3, slice(16300, 16384))):
        d2 = torch.cdist(x[l, :, rows].t().double(), z.t().double(), p=2.0) ** 2
        truth = torch.exp(-d2 / (2 * 9.0 ** 2)) @ coef[l].double()
        assert_close_to_truth(out[l, rows], truth, rtol=1e-5, atol=atol_for(truth, 1e-5), what=f"256 columns, slab of batch {l}")
