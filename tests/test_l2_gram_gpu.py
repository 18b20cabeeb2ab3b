"""GPU tests of the opt-in matrix-core path for squared-difference descriptors
(``kermac_amd.set_l2_mode("gram")`` and ``"gram_bf16"``): |a|^2 + |b|^2 - 2 a.b on the
MFMA units (fp32 operands, or three bf16 pieces per operand) with automatic repair of
ill-conditioned tiles by the direct kernel.

Stated tolerance: the same 1e-5 relative to the float64 truth as the direct p = 2
path -- trusted tiles by the error bound of the expansion, repaired tiles because
they are recomputed with the direct arithmetic.
"""
import pytest
import torch

import kermac_amd as kermac
from oracle import oracle
from tests.helpers import assert_close_to_truth, make_operand

pytestmark = pytest.mark.gpu


@pytest.fixture(params=["gram", "gram_bf16"])
def gram_mode(request):
    kermac.set_l2_mode(request.param, min_k=0)      # also the short contractions, which would stay direct
    yield
    kermac.set_l2_mode(kermac.DEFAULT_L2_MODE)


def test_mode_switch_validation():
    with pytest.raises(ValueError):
        kermac.set_l2_mode("fast")
    with pytest.raises(ValueError):
        kermac.set_l2_mode("gram", trust=0.0)
    with pytest.raises(ValueError):
        kermac.set_l2_mode("gram", min_k=-1)
    assert kermac.get_l2_mode() == kermac.DEFAULT_L2_MODE


@pytest.mark.parametrize("M,N,K", [(1, 1, 1), (128, 128, 16), (129, 127, 17), (300, 515, 70), (1000, 1000, 64),
                                   (257, 64, 1024),
                                   # K ragged but a multiple of 4: row-major operands keep their 128-bit loads
                                   # and take the kernels built for a ragged K
                                   (260, 300, 100), (384, 130, 36), (128, 256, 20)])
@pytest.mark.parametrize("layout", ["cc", "rr", "cr", "rc"])
def test_random_data_matches_truth(device, gram_mode, M, N, K, layout):
    g = torch.Generator().manual_seed(M + 3 * N + 7 * K)
    a = make_operand(1, M, K, layout[0] == "c", device, g, batch=False)
    b = make_operand(1, N, K, layout[1] == "c", device, g, batch=False)
    for c_col in (False, True):
        out = torch.empty(N, M, device=device).t() if c_col else torch.empty(M, N, device=device)
        got = kermac.cdist(a, b, out=out, p=2.0)
        assert_close_to_truth(got, oracle.cdist(a.cpu(), b.cpu(), p=2.0)[0], rtol=1e-5,
                              what=f"gram {M}x{N}x{K} {layout} out col-major={c_col}")


def test_misaligned_operands(device, gram_mode):
    g = torch.Generator().manual_seed(3)
    M, N, K = 200, 150, 37
    flat = torch.randn(K * (M + 3) + 1, generator=g).to(device)
    a = flat[1:].view(K, M + 3)[:, :M].t()
    b = torch.randn(N, K + 5, generator=g).to(device)[:, 2:2 + K]
    got = kermac.cdist(a, b, p=2.0)
    assert_close_to_truth(got, oracle.cdist(a.cpu(), b.cpu(), p=2.0), rtol=1e-5, what="gram misaligned")


def test_near_duplicates_are_repaired(device, gram_mode):
    # 40 cluster centres far from the origin, points = centre + tiny noise: most
    # distances inside a cluster are 1e-4 of the norms, hopeless for the expansion.
    g = torch.Generator().manual_seed(4)
    K = 96
    centres = torch.randn(40, K, generator=g) * 3 + 5
    pts = centres[torch.randint(0, 40, (700,), generator=g)] + 1e-3 * torch.randn(700, K, generator=g)
    x = pts.to(device)
    got = kermac.cdist(x, x, p=2.0)[0]
    truth = oracle.cdist(pts, pts, p=2.0)[0]
    assert_close_to_truth(got, truth, rtol=1e-5, what="gram clustered")
    assert torch.all(torch.diagonal(got) == 0), "identical points must give exactly 0"
    assert torch.equal(got, got.t())
    # every tile is repaired here, so the result is bit-identical to the direct path
    kermac.set_l2_mode("direct")
    assert torch.equal(got, kermac.cdist(x, x, p=2.0)[0])


def test_offset_data_falls_back_everywhere(device, gram_mode):
    g = torch.Generator().manual_seed(5)
    a = (torch.rand(300, 50, generator=g) + 100).to(device)
    b = (torch.rand(260, 50, generator=g) + 100).to(device)
    got = kermac.cdist(a, b, p=2.0)
    assert_close_to_truth(got, oracle.cdist(a.cpu(), b.cpu(), p=2.0), rtol=1e-5, what="gram offset data")


def test_kernels_batches_and_regularisation(device, gram_mode):
    g = torch.Generator().manual_seed(6)
    L, N, K = 3, 333, 24
    data = torch.randn(L, N, K, generator=g).to(device)
    bw = torch.tensor([2.0, 5.0, 9.0], device=device)
    got = kermac.run_kernel(kermac.kernel_descriptor_laplace_l2, data, data, bandwidth=bw, regularization=0.125,
                            regularization_offset_x=2, regularization_offset_y=0)
    truth = oracle.run_kernel("DIFF", "SQUARE", "SQRT", "LAPLACE", data.cpu(), data.cpu(), bandwidth=bw.cpu(),
                              regularization=0.125, regularization_offset_x=2, regularization_offset_y=0)
    assert_close_to_truth(got, truth, rtol=1e-5, what="gram laplace-l2")
    gaussian = kermac.KernelDescriptor(kermac.InnerOperator.DIFF, kermac.PowerType.SQUARE, kermac.PowerType.NOOP,
                                       kermac.KernelType.GAUSSIAN)
    got = kermac.run_kernel(gaussian, data, data[0], bandwidth=3.0)
    truth = oracle.build_kernel("DIFF", "SQUARE", "NOOP", "GAUSSIAN", data.cpu(), data[0].cpu(), bandwidth=3.0)
    assert_close_to_truth(got, truth, rtol=2e-5, what="gram gaussian")   # exp(-d^2 / 18): doubles the error of d
    skipped = kermac.cdist(data, data[0], p=2.0, skip_epilogue=True)
    assert_close_to_truth(skipped, oracle.cdist(data.cpu(), data[0].cpu(), p=2.0, skip_epilogue=True), rtol=1e-5,
                          atol=1e-4, what="gram squared distances")


def test_empty_contraction_gives_zeros(device, gram_mode):
    a = torch.empty(200, 0, device=device)
    b = torch.empty(150, 0, device=device)
    out = torch.full((1, 200, 150), 7.0, device=device)
    assert kermac.cdist(a, b, out=out, p=2.0) is out
    assert torch.count_nonzero(out) == 0


def test_bf16_flag_alone_through_the_c_abi(device, monkeypatch):
    """KMC_FLAG_L2_GRAM_BF16 implies the matrix-core path; a caller of the C ABI need not set both flags."""
    from kermac_amd import _backend
    from kermac_amd.build_a_kernel import _plan_run_kernel
    g = torch.Generator().manual_seed(8)
    a = torch.randn(300, 48, generator=g).to(device)
    b = torch.randn(257, 48, generator=g).to(device)
    out = torch.empty(1, 300, 257, device=device)
    plan = _plan_run_kernel(kermac.kernel_descriptor_l2_norm, a, b, out, None, None, None, None, None, None, 0, 0, False)
    assert plan.params.flags & (_backend.FLAG_L2_GRAM | _backend.FLAG_L2_GRAM_BF16) == 0
    plan.params.flags |= _backend.FLAG_L2_GRAM_BF16
    plan.params.gram_trust = 0.25
    _backend.build_kernel(plan.params, torch.cuda.current_stream(device).cuda_stream)
    assert_close_to_truth(out, oracle.cdist(a.cpu(), b.cpu(), p=2.0), rtol=1e-5, what="bf16 flag alone")
    monkeypatch.setenv("KERMAC_AMD_L2_CENTRE", "0")          # the call above gave no gram_centre either
    with kermac.l2_mode("gram_bf16", min_k=0):
        assert torch.equal(out, kermac.cdist(a, b, p=2.0))


def test_full_size(device, gram_mode):
    M = N = 30000
    K = 1024
    torch.manual_seed(1)
    a_store = torch.randn(K, M, device=device)
    b_store = torch.randn(K, N, device=device)
    out_store = torch.empty(N, M, device=device)
    out = kermac.cdist(a_store.t(), b_store.t(), out=out_store.t(), p=2.0)
    for ms, ns in ((slice(0, 300), slice(0, 2000)), (slice(29900, 30000), slice(29800, 30000))):
        truth = torch.cdist(a_store.t()[ms].double(), b_store.t()[ns].double(), p=2.0)
        assert_close_to_truth(out[ms, ns], truth, rtol=1e-5, what="gram slab")
    assert not torch.isnan(out_store[::128, ::128]).any(), "a repair marker was left behind"
    del out_store, out
    self_out = kermac.cdist(a_store.t()[:5000], a_store.t()[:5000], p=2.0)[0]
    assert torch.all(torch.diagonal(self_out) == 0)
    assert torch.equal(self_out, self_out.t())


@pytest.mark.parametrize("layout", ["cc", "rr", "cr", "rc"])
def test_data_with_a_common_offset_stays_on_the_matrix_cores(device, gram_mode, monkeypatch, layout):
    """Points in [100, 101]^K: around the origin the expansion |a|^2 + |b|^2 - 2 a.b cancels four
    digits and every tile is recomputed by the direct kernel; around the centre that the Python
    layer hands to the library (the mean of a sample of the rows of the first operand) the norms
    are those of the spread, the tiles stay trusted, and the result keeps the stated tolerance.
    That the matrix-core values were kept shows in the bits: a repaired tile equals the direct
    kernel's result exactly."""
    g = torch.Generator().manual_seed(17)
    M, N, K = 300, 260, 96
    a = make_operand(1, M, K, layout[0] == "c", device, g, batch=False, dist="rand") + 100.0
    b = make_operand(1, N, K, layout[1] == "c", device, g, batch=False, dist="rand") + 100.0
    truth = oracle.cdist(a.cpu(), b.cpu(), p=2.0)[0]
    with kermac.l2_mode("direct"):
        direct = kermac.cdist(a, b, p=2.0)[0]
    centred = kermac.cdist(a, b, p=2.0)[0]
    assert_close_to_truth(centred, truth, rtol=1e-5, what=f"offset data, centred, {layout}")
    assert not torch.equal(centred, direct), "every tile was repaired: the centre did not take effect"
    monkeypatch.setenv("KERMAC_AMD_L2_CENTRE", "0")
    uncentred = kermac.cdist(a, b, p=2.0)[0]
    assert torch.equal(uncentred, direct), "without a centre every tile of this data must be distrusted and repaired"
    # batched, the centre per batch entry; a broadcast first operand has one
    monkeypatch.setenv("KERMAC_AMD_L2_CENTRE", "1")
    shifts = torch.tensor([0.0, 50.0, -30.0], device=device)[:, None, None]
    ab = (a - 100.0)[None] + shifts
    bb = (b - 100.0)[None] + shifts
    got = kermac.cdist(ab, bb, p=2.0)
    for l in range(3):
        assert_close_to_truth(got[l], oracle.cdist(ab[l].cpu(), bb[l].cpu(), p=2.0)[0], rtol=1e-5, what=f"batch {l}")
    got = kermac.cdist(a, bb + 100.0 - shifts, p=2.0)
    assert_close_to_truth(got[2], truth, rtol=1e-5, what="broadcast first operand")


def test_sample_mean_through_the_c_abi(device):
    """kmc_sample_mean: whole panels up to 4096 rows, 16 runs of 256 rows beyond; zero padding to 64,
    then the flag (subtract or not) and, 64 floats on, the variance per k of the sampled rows."""
    from kermac_amd import _backend
    g = torch.Generator().manual_seed(23)
    stream = torch.cuda.current_stream(device).cuda_stream
    cases = ((1, 1, False, 1, 3.0), (300, 70, False, 2, 3.0), (300, 70, True, 2, 0.0), (5000, 33, True, 1, 3.0),
             (9000, 130, False, 3, 0.01), (9000, 130, True, 2, 0.2))
    for rows, K, col_major, L, shift in cases:
        x = make_operand(L, rows, K, col_major, device, g, dist="randn") + shift
        padded = -(-K // 64) * 64
        width = 2 * padded + 64
        mean = torch.full((L, width + 5), -1.0, device=device)
        ld = x.stride(2) if col_major else x.stride(1)
        _backend.sample_mean(x.data_ptr(), _backend.COL_MAJOR if col_major else _backend.ROW_MAJOR, rows, K, ld, x.stride(0), L,
                             mean.data_ptr(), width + 5, stream)
        torch.cuda.synchronize()
        if rows <= 4096:
            sample = x
        else:
            starts = [(j * (rows - 256)) // 15 for j in range(16)]
            sample = torch.cat([x[:, s:s + 256] for s in starts], dim=1)
        assert_close_to_truth(mean[:, :K], sample.double().mean(dim=1), rtol=1e-5, atol=1e-6,      # sums of values of order 1
                              what=f"sample mean rows={rows} K={K}")
        assert torch.all(mean[:, K:padded] == 0.0) and torch.all(mean[:, width:] == -1.0)
        variance = mean[:, padded + 64:padded + 64 + K]
        assert_close_to_truth(variance, sample.double().var(dim=1, unbiased=False), rtol=1e-3, atol=1e-6,
                              what=f"sample variance rows={rows} K={K}")
        # shift^2 * K against K / 64: only a centre well inside the cloud of points is left out
        expect = 0.0 if shift * shift <= 1.0 / 256 else 1.0
        assert torch.all(mean[:, padded] == expect), f"flag rows={rows} K={K} shift={shift}: {mean[:, padded].tolist()}"
    with pytest.raises(_backend.BackendError, match="mean_bs"):
        _backend.sample_mean(x.data_ptr(), _backend.ROW_MAJOR, rows, K, ld, x.stride(0), 2, mean.data_ptr(), padded, stream)


def test_a_negligible_centre_is_left_out(device, gram_mode, monkeypatch):
    """Points spread around the origin: the library sees that the sample mean is negligible against
    the spread and runs the walk that subtracts nothing -- the bits equal those of a call without a
    centre.  A centre that matters changes them."""
    g = torch.Generator().manual_seed(31)
    a = torch.randn(700, 256, generator=g).to(device)
    b = torch.randn(650, 256, generator=g).to(device)
    with_centre = kermac.cdist(a, b, p=2.0)
    shifted = kermac.cdist(a + 1.0, b + 1.0, p=2.0)
    monkeypatch.setenv("KERMAC_AMD_L2_CENTRE", "0")
    assert torch.equal(with_centre, kermac.cdist(a, b, p=2.0))
    assert not torch.equal(shifted, kermac.cdist(a + 1.0, b + 1.0, p=2.0))


def test_auto_mode_picks_the_kernel_by_shape(device):
    """The default mode: squared differences go to the matrix cores (split-bf16 for a stored
    matrix, fp32 for the fused coefficient product) when the problem is large enough to pay for
    the two extra launches, to the direct kernel when it is small or when its grid is one that
    the direct path would cut over k; everything else is untouched."""
    from kermac_amd import _backend, build_a_kernel as module
    from kermac_amd.kernel_coefficients import _plan_run_kernel_coefficients
    assert kermac.get_l2_mode() == kermac.DEFAULT_L2_MODE == "auto"
    core = _backend.FLAG_L2_GRAM | _backend.FLAG_L2_GRAM_BF16

    def planned(M, N, K, descriptor=kermac.kernel_descriptor_l2_norm, **kw):
        a = torch.empty(M, K, device=device)
        b = torch.empty(N, K, device=device)
        return module._plan_run_kernel(descriptor, a, b, None, kw.get("p"), None, None, kw.get("bandwidth"), None, None, 0, 0, False)

    def chosen(M, N, K, descriptor=kermac.kernel_descriptor_l2_norm, **kw):
        plan = planned(M, N, K, descriptor, **kw)
        asked = plan.params.flags & core
        return module._auto_matrix_core_flags(plan.params, asked) if plan.l2_auto and asked else 0

    big = planned(8000, 8000, 128)
    assert big.l2_auto and big.params.flags & core == core and big.params.gram_trust > 0
    assert chosen(8000, 8000, 128) == core                                       # the route through a workspace
    assert chosen(500, 500, 112) == 0                                            # a short contraction: direct
    assert chosen(500, 500, 256) == core                                         # one step, from K = 128 on
    assert planned(16000, 16000, 32).params.flags & core == 0                    # K below min_k: direct
    assert planned(8000, 8000, 128, kermac.kernel_descriptor_l1_norm).params.flags & core == 0
    assert chosen(8000, 8000, 128, kermac.kernel_descriptor_laplace_l2, bandwidth=2.0) == core
    a = torch.empty(8000, 128, device=device)
    fused = _plan_run_kernel_coefficients(kermac.kernel_descriptor_laplace_l2, a, a, torch.empty(8000, 8, device=device), None,
                                          None, None, None, 2.0, None, None, 0, 0)
    assert fused.params.kernel.flags & core == _backend.FLAG_L2_GRAM            # fp32 matrix instruction there
    # a small result over a long contraction: marked, then handed back to the direct kernel and cut over k
    g = torch.Generator().manual_seed(5)
    x = torch.randn(400, 40000, generator=g).to(device)
    y = torch.randn(380, 40000, generator=g).to(device)
    assert planned(400, 380, 40000).params.flags & core == core and chosen(400, 380, 40000) == 0
    got = kermac.cdist(x, y, p=2.0)[0]
    with kermac.l2_mode("direct"):
        assert torch.equal(got, kermac.cdist(x, y, p=2.0)[0])
    assert_close_to_truth(got, oracle.cdist(x.cpu(), y.cpu(), p=2.0)[0], rtol=1e-5, what="auto, long contraction")
    # results the direct path would cut over k, but large enough for the matrix cores uncut: with the rows contiguous
    # 144 tiles of 128 x 128 on the split one-step kernel (36 of 256 x 256 are too few for the route through a
    # workspace); with k contiguous 144 tiles of 256 x 256 on that route, and 144 of 128 x 128 left to the direct path
    for rows, depth, mode, rows_contiguous in ((1500, 2048, "gram_bf16", True), (3000, 2048, "gram_bf16", False), (1500, 2048, "direct", False)):
        x = torch.randn(rows, depth, generator=g).to(device)
        y = torch.randn(rows, depth, generator=g).to(device)
        if rows_contiguous:
            x, y = x.t().contiguous().t(), y.t().contiguous().t()
        assert module._cut_over_contraction(planned(rows, rows, depth, kermac.kernel_descriptor_l1_norm).params) is not None
        got = kermac.cdist(x, y, p=2.0)[0]
        with kermac.l2_mode(mode):
            assert torch.equal(got, kermac.cdist(x, y, p=2.0)[0]), f"{rows} x {rows} x {depth}: expected {mode}"
        truth = torch.cdist(x[:64].double(), y[:64].double(), p=2.0)
        assert_close_to_truth(got[:64, :64], truth, rtol=1e-5, what="auto on results the direct path would cut")
    # a large problem in auto mode equals the explicit split-bf16 mode, near-duplicate tiles included
    g = torch.Generator().manual_seed(6)
    points = torch.randn(4400, 256, generator=g)
    points[2200:] = points[:2200] + 1e-4 * torch.randn(2200, 256, generator=g)       # every point has a near twin
    points = points.to(device)
    got = kermac.cdist(points, points.clone(), p=2.0)[0]
    with kermac.l2_mode("gram_bf16"):
        assert torch.equal(got, kermac.cdist(points, points.clone(), p=2.0)[0])
    assert_close_to_truth(got, oracle.cdist(points.cpu(), points.cpu(), p=2.0)[0], rtol=1e-5, atol=1e-30,
                          what="auto, near-duplicate points")


def test_the_one_step_kernels_look_before_they_multiply(device, monkeypatch):
    """A problem of 8.6e9 terms that the default mode gives to a one-step matrix-core kernel (256 tiles of 256 x 256 at
    K = 512: too few for the route through a workspace): the Python layer hands the library KMC_SAMPLE_BYTES of workspace,
    and the library samples the result first.  Points drawn around 64 centres in any order have a near-duplicate pair in
    every tile: the kernel only stamps its tiles, and the result is the direct kernel's bit for bit.  The same points stored
    cluster by cluster have them in the blocks on the diagonal only: the matrix cores keep the call.  Without the sample
    (KERMAC_AMD_L2_PROBE=0) every tile is multiplied, checked and recomputed: the same bits as with it."""
    from kermac_amd import _backend, build_a_kernel as module
    M = N = 4096
    K = 512
    g = torch.Generator().manual_seed(21)
    middle = 10.0 * torch.randn(64, K, generator=g)

    def clustered(rows, cluster_by_cluster):
        which = torch.randint(0, 64, (rows,), generator=g)
        if cluster_by_cluster:
            which = which.sort().values
        # rows contiguous (the benchmark's storage): with k contiguous this shape would take the route through a workspace
        return (middle[which] + 1e-3 * torch.randn(rows, K, generator=g)).to(device).t().contiguous().t()

    assert kermac.get_l2_mode() == "auto"
    a, b = clustered(M, False), clustered(N, False)
    plan = module._plan_run_kernel(kermac.kernel_descriptor_l2_norm, a, b, None, None, None, None, None, None, None, 0, 0, False)
    plan.params.flags = (plan.params.flags & ~(_backend.FLAG_L2_GRAM | _backend.FLAG_L2_GRAM_BF16)) | module._auto_matrix_core_flags(
        plan.params, plan.params.flags & (_backend.FLAG_L2_GRAM | _backend.FLAG_L2_GRAM_BF16))
    assert plan.params.flags & (_backend.FLAG_L2_GRAM | _backend.FLAG_L2_GRAM_BF16) and _backend.gram_workspace_bytes(plan.params) == 0
    workspace = module._attach_gram_workspace(plan.params, device)
    assert workspace is not None and workspace.numel() == _backend.SAMPLE_BYTES

    got = kermac.cdist(a, b, p=2.0)[0]
    with kermac.l2_mode("direct"):
        plain = kermac.cdist(a, b, p=2.0)[0]
    assert torch.equal(got, plain)
    assert_close_to_truth(got[:256, :256], torch.cdist(a[:256].double(), b[:256].double()), rtol=1e-5, atol=1e-30, what="clusters, any order")
    monkeypatch.setenv("KERMAC_AMD_L2_PROBE", "0")
    assert torch.equal(kermac.cdist(a, b, p=2.0)[0], plain)
    monkeypatch.delenv("KERMAC_AMD_L2_PROBE")

    a, b = clustered(M, True), clustered(N, True)
    got = kermac.cdist(a, b, p=2.0)[0]
    with kermac.l2_mode("direct"):
        plain = kermac.cdist(a, b, p=2.0)[0]
    same = got == plain
    assert same[:32, :32].all() and not same[:64, -64:].all() and (~same).float().mean().item() > 0.2
    rows = torch.cat([torch.arange(0, 256), torch.arange(M - 128, M)]).to(device)
    assert_close_to_truth(got[rows][:, :512], torch.cdist(a[rows].double(), b[:512].double()), rtol=1e-5, atol=1e-30,
                          what="clusters stored one after the other")

    # spread-out data of the same shape: the sample finds nothing, the matrix cores' bits
    x, y = torch.randn(K, M, generator=g).to(device).t(), torch.randn(K, N, generator=g).to(device).t()
    got = kermac.cdist(x, y, p=2.0)[0]
    with kermac.l2_mode("direct"):
        assert not torch.equal(got, kermac.cdist(x, y, p=2.0)[0])
    assert_close_to_truth(got[:256, :256], torch.cdist(x[:256].double(), y[:256].double()), rtol=1e-5, what="spread-out data")
