"""GPU tests of the route that large squared-difference problems take in the split-bf16 mode when
the caller brings a workspace (include/kermac_amd.h, gram_workspace): row statistics, both
operands split once into two fp16 pieces per value with a power-of-two scale per row, then
256 x 256 tiles on the fp16 matrix instruction.  Same stated tolerance as every p = 2 path: 1e-5
relative to the float64 truth -- trusted 128 x 128 parts by the error bound of the expansion,
distrusted parts because the direct kernel recomputes them.

KERMAC_AMD_WIDE_MIN_TILES=1 sends the small shapes of these tests down the route, which by itself
only takes problems of at least 128 tiles of 256 x 256 (and K >= 64, several tiles in both directions
of every batch entry, little padding: kmc_gram_workspace_bytes in include/kermac_amd.h).
"""
import pytest
import torch

import kermac_amd as kermac
from kermac_amd import _backend, build_a_kernel as module
from oracle import oracle
from tests.helpers import assert_close_to_truth, make_operand

pytestmark = pytest.mark.gpu


@pytest.fixture
def wide(monkeypatch):
    monkeypatch.setenv("KERMAC_AMD_WIDE_MIN_TILES", "1")
    kermac.set_l2_mode("gram_bf16", min_k=0)
    yield
    kermac.set_l2_mode(kermac.DEFAULT_L2_MODE)


def one_step(fn, monkeypatch):
    """The same call on the one-step kernel."""
    monkeypatch.setenv("KERMAC_AMD_L2_WORKSPACE", "0")
    try:
        return fn()
    finally:
        monkeypatch.setenv("KERMAC_AMD_L2_WORKSPACE", "1")


def workspace_bytes(a, b, descriptor=kermac.kernel_descriptor_l2_norm, **kw):
    plan = module._plan_run_kernel(descriptor, a, b, None, None, None, None, kw.get("bandwidth"), None, None, 0, 0, False)
    return _backend.gram_workspace_bytes(plan.params)


@pytest.mark.parametrize("M,N,K", [(300, 260, 96), (515, 770, 70), (1000, 900, 200), (257, 255, 33), (256, 512, 1024),
                                   (1, 700, 64), (640, 3, 48), (300, 200, 5), (128, 128, 16), (513, 257, 1)])
@pytest.mark.parametrize("layout", ["cc", "rr", "cr", "rc"])
def test_random_data_matches_truth(device, wide, M, N, K, layout):
    g = torch.Generator().manual_seed(M + 3 * N + 7 * K)
    a = make_operand(1, M, K, layout[0] == "c", device, g, batch=False)
    b = make_operand(1, N, K, layout[1] == "c", device, g, batch=False)
    assert workspace_bytes(a, b) > 0
    for c_col in (False, True):
        out = torch.empty(N, M, device=device).t() if c_col else torch.empty(M, N, device=device)
        got = kermac.cdist(a, b, out=out, p=2.0)
        assert_close_to_truth(got, oracle.cdist(a.cpu(), b.cpu(), p=2.0)[0], rtol=1e-5,
                              what=f"wide {M}x{N}x{K} {layout} out col-major={c_col}")


def test_when_the_route_applies(device, monkeypatch):
    """kmc_gram_workspace_bytes: 0 without the split-bf16 flag, for
    short contractions and for problems of too few tiles of 256 x 256 over the batch for their k."""
    a = torch.empty(7000, 512, device=device)
    b = torch.empty(4000, 512, device=device)
    with kermac.l2_mode("gram_bf16"):
        assert workspace_bytes(a, b) > 0                                         # 28 x 16 tiles
        assert workspace_bytes(a, b, kermac.kernel_descriptor_laplace_l2, bandwidth=2.0) > 0
        assert workspace_bytes(a, b, kermac.kernel_descriptor_l1_norm) == 0
        assert 0 < workspace_bytes(a, a) < 0.6 * workspace_bytes(a, a.clone())   # 406 tiles of the triangle; one panel, split once
        assert workspace_bytes(a[:2500], b[:2500]) > 0                           # 100 tiles, k contiguous: from 48 tiles on
        assert workspace_bytes(a[:1500], b[:1500]) == 0                          # 36 tiles
        at, bt = torch.empty(512, 7000, device=device).t(), torch.empty(512, 4000, device=device).t()
        assert workspace_bytes(at, bt) > 0                                       # rows contiguous: from 128 tiles on
        assert workspace_bytes(at[:3500], at[:3500]) == 0                        # 14 * 15 / 2 = 105 tiles of the triangle
        assert workspace_bytes(at[:2500], bt[:2500]) == 0                        # 100 tiles
        assert workspace_bytes(a[:, :32], b[:, :32]) == 0                        # k < 64
        assert workspace_bytes(a[:, :128], b[:, :128]) == 0                      # 320 tiles at k = 128
        assert workspace_bytes(a[:2500].expand(3, 2500, 512), b[:2500].expand(3, 2500, 512)) > 0    # 300 over the batch
        needed = workspace_bytes(a, b)
        operands = (7000 + 4000) * 512 * 4
        assert operands <= needed <= 2 * operands
    with kermac.l2_mode("gram"):
        assert workspace_bytes(a, b) == 0
    with kermac.l2_mode("direct"):
        assert workspace_bytes(a, b) == 0


def test_without_a_workspace_the_one_step_kernel_runs(device, wide, monkeypatch):
    g = torch.Generator().manual_seed(2)
    a = torch.randn(700, 96, generator=g).to(device)
    b = torch.randn(600, 96, generator=g).to(device)
    reference = one_step(lambda: kermac.cdist(a, b, p=2.0), monkeypatch)
    plan = module._plan_run_kernel(kermac.kernel_descriptor_l2_norm, a, b, None, None, None, None, None, None, None, 0, 0, False)
    stream = torch.cuda.current_stream(device).cuda_stream
    keep = module._attach_gram_centre(plan.params, stream, device)
    needed = _backend.gram_workspace_bytes(plan.params)
    assert needed > 0
    workspace = torch.empty(needed, dtype=torch.uint8, device=device)
    for pointer, size in ((0, 0), (workspace.data_ptr(), needed - 1), (workspace.data_ptr() + 16, needed)):
        plan.out.fill_(-1.0)
        plan.params.gram_workspace, plan.params.gram_workspace_bytes = pointer, size
        _backend.build_kernel(plan.params, stream)
        assert torch.equal(plan.out, reference), "null, short or misaligned workspace: expected the one-step kernel's bits"
    plan.params.gram_workspace, plan.params.gram_workspace_bytes = workspace.data_ptr(), needed
    _backend.build_kernel(plan.params, stream)
    assert_close_to_truth(plan.out, oracle.cdist(a.cpu(), b.cpu(), p=2.0), rtol=1e-5, what="with the workspace")
    del keep


def test_rows_of_very_different_magnitude(device, wide):
    """The scale is per row: a row of values around 1e-6 beside rows around 1e+5, and eight orders
    of magnitude inside every row, keep the tolerance (one scale per operand would put the small
    rows into fp16's subnormals)."""
    g = torch.Generator().manual_seed(9)
    M, N, K = 520, 390, 150
    within = torch.pow(2.0, -(torch.arange(K) % 27).float())
    a = torch.randn(M, K, generator=g) * within * torch.pow(2.0, (torch.arange(M) % 37 - 18).float())[:, None]
    b = torch.randn(N, K, generator=g) * within * torch.pow(2.0, (torch.arange(N) % 37 - 18).float())[:, None]
    a, b = a.to(device), b.to(device)
    got = kermac.cdist(a, b, p=2.0)
    assert_close_to_truth(got, oracle.cdist(a.cpu(), b.cpu(), p=2.0), rtol=1e-5, what="rows of different magnitude")


def test_near_duplicates_are_repaired_part_by_part(device, wide, monkeypatch):
    """Every point of b has a twin in a: the parts of 128 x 128 that hold a twin pair are distrusted
    and come from the direct kernel bit for bit; no marker is left behind."""
    g = torch.Generator().manual_seed(4)
    a = torch.randn(600, 128, generator=g)
    b = a[:500] + 1e-5 * torch.randn(500, 128, generator=g)
    a, b = a.to(device), b.to(device)
    got = kermac.cdist(a, b, p=2.0)[0]
    with kermac.l2_mode("direct"):
        direct = kermac.cdist(a, b, p=2.0)[0]
    assert not torch.isnan(got).any()
    assert_close_to_truth(got, oracle.cdist(a.cpu(), b.cpu(), p=2.0)[0], rtol=1e-5, atol=1e-30, what="near duplicates")
    for part in range(0, 500, 128):                      # the parts on the diagonal hold the twins
        stop = min(part + 128, 500)
        assert torch.equal(got[part:stop, part:stop], direct[part:stop, part:stop])
    assert not torch.equal(got, direct), "every part was repaired: the matrix-core values were not kept"


def test_data_that_is_not_a_number(device, wide):
    """A NaN and an infinity in a: their rows come out as the direct kernel gives them."""
    g = torch.Generator().manual_seed(6)
    a = torch.randn(300, 64, generator=g)
    b = torch.randn(280, 64, generator=g)
    a[17, 3] = float("nan")
    a[200, 40] = float("inf")
    a, b = a.to(device), b.to(device)
    got = kermac.cdist(a, b, p=2.0)[0]
    with kermac.l2_mode("direct"):
        direct = kermac.cdist(a, b, p=2.0)[0]
    assert torch.equal(torch.isnan(got), torch.isnan(direct)) and torch.equal(torch.isinf(got), torch.isinf(direct))
    finite = torch.isfinite(direct)
    rows = torch.ones(300, dtype=torch.bool)
    rows[17] = rows[200] = False
    assert torch.equal(finite.cpu(), rows[:, None].expand(300, 280))
    truth = oracle.cdist(a.cpu(), b.cpu(), p=2.0)[0]
    assert_close_to_truth(got[rows.to(device)], truth[rows], rtol=1e-5, what="rows without NaN or infinity")


@pytest.mark.parametrize("layout", ["cc", "rr"])
def test_offset_data_and_batches(device, wide, monkeypatch, layout):
    """Points in [100, 101]^K: the centre is subtracted by the split, per batch entry; a first
    operand that is the same for every batch entry is split once, or once per entry when the
    centres differ."""
    g = torch.Generator().manual_seed(17)
    M, N, K = 300, 260, 96
    a = make_operand(1, M, K, layout[0] == "c", device, g, batch=False, dist="rand") + 100.0
    b = make_operand(1, N, K, layout[1] == "c", device, g, batch=False, dist="rand") + 100.0
    truth = oracle.cdist(a.cpu(), b.cpu(), p=2.0)[0]
    with kermac.l2_mode("direct"):
        direct = kermac.cdist(a, b, p=2.0)[0]
    got = kermac.cdist(a, b, p=2.0)[0]
    assert_close_to_truth(got, truth, rtol=1e-5, what=f"offset data {layout}")
    assert not torch.equal(got, direct), "every part was repaired: the centre did not take effect"
    shifts = torch.tensor([0.0, 50.0, -30.0], device=device)[:, None, None]
    ab = (a - 100.0)[None] + shifts
    bb = (b - 100.0)[None] + shifts
    batched = kermac.cdist(ab, bb, p=2.0)
    for l in range(3):
        assert_close_to_truth(batched[l], oracle.cdist(ab[l].cpu(), bb[l].cpu(), p=2.0)[0], rtol=1e-5, what=f"batch {l}")
    broadcast = kermac.cdist(a, bb + 100.0 - shifts, p=2.0)                  # a for every entry, one centre
    assert_close_to_truth(broadcast[2], truth, rtol=1e-5, what="first operand for every batch entry")
    broadcast = kermac.cdist(ab, b - 100.0, p=2.0)                           # b for every entry, a centre per entry
    for l in range(3):
        assert_close_to_truth(broadcast[l], oracle.cdist(ab[l].cpu(), (b - 100.0).cpu(), p=2.0)[0], rtol=1e-5,
                              what=f"second operand for every batch entry, entry {l}")


def test_kernel_functions_and_regularisation(device, wide):
    g = torch.Generator().manual_seed(12)
    M, N, K = 400, 330, 80
    a = torch.randn(M, K, generator=g).to(device)
    b = torch.randn(N, K, generator=g).to(device)
    gaussian = kermac.KernelDescriptor(kermac.InnerOperator.DIFF, kermac.PowerType.SQUARE, kermac.PowerType.NOOP,
                                       kermac.KernelType.GAUSSIAN)
    for descriptor, outer, kernel, bandwidth, rtol in ((kermac.kernel_descriptor_laplace_l2, "SQRT", "LAPLACE", float(K), 1e-5),
                                                       (gaussian, "NOOP", "GAUSSIAN", 10.0, 2e-5)):     # exp(-d^2 / 200) doubles the error of d
        assert workspace_bytes(a, b, descriptor, bandwidth=bandwidth) > 0
        got = kermac.run_kernel(descriptor, a, b, bandwidth=bandwidth, regularization=0.25, regularization_offset_x=2,
                                regularization_offset_y=70)
        want = oracle.run_kernel("DIFF", "SQUARE", outer, kernel, a.cpu(), b.cpu(), bandwidth=bandwidth, regularization=0.25,
                                 regularization_offset_x=2, regularization_offset_y=70)
        assert_close_to_truth(got, want, rtol=rtol, what=kernel)
        assert (got == 1.25).sum() > 0
    squares = kermac.cdist(a, b, p=2.0, skip_epilogue=True)
    assert_close_to_truth(squares, oracle.cdist(a.cpu(), b.cpu(), p=2.0, skip_epilogue=True), rtol=1e-5, what="squared distances")


def test_unaligned_result_and_operands(device, wide):
    g = torch.Generator().manual_seed(3)
    M, N, K = 310, 270, 37
    flat = torch.randn(K * (M + 3) + 1, generator=g).to(device)
    a = flat[1:].view(K, M + 3)[:, :M].t()
    b = torch.randn(N, K + 5, generator=g).to(device)[:, 2:2 + K]
    out = torch.empty(N, M + 1, device=device)[:, :M].t()
    got = kermac.cdist(a, b, out=out, p=2.0)
    assert_close_to_truth(got, oracle.cdist(a.cpu(), b.cpu(), p=2.0)[0], rtol=1e-5, what="unaligned")


def test_large_problem_takes_the_route_by_itself(device):
    """The default mode at a size above the threshold: the result equals the explicit mode with the
    workspace and differs from the one-step kernel's, and keeps the tolerance on slabs."""
    assert kermac.get_l2_mode() == "auto"
    g = torch.Generator().manual_seed(8)
    a = torch.randn(512, 4700, generator=g).to(device).t()
    b = torch.randn(512, 4200, generator=g).to(device).t()
    assert workspace_bytes(a, b) > 0
    got = kermac.cdist(a, b, p=2.0)[0]
    truth = torch.cdist(a[:300].double(), b.double(), p=2.0)
    assert_close_to_truth(got[:300], truth, rtol=1e-5, what="auto, wide")
    assert not torch.isnan(got[::128, ::128]).any()


@pytest.mark.parametrize("rows,K,col_major", [(129, 20, True), (700, 48, True), (515, 33, False), (1024, 64, False), (300, 200, True)])
def test_a_panel_against_itself(device, wide, monkeypatch, rows, K, col_major):
    """One workgroup per 256 x 256 tile on or below the diagonal; the result is symmetric bit for bit,
    equals the full computation to rounding and the truth to the stated tolerance."""
    g = torch.Generator().manual_seed(rows + K)
    x = torch.randn(K, rows, generator=g).to(device).t() if col_major else torch.randn(rows, K, generator=g).to(device)
    assert workspace_bytes(x, x) > 0
    for out_col_major in (True, False):
        store = torch.full((rows, rows + 4), float("nan"), device=device)
        out = store[:, :rows].t() if out_col_major else store[:, :rows]
        got = kermac.cdist(x, x, out=out, p=2.0)
        assert got.shape == (rows, rows)
        assert torch.equal(got, got.t()), "not symmetric"
        assert torch.all(torch.diagonal(got) == 0)
        assert torch.isnan(store[:, rows:]).all(), "wrote outside the out view"
        full = kermac.cdist(x, x.clone(memory_format=torch.preserve_format), p=2.0)[0]
        torch.testing.assert_close(got, full, rtol=2e-6, atol=1e-6)
        assert_close_to_truth(got, oracle.cdist(x.cpu(), x.cpu(), p=2.0)[0], rtol=1e-5, atol=1e-30, what=f"self {rows}x{K}")


def test_a_batch_of_panels_against_themselves_with_near_twins(device, wide):
    g = torch.Generator().manual_seed(11)
    L, rows, K = 3, 400, 40
    x = torch.randn(L, K, rows, generator=g).to(device).transpose(1, 2)
    bw = torch.tensor([5.0, 9.0, 14.0], device=device)
    got = kermac.run_kernel(kermac.kernel_descriptor_laplace_l2, x, x, bandwidth=bw, regularization=1e-3)
    assert torch.equal(got, got.transpose(1, 2))
    truth = oracle.build_kernel("DIFF", "SQUARE", "SQRT", "LAPLACE", x.cpu().contiguous(), x.cpu().contiguous(),
                                bandwidth=bw.cpu(), regularization=1e-3)
    assert_close_to_truth(got, truth, rtol=1e-5, atol=1e-7, what="batched self matrix")
    # near-duplicate rows: those parts are recomputed, and mirrored, by the repair launch
    y = torch.randn(600, 24, generator=g).to(device)
    y[300:] = y[:300] + 1e-4 * torch.randn(300, 24, generator=g).to(device)
    d_self = kermac.cdist(y, y, p=2.0)[0]
    assert torch.equal(d_self, d_self.t())
    assert not torch.isnan(d_self).any()
    assert_close_to_truth(d_self, oracle.cdist(y.cpu(), y.cpu(), p=2.0)[0], rtol=1e-5, atol=1e-30, what="near duplicates")


def clustered(rows, middle, device, seed, cluster_by_cluster=False):
    """Every row one of the points `middle` plus noise of 1e-3: two rows of one cluster are near-duplicates."""
    g = torch.Generator().manual_seed(seed)
    which = torch.randint(0, middle.size(0), (rows,), generator=g)
    if cluster_by_cluster:
        which = which.sort().values
    return (middle[which] + 1e-3 * torch.randn(rows, middle.size(1), generator=g)).to(device)


def test_sets_of_near_duplicates_go_to_the_direct_kernel_whole(device):
    """The default mode on data that the trust rule rejects nearly everywhere (64 tight clusters: one pair in 64 is a
    pair of near-duplicates, so every 128 x 128 part holds some): the sample of pairs sees it, the matrix-core kernel only
    stamps its parts, and the result is the direct kernel's, bit for bit, at its tolerance -- for the direct kernel's
    time, not for both."""
    M, N, K = 8192, 8192, 1024          # 1024 tiles of 256 x 256, 64 slices: the route applies and the sample is taken
    middle = 10.0 * torch.randn(64, K, generator=torch.Generator().manual_seed(4))
    a, b = clustered(M, middle, device, 5), clustered(N, middle, device, 6)
    out = torch.empty(N, M, device=device).t()
    assert kermac.get_l2_mode() == "auto"
    with kermac.l2_mode("gram_bf16"):
        assert workspace_bytes(a.t().contiguous().t(), b.t().contiguous().t()) > 0
    at, bt = a.t().contiguous().t(), b.t().contiguous().t()       # rows contiguous: the benchmark's storage
    got = kermac.cdist(at, bt, out=out, p=2.0)
    with kermac.l2_mode("direct"):
        plain = kermac.cdist(at, bt, p=2.0)[0]
    assert torch.equal(got, plain)
    truth = torch.cdist(a[:512].double(), b[:768].double(), p=2.0)
    assert_close_to_truth(got[:512, :768], truth, rtol=1e-5, atol=1e-30, what="clustered data")
    # and spread-out data of the same shape still takes the matrix cores (different bits than the direct kernel)
    g = torch.Generator().manual_seed(7)
    a2, b2 = torch.randn(K, M, generator=g).to(device).t(), torch.randn(K, N, generator=g).to(device).t()
    got2 = kermac.cdist(a2, b2, p=2.0)
    with kermac.l2_mode("direct"):
        plain2 = kermac.cdist(a2, b2, p=2.0)
    assert not torch.equal(got2, plain2)
    assert_close_to_truth(got2[0][:512, :768], torch.cdist(a2[:512].double(), b2[:768].double(), p=2.0), rtol=1e-5, what="spread-out data")


def test_near_duplicates_stored_cluster_by_cluster_stay_on_the_matrix_cores(device):
    """The same 64 clusters with the points stored cluster by cluster: as many pairs are near-duplicates, but they fill
    the blocks on the diagonal (one part in 64) instead of sitting in every part.  The sample tells the two apart by
    the number of sampled parts that show such a pair, the matrix-core kernel does its work, and the repair launch
    recomputes the blocks on the diagonal only: parts between different clusters carry the matrix cores' bits, parts
    inside a cluster the direct kernel's, and everything keeps the tolerance."""
    M, N, K = 8192, 8192, 1024
    middle = 10.0 * torch.randn(64, K, generator=torch.Generator().manual_seed(4))
    a = clustered(M, middle, device, 5, cluster_by_cluster=True)
    b = clustered(N, middle, device, 6, cluster_by_cluster=True)
    at, bt = a.t().contiguous().t(), b.t().contiguous().t()
    assert kermac.get_l2_mode() == "auto"
    got = kermac.cdist(at, bt, p=2.0)[0]
    with kermac.l2_mode("direct"):
        plain = kermac.cdist(at, bt, p=2.0)[0]
    same = (got == plain)
    # first cluster against first cluster: near-duplicates, recomputed by the direct kernel
    assert same[:64, :64].all()
    # first cluster against last: far apart, trusted, the matrix cores' own rounding
    assert not same[:64, -64:].all()
    assert 0.2 < (~same).float().mean().item()
    rows = torch.cat([torch.arange(0, 384), torch.arange(M - 128, M)]).to(device)
    truth = torch.cdist(a[rows].double(), b[:768].double(), p=2.0)
    assert_close_to_truth(got[rows][:, :768], truth, rtol=1e-5, atol=1e-30, what="clusters stored one after the other")


def test_a_clustered_set_against_itself_and_a_batch_of_clustered_sets(device):
    """The sample in front of the product kernel on a panel against itself (only the tiles on and below the diagonal are
    stamped; the repair launch computes them and mirrors them) and on a batch (the sampled tiles are spread over the
    entries): clustered points in any order, so everything is left to the direct kernel -- its bits, a symmetric result,
    the tolerance."""
    K = 1024
    middle = 10.0 * torch.randn(64, K, generator=torch.Generator().manual_seed(14))
    x = clustered(8192, middle, device, 15).t().contiguous().t()
    assert kermac.get_l2_mode() == "auto"
    got = kermac.cdist(x, x, p=2.0)[0]
    with kermac.l2_mode("direct"):
        plain = kermac.cdist(x, x, p=2.0)[0]
    assert torch.equal(got, plain) and torch.equal(got, got.t())
    truth = torch.cdist(x[:256].double(), x[4096:4608].double(), p=2.0)
    assert_close_to_truth(got[:256, 4096:4608], truth, rtol=1e-5, atol=1e-30, what="a clustered set against itself")

    a = torch.stack([clustered(4096, middle, device, 16 + i) for i in range(4)]).transpose(1, 2).contiguous().transpose(1, 2)
    b = torch.stack([clustered(4096, middle, device, 26 + i) for i in range(4)]).transpose(1, 2).contiguous().transpose(1, 2)
    with kermac.l2_mode("gram_bf16"):
        assert workspace_bytes(a, b) > 0
    got = kermac.cdist(a, b, p=2.0)
    with kermac.l2_mode("direct"):
        plain = kermac.cdist(a, b, p=2.0)
    assert torch.equal(got, plain)
    truth = torch.cdist(a[3, :256].double(), b[3, :256].double(), p=2.0)
    assert_close_to_truth(got[3, :256, :256], truth, rtol=1e-5, atol=1e-30, what="a batch of clustered sets")


def test_the_kept_split_is_made_again_when_it_is_not_the_one_needed(device, wide):
    """KMC_FLAG_GRAM_A_KEPT on a workspace that holds no split of this `a` (never used, used for another `a`, used by
    another route in between): the library notices from its record of the workspace and makes the split; the result is
    that of a call without the flag, bit for bit."""
    g = torch.Generator().manual_seed(41)
    a1 = torch.randn(600, 96, generator=g).to(device)
    a2 = torch.randn(600, 96, generator=g).to(device)
    b = torch.randn(500, 96, generator=g).to(device)
    stream = torch.cuda.current_stream(device).cuda_stream

    def plan_for(a):
        plan = module._plan_run_kernel(kermac.kernel_descriptor_l2_norm, a, b, None, None, None, None, None, None, None, 0, 0, False)
        plan.keepalive.append(module._attach_gram_centre(plan.params, stream, device))
        return plan

    plan1, plan2 = plan_for(a1), plan_for(a2)
    needed = _backend.gram_workspace_bytes(plan1.params)
    assert needed > 0 and needed == _backend.gram_workspace_bytes(plan2.params)
    workspace = torch.zeros(needed, dtype=torch.uint8, device=device)
    for plan in (plan1, plan2):
        plan.params.gram_workspace, plan.params.gram_workspace_bytes = workspace.data_ptr(), needed
    expected1 = kermac.cdist(a1, b, p=2.0).clone()
    expected2 = kermac.cdist(a2, b, p=2.0).clone()
    # the workspace has never held a split: the flag is set all the same
    plan1.params.flags |= _backend.FLAG_GRAM_A_KEPT
    _backend.build_kernel(plan1.params, stream)
    assert torch.equal(plan1.out, expected1)
    # now it holds the split of a1: kept for a1 (same bits), made again for a2
    plan1.out.fill_(-1.0)
    _backend.build_kernel(plan1.params, stream)
    assert torch.equal(plan1.out, expected1)
    plan2.params.flags |= _backend.FLAG_GRAM_A_KEPT
    _backend.build_kernel(plan2.params, stream)
    assert torch.equal(plan2.out, expected2)
    # another route writes into the workspace in between (the fixed-point route of absolute differences)
    l1 = module._plan_run_kernel(kermac.kernel_descriptor_l1_norm, a2, b, None, None, None, None, None, None, None, 0, 0, False)
    l1.params.flags |= _backend.FLAG_L1_FIXED | _backend.FLAG_GRAM_WORKSPACE_ANY_SIZE
    assert 0 < _backend.gram_workspace_bytes(l1.params) <= needed
    l1.params.gram_workspace, l1.params.gram_workspace_bytes = workspace.data_ptr(), needed
    _backend.build_kernel(l1.params, stream)
    plan2.out.fill_(-1.0)
    _backend.build_kernel(plan2.params, stream)
    assert torch.equal(plan2.out, expected2)
