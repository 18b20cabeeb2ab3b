"""GPU tests of the opt-in fixed-point route for sums of absolute differences (include/kermac_amd.h,
KMC_FLAG_L1_FIXED; kermac.set_l1_mode("fixed")): both operands rounded once to a common power-of-two
grid, |qb - qa| summed exactly on integers, every element whose relative error bound exceeds 8e-6
recomputed (its 128 x 128 tile) by the direct fp32 kernel.  Stated tolerance: the 1e-5 of every p = 1
path, relative to the float64 truth.

KERMAC_AMD_L1_FIXED_ANY_SIZE=1 sends the small shapes of these tests down the route, which by itself only
takes problems of at least 2048 tiles of 128 x 128 with K >= 128.
"""
import pytest
import torch

import kermac_amd as kermac
from kermac_amd import _backend, build_a_kernel as module
from oracle import oracle
from tests.helpers import assert_close_to_truth, make_operand, l1_distances_float64

pytestmark = pytest.mark.gpu


@pytest.fixture
def fixed(monkeypatch):
    monkeypatch.setenv("KERMAC_AMD_L1_FIXED_ANY_SIZE", "1")
    kermac.set_l1_mode("fixed")
    yield
    kermac.set_l1_mode(kermac.DEFAULT_L1_MODE)


def direct(fn):
    with kermac.l1_mode("direct"):
        return fn()


def workspace_bytes(a, b, descriptor=kermac.kernel_descriptor_l1_norm, **kw):
    plan = module._plan_run_kernel(descriptor, a, b, None, None, None, None, kw.get("bandwidth"), None, None, 0, 0, False)
    return _backend.gram_workspace_bytes(plan.params)


@pytest.mark.parametrize("M,N,K", [(300, 260, 96), (515, 770, 70), (1000, 900, 200), (257, 255, 33), (256, 512, 1024),
                                   (1, 700, 64), (640, 3, 48), (300, 200, 5), (128, 128, 16), (513, 257, 1),
                                   (260, 130, 1030), (200, 300, 2500)])
@pytest.mark.parametrize("layout", ["cc", "rr", "cr", "rc"])
def test_random_data_matches_truth(device, fixed, M, N, K, layout):
    """All three grid widths (26, 24 and 22 bits), contractions longer than one accumulator holds (1030, 2500:
    partial sums through the result), ragged tiles, every storage order of operands and result."""
    g = torch.Generator().manual_seed(M + 3 * N + 7 * K)
    a = make_operand(1, M, K, layout[0] == "c", device, g, batch=False)
    b = make_operand(1, N, K, layout[1] == "c", device, g, batch=False)
    assert workspace_bytes(a, b) > 0
    truth = oracle.cdist(a.cpu(), b.cpu(), p=1.0)[0]
    for c_col in (False, True):
        out = torch.empty(N, M, device=device).t() if c_col else torch.empty(M, N, device=device)
        got = kermac.cdist(a, b, out=out, p=1.0)
        assert_close_to_truth(got, truth, rtol=1e-5, what=f"fixed {M}x{N}x{K} {layout} out col-major={c_col}")


def test_the_route_is_the_one_that_ran(device, fixed):
    """On spread-out data nothing is distrusted, so the result is the integer sum: exact up to the rounding of
    the operands, and not the bits of the fp32 kernel, whose own rounding at K = 1024 is ten times larger."""
    g = torch.Generator().manual_seed(5)
    a, b = torch.randn(384, 1024, generator=g).to(device), torch.randn(256, 1024, generator=g).to(device)
    got = kermac.cdist(a, b, p=1.0)
    plain = direct(lambda: kermac.cdist(a, b, p=1.0))
    truth = l1_distances_float64(a, b)
    assert not torch.equal(got, plain)
    fixed_err = ((got.double() - truth).abs() / truth).max().item()
    direct_err = ((plain.double() - truth).abs() / truth).max().item()
    assert fixed_err < 5e-7, fixed_err
    assert fixed_err < direct_err, (fixed_err, direct_err)


def test_when_the_route_applies(device):
    a = torch.empty(7000, 512, device=device)
    b = torch.empty(6000, 512, device=device)
    with kermac.l1_mode("fixed"):
        needed = workspace_bytes(a, b)                                           # 55 x 47 tiles
        padded = (7040 + 6016) * 512 * 4
        assert padded <= needed <= padded + 1024
        assert workspace_bytes(a, b, kermac.kernel_descriptor_laplace_l1, bandwidth=2.0) == needed
        assert workspace_bytes(a, b, kermac.kernel_descriptor_l2_norm) != needed   # squared differences: not this route
        assert workspace_bytes(a[:5000], b[:5000]) == 0                          # 40 x 40 tiles
        assert workspace_bytes(a[:, :100], b[:, :100]) == 0                      # k < 128
        assert workspace_bytes(a[:3000].expand(4, 3000, 512), b[:3000].expand(4, 3000, 512)) > 0    # 2304 tiles over the batch
        big = torch.empty(9000, 512, device=device)
        assert 0 < workspace_bytes(big, big) < 0.6 * workspace_bytes(big, big.clone())   # 2556 tiles of the triangle; one panel, converted once
        assert workspace_bytes(a, a) == 0                                        # 1540 tiles of the triangle
    with kermac.l1_mode("direct"):
        assert workspace_bytes(a, b) == 0


def test_without_a_workspace_the_direct_kernel_runs(device, fixed):
    g = torch.Generator().manual_seed(2)
    a = torch.randn(700, 96, generator=g).to(device)
    b = torch.randn(600, 96, generator=g).to(device)
    reference = direct(lambda: kermac.cdist(a, b, p=1.0))
    plan = module._plan_run_kernel(kermac.kernel_descriptor_l1_norm, a, b, None, None, None, None, None, None, None, 0, 0, False)
    stream = torch.cuda.current_stream(device).cuda_stream
    needed = _backend.gram_workspace_bytes(plan.params)
    assert needed > 0
    workspace = torch.empty(needed, dtype=torch.uint8, device=device)
    for pointer, size in ((0, 0), (workspace.data_ptr(), needed - 1), (workspace.data_ptr() + 16, needed)):
        plan.out.fill_(-1.0)
        plan.params.gram_workspace, plan.params.gram_workspace_bytes = pointer, size
        _backend.build_kernel(plan.params, stream)
        assert torch.equal(plan.out, reference), "null, short or misaligned workspace: expected the direct kernel's bits"
    plan.params.gram_workspace, plan.params.gram_workspace_bytes = workspace.data_ptr(), needed
    _backend.build_kernel(plan.params, stream)
    assert not torch.equal(plan.out, reference)
    assert_close_to_truth(plan.out, oracle.cdist(a.cpu(), b.cpu(), p=1.0), rtol=1e-5, what="with the workspace")


def test_near_duplicates_are_recomputed_directly(device, fixed):
    """Points that differ by 1e-6 of the data range: their distances are a few grid steps, the tiles that hold
    them come from the direct kernel (bit-equal to it), the others from the integer sums."""
    g = torch.Generator().manual_seed(11)
    M, N, K = 512, 384, 300
    a = torch.randn(M, K, generator=g)
    b = torch.randn(N, K, generator=g)
    b[:100] = a[50:150] + 1e-6 * torch.randn(100, K, generator=g)      # tiles (0, 0) and (1, 0) of the [M, N] result
    a, b = a.to(device), b.to(device)
    out = torch.empty(N, M, device=device).t()
    got = kermac.cdist(a, b, out=out, p=1.0)
    plain = direct(lambda: kermac.cdist(a, b, p=1.0))[0]
    assert torch.equal(got[:256, :128], plain[:256, :128])
    assert not torch.equal(got[256:, 128:], plain[256:, 128:])
    assert_close_to_truth(got, l1_distances_float64(a, b), rtol=1e-5, what="near-duplicates")


def test_identical_points_and_a_set_against_itself(device, fixed):
    g = torch.Generator().manual_seed(12)
    x = torch.randn(700, 200, generator=g).to(device)
    got = kermac.cdist(x, x, p=1.0)[0]
    assert torch.equal(got, got.t()), "a set against itself is symmetric bit for bit"
    assert torch.all(torch.diagonal(got) == 0.0)
    assert_close_to_truth(got, l1_distances_float64(x, x), rtol=1e-5, what="x against x")
    other = kermac.cdist(x, x.clone(), p=1.0)[0]
    assert_close_to_truth(other, l1_distances_float64(x, x), rtol=1e-5, what="x against a copy of x")


def test_outliers_and_values_that_are_not_numbers(device, fixed):
    """One huge value stretches the grid until nothing can be trusted: the sample of pairs says so and the whole
    result is the direct kernel's.  A NaN or an infinity in the data likewise."""
    g = torch.Generator().manual_seed(13)
    a = torch.randn(400, 256, generator=g).to(device)
    b = torch.randn(300, 256, generator=g).to(device)
    for value in (1e9, float("inf"), float("nan")):
        spoiled = a.clone()
        spoiled[17, 5] = value
        got = kermac.cdist(spoiled, b, p=1.0)
        plain = direct(lambda: kermac.cdist(spoiled, b, p=1.0))
        assert torch.equal(torch.nan_to_num(got, nan=-1.0), torch.nan_to_num(plain, nan=-1.0)), value
    zeros = torch.zeros(300, 256, device=device)
    assert torch.equal(kermac.cdist(zeros, zeros.clone(), p=1.0)[0], torch.zeros(300, 300, device=device))


def test_rows_of_very_different_magnitude(device, fixed):
    """One grid for the whole batch entry: rows far below the largest magnitude have distances of few grid steps and
    are recomputed; the tolerance holds everywhere."""
    g = torch.Generator().manual_seed(9)
    M, N, K = 520, 390, 150
    a = torch.randn(M, K, generator=g) * torch.pow(2.0, -(torch.arange(M) // 130 * 9).float())[:, None]
    b = torch.randn(N, K, generator=g) * torch.pow(2.0, -(torch.arange(N) // 130 * 9).float())[:, None]
    a, b = a.to(device), b.to(device)
    got = kermac.cdist(a, b, p=1.0)[0]
    assert_close_to_truth(got, l1_distances_float64(a, b), rtol=1e-5, what="rows spread over 27 binades")


def test_batches_kernels_and_offsets(device, fixed):
    """Laplace kernel on L1 distances, a batch with a broadcast operand and a scale per entry, per-entry bandwidth,
    regularised off-diagonal; against the oracle."""
    g = torch.Generator().manual_seed(21)
    L, M, N, K = 3, 300, 280, 140
    a = make_operand(L, M, K, True, device, g) * torch.tensor([1.0, 100.0, 0.01], device=device)[:, None, None]
    b = make_operand(1, N, K, False, device, g, batch=False)
    bandwidth = torch.tensor([3.0, 200.0, 1.5], device=device)
    got = kermac.run_kernel(kermac.kernel_descriptor_laplace_l1, a, b, bandwidth=bandwidth, regularization=0.5,
                            regularization_offset_x=3, regularization_offset_y=1)
    truth = oracle.run_kernel("DIFF", "ABS", "NOOP", "LAPLACE", a.cpu(), b.cpu(), bandwidth=bandwidth.cpu(), regularization=0.5,
                              regularization_offset_x=3, regularization_offset_y=1)
    assert_close_to_truth(got, truth, rtol=1e-5, atol=1e-7, what="laplace, batch of 3")


def test_the_sample_tells_near_duplicates_everywhere_from_near_duplicates_in_few_tiles(device):
    """4096 tiles by the route's own rule.  Points drawn around 64 centres in any order: every tile holds pairs whose
    distance is a few grid steps, the sample sees them spread over its tiles, the conversion and the walk do nothing and
    the result is the direct kernel's.  The same points stored cluster by cluster: those pairs fill the blocks on the
    diagonal, one tile in 64, the walk runs and only those blocks are recomputed.  Every other feature constant: one
    pair in two thousand just below the threshold, spread evenly -- eight per tile -- and the call is left to the
    direct kernel as well.  The tolerance holds in all three."""
    M = N = 8192
    K = 512
    g = torch.Generator().manual_seed(33)
    middle = 10.0 * torch.randn(64, K, generator=g)

    def clustered(rows, cluster_by_cluster):
        which = torch.randint(0, 64, (rows,), generator=g)
        if cluster_by_cluster:
            which = which.sort().values
        return (middle[which] + 1e-3 * torch.randn(rows, K, generator=g)).to(device).t().contiguous().t()

    def both(a, b):
        with kermac.l1_mode("fixed"):
            assert workspace_bytes(a, b) > 0         # the route applies by its own rule
            got = kermac.cdist(a, b, p=1.0)[0]
        return got, direct(lambda: kermac.cdist(a, b, p=1.0))[0]

    a, b = clustered(M, False), clustered(N, False)
    got, plain = both(a, b)
    assert torch.equal(got, plain)
    assert_close_to_truth(got[:200, :300], l1_distances_float64(a[:200], b[:300]), rtol=1e-5, atol=1e-30, what="clusters in any order")

    a, b = clustered(M, True), clustered(N, True)
    got, plain = both(a, b)
    same = got == plain
    assert same[:32, :32].all() and not same[:64, -64:].all() and (~same).float().mean().item() > 0.2
    rows = torch.cat([torch.arange(0, 150), torch.arange(M - 50, M)]).to(device)
    assert_close_to_truth(got[rows][:, :300], l1_distances_float64(a[rows], b[:300]), rtol=1e-5, atol=1e-30, what="clusters one after the other")

    a = torch.randn(K, M, generator=g); a[::2] = 3.0
    b = torch.randn(K, N, generator=g); b[::2] = 3.0
    a, b = a.to(device).t(), b.to(device).t()
    got, plain = both(a, b)
    assert torch.equal(got, plain)
    assert_close_to_truth(got[:200, :300], l1_distances_float64(a[:200], b[:300]), rtol=1e-5, what="every other feature constant")


def test_a_tighter_tolerance_repairs_more(device, monkeypatch):
    monkeypatch.setenv("KERMAC_AMD_L1_FIXED_ANY_SIZE", "1")
    g = torch.Generator().manual_seed(3)
    a, b = torch.randn(256, 256, generator=g).to(device), torch.randn(256, 256, generator=g).to(device)
    plain = kermac.cdist(a, b, p=1.0)
    with kermac.l1_mode("fixed", tolerance=1e-7):       # 24 bits cannot promise that at K = 256: everything is recomputed
        assert torch.equal(kermac.cdist(a, b, p=1.0), plain)
    with kermac.l1_mode("fixed"):
        assert not torch.equal(kermac.cdist(a, b, p=1.0), plain)


@pytest.mark.parametrize("rows_contiguous", [True, False])
def test_full_size(device, rows_contiguous):
    """BASELINE's cdist p = 1 problem by the route's own rule (no size override): float64 slabs, 1e-5."""
    M = N = 30000
    K = 1024
    torch.manual_seed(1)
    if rows_contiguous:
        a, b = torch.randn(K, M, device=device).t(), torch.randn(K, N, device=device).t()
    else:
        a, b = torch.randn(M, K, device=device), torch.randn(N, K, device=device)
    out = torch.empty(N, M, device=device).t()
    with kermac.l1_mode("fixed"):
        assert workspace_bytes(a, b) > 0
        kermac.cdist(a, b, out=out, p=1.0)
    for ms, ns in ((slice(0, 256), slice(0, 2048)), (slice(29900, 30000), slice(29744, 30000)), (slice(15000, 15100), slice(7, 1000))):
        truth = l1_distances_float64(a[ms], b[ns])
        err = ((out[ms, ns].double() - truth).abs() / truth).max().item()
        assert err < 1e-6, err          # nothing is distrusted on this data; the integer sums are ten times closer than fp32
