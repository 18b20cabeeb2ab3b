"""GPU tests of the copies that let the direct kernel with b in scalar registers run on operands in any storage
(csrc/kernels/panel_copy.hip, KMC_FLAG_DIRECT_PANELS): absolute and squared differences of operands with k contiguous
(as torch allocates them), misaligned views, K and N that are not multiples of 16.  By its own rule the library makes
the copies from 5400 tiles of 256 x 64 per batch entry on; KERMAC_AMD_DIRECT_PANELS_ANY_SIZE=1 sends the small shapes
of these tests down the route, KERMAC_AMD_DIRECT_PANELS=0 keeps a call on the operands as they are.  The copies hold
the same numbers and the kernel sums them in the ordinary kernel's order (include/build_a_kernel.cuh:339-370 has one
kernel for all storage orders), so beside the oracle the tests ask for that kernel's bits.
"""
import pytest
import torch

import kermac_amd as kermac
from oracle import oracle
from tests.helpers import assert_close_to_truth, l1_distances_float64

pytestmark = pytest.mark.gpu


@pytest.fixture
def panels(monkeypatch):
    monkeypatch.setenv("KERMAC_AMD_DIRECT_PANELS_ANY_SIZE", "1")
    kermac.set_l2_mode("direct")
    yield monkeypatch
    kermac.set_l2_mode(kermac.DEFAULT_L2_MODE)


def without_copies(monkeypatch, call):
    monkeypatch.setenv("KERMAC_AMD_DIRECT_PANELS", "0")
    try:
        return call()
    finally:
        monkeypatch.delenv("KERMAC_AMD_DIRECT_PANELS")


def operand(rows, K, device, generator, k_contiguous, L=None, misaligned=False):
    """[L?, rows, K] with k contiguous or with the rows contiguous; `misaligned`: one float off a 16-byte boundary."""
    batch = () if L is None else (L,)
    shape = batch + ((rows, K) if k_contiguous else (K, rows))
    count = 1
    for extent in shape:
        count *= extent
    store = torch.randn(count + 1, generator=generator).to(device)
    x = (store[1:] if misaligned else store[:-1]).view(shape)
    return x if k_contiguous else x.transpose(-1, -2)


def truth_of(a, b, p):
    if a.dim() == 3 or b.dim() == 3:
        L = max(a.size(0) if a.dim() == 3 else 1, b.size(0) if b.dim() == 3 else 1)
        pick = lambda x, entry: x[entry] if x.dim() == 3 else x
        return torch.stack([truth_of(pick(a, entry), pick(b, entry), p) for entry in range(L)])
    if p == 1.0:
        return l1_distances_float64(a, b)
    return torch.cdist(a.double(), b.double(), p=2.0, compute_mode="donot_use_mm_for_euclid_dist")


@pytest.mark.parametrize("M,N,K", [(300, 200, 5), (256, 64, 16), (1000, 911, 70), (1, 1, 1), (3, 17, 1030), (2050, 1500, 129), (700, 2049, 256)])
@pytest.mark.parametrize("layout", ["kk", "mk", "km"])
@pytest.mark.parametrize("p", [1.0, 2.0])
def test_matches_truth_and_the_ordinary_kernel(device, panels, M, N, K, layout, p):
    g = torch.Generator().manual_seed(M + 3 * N + 7 * K)
    a = operand(M, K, device, g, layout[0] == "k")
    b = operand(N, K, device, g, layout[1] == "k")
    got = kermac.cdist(a, b, p=p)
    assert_close_to_truth(got[0], truth_of(a, b, p), rtol=1e-5, atol=1e-30, what=f"p={p} {M}x{N}x{K} {layout}")
    plain = without_copies(panels, lambda: kermac.cdist(a, b, p=p))
    assert torch.equal(got, plain), "not the ordinary kernel's bits"


@pytest.mark.parametrize("p", [3.0, 4.0])
def test_cubes_and_fourth_powers_take_the_copies_too(device, panels, p):
    g = torch.Generator().manual_seed(17)
    a, b = operand(700, 70, device, g, True), operand(333, 70, device, g, True)
    got = kermac.cdist(a, b, p=p)
    assert_close_to_truth(got[0], torch.cdist(a.double(), b.double(), p=p), rtol=1e-5, atol=1e-30, what=f"p={p}")
    assert torch.equal(got, without_copies(panels, lambda: kermac.cdist(a, b, p=p))), "not the ordinary kernel's bits"


@pytest.mark.parametrize("M,K,k_contiguous", [(700, 70, True), (1030, 48, True), (523, 20, False), (2051, 16, True)])
@pytest.mark.parametrize("p", [1.0, 2.0])
def test_a_panel_against_itself_is_copied_once(device, panels, M, K, k_contiguous, p):
    """One copy serves both sides; the kernel runs the tiles that reach the diagonal or lie below it and stores each twice:
    symmetric bit for bit, zero diagonal, the ordinary kernels' result."""
    g = torch.Generator().manual_seed(M + K)
    a = operand(M, K, device, g, k_contiguous)
    out = torch.full((M, M), float("nan"), device=device).t()
    got = kermac.cdist(a, a, out=out, p=p)
    assert not torch.isnan(got).any(), "elements left out"
    assert torch.equal(got, got.t()) and (torch.diagonal(got) == 0).all()
    assert torch.equal(got, without_copies(panels, lambda: kermac.cdist(a, a, p=p))[0]), "not the ordinary kernel's bits"
    rows = slice(0, M, 5)
    assert_close_to_truth(got[rows], truth_of(a[rows], a, p), rtol=1e-5, atol=1e-5, what=f"a against a {M}x{K}")


def test_the_route_is_taken_where_the_library_says_so(device, panels):
    """The workspace the library asks for is what the call allocates: with the cap on scratch memory at zero nothing is
    copied and the result is the same; a call whose operands the kernel takes as they are asks for nothing."""
    g = torch.Generator().manual_seed(5)
    a, b = operand(520, 48, device, g, True), operand(336, 48, device, g, True)
    before = torch.cuda.memory_stats(device)["allocation.all.allocated"]
    out = torch.empty(336, 520, device=device).t()
    allocated_for_out = torch.cuda.memory_stats(device)["allocation.all.allocated"] - before
    kermac.cdist(a, b, out=out, p=1.0)
    with_copies = torch.cuda.memory_stats(device)["allocation.all.allocated"] - before - allocated_for_out
    assert with_copies >= 1
    kermac.set_max_scratch_bytes(0)
    try:
        before = torch.cuda.memory_stats(device)["allocation.all.allocated"]
        capped = kermac.cdist(a, b, out=torch.empty_like(out.t()).t(), p=1.0)
        assert torch.cuda.memory_stats(device)["allocation.all.allocated"] - before == 1       # the result alone
    finally:
        kermac.set_max_scratch_bytes(None)
    assert torch.equal(capped, out)
    fits = operand(512, 48, device, g, False), operand(320, 48, device, g, False)
    before = torch.cuda.memory_stats(device)["allocation.all.allocated"]
    kermac.cdist(*fits, out=torch.empty(320, 512, device=device).t(), p=1.0)
    assert torch.cuda.memory_stats(device)["allocation.all.allocated"] - before == 1


def test_kernel_functions_batches_views_and_a_row_major_result(device, panels):
    """Laplace kernels with a regularised off-diagonal and per-entry bandwidths, a batch with an operand that every entry
    shares, misaligned views, and a result with n contiguous (the operands change sides); against the oracle, float64
    and the ordinary kernel."""
    g = torch.Generator().manual_seed(11)
    L, M, N, K = 3, 530, 340, 52
    a = operand(M, K, device, g, True, L=L)
    b = operand(N, K, device, g, True, misaligned=True)
    bandwidth = torch.tensor([3.0, 7.0, 1.5], device=device)
    for descriptor, names in ((kermac.kernel_descriptor_laplace_l1, ("DIFF", "ABS", "NOOP", "LAPLACE")),
                              (kermac.kernel_descriptor_laplace_l2, ("DIFF", "SQUARE", "SQRT", "LAPLACE"))):
        def call():
            return kermac.run_kernel(descriptor, a, b, bandwidth=bandwidth, regularization=0.25, regularization_offset_x=3,
                                     regularization_offset_y=1)
        got = call()
        truth = oracle.run_kernel(*names, a.cpu(), b.cpu(), bandwidth=bandwidth.cpu(), regularization=0.25,
                                  regularization_offset_x=3, regularization_offset_y=1)
        assert_close_to_truth(got, truth, rtol=1e-5, atol=1e-7, what=str(descriptor))
        assert torch.equal(got, without_copies(panels, call)), "not the ordinary kernel's bits"
    a2, b2 = operand(M, K, device, g, False, misaligned=True), operand(N, K, device, g, True)
    out = torch.empty(M, N, device=device)
    got = kermac.cdist(a2, b2, out=out, p=1.0)
    assert got.data_ptr() == out.data_ptr()
    assert_close_to_truth(got, truth_of(a2, b2, 1.0), rtol=1e-5, atol=1e-30, what="row-major result")
    assert torch.equal(got, without_copies(panels, lambda: kermac.cdist(a2, b2, out=torch.empty(M, N, device=device), p=1.0)))


def test_large_problem_by_the_librarys_own_rule(device):
    """10000 x 10008 x 200 with k contiguous is above the rule's size (5400 tiles per entry): the copies are made without
    any switch, and the result is the direct kernel's."""
    g = torch.Generator().manual_seed(3)
    a, b = operand(10000, 200, device, g, True), operand(10008, 200, device, g, True)
    before = torch.cuda.memory_stats(device)["allocation.all.allocated"]
    got = kermac.cdist(a, b, p=1.0)
    assert torch.cuda.memory_stats(device)["allocation.all.allocated"] - before == 2       # the result and the copies
    sample = slice(0, 10000, 131)
    assert_close_to_truth(got[0, sample], l1_distances_float64(a[sample], b), rtol=1e-5, atol=1e-30, what="10000 x 10008 x 200")


def test_random_calls_with_both_variants_forced(device, monkeypatch):
    """300 seeded random calls -- shapes around the tile edges, both storage orders, misaligned views, batches with shared
    operands, a set against itself, row-major results, Laplace kernels with an offset diagonal -- once with the copies and the
    kernel with b in scalar registers forced wherever they can run, once with both switched off: the same bits, no NaN."""
    import random
    rng = random.Random(20240521)
    g = torch.Generator().manual_seed(99)
    kermac.set_l2_mode("direct")
    try:
        for case in range(300):
            M = rng.choice([1, 3, 64, 255, 256, 257, 300, 512, 777, 1024, 1500, 2049])
            N = rng.choice([1, 16, 17, 48, 64, 65, 100, 256, 300, 640, 1000])
            K = rng.choice([1, 5, 16, 17, 32, 48, 100, 128, 130])
            L = rng.choice([None, None, 2, 3])
            p = rng.choice([1.0, 2.0])
            same = rng.random() < 0.15
            shared_a = L is not None and rng.random() < 0.2
            shared_b = L is not None and not shared_a and rng.random() < 0.2
            a = operand(M, K, device, g, rng.random() < 0.5, L=None if shared_a else L, misaligned=rng.random() < 0.2)
            b = a if same else operand(N, K, device, g, rng.random() < 0.5, L=None if shared_b else L, misaligned=rng.random() < 0.2)
            columns = M if same else N
            row_major_out = L is None and rng.random() < 0.3
            laplace = rng.random() < 0.5
            offsets = (0, 0) if same else (rng.choice([0, 0, 2]), rng.choice([0, 0, 1]))

            def call():
                if laplace:
                    descriptor = kermac.kernel_descriptor_laplace_l1 if p == 1.0 else kermac.kernel_descriptor_laplace_l2
                    return kermac.run_kernel(descriptor, a, b, bandwidth=3.0, regularization=0.5, regularization_offset_x=offsets[0],
                                             regularization_offset_y=offsets[1])
                out = torch.full((M, columns), float("nan"), device=device) if row_major_out else None
                return kermac.cdist(a, b, p=p, out=out)

            monkeypatch.setenv("KERMAC_AMD_DIRECT_PANELS_ANY_SIZE", "1")
            monkeypatch.setenv("KERMAC_AMD_SCALAR_B_MIN_TILES", "1")
            forced = call()
            monkeypatch.delenv("KERMAC_AMD_DIRECT_PANELS_ANY_SIZE")
            monkeypatch.setenv("KERMAC_AMD_SCALAR_B_MIN_TILES", "2000000000")
            monkeypatch.setenv("KERMAC_AMD_DIRECT_PANELS", "0")
            plain = call()
            monkeypatch.delenv("KERMAC_AMD_DIRECT_PANELS")
            what = f"case {case}: {M} x {columns} x {K}, L = {L}, p = {p}, a against itself {same}, laplace {laplace}"
            assert not torch.isnan(forced).any(), what
            assert torch.equal(forced, plain), what
    finally:
        kermac.set_l2_mode(kermac.DEFAULT_L2_MODE)
