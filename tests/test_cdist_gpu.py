"""GPU parity tests of cdist / run_kernel against the CPU oracle (float64 mode),
the golden vectors and torch.cdist.  Every call goes through the public operator,
i.e. through the C ABI of libkermac_amd.so.

Tolerances (relative to the float64 truth): 1e-5 for p = 1 and p = 2, 1e-4 for
fractional p, as the acceptance criteria of this path state.
"""
from itertools import product
from pathlib import Path

import numpy as np
import pytest
import torch

import kermac_amd as kermac
from oracle import oracle
from tests.helpers import assert_close_to_truth, make_operand

pytestmark = pytest.mark.gpu

GOLDEN = np.load(Path(__file__).resolve().parent / "golden" / "hot_path_vectors.npz")
RTOL = {1.0: 1e-5, 2.0: 1e-5}


def rtol_for(p):
    return RTOL.get(p, 1e-4)


def G(name, device):
    return torch.from_numpy(GOLDEN[name]).to(device)


@pytest.mark.parametrize("p", [1.0, 1.3, 2.0, 0.5, 3.0])
@pytest.mark.parametrize("skip", [False, True])
def test_cdist_golden_vectors(device, p, skip):
    a, b = G("a", device), G("b", device)
    got = kermac.cdist(a, b, p=p, skip_epilogue=skip)
    truth = GOLDEN[f"cdist_p{p}" + ("_skip" if skip else "")]
    assert_close_to_truth(got, torch.from_numpy(truth), rtol=rtol_for(p), what=f"cdist golden p={p} skip={skip}")


@pytest.mark.parametrize("a_col,b_col,c_col", list(product([False, True], repeat=3)))
@pytest.mark.parametrize("p", [1.0, 1.3, 2.0])
@pytest.mark.parametrize("try_to_align", [False, True])
def test_cdist_transposes(device, a_col, b_col, c_col, p, try_to_align):
    """The reference's own test matrix (tests/test_cdist.py:48-88): L=2, M=N=1000,
    K=64, all 8 majorness combinations x 3 p x try_to_align, against torch.cdist
    with its RMSE / max-abs < 1e-4 criterion, plus the oracle at 1e-5 / 1e-4."""
    g = torch.Generator().manual_seed(1000 + 4 * a_col + 2 * b_col + c_col)
    L, M, N, K = 2, 1000, 1000, 64
    a = make_operand(L, M, K, a_col, device, g)
    b = make_operand(L, N, K, b_col, device, g)
    c = make_operand(L, M, N, c_col, device, g)
    out = kermac.cdist(a, b, p=p, out=c, skip_epilogue=False, try_to_align=try_to_align)
    assert out is c
    torch_out = torch.cdist(a, b, p=p)
    diff = out - torch_out
    assert torch.sqrt(torch.mean(diff ** 2)).item() < 1e-4
    assert diff.abs().max().item() < 1e-4
    truth = oracle.cdist(a.cpu(), b.cpu(), p=p)
    assert_close_to_truth(out, truth, rtol=rtol_for(p), what=f"cdist vs oracle p={p}")


@pytest.mark.parametrize("M,N,K", [(1, 1, 1), (5, 3, 2), (128, 128, 16), (129, 127, 17), (130, 260, 6), (300, 70, 33),
                                   (64, 513, 1), (257, 1, 40)])
@pytest.mark.parametrize("p", [1.0, 2.0, 1.7])
def test_cdist_ragged_shapes_and_k_residue(device, M, N, K, p):
    g = torch.Generator().manual_seed(M * 7 + N * 3 + K)
    for a_col, b_col in ((True, True), (False, False), (True, False)):
        a = make_operand(1, M, K, a_col, device, g, batch=False)
        b = make_operand(1, N, K, b_col, device, g, batch=False)
        out = kermac.cdist(a, b, p=p)
        assert out.shape == (1, M, N)
        truth = oracle.cdist(a.cpu(), b.cpu(), p=p)
        assert_close_to_truth(out, truth, rtol=rtol_for(p), what=f"ragged {M}x{N}x{K} p={p} {a_col}{b_col}")


def test_cdist_misaligned_and_padded_operands(device):
    g = torch.Generator().manual_seed(77)
    M, N, K = 200, 150, 37
    # pointer 4 bytes past a 16-byte boundary, leading dimension not a multiple of 4
    flat = torch.randn(K * (M + 3) + 1, generator=g).to(device)
    a = flat[1:].view(K, M + 3)[:, :M].t()                  # column-major, ld = M + 3, misaligned base
    b_store = torch.randn(N, K + 5, generator=g).to(device)
    b = b_store[:, 2:2 + K]                                 # row-major, ld = K + 5, misaligned base
    out_store = torch.full((N, M + 1), -1.0, device=device)
    out = out_store[:, :M].t()                              # column-major out with padding column
    for p in (1.0, 2.0, 1.3):
        got = kermac.cdist(a, b, p=p, out=out)
        truth = oracle.cdist(a.cpu(), b.cpu(), p=p)
        assert_close_to_truth(got, truth[0], rtol=rtol_for(p), what=f"misaligned p={p}")
        assert torch.all(out_store[:, M] == -1.0), "wrote outside the out view"


def test_cdist_broadcast_batches_and_out_none(device):
    g = torch.Generator().manual_seed(78)
    L, M, N, K = 3, 140, 90, 20
    a = make_operand(L, M, K, True, device, g)
    b = make_operand(1, N, K, True, device, g, batch=False)   # shared by all batches
    out = kermac.cdist(a, b, p=1.0)
    assert out.shape == (L, M, N) and out.dtype == torch.float32
    truth = oracle.cdist(a.cpu(), b.cpu(), p=1.0)
    assert_close_to_truth(out, truth, rtol=1e-5, what="broadcast b")
    b1 = b.unsqueeze(0)                                        # explicit batch of 1 also broadcasts
    assert torch.equal(kermac.cdist(a, b1, p=1.0), out)
    out2 = torch.empty(L, M, N, device=device)
    assert kermac.cdist(a[0], b, p=2.0, out=out2) is out2      # out's batch makes L = 3
    truth = oracle.cdist(a[0].cpu(), b.cpu(), p=2.0)
    assert_close_to_truth(out2, truth.expand(L, -1, -1), rtol=1e-5, what="out-driven batch")


def test_cdist_empty_and_degenerate(device):
    a = torch.zeros(0, 5, device=device)
    b = torch.zeros(7, 5, device=device)
    assert kermac.cdist(a, b).shape == (1, 0, 7)
    assert kermac.cdist(b, a).shape == (1, 7, 0)
    # K = 0: empty sums
    a0, b0 = torch.zeros(4, 0, device=device), torch.zeros(6, 0, device=device)
    assert torch.all(kermac.cdist(a0, b0, p=1.0) == 0)
    # identical points: exact zeros, symmetric result
    x = torch.randn(150, 40, device=device)
    for p in (1.0, 2.0):
        d = kermac.cdist(x, x, p=p)[0]
        assert torch.all(torch.diagonal(d) == 0)
        assert torch.equal(d, d.t())


def test_cdist_skip_epilogue_does_not_leak_between_calls(device):
    g = torch.Generator().manual_seed(79)
    a = make_operand(1, 60, 12, False, device, g, batch=False)
    b = make_operand(1, 50, 12, False, device, g, batch=False)
    for p in (2.0, 1.3):
        plain_before = kermac.cdist(a, b, p=p).clone()
        skipped = kermac.cdist(a, b, p=p, skip_epilogue=True)
        plain_after = kermac.cdist(a, b, p=p)
        assert torch.equal(plain_before, plain_after)
        assert_close_to_truth(skipped, plain_before.double() ** p, rtol=2e-5 if p == 2.0 else 2e-4,
                              what=f"skip_epilogue p={p}")


def test_cdist_runs_on_the_current_stream(device):
    g = torch.Generator().manual_seed(80)
    a = make_operand(1, 500, 64, True, device, g, batch=False)
    b = make_operand(1, 400, 64, True, device, g, batch=False)
    side = torch.cuda.Stream(device=device)
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        a2 = a * 2.0                                           # produced on the side stream
        out = kermac.cdist(a2, b * 2.0, p=1.0)                 # must be ordered after it
    side.synchronize()
    assert_close_to_truth(out, 2.0 * oracle.cdist(a.cpu(), b.cpu(), p=1.0), rtol=1e-5, what="side stream")


# ------------------------------------------------------------------- run_kernel

def test_run_kernel_golden_kernel_functions(device):
    a, b = G("a", device), G("b", device)
    got = kermac.run_kernel(kermac.kernel_descriptor_laplace_l1, a, b, bandwidth=3.0)
    assert_close_to_truth(got, torch.from_numpy(GOLDEN["laplace_l1_bw3"]), rtol=1e-5, what="laplace l1")
    got = kermac.run_kernel(kermac.kernel_descriptor_laplace_l2, a, b, bandwidth=3.0)
    assert_close_to_truth(got, torch.from_numpy(GOLDEN["laplace_l2_bw3"]), rtol=1e-5, what="laplace l2")
    gaussian = kermac.KernelDescriptor(kermac.InnerOperator.DIFF, kermac.PowerType.SQUARE, kermac.PowerType.NOOP,
                                       kermac.KernelType.GAUSSIAN)
    got = kermac.run_kernel(gaussian, a, b, bandwidth=3.0)
    assert_close_to_truth(got, torch.from_numpy(GOLDEN["gaussian_sq_bw3"]), rtol=1e-5, what="gaussian")
    got = kermac.run_kernel(kermac.kernel_descriptor_mma, a, b)
    assert_close_to_truth(got, torch.from_numpy(GOLDEN["dot"]), rtol=1e-5, atol=1e-5, what="dot")
    x = a[0]
    got = kermac.run_kernel(kermac.kernel_descriptor_laplace_l1, x, x, bandwidth=3.0, regularization=0.25)[0]
    assert_close_to_truth(got, torch.from_numpy(GOLDEN["laplace_l1_self_bw3_reg0.25"]), rtol=1e-5, what="regularised")
    for c_col in (False, True):
        out = torch.empty(x.shape[0], x.shape[0], device=device)
        out = out.t() if c_col else out
        got = kermac.run_kernel(kermac.kernel_descriptor_laplace_l1, x, x, out=out, bandwidth=3.0, regularization=0.25,
                                regularization_offset_x=3, regularization_offset_y=1)
        # The reference's examples/broadcast_kernel.py passes offsets (3, 1) with out=None: its
        # row-major result has 1 + regularization where 3 + n == 1 + m, i.e. at [n + 2, n], below
        # the diagonal (the golden vector holds the kernel-level position [m, m + 2]; x against
        # x is symmetric elsewhere, so the expected matrix is its transpose).  Same for every out.
        assert_close_to_truth(got, torch.from_numpy(GOLDEN["laplace_l1_self_bw3_reg0.25_off3_1"]).t(), rtol=1e-5,
                              what=f"offset diagonal, out col-major={c_col}")
        assert got[2, 0].item() == 1.25 and got[0, 2].item() < 1.0


def test_run_kernel_batched_hyper_parameters(device):
    """examples/broadcast_kernel.py of the reference: per-batch p / bandwidth /
    regularisation tensors, K = 6 (K residue), a tiled diagonal."""
    g = torch.Generator().manual_seed(81)
    N, K = 333, 6
    data = torch.randn(N, K, generator=g).to(device)
    desc = kermac.KernelDescriptor(kermac.InnerOperator.DIFF, kermac.PowerType.POW, kermac.PowerType.POW,
                                   kermac.KernelType.LAPLACE)
    p = torch.tensor([0.5, 0.6, 0.7, 2.0], device=device)
    bw = torch.tensor(10.0, device=device)
    reg = torch.tensor([1e-3, 1e-2, 1e-1, 1.0], device=device)
    out = kermac.run_kernel(desc, data, data, p=p, bandwidth=bw, regularization=reg)
    assert out.shape == (4, N, N)
    truth = oracle.build_kernel("DIFF", "POW", "POW", "LAPLACE", data.cpu(), data.cpu(), p_inner=p.cpu(),
                                p_outer=(1.0 / p).cpu(), bandwidth=10.0, regularization=reg.cpu())
    assert_close_to_truth(out, truth, rtol=1e-4, what="per-batch p and regularisation")
    bw2 = torch.tensor([10.0, 20.0], device=device)
    out = kermac.run_kernel(kermac.kernel_descriptor_laplace_l2, data, data, bandwidth=bw2, regularization=10.0,
                            regularization_offset_x=3, regularization_offset_y=1)
    truth = oracle.run_kernel("DIFF", "SQUARE", "SQRT", "LAPLACE", data.cpu(), data.cpu(), bandwidth=bw2.cpu(),
                              regularization=10.0, regularization_offset_x=3, regularization_offset_y=1)
    assert out.shape == (2, N, N)
    assert_close_to_truth(out, truth, rtol=1e-5, what="per-batch bandwidth, offset diagonal")
    # independent inner / outer powers (examples/build_a_kernel.py: Gaussian p-norm)
    gp = kermac.KernelDescriptor(kermac.InnerOperator.DIFF, kermac.PowerType.POW, kermac.PowerType.POW,
                                 kermac.KernelType.GAUSSIAN)
    out = kermac.run_kernel(gp, data, data, inner_p=1.3, outer_p=1.0 / 1.3, bandwidth=10.0)
    truth = oracle.build_kernel("DIFF", "POW", "POW", "GAUSSIAN", data.cpu(), data.cpu(), p_inner=1.3,
                                p_outer=1.0 / 1.3, bandwidth=10.0)
    assert_close_to_truth(out, truth, rtol=1e-4, what="gaussian p-norm")


@pytest.mark.parametrize("p", [0.5, 1.5, 3.0, 4.0])
def test_scalar_exponents_with_exact_forms(device, p):
    """A float exponent of 0.5, 1.5, 3 or 4 is evaluated as sqrt|x|, |x| sqrt|x|,
    |x| x^2, (x^2)^2 inside the library; the same exponent as a tensor takes the
    generic exp2(p log2|x|).  Both must meet the fractional-p tolerance against the
    float64 oracle, for every layout, ragged shapes, zeros and the kernel epilogues."""
    g = torch.Generator().manual_seed(int(p * 10) + 83)
    for (M, N, K), a_col, b_col in (((300, 170, 70), True, True), ((129, 257, 33), False, False),
                                    ((64, 200, 16), True, False)):
        a = make_operand(1, M, K, a_col, device, g, batch=False)
        b = make_operand(1, N, K, b_col, device, g, batch=False)
        b[:3] = a[:3]                                                # exact zeros among the differences
        truth = oracle.cdist(a.cpu(), b.cpu(), p=p)
        special = kermac.cdist(a, b, p=p)
        assert_close_to_truth(special, truth, rtol=1e-4, what=f"exact form p={p} {M}x{N}x{K}")
        generic = kermac.run_kernel(kermac.kernel_descriptor_p_norm, a, b, p=torch.tensor(p, device=device))
        assert_close_to_truth(generic, truth, rtol=1e-4, what=f"generic power p={p}")
        assert_close_to_truth(special, generic.double(), rtol=2e-5, what=f"exact form vs generic p={p}")
        skipped = kermac.cdist(a, b, p=p, skip_epilogue=True)
        assert_close_to_truth(skipped, truth.double() ** p, rtol=1e-4, what=f"skip_epilogue p={p}")
    desc = kermac.KernelDescriptor(kermac.InnerOperator.DIFF, kermac.PowerType.POW, kermac.PowerType.POW,
                                   kermac.KernelType.LAPLACE)
    out = kermac.run_kernel(desc, a, b, p=p, bandwidth=5.0)
    truth = oracle.build_kernel("DIFF", "POW", "POW", "LAPLACE", a.cpu(), b.cpu(), p_inner=p, p_outer=1.0 / p,
                                bandwidth=5.0)
    # exp(-d / bw) turns a relative error of d into d / bw times as much: absolute floor for tiny values
    assert_close_to_truth(out, truth, rtol=1e-4, atol=1e-7, what=f"laplace on the {p}-norm")


def test_run_kernel_epsilon_mask(device):
    a = torch.zeros(1, 2, device=device)
    b = torch.tensor([[1e-6, 0.0], [1.0, 0.0]], device=device)
    out = kermac.run_kernel(kermac.kernel_descriptor_laplace_l1, a, b, bandwidth=1.0)[0]
    assert out[0, 0].item() == 1.0
    assert out[0, 1].item() == pytest.approx(np.exp(-1.0), rel=1e-6)
    out = kermac.run_kernel(kermac.kernel_descriptor_laplace_l1, a, b, bandwidth=1.0, epsilon=1e-9)[0]
    assert out[0, 0].item() == pytest.approx(np.exp(-1e-6), rel=1e-6) and out[0, 0].item() < 1.0


def test_signed_inner_operator_with_row_major_out(device):
    # DIFF + NOOP is sign sensitive: a[m] - b[n], what the reference returns for out=None
    # (src/kermac/build_a_kernel.py:323-336 swap the operands in front of a kernel that
    # computes B - A), here for every layout of out.
    g = torch.Generator().manual_seed(82)
    a, b = torch.randn(70, 9, generator=g).to(device), torch.randn(50, 9, generator=g).to(device)
    signed = kermac.KernelDescriptor(kermac.InnerOperator.DIFF, kermac.PowerType.NOOP, kermac.PowerType.NOOP,
                                     kermac.KernelType.NONE)
    truth = (a.double()[:, None] - b.double()[None]).sum(-1).cpu()
    assert_close_to_truth(kermac.run_kernel(signed, a, b)[0], truth, rtol=1e-5, atol=1e-5, what="signed diff, out=None")
    for c_col in (False, True):
        out = torch.empty(50, 70, device=device).t() if c_col else torch.empty(70, 50, device=device)
        got = kermac.run_kernel(signed, a, b, out=out)
        assert_close_to_truth(got, truth, rtol=1e-5, atol=1e-5, what=f"signed diff, out col-major={c_col}")


@pytest.mark.parametrize("l2_mode", ["direct", "gram", "gram_bf16"])
def test_cdist_cpu_oracle_configuration(device, l2_mode):
    """The reference's CPU-runnable case exactly: a_store[K=64, M=1024], b_store[64, N=1024]
    ~ U(0,1) from torch.manual_seed(0), K-major panels, p = 2 with the square root, one
    batch, out[N, M]; against the float64 oracle at rtol 1e-5 and against torch.cdist under
    the reference test's criterion (tests/test_cdist.py:75-88), in every L2 mode."""
    torch.manual_seed(0)
    a_store = torch.rand(64, 1024)
    b_store = torch.rand(64, 1024)
    out_store = torch.empty(1024, 1024, device=device)
    a, b = a_store.to(device).t(), b_store.to(device).t()
    with kermac.l2_mode(l2_mode, min_k=0):
        out = kermac.cdist(a, b, out=out_store.t(), p=2.0)
    assert out.data_ptr() == out_store.data_ptr() and tuple(out.shape) == (1024, 1024)
    truth = oracle.cdist(a_store.t(), b_store.t(), p=2.0)[0]
    assert_close_to_truth(out, truth, rtol=1e-5, what=f"configs[0], l2 mode {l2_mode}")
    assert_close_to_truth(out, torch.cdist(a_store.t().double(), b_store.t().double(), p=2.0), rtol=1e-5,
                          what=f"configs[0] vs float64 torch.cdist, l2 mode {l2_mode}")
    diff = out.cpu() - torch.cdist(a_store.t(), b_store.t(), p=2.0)
    assert torch.sqrt(torch.mean(diff ** 2)).item() < 1e-4 and diff.abs().max().item() < 1e-4


# ------------------------------------------------- full-size, size-independent checks

@pytest.mark.parametrize("p", [1.0, 2.0, 1.3])
def test_cdist_full_size_properties(device, p):
    """M = N = 30000, K = 1024 (the benchmark configuration): the float64 truth of
    the whole 30000 x 30000 matrix is out of reach, so check a float64 slab, random
    entries, symmetry under exchanging the operands and the zero diagonal of a
    self-distance block."""
    M = N = 30000
    K = 1024
    torch.manual_seed(1)
    a_store = torch.randn(K, M, device=device)
    b_store = torch.randn(K, N, device=device)
    out_store = torch.empty(N, M, device=device)
    out = kermac.cdist(a_store.t(), b_store.t(), out=out_store.t(), p=p)
    assert out.data_ptr() == out_store.data_ptr()
    # slab and edge tile in float64 on the GPU
    for ms, ns in ((slice(0, 300), slice(0, 2000)), (slice(29900, 30000), slice(29800, 30000))):
        truth = torch.cdist(a_store.t()[ms].double(), b_store.t()[ns].double(), p=p)
        assert_close_to_truth(out[ms, ns], truth, rtol=rtol_for(p), what=f"slab p={p}")
    if p == 1.3:
        # the same launch without the 1/p power (the reference raises here; its README
        # documents the bare sum): float64 slabs of cdist ** p at the fractional tolerance
        raw = kermac.cdist(a_store.t(), b_store.t(), out=out_store.t(), p=p, skip_epilogue=True)
        assert raw.data_ptr() == out_store.data_ptr()
        for ms, ns in ((slice(0, 300), slice(0, 2000)), (slice(29900, 30000), slice(29800, 30000)),
                       (slice(14000, 14200), slice(7000, 7600))):
            truth = torch.cdist(a_store.t()[ms].double(), b_store.t()[ns].double(), p=p) ** p
            assert_close_to_truth(raw[ms, ns], truth, rtol=1e-4, what="slab p=1.3, skip_epilogue")
        out = kermac.cdist(a_store.t(), b_store.t(), out=out_store.t(), p=p)
    # exchanging the operands transposes the result exactly (same sums, |b-a| = |a-b|)
    swapped = torch.empty(4000, 3000, device=device)
    kermac.cdist(b_store.t()[:3000], a_store.t()[:4000], out=swapped.t(), p=p)
    assert_close_to_truth(swapped.t(), out[:4000, :3000].t(), rtol=2e-6, what="operand exchange")
    # self-distance block: zero diagonal, symmetric
    del out_store, out
    self_out = kermac.cdist(a_store.t()[:5000], a_store.t()[:5000], p=p)[0]
    assert torch.all(torch.diagonal(self_out) == 0)
    assert torch.equal(self_out, self_out.t())


def test_cdist_full_size_direct_kernel_for_squared_differences(device):
    """M = N = 30000, K = 1024, p = 2 on the kernel with the reference's arithmetic (subtract, square, accumulate:
    include/build_a_kernel.cuh:339-370), which the default mode no longer runs at this size: float64 slabs at 1e-5, also
    without the square root."""
    M = N = 30000
    K = 1024
    torch.manual_seed(1)
    a_store = torch.randn(K, M, device=device)
    b_store = torch.randn(K, N, device=device)
    out_store = torch.empty(N, M, device=device)
    slabs = ((slice(0, 300), slice(0, 2000)), (slice(29900, 30000), slice(29800, 30000)), (slice(14000, 14200), slice(7000, 7600)))
    with kermac.l2_mode("direct"):
        out = kermac.cdist(a_store.t(), b_store.t(), out=out_store.t(), p=2.0)
        for ms, ns in slabs:
            truth = torch.cdist(a_store.t()[ms].double(), b_store.t()[ns].double(), p=2.0)
            assert_close_to_truth(out[ms, ns], truth, rtol=1e-5, what="direct kernel, slab p=2")
        default = torch.empty(2000, 300, device=device)
    kermac.cdist(a_store.t()[:300], b_store.t()[:2000], out=default.t(), p=2.0)
    with kermac.l2_mode("direct"):
        raw = kermac.cdist(a_store.t(), b_store.t(), out=out_store.t(), p=2.0, skip_epilogue=True)
        for ms, ns in slabs:
            truth = torch.cdist(a_store.t()[ms].double(), b_store.t()[ns].double(), p=2.0) ** 2
            assert_close_to_truth(raw[ms, ns], truth, rtol=1e-5, what="direct kernel, slab p=2, skip_epilogue")
