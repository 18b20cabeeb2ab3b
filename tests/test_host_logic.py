"""CPU tests of the host side: layout analysis, batch merging, validation,
parameter marshalling, the C-ABI surface and the kernel cache.

No kernel is launched here.  The marshalling tests take the parameter block that
``run_kernel`` / ``cdist_grad`` would hand to the GPU library and interpret it with
the CPU oracle on the same host memory, so a wrong stride, a missing operand swap
or a wrong enum value shows up without a GPU.
"""
import ctypes
import re
import sys
from ctypes import POINTER, c_float, c_int, c_int64
from itertools import product
from pathlib import Path

import pytest
import torch

import kermac_amd as kermac
from kermac_amd import _backend
from kermac_amd.build_a_kernel import _plan_run_kernel
from kermac_amd.cdist_grad import _plan_cdist_grad
from oracle import oracle
from tests.helpers import assert_close_to_truth, make_operand

ROOT = Path(__file__).resolve().parents[1]


# ------------------------------------------------------------------ TensorStats

def test_tensor_stats_majorness_alignment_and_batch():
    t = torch.zeros(3, 8, 12)
    s = kermac.tensor_stats(t)
    assert s.shape == (3, 8, 12) and s.majorness is kermac.Majorness.ROW_MAJOR
    assert s.alignment is kermac.Alignment.ALIGN_1          # row major is never ALIGN_4
    assert s.batch_stride == 96 and s.leading_dimension_stride == 12 and s.num_batches == 3

    s = kermac.tensor_stats(t.transpose(1, 2))              # [3, 12, 8] view, rows contiguous
    assert s.shape == (3, 12, 8) and s.majorness is kermac.Majorness.COL_MAJOR
    assert s.alignment is kermac.Alignment.ALIGN_4 and s.leading_dimension_stride == 12

    s = kermac.tensor_stats(torch.zeros(7, 5).t())          # ld = 5: not a multiple of 4
    assert s.majorness is kermac.Majorness.COL_MAJOR and s.alignment is kermac.Alignment.ALIGN_1
    assert s.batch_stride == 0 and s.num_batches == 1

    base = torch.zeros(8 * 12 + 1)
    off = base[1:].view(8, 12).t()                          # pointer 4 bytes off a 16-byte boundary
    assert kermac.tensor_stats(off).alignment is kermac.Alignment.ALIGN_1

    assert kermac.tensor_stats(torch.zeros(1, 4, 4)).batch_stride == 0   # batch of 1 broadcasts

    with pytest.raises(ValueError):
        kermac.tensor_stats(torch.zeros(4, 8)[:, ::2])      # neither dimension contiguous
    with pytest.raises(ValueError):
        kermac.tensor_stats(torch.zeros(4))
    with pytest.raises(TypeError):
        kermac.tensor_stats(torch.zeros(4, 4, dtype=torch.float64))


def test_merge_batch_size_rules():
    m = kermac.merge_batch_size
    assert m("x", 1, None, 2, can_be_none=True) == 1
    with pytest.raises(ValueError):
        m("x", 1, None, 2)
    assert m("p", 4, 1.5, 0) == 4
    with pytest.raises(ValueError):
        m("a", 1, 1.5, 2)
    assert m("a", 1, torch.zeros(3, 3), 2) == 1
    assert m("a", 1, torch.zeros(5, 3, 3), 2) == 5
    assert m("a", 5, torch.zeros(1, 3, 3), 2) == 5
    assert m("a", 5, torch.zeros(5, 3, 3), 2) == 5
    with pytest.raises(ValueError):
        m("a", 5, torch.zeros(4, 3, 3), 2)
    with pytest.raises(ValueError):
        m("a", 1, torch.zeros(2, 2, 3, 3), 2)
    assert m("p", 1, torch.zeros(6), 0) == 6
    assert kermac.ceil_div(1000, 128) == 8 and kermac.ceil_div(1024, 128) == 8 and kermac.ceil_div(0, 32) == 0


# ------------------------------------------------------------------- validation

def test_run_kernel_validation_errors():
    a, b = torch.zeros(4, 3), torch.zeros(5, 3)
    plan = lambda d, *args, **kw: _plan_run_kernel(
        d, kw.pop("a", a), kw.pop("b", b), kw.pop("out", None), kw.pop("p", None), kw.pop("inner_p", None),
        kw.pop("outer_p", None), kw.pop("bandwidth", None), kw.pop("epsilon", None), kw.pop("regularization", None),
        0, 0, False, require_device=False)
    with pytest.raises(ValueError):
        plan(kermac.kernel_descriptor_p_norm)                          # POW without p
    with pytest.raises(ValueError):
        plan(kermac.kernel_descriptor_l1_norm, p=1.3)                  # p without POW
    with pytest.raises(ValueError):
        plan(kermac.kernel_descriptor_l1_norm, bandwidth=1.0)          # bandwidth without kernel
    with pytest.raises(ValueError):
        plan(kermac.kernel_descriptor_laplace_l1)                      # kernel without bandwidth
    with pytest.raises(ValueError):
        plan(kermac.kernel_descriptor_p_norm, p=1.3, inner_p=1.3)
    with pytest.raises(ValueError):
        plan(kermac.kernel_descriptor_p_norm, p=1.3, outer_p=1.3)
    with pytest.raises(TypeError):
        plan(kermac.kernel_descriptor_l1_norm, a=[[1.0]])
    with pytest.raises(TypeError):
        plan(kermac.kernel_descriptor_l1_norm, a=torch.zeros(4, 3, dtype=torch.float64))
    with pytest.raises(ValueError):
        plan(kermac.kernel_descriptor_l1_norm, b=torch.zeros(5, 4))    # K mismatch
    with pytest.raises(ValueError):
        plan(kermac.kernel_descriptor_l1_norm, out=torch.zeros(5, 4))  # out is [M, N], not [N, M]
    with pytest.raises(ValueError):
        plan(kermac.kernel_descriptor_l1_norm, a=torch.zeros(2, 4, 3), b=torch.zeros(3, 5, 3))  # batch 2 vs 3
    with pytest.raises(ValueError):
        plan(kermac.kernel_descriptor_l1_norm, a=torch.zeros(2, 4, 3), out=torch.zeros(1, 4, 5))
    with pytest.raises(TypeError):
        plan(kermac.kernel_descriptor_laplace_l1, bandwidth=torch.zeros((), dtype=torch.float64))
    with pytest.raises(ValueError):
        plan(kermac.kernel_descriptor_laplace_l1, a=torch.zeros(2, 4, 3), bandwidth=torch.ones(3))
    # the real entry points refuse CPU tensors, as the reference does
    with pytest.raises(ValueError):
        kermac.run_kernel(kermac.kernel_descriptor_l1_norm, a, b)
    with pytest.raises(ValueError):
        kermac.cdist(a, b)
    with pytest.raises(ValueError):
        kermac.cdist_grad(torch.zeros(3, 4), torch.zeros(5, 3), torch.zeros(2, 3), torch.zeros(5, 4))


def test_cdist_grad_validation_errors():
    a, b, c, d = torch.zeros(6, 4), torch.zeros(5, 6), torch.zeros(2, 6), torch.zeros(5, 4)
    plan = lambda *t, **kw: _plan_cdist_grad(*t, kw.get("out"), kw.get("p", 2.0), require_device=False)
    assert plan(a, b, c, d).out.shape == (1, 2, 5, 4)
    with pytest.raises(TypeError):
        plan(a, b, c, [1.0])
    with pytest.raises(TypeError):
        plan(a.double(), b, c, d)
    with pytest.raises(ValueError):
        plan(a, torch.zeros(5, 7), c, d)                    # K mismatch
    with pytest.raises(ValueError):
        plan(a, b, torch.zeros(2, 7), d)
    with pytest.raises(ValueError):
        plan(a, b, c, torch.zeros(4, 5))                    # d must be [N, M]
    with pytest.raises(ValueError):
        plan(a, b, c, d, out=torch.zeros(2, 4, 5))          # out must be [O, N, M]
    with pytest.raises(ValueError):
        plan(a.t().contiguous().t(), b, c, d)               # a not contiguous in M
    with pytest.raises(ValueError):
        plan(torch.zeros(6), b, c, d)
    with pytest.raises(ValueError):
        plan(torch.zeros(2, 6, 4), torch.zeros(3, 5, 6), c, d)


def test_skip_epilogue_does_not_modify_shared_descriptors():
    # The reference mutates its module-level descriptor (cdist.py:65,75); here the
    # predefined descriptors must be untouched by any call.
    before = (kermac.kernel_descriptor_l2_norm._outer_power, kermac.kernel_descriptor_p_norm._outer_power)
    for p in (2.0, 1.3):
        with pytest.raises(ValueError):                     # CPU tensors: rejected after descriptor handling
            kermac.cdist(torch.zeros(2, 2), torch.zeros(2, 2), p=p, skip_epilogue=True)
    assert before == (kermac.PowerType.SQRT, kermac.PowerType.POW)
    assert (kermac.kernel_descriptor_l2_norm._outer_power, kermac.kernel_descriptor_p_norm._outer_power) == before


# ---------------------------------------------- marshalling, interpreted on the CPU

_lib = ctypes.CDLL(str(oracle.build()))
_OP = ["DIFF", "DOT"]
_POWER = ["NOOP", "ABS", "SQUARE", "SQRT", "POW"]
_KERNEL = ["NONE", "LAPLACE", "GAUSSIAN"]


def _fp(address):
    return ctypes.cast(ctypes.c_void_p(address), POINTER(c_float)) if address else None


def interpret_build_params(p: _backend.BuildKernelParams):
    """Execute a build-kernel parameter block with the CPU oracle, in place, the way
    the device kernel is specified to (include/kermac_amd.h)."""
    def strides(ld, majorness):
        return (1, ld) if majorness == _backend.COL_MAJOR else (ld, 1)
    a_sm, a_sk = strides(p.a_ld, p.a_majorness)
    b_sn, b_sk = strides(p.b_ld, p.b_majorness)
    args_a = (_fp(p.a), c_int64(a_sm), c_int64(a_sk), c_int64(p.a_bs))
    args_b = (_fp(p.b), c_int64(b_sn), c_int64(b_sk), c_int64(p.b_bs))
    m, n, c_sm, c_sn, off_x, off_y = p.m, p.n, 1, p.c_ld, p.regularization_offset_x, p.regularization_offset_y
    if p.flags & _backend.FLAG_NEGATE_DIFF:
        # value(m, n) uses A - B: evaluate with the operands exchanged and write transposed
        args_a, args_b = args_b, args_a
        m, n, c_sm, c_sn, off_x, off_y = n, m, c_sn, c_sm, off_y, off_x
    hyper = []
    for ptr, bs, val in ((p.p_inner, p.p_inner_bs, p.p_inner_value), (p.p_outer, p.p_outer_bs, p.p_outer_value),
                         (p.bandwidth, p.bandwidth_bs, p.bandwidth_value),
                         (p.regularization, p.regularization_bs, p.regularization_value)):
        if ptr:
            hyper += [_fp(ptr), c_int64(bs)]
        else:
            keep = (c_float * 1)(val)
            hyper += [keep, c_int64(0)]
    _lib.kmo_build_kernel(
        c_int(p.inner_operator), c_int(p.inner_power), c_int(p.outer_power), c_int(p.kernel_type),
        c_int(m), c_int(n), c_int(p.k), c_int(p.l), *args_a, *args_b,
        _fp(p.c), c_int64(c_sm), c_int64(c_sn), c_int64(p.c_bs), *hyper,
        c_int(off_x), c_int(off_y), c_float(p.epsilon), c_int(1))


def cpu_run_kernel(descriptor, a, b, out=None, p=None, inner_p=None, outer_p=None, bandwidth=None, epsilon=None,
                   regularization=None, regularization_offset_x=0, regularization_offset_y=0):
    plan = _plan_run_kernel(descriptor, a, b, out, p, inner_p, outer_p, bandwidth, epsilon, regularization,
                            regularization_offset_x, regularization_offset_y, False, require_device=False)
    interpret_build_params(plan.params)
    return plan.out


@pytest.mark.parametrize("a_col,b_col,c_col", list(product([False, True], repeat=3)))
@pytest.mark.parametrize("p", [1.0, 1.3, 2.0])
def test_marshalling_all_majorness_combinations(a_col, b_col, c_col, p):
    # The reference's test matrix (tests/test_cdist.py:50-57) at a small size.
    g = torch.Generator().manual_seed(11)
    L, M, N, K = 2, 21, 17, 9
    a = make_operand(L, M, K, a_col, "cpu", g)
    b = make_operand(L, N, K, b_col, "cpu", g)
    out = torch.full((L, N, M), float("nan")).transpose(1, 2) if c_col else torch.full((L, M, N), float("nan"))
    descriptor, kwargs = {
        1.0: (kermac.kernel_descriptor_l1_norm, {}),
        2.0: (kermac.kernel_descriptor_l2_norm, {}),
        1.3: (kermac.kernel_descriptor_p_norm, {"p": 1.3}),
    }[p]
    got = cpu_run_kernel(descriptor, a, b, out=out, **kwargs)
    assert got is out
    assert_close_to_truth(got, torch.cdist(a.double(), b.double(), p=p), rtol=1e-6, what="marshalled cdist")


@pytest.mark.parametrize("c_col", [False, True])
def test_marshalling_sign_and_offsets_survive_the_swap(c_col):
    g = torch.Generator().manual_seed(12)
    M, N, K = 13, 10, 6
    a, b = torch.randn(M, K, generator=g), torch.randn(N, K, generator=g)
    out = torch.empty(N, M).t() if c_col else torch.empty(M, N)
    signed = kermac.KernelDescriptor(kermac.InnerOperator.DIFF, kermac.PowerType.NOOP, kermac.PowerType.NOOP,
                                     kermac.KernelType.NONE)
    got = cpu_run_kernel(signed, a, b, out=out)
    truth = (a.double()[:, None, :] - b.double()[None, :, :]).sum(-1)        # sum_k (a[m] - b[n]), signed
    assert_close_to_truth(got, truth, rtol=1e-6, atol=1e-9, what="signed difference")
    got = cpu_run_kernel(kermac.kernel_descriptor_laplace_l1, a, b, out=out, bandwidth=2.0, regularization=0.5,
                         regularization_offset_x=4, regularization_offset_y=1)
    truth = torch.exp(-torch.cdist(a.double(), b.double(), p=1.0) / 2.0)
    for n in range(N):                      # offset_x + n == offset_y + m: the reference's out=None result
        if 0 <= n + 3 < M:
            truth[n + 3, n] = 1.5
    assert_close_to_truth(got, truth, rtol=1e-6, what="offset diagonal")


def test_marshalling_broadcast_and_hyper_parameter_tensors():
    g = torch.Generator().manual_seed(13)
    L, M, N, K = 3, 8, 7, 5
    a = torch.randn(L, M, K, generator=g)
    b = torch.randn(N, K, generator=g)                       # broadcast over the batch
    p = torch.tensor([1.5, 2.5, 0.7])
    got = cpu_run_kernel(kermac.kernel_descriptor_p_norm, a, b, p=p)
    assert got.shape == (L, M, N)
    truth = torch.stack([torch.cdist(a[i].double(), b.double(), p=float(p[i])) for i in range(L)])
    assert_close_to_truth(got, truth, rtol=2e-6, what="per-batch p")
    bw = torch.tensor([1.0, 2.0, 4.0])
    got = cpu_run_kernel(kermac.kernel_descriptor_laplace_l2, a, b, bandwidth=bw, regularization=torch.tensor(0.0))
    truth = torch.exp(-torch.cdist(a.double(), b.double().expand(L, -1, -1), p=2.0) / bw.double()[:, None, None])
    assert_close_to_truth(got, truth, rtol=2e-6, what="per-batch bandwidth")
    # a one-element 1-D tensor broadcasts (the reference reads out of bounds here)
    got = cpu_run_kernel(kermac.kernel_descriptor_laplace_l2, a, b, bandwidth=torch.tensor([2.0]))
    truth = torch.exp(-torch.cdist(a.double(), b.double().expand(L, -1, -1), p=2.0) / 2.0)
    assert_close_to_truth(got, truth, rtol=2e-6, what="1-element bandwidth")
    # out=None allocates [L, M, N] zeros-initialised storage and 2-D inputs give L = 1
    got = cpu_run_kernel(kermac.kernel_descriptor_l1_norm, a[0], b)
    assert got.shape == (1, M, N)


def test_scalar_p_rounding_matches_fp32_division():
    plan = _plan_run_kernel(kermac.kernel_descriptor_p_norm, torch.zeros(2, 2), torch.zeros(2, 2), None, 1.3, None,
                            None, None, None, None, 0, 0, False, require_device=False)
    expect_inner = torch.tensor(1.3, dtype=torch.float32)
    assert plan.params.p_inner_value == expect_inner.item()
    assert plan.params.p_outer_value == (1.0 / expect_inner).item()
    assert plan.params.p_inner is None and plan.params.p_outer is None
    assert plan.params.epsilon == pytest.approx(1e-5)


def test_l2_mode_sets_the_gram_flag_only_for_squared_differences():
    a, b = torch.zeros(4, 64), torch.zeros(5, 64)
    def flags(descriptor, **kw):
        plan = _plan_run_kernel(descriptor, a, b, None, kw.get("p"), None, None, kw.get("bandwidth"), None, None, 0, 0,
                                False, require_device=False)
        return plan.params.flags, plan.params.gram_trust
    # the default mode "auto" marks a stored matrix of squared differences as a candidate; run_kernel decides
    assert flags(kermac.kernel_descriptor_l2_norm)[0] & _backend.FLAG_L2_GRAM
    assert flags(kermac.kernel_descriptor_l1_norm)[0] & _backend.FLAG_L2_GRAM == 0
    kermac.set_l2_mode("direct")
    assert flags(kermac.kernel_descriptor_l2_norm)[0] & _backend.FLAG_L2_GRAM == 0
    kermac.set_l2_mode("gram")
    try:
        f, trust = flags(kermac.kernel_descriptor_l2_norm)
        assert f & _backend.FLAG_L2_GRAM and trust == pytest.approx(0.25)
        assert flags(kermac.kernel_descriptor_laplace_l2, bandwidth=1.0)[0] & _backend.FLAG_L2_GRAM
        assert flags(kermac.kernel_descriptor_l1_norm)[0] & _backend.FLAG_L2_GRAM == 0
        assert flags(kermac.kernel_descriptor_p_norm, p=1.3)[0] & _backend.FLAG_L2_GRAM == 0
        kermac.set_l2_mode("gram", trust=0.5)
        assert flags(kermac.kernel_descriptor_l2_norm)[1] == pytest.approx(0.5)
        assert flags(kermac.kernel_descriptor_l2_norm)[0] & _backend.FLAG_L2_GRAM_BF16 == 0
        # short contractions stay on the direct kernel unless min_k says otherwise (K = 64 here)
        kermac.set_l2_mode("gram", min_k=65)
        assert flags(kermac.kernel_descriptor_l2_norm)[0] & _backend.FLAG_L2_GRAM == 0
        kermac.set_l2_mode("gram_bf16")
        f, trust = flags(kermac.kernel_descriptor_l2_norm)
        assert f & _backend.FLAG_L2_GRAM and f & _backend.FLAG_L2_GRAM_BF16 and trust == pytest.approx(0.25)
        assert flags(kermac.kernel_descriptor_l1_norm)[0] & (_backend.FLAG_L2_GRAM | _backend.FLAG_L2_GRAM_BF16) == 0
    finally:
        kermac.set_l2_mode(kermac.DEFAULT_L2_MODE)
    # the default trust grows with K so that very long sums fall back to the direct kernel
    from kermac_amd.build_a_kernel import _gram_trust
    default = {"trust": None}
    assert _gram_trust(1024, default) == pytest.approx(0.25) and _gram_trust(1 << 20, default) > 2.0
    # the C ABI refuses the flag for other inner powers
    params = _backend.BuildKernelParams()
    params.inner_power, params.flags, params.l = 1, _backend.FLAG_L2_GRAM, 1
    params.m = params.n = params.k = 0
    _backend.build_kernel(params, 0)          # empty problem: accepted, nothing launched


def test_auto_mode_picks_the_kernel_by_shape_without_a_gpu(monkeypatch):
    """The l2 mode "auto" decides from the parameter block (and the library's answer about its
    workspace route, which needs no device): the route through a workspace where the library takes
    it, the one-step kernels from K = 128 on (the fp32 one for long contractions over few tiles),
    the direct kernel for short contractions, for grids it would rather cut over k, and for
    contractions so long that the one-step kernels would trust nothing."""
    from kermac_amd import build_a_kernel as module
    for name in ("KERMAC_AMD_WIDE_MIN_TILES", "KERMAC_AMD_L2_WORKSPACE", "KERMAC_AMD_NO_CUT"):
        monkeypatch.delenv(name, raising=False)
    core = _backend.FLAG_L2_GRAM | _backend.FLAG_L2_GRAM_BF16

    def chosen(m, n, k, l=1, dot=False, rows_contiguous=False):
        params = _backend.BuildKernelParams()
        params.a_majorness = params.b_majorness = _backend.COL_MAJOR if rows_contiguous else _backend.ROW_MAJOR
        params.inner_operator, params.inner_power, params.outer_power = (1, 0, 0) if dot else (0, 2, 3)
        params.m, params.n, params.k, params.l = m, n, k, l
        params.a, params.a_ld, params.a_bs = 4096, (m if rows_contiguous else k), m * k
        params.b, params.b_ld, params.b_bs = 4096 + 4 * m * k * l, (n if rows_contiguous else k), n * k
        params.c, params.c_ld, params.c_bs = 256, m, m * n
        params.gram_trust = module._gram_trust(k, {"trust": None})
        return module._auto_matrix_core_flags(params, _backend.FLAG_DOT_PIECES if dot else core)

    assert chosen(128, 128, 200) == core                         # one step, split pieces
    assert chosen(100, 50000, 256, l=4) == _backend.FLAG_L2_GRAM   # one long row of tiles: fp32
    assert chosen(1500, 1500, 384) == _backend.FLAG_L2_GRAM      # one step, fp32: 144 tiles, a contraction the direct path does not cut
    assert chosen(1500, 1500, 784) == 0                          # ... one it does cut: 144 tiles with k contiguous stay with it
    assert chosen(512, 512, 1024, l=8) == core                   # 128 tiles in entries of 16: split pieces, not fp32
    assert chosen(700, 700, 1024, l=4) == _backend.FLAG_L2_GRAM  # 144 tiles in entries of 36: fp32
    assert chosen(2000, 2000, 784) == core                       # 64 tiles of 256 x 256, k contiguous: the workspace route
    assert chosen(4096, 4096, 512) == core                       # 1024 tiles: split pieces
    assert chosen(4096, 4096, 64) == 0 and chosen(1000, 30000, 120) == 0 and chosen(1000, 30000, 128) == core
    assert chosen(10000, 10000, 96) == core                      # the library's workspace route
    assert chosen(4096, 4096, 4096) == core                      # ... also where the direct path would cut over k
    assert chosen(4096, 4096, 20000) == core                     # ... and for contractions the one-step kernels would not trust
    assert chosen(1500, 1500, 20000) == 0
    assert chosen(1024, 1024, 32768) == 0                        # 64 tiles: cut over k by the direct path
    assert chosen(1536, 1536, 4096) == 0                         # 144 tiles, k contiguous: cut over k as well
    assert chosen(1536, 1536, 4096, rows_contiguous=True) == core  # rows contiguous: uncut on the matrix cores from 128 tiles on
    assert chosen(256, 256, 512, l=8) == core
    # operands stored with the rows contiguous: the split kernel instead of the fp32 one
    assert chosen(5000, 5000, 128, rows_contiguous=True) == core and chosen(5000, 5000, 128) == core and chosen(5000, 5000, 112) == 0
    assert chosen(1500, 1500, 1024, rows_contiguous=True) == core and chosen(1500, 1500, 400) == _backend.FLAG_L2_GRAM
    assert chosen(2000, 2000, 784, rows_contiguous=True) == core              # the split one-step kernel there
    assert chosen(8192, 4096, 512, dot=True) == _backend.FLAG_DOT_PIECES
    assert chosen(300, 300, 512, dot=True) == 0
    # from K = 256 on: 32 tiles over a batch, 64 of a single problem (which the direct path would cut over k), any padding
    assert chosen(512, 512, 784, l=8, dot=True) == _backend.FLAG_DOT_PIECES
    assert chosen(1500, 1500, 784, dot=True) == 0 and chosen(2000, 2000, 784, dot=True) == _backend.FLAG_DOT_PIECES
    assert chosen(300, 30000, 784, dot=True) == _backend.FLAG_DOT_PIECES
    assert chosen(1000, 1000, 256, l=4, dot=True) == 0                          # tiles * k below 24576
    monkeypatch.setenv("KERMAC_AMD_L2_WORKSPACE", "0")
    assert chosen(8192, 4096, 512, dot=True) == 0 and chosen(10000, 10000, 96) == 0 and chosen(10000, 10000, 256) == core


def interpret_grad_params(p: _backend.NormGradientParams):
    keep = (c_float * 1)(p.p_value)
    _lib.kmo_norm_kernel_gradient(
        c_int(p.norm_type), c_int(p.m), c_int(p.n), c_int(p.o), c_int(p.k), c_int(p.l),
        _fp(p.a), c_int64(p.a_ld), c_int64(1), c_int64(p.a_bs),
        _fp(p.b), c_int64(p.b_ld), c_int64(1), c_int64(p.b_bs),
        _fp(p.c), c_int64(p.c_ld), c_int64(1), c_int64(p.c_bs),
        _fp(p.d), c_int64(p.d_ld), c_int64(1), c_int64(p.d_bs),
        _fp(p.e), c_int64(p.e_ld_o), c_int64(p.e_ld_n), c_int64(1), c_int64(p.e_bs),
        _fp(p.p) if p.p else keep, c_int64(p.p_bs), c_int(1))


@pytest.mark.parametrize("p", [1.0, 2.0, 1.3, "tensor"])
def test_gradient_marshalling(p):
    g = torch.Generator().manual_seed(14)
    L, M, N, O, K = 2, 12, 7, 3, 10
    a = torch.rand(L, K, M, generator=g)
    b = torch.randn(N, K, generator=g)                       # broadcast
    c = torch.randn(L, O, K + 2, generator=g)[:, :, :K]      # leading dimension larger than K
    d = torch.randn(L, N, M, generator=g)
    out = torch.full((L, O, N, M), float("nan"))
    p_arg = torch.tensor([1.5, 3.0]) if p == "tensor" else p
    plan = _plan_cdist_grad(a, b, c, d, out, p_arg, require_device=False)
    assert plan.params.norm_type == {1.0: 0, 2.0: 1}.get(p, 2)
    interpret_grad_params(plan.params)
    truth = oracle.cdist_grad(a, b, c.contiguous(), d, p=p_arg)
    assert_close_to_truth(out, truth, rtol=1e-6, atol=1e-6, what="marshalled gradient")


# ------------------------------------------------------------------ C ABI surface

def test_library_exports_every_declared_symbol():
    header = (ROOT / "include" / "kermac_amd.h").read_text()
    declared = set(re.findall(r"^\s*(?:int|void|const char \*)\s*\*?(kmc_[a-z0-9_]+)\s*\(", header, flags=re.M))
    assert len(declared) >= 14, declared
    assert declared == set(_backend.SIGNATURES), declared ^ set(_backend.SIGNATURES)
    lib = _backend.library()                                # raises if the library is not built
    for name in declared:
        assert hasattr(lib, name), f"{name} is declared in kermac_amd.h but not exported"
    assert lib.kmc_abi_version() == _backend.ABI_VERSION
    # struct layout agreed between header and binding: spot-check sizes
    assert ctypes.sizeof(_backend.BuildKernelParams) % 8 == 0
    assert _backend.build_kernel_has_variant(0, 1) and _backend.build_kernel_has_variant(0, 2)
    assert _backend.build_kernel_has_variant(0, 4) and _backend.build_kernel_has_variant(1, 0)


def test_header_is_plain_c_and_agrees_with_the_binding(tmp_path):
    """include/kermac_amd.h must compile as C11 on its own, and every struct must
    have, field by field, the size and offsets the ctypes binding assumes.  The
    probe program is generated from the binding's field names, so a field that is
    missing, renamed or reordered in either place fails here."""
    import shutil
    import subprocess
    gcc = shutil.which("gcc")
    if gcc is None:
        pytest.skip("no C compiler")
    structs = {"kmc_build_kernel_params": _backend.BuildKernelParams,
               "kmc_norm_gradient_params": _backend.NormGradientParams,
               "kmc_kernel_coefficients_params": _backend.KernelCoefficientsParams,
               "kmc_matrix_coefficients_params": _backend.MatrixCoefficientsParams}
    lines = ['#include "kermac_amd.h"', "#include <stddef.h>", "#include <stdio.h>", "int main(void) {"]
    for c_name, binding in structs.items():
        lines.append(f'  printf("{c_name} size %zu\\n", sizeof(struct {c_name}));')
        for field, _ in binding._fields_:
            lines.append(f'  printf("{c_name} {field} %zu\\n", offsetof(struct {c_name}, {field}));')
    for flag in ("FORCE_SCALAR_ACCESS", "NEGATE_DIFF", "L2_GRAM", "GENERIC_POWER", "NO_SYMMETRY", "L2_GRAM_BF16", "GRAM_A_KEPT",
                 "DOT_PIECES", "GRAM_WORKSPACE_ANY_SIZE", "L1_FIXED", "NO_PROBE"):
        lines.append(f'  printf("flag {flag} %d\\n", (int)KMC_FLAG_{flag});')
    lines += ['  printf("err WRONG_DEVICE %d\\n", (int)KMC_ERR_WRONG_DEVICE);', "  return 0;", "}"]
    source = tmp_path / "probe.c"
    source.write_text("\n".join(lines))
    exe = tmp_path / "probe"
    subprocess.run([gcc, "-std=c11", "-Wall", "-Wextra", "-Werror", "-pedantic", f"-I{ROOT / 'include'}", str(source),
                    "-o", str(exe)], check=True)
    reported = {}
    for line in subprocess.run([str(exe)], check=True, capture_output=True, text=True).stdout.splitlines():
        *key, value = line.split()
        reported[tuple(key)] = int(value)
    for c_name, binding in structs.items():
        assert reported[(c_name, "size")] == ctypes.sizeof(binding), c_name
        for field, _ in binding._fields_:
            assert reported[(c_name, field)] == getattr(binding, field).offset, f"{c_name}.{field}"
    for flag in ("FORCE_SCALAR_ACCESS", "NEGATE_DIFF", "L2_GRAM", "GENERIC_POWER", "NO_SYMMETRY", "L2_GRAM_BF16", "GRAM_A_KEPT",
                 "DOT_PIECES", "GRAM_WORKSPACE_ANY_SIZE", "L1_FIXED", "NO_PROBE"):
        assert reported[("flag", flag)] == getattr(_backend, f"FLAG_{flag}")
    assert reported[("err", "WRONG_DEVICE")] == _backend.ERR_WRONG_DEVICE


def test_c_abi_rejects_bad_arguments_without_a_gpu():
    params = _backend.BuildKernelParams()
    params.inner_operator = 7
    with pytest.raises(_backend.BackendError) as info:
        _backend.build_kernel(params, 0)
    assert info.value.status == _backend.ERR_INVALID_ARGUMENT and "inner_operator" in str(info.value)
    params = _backend.BuildKernelParams()
    params.inner_power = 1
    params.m = params.n = params.k = 4
    params.l = 1
    with pytest.raises(_backend.BackendError) as info:      # null operand pointers
        _backend.build_kernel(params, 0)
    assert info.value.status == _backend.ERR_INVALID_ARGUMENT
    grad = _backend.NormGradientParams()
    grad.norm_type = 9
    with pytest.raises(_backend.BackendError):
        _backend.norm_kernel_gradient(grad, 0)
    # the finishing step of a contraction cut over k: host pointers are never dereferenced, so
    # fake non-null addresses are enough to reach the checks of the partial-sum arguments
    fake = 4096
    params = _backend.BuildKernelParams()
    params.inner_power = 1
    params.m = params.n = params.k = 8
    params.l = 1
    params.a = params.b = params.c = fake
    params.a_ld = params.b_ld = params.c_ld = 8
    for partials, ld, slices, word in ((0, 8, 3, "null"), (fake, 4, 3, "leading dimension"), (fake, 8, -1, "slice count")):
        with pytest.raises(_backend.BackendError) as info:
            _backend.build_kernel_finish(params, partials, ld, 0, 64, slices, 0)
        assert info.value.status == _backend.ERR_INVALID_ARGUMENT and word in str(info.value), str(info.value)
    # ranges of one contraction as batch entries: k_total must be covered by l ranges of k, the last not empty
    for l, k, k_total, flags, word in ((3, 8, -1, 0, "k_total"), (3, 8, 30, 0, "not covered"), (3, 8, 16, 0, "not covered"),
                                       (3, 8, 20, _backend.FLAG_L2_GRAM, "matrix-core")):
        ranged = _backend.BuildKernelParams.from_buffer_copy(params)
        ranged.inner_power = 2
        ranged.l, ranged.k, ranged.k_total, ranged.flags = l, k, k_total, flags
        with pytest.raises(_backend.BackendError) as info:
            _backend.build_kernel(ranged, 0)
        assert info.value.status == _backend.ERR_INVALID_ARGUMENT and word in str(info.value), str(info.value)
    fused = _backend.KernelCoefficientsParams()
    fused.kernel = _backend.BuildKernelParams.from_buffer_copy(params)
    fused.kernel.k_total = 8
    with pytest.raises(_backend.BackendError) as info:
        _backend.kernel_times_coefficients(fused, 0)
    assert "k_total" in str(info.value)
    params.m = 0
    _backend.build_kernel_finish(params, 0, 0, 0, 0, 0, 0)      # empty result: accepted, nothing launched
    # a device that is not a gfx950 is a ValueError, as an unsupported compute capability is in
    # the reference (src/kermac/module_cache/module_cache.py:166-167), and still a BackendError
    with pytest.raises(ValueError) as info:
        _backend.check(_backend.ERR_WRONG_DEVICE)
    assert isinstance(info.value, _backend.BackendError) and info.value.status == _backend.ERR_WRONG_DEVICE


def test_workspace_queries_need_no_gpu(monkeypatch):
    """kmc_gram_workspace_bytes and kmc_norm_gradient_workspace_bytes decide from the parameter block
    alone (no device call, no pointer dereferenced, the result need not be allocated yet): which
    problems take the routes through a workspace, and how much they want."""
    monkeypatch.delenv("KERMAC_AMD_WIDE_MIN_TILES", raising=False)
    monkeypatch.delenv("KERMAC_AMD_GRADIENT_F16_MIN_TERMS", raising=False)
    fake = 4096

    def squared_differences(m, n, k, l=1, flags=_backend.FLAG_L2_GRAM | _backend.FLAG_L2_GRAM_BF16, same=False, k_contiguous=False):
        params = _backend.BuildKernelParams()
        params.inner_operator, params.inner_power, params.outer_power = 0, 2, 3      # DIFF, SQUARE, SQRT
        params.m, params.n, params.k, params.l = m, n, k, l
        params.a, params.a_ld, params.a_bs = fake, (k if k_contiguous else m), m * k
        params.b, params.b_ld, params.b_bs = (fake if same else fake + 4 * m * k * l), (k if k_contiguous else n), n * k
        params.a_majorness = params.b_majorness = _backend.ROW_MAJOR if k_contiguous else _backend.COL_MAJOR
        params.c_ld, params.c_bs = m, m * n                                          # c stays null: not allocated yet
        params.flags = flags
        return _backend.gram_workspace_bytes(params)

    full = squared_differences(8192, 8192, 512)
    operands = 2 * 8192 * 512 * 4
    assert operands < full < 1.3 * operands                                          # two fp16 pieces per value, padding, statistics
    assert squared_differences(8192, 8192, 512, flags=_backend.FLAG_L2_GRAM) == 0    # fp32 matrix instruction: one step
    assert squared_differences(8192, 8192, 32) == 0                                  # k < 64
    assert squared_differences(2048, 2048, 512) == 0                                 # 64 tiles
    assert squared_differences(2048, 2048, 512, l=5) > 0                             # 320 tiles over the batch
    assert 0 < squared_differences(8192, 8192, 512, same=True) < 0.6 * full          # a panel against itself: split once
    assert squared_differences(512, 512, 1024, l=64) == 0                            # 256 tiles, but 2 x 2 per entry: the split is not earned back
    assert squared_differences(30000, 512, 1024) == 0 and squared_differences(30000, 1024, 1024) > 0
    assert squared_differences(1290, 1290, 1024, l=8) == 0                           # 6 x 6 tiles, 30 % of them padding
    assert squared_differences(1280, 1280, 1024, l=8) > 0
    assert squared_differences(0, 8192, 512) == 0
    # both operands with k contiguous: from 48 tiles on at k >= 256, whatever the shape of a batch entry,
    # unless half a tile holds a dimension
    assert squared_differences(2048, 2048, 1024, k_contiguous=True) > 0
    assert squared_differences(512, 512, 1024, l=16, k_contiguous=True) > 0
    assert squared_differences(1500, 1500, 512, k_contiguous=True) == 0              # 36 tiles
    assert squared_differences(2048, 2048, 128, k_contiguous=True) == 0
    assert squared_differences(128, 50000, 1024, k_contiguous=True) == 0 and squared_differences(129, 50000, 1024, k_contiguous=True) > 0
    # the caller's own rule
    any_size = _backend.FLAG_L2_GRAM_BF16 | _backend.FLAG_GRAM_WORKSPACE_ANY_SIZE
    assert squared_differences(300, 200, 5, flags=any_size) > 0
    assert squared_differences(300, 200, 0, flags=any_size) == 0
    assert squared_differences(300, 200, 5, flags=_backend.FLAG_L2_GRAM | _backend.FLAG_GRAM_WORKSPACE_ANY_SIZE) == 0
    monkeypatch.setenv("KERMAC_AMD_WIDE_MIN_TILES", "1")
    assert squared_differences(300, 200, 5) > 0

    def gradient(m, n, o, k, norm_type=0):
        grad = _backend.NormGradientParams()
        grad.norm_type = norm_type
        grad.m, grad.n, grad.o, grad.k, grad.l = m, n, o, k, 1
        grad.a, grad.b, grad.c, grad.d, grad.e = fake, fake, fake, fake, fake
        grad.a_ld, grad.b_ld, grad.c_ld, grad.d_ld, grad.e_ld_n, grad.e_ld_o = m, k, k, m, m, m * n
        return _backend.norm_gradient_workspace_bytes(grad)

    assert gradient(8192, 512, 16, 8192) > 4 * 8192 * 8192                           # the pieces of a alone
    assert gradient(8192, 512, 16, 8192, norm_type=2) == 0
    # the L2 norm: one product of (o n) x k by k x m on the fp16 matrix instruction, by a model of both times
    monkeypatch.delenv("KERMAC_AMD_GRADIENT_L2_MIN_TERMS", raising=False)
    assert gradient(8192, 512, 16, 8192, norm_type=1) > 3 * 4 * 8192 * 8192          # c b in fp32 and in pieces, the pieces of a
    assert gradient(8192, 512, 16, 256, norm_type=1) == 0                            # a short contraction
    assert gradient(8192, 8, 16, 8192, norm_type=1) == 0                             # 32 x 1 tiles
    assert gradient(512, 512, 16, 8192, norm_type=1) == 0                            # 2 x 32 tiles
    assert gradient(8192, 512, 1, 8192, norm_type=1) > 0                             # one output: the fp32 kernel is slow there
    assert gradient(8192, 512, 2, 8192) == 0                                         # two outputs: the vector kernel
    assert gradient(1024, 64, 16, 1024) == 0                                         # 6.7e7 terms
    assert gradient(1024, 64, 17, 1024) > 0 and gradient(512, 64, 64, 512) > 0       # more than 16 outputs: from 1.5e7 terms on
    assert gradient(256, 64, 64, 512) == 0                                           # 8.4e6 terms
    assert gradient(8192, 16, 16, 8192) == 0                                         # half of every tile of 32 columns unused
    assert gradient(2048, 128, 4, 2048) == 0 and gradient(2048, 128, 16, 2048) > 0   # 5.4e8 terms: enough for 16 outputs, not for 4
    # a row n is a workgroup row of the route's padding kernel: beyond 65535 of them the fp32 kernels run
    assert gradient(1000, 65000, 16, 100) > 0 and gradient(1000, 70000, 16, 100) == 0

    def absolute_differences(m, n, k, l=1, flags=_backend.FLAG_L1_FIXED, same=False):
        params = _backend.BuildKernelParams()
        params.inner_operator, params.inner_power, params.outer_power = 0, 1, 0      # DIFF, ABS, NOOP
        params.m, params.n, params.k, params.l = m, n, k, l
        params.a, params.a_ld, params.a_bs = fake, m, m * k
        params.b, params.b_ld, params.b_bs = (fake if same else fake + 4 * m * k * l), n, n * k
        params.c_ld, params.c_bs = m, m * n
        params.flags = flags
        return _backend.gram_workspace_bytes(params)

    # the fixed-point route of sums of absolute differences: 2048 tiles of 128 x 128 over the batch, k >= 128
    padded = (6016 + 6016) * 512 * 4
    assert padded <= absolute_differences(6000, 6000, 512) <= padded + 1024         # 47 x 47 tiles, 4 bytes per padded element
    assert absolute_differences(6000, 6000, 512, flags=0) == 0
    assert absolute_differences(5000, 5000, 512) == 0 and absolute_differences(5000, 5000, 512, l=2) > 0
    assert absolute_differences(6000, 6000, 100) == 0
    assert 0 < absolute_differences(9000, 9000, 512, same=True) < 0.6 * absolute_differences(9000, 9000, 512)
    assert absolute_differences(300, 200, 5, flags=_backend.FLAG_L1_FIXED | _backend.FLAG_GRAM_WORKSPACE_ANY_SIZE) > 0
    assert squared_differences(6000, 6000, 512, flags=_backend.FLAG_L1_FIXED) == 0  # squared differences: not this route
    monkeypatch.setenv("KERMAC_AMD_GRADIENT_F16_MIN_TERMS", "1")
    assert gradient(3, 2, 1, 5) > 0

    def panels(m, n, k, l=1, power=1, flags=_backend.FLAG_DIRECT_PANELS, k_contiguous=(True, True), same=False, misaligned=False):
        params = _backend.BuildKernelParams()
        params.inner_operator, params.inner_power, params.outer_power = 0, power, 0
        params.m, params.n, params.k, params.l = m, n, k, l
        params.a, params.a_ld, params.a_bs = fake + (4 if misaligned else 0), (k if k_contiguous[0] else m), m * k
        params.b, params.b_ld, params.b_bs = (params.a if same else fake + 4 * m * k * l), (k if k_contiguous[1] else n), n * k
        params.a_majorness = _backend.ROW_MAJOR if k_contiguous[0] else _backend.COL_MAJOR
        params.b_majorness = _backend.ROW_MAJOR if k_contiguous[1] else _backend.COL_MAJOR
        params.c_ld, params.c_bs = m, m * n
        params.flags = flags
        return _backend.gram_workspace_bytes(params)

    # copies of the operands for the direct kernel with b in scalar registers: 5400 tiles of 256 x 64 per batch entry,
    # k >= 64, absolute or squared differences, an operand the kernel cannot take as it is; 4 bytes per padded element
    assert panels(30000, 30000, 1024) == 2 * 1024 * 30016 * 4
    assert panels(30000, 30000, 1024, power=2) == panels(30000, 30000, 1024) and panels(30000, 30000, 1024, power=4) == 0
    assert panels(30000, 30000, 1024, k_contiguous=(False, False)) == 0             # the kernel takes these by itself
    assert panels(30000, 30000, 1024, k_contiguous=(False, True)) == 1024 * 30016 * 4
    assert panels(30000, 30008, 1024, k_contiguous=(False, False)) == 1024 * 30016 * 4        # n not a multiple of 16: b
    assert panels(30000, 30000, 1000, k_contiguous=(False, False)) == 2 * 1008 * 30016 * 4    # k not a multiple of 16: both
    assert panels(30000, 30000, 1024, k_contiguous=(False, False), misaligned=True) == 1024 * 30016 * 4
    assert panels(10000, 10000, 1024) > 0 and panels(9000, 9000, 1024) == 0         # 6280 and 5076 tiles
    assert panels(9000, 9000, 1024, l=4) == 0                                       # per batch entry
    assert panels(30000, 30000, 48) == 0
    assert panels(30000, 30000, 1024, same=True) == 1024 * 30016 * 4               # a set against itself: one copy, from 16000 tiles of the triangle on
    assert panels(16384, 16384, 1024, same=True) == 0                              # 8320 tiles
    assert panels(30000, 30000, 1024, flags=0) == 0
    assert panels(30000, 30000, 1024, flags=_backend.FLAG_DIRECT_PANELS | _backend.FLAG_L1_FIXED) == absolute_differences(30000, 30000, 1024)   # that route's own
    assert panels(300, 200, 5, flags=_backend.FLAG_DIRECT_PANELS | _backend.FLAG_GRAM_WORKSPACE_ANY_SIZE) == 16 * (320 + 256) * 4


def test_auto_mode_of_the_coefficient_product_without_a_gpu(monkeypatch):
    """l2 mode "auto", run_kernel(..., coefficients=...) of squared differences: panels where the
    library's rule or the rule for this product takes them, else the matrix-core variant of the
    fused kernel or the direct one, by K, the number of coefficient columns and the size."""
    from kermac_amd import kernel_coefficients as module
    for name in ("KERMAC_AMD_WIDE_MIN_TILES", "KERMAC_AMD_COEFFICIENT_PANEL_BYTES"):
        monkeypatch.delenv(name, raising=False)
    assert kermac.get_l2_mode() == "auto"
    any_size = _backend.FLAG_GRAM_WORKSPACE_ANY_SIZE

    def plan(M, N, K, O, L=1, k_contiguous=True, descriptor=kermac.kernel_descriptor_laplace_l2):
        a = torch.empty(L, M, K) if k_contiguous else torch.empty(L, K, M).transpose(1, 2)
        b = torch.empty(L, N, K) if k_contiguous else torch.empty(L, K, N).transpose(1, 2)
        bandwidth = None if descriptor._kernel_type is kermac.KernelType.NONE else 2.0
        return module._plan_run_kernel_coefficients(descriptor, a, b, torch.empty(L, N, O), None, None, None, None, bandwidth,
                                                    None, None, 0, 0, require_device=False)

    def chosen(*shape, **kw):
        p = plan(*shape, **kw)
        assert p.l2_auto and p.params.kernel.flags & _backend.FLAG_L2_GRAM
        panels = module._panel_shape(p, _backend.FLAG_L2_GRAM_BF16)
        if panels is not None:
            return "panels, any size" if panels[4] & any_size else "panels"
        return "fused, matrix cores" if module._auto_fused_on_matrix_cores(p) else "fused, direct"

    assert chosen(4096, 4096, 256, 32) == "panels"
    assert chosen(4096, 4096, 256, 32, k_contiguous=False) == "panels, any size"       # 256 tiles
    assert chosen(4096, 4096, 128, 32, k_contiguous=False) == "fused, matrix cores"    # 256 tiles at K = 128: no panels; 2.1e9 terms
    assert chosen(4096, 4096, 128, 32, L=4, k_contiguous=False) == "panels"            # 1024 tiles
    assert chosen(10000, 10000, 64, 32) == "fused, direct"                             # K below 128
    assert chosen(500, 500, 256, 32) == "fused, matrix cores"
    assert chosen(500, 500, 128, 32) == "fused, direct"                                # 3.2e7 terms
    assert chosen(500, 500, 256, 40) == "fused, matrix cores"                          # a small problem: the second chunk of columns runs beside the first
    assert chosen(500, 500, 3072, 8) == "panels, any size"                             # a long contraction
    assert chosen(2000, 2000, 784, 32, k_contiguous=False) == "fused, matrix cores"    # 64 tiles
    assert chosen(2000, 2000, 784, 40, k_contiguous=False) == "panels, any size"
    assert chosen(100, 50000, 784, 32) == "fused, matrix cores"                        # 61 % of every tile padding
    assert chosen(100, 50000, 784, 40) == "panels, any size"
    assert chosen(100, 50000, 256, 40) == "fused, direct"
    monkeypatch.setenv("KERMAC_AMD_COEFFICIENT_PANEL_BYTES", "0")
    assert chosen(4096, 4096, 256, 32) == "fused, matrix cores"
    assert chosen(4096, 4096, 256, 40) == "fused, direct"
    monkeypatch.delenv("KERMAC_AMD_COEFFICIENT_PANEL_BYTES")
    with kermac.l2_mode("gram_bf16"):                                                   # the explicit mode: the library's rule alone
        p = plan(4096, 4096, 256, 32, k_contiguous=False)
        assert not p.l2_auto and module._panel_shape(p, _backend.FLAG_L2_GRAM_BF16) is None
        p = plan(8192, 8192, 256, 32, k_contiguous=False)
        assert module._panel_shape(p, _backend.FLAG_L2_GRAM_BF16)[4] == _backend.FLAG_L2_GRAM_BF16
    # sums of products have rules of their own (their fused kernel has no matrix-core variant)
    products = kermac.KernelDescriptor(kermac.InnerOperator.DOT, kermac.PowerType.NOOP, kermac.PowerType.NOOP, kermac.KernelType.NONE)

    def product_panels(*shape, **kw):
        p = plan(*shape, descriptor=products, **kw)
        if not module._products_in_panels(p):
            return None
        panels = module._panel_shape(p, _backend.FLAG_DOT_PIECES)
        return None if panels is None else bool(panels[4] & any_size)

    assert product_panels(8192, 8192, 512, 8) is False                                 # the library's rule takes them
    assert product_panels(500, 500, 784, 8) is True and product_panels(500, 500, 256, 8) is None
    assert product_panels(4096, 4096, 64, 40) is True and product_panels(4096, 4096, 64, 32) is None
    assert product_panels(2000, 2000, 64, 40) is None                                  # 4e6 elements
    assert product_panels(100, 50000, 784, 8) is None and product_panels(100, 50000, 784, 40) is False
    assert product_panels(4096, 4096, 32, 40) is None                                  # K below 64
    with kermac.l2_mode("direct"):
        assert plan(4096, 4096, 256, 32).params.kernel.flags & _backend.FLAG_L2_GRAM == 0
        assert product_panels(8192, 8192, 512, 8) is None
        # more than 64 columns: plain panels (no route flag) in any mode, for any descriptor
        rows, panels, ld, splits, flags = module._panel_shape(plan(4096, 20000, 256, 100, descriptor=kermac.kernel_descriptor_laplace_l1), 0)
        assert (rows, panels, ld, flags) == (20000, 1, 4096, 0) and splits >= 1
    # partial products beyond 512 MiB are not kept: the panels are added to the result one after the other
    monkeypatch.setenv("KERMAC_AMD_COEFFICIENT_PANEL_BYTES", str(1 << 26))
    assert module._panel_shape(plan(16384, 16384, 256, 1000, L=4, descriptor=kermac.kernel_descriptor_laplace_l1), 0)[3] == 0
    monkeypatch.delenv("KERMAC_AMD_COEFFICIENT_PANEL_BYTES")
    assert plan(4096, 4096, 256, 32, descriptor=kermac.kernel_descriptor_laplace_l1).params.kernel.flags & _backend.FLAG_L2_GRAM == 0


def test_which_products_contract_their_panels_from_fp16_pieces(monkeypatch):
    """At least 256 coefficient columns and 128 tiles of 256 x 256 over (columns, rows, batch); the
    environment variable replaces both conditions by a number of columns."""
    from kermac_amd.kernel_coefficients import _contraction_by_pieces_pays as pays
    monkeypatch.delenv("KERMAC_AMD_COEFFICIENT_PIECES_MIN_COLUMNS", raising=False)
    assert not pays(4, 16384, 128) and pays(4, 16384, 256)
    assert not pays(1, 10000, 256) and pays(1, 10000, 1000)             # 40 and 160 tiles
    assert not pays(1, 2000, 1000)                                      # 32 tiles
    monkeypatch.setenv("KERMAC_AMD_COEFFICIENT_PIECES_MIN_COLUMNS", "5")
    assert pays(1, 10, 5) and not pays(4, 16384, 4)


def test_matrix_times_coefficients_checks_its_arguments_before_any_device_call():
    """kmc_matrix_times_coefficients: extents, strides and the l * n_splits limit are checked
    first, and an empty product returns without touching a device."""
    def params(m=64, n=100, o=8, l=1, **fields):
        block = _backend.MatrixCoefficientsParams()
        block.m, block.n, block.o, block.l = m, n, o, l
        block.matrix, block.matrix_ld, block.matrix_bs = 4096, m, m * n
        block.coef, block.coef_ld, block.coef_bs = 4096, o, n * o
        block.out, block.out_ld, block.out_bs = 4096, o, m * o
        for name, value in fields.items():
            setattr(block, name, value)
        return block

    for bad in (params(m=-1), params(matrix_ld=32), params(coef_ld=4), params(out_ld=4), params(out=None),
                params(matrix=None), params(l=70000), params(l=300, n_splits=300), params(n_splits=-2),
                params(out_split_stride=-1)):
        with pytest.raises(_backend.BackendError) as info:
            _backend.matrix_times_coefficients(bad, 0)
        assert info.value.status == _backend.ERR_INVALID_ARGUMENT
    for empty in (params(m=0), params(o=0), params(l=0)):
        _backend.matrix_times_coefficients(empty, 0)
    # the Python mirror cuts the n of a panel so that the contraction has a workgroup per CU
    from kermac_amd.kernel_coefficients import _panel_splits
    assert _panel_splits(16384, 32, 4, 4096) == 1            # 512 workgroups of 128 rows
    assert _panel_splits(8192, 8, 1, 4096) == 4              # 64 workgroups
    assert _panel_splits(8192, 8, 1, 1024) == 2              # at least 512 rows per range
    assert _panel_splits(30000, 16, 1, 16384) == 4           # sums of at most 4096 rows per workgroup
    assert _panel_splits(128, 1, 60000, 1 << 20) == 1        # l * n_splits stays below 65536


def test_launch_cuts_follow_the_shape_and_the_environment_switch(monkeypatch):
    """The cut over k is decided from the parameter block alone: small and middling results over a
    long contraction are cut, batches, short contractions and large results are not, and
    KERMAC_AMD_NO_CUT=1 switches every cut off."""
    from kermac_amd import _backend
    from kermac_amd import build_a_kernel as module

    def block(m, n, k, l=1, same=False, flags=0):
        params = _backend.BuildKernelParams()
        params.m, params.n, params.k, params.l, params.flags = m, n, k, l, flags
        params.a, params.b = 4096, 4096 if same else 8192
        params.a_ld = params.b_ld = max(m, n)
        return params

    monkeypatch.delenv("KERMAC_AMD_NO_CUT", raising=False)
    ranges, depth = module._cut_over_contraction(block(100, 100, 100000))
    assert ranges * depth >= 100000 > (ranges - 1) * depth and depth % 16 == 0 and ranges > 100
    ranges, depth = module._cut_over_contraction(block(3072, 3072, 1000))
    assert 2 <= ranges <= 8 and ranges * depth >= 1000 > (ranges - 1) * depth
    assert module._cut_over_contraction(block(3072, 3072, 1000, l=2)) is None                 # batched
    assert module._cut_over_contraction(block(3072, 3072, 256)) is None                       # short contraction
    assert module._cut_over_contraction(block(30000, 30000, 1024)) is None                    # the chip is full
    assert module._cut_over_contraction(block(3072, 3072, 4096, flags=_backend.FLAG_L2_GRAM)) is None
    # a set against itself counts the tiles of one triangle: 64 x 64 tiles are 2080 to compute, 2048 cut nothing
    assert module._cut_over_contraction(block(8192, 8192, 4096, same=True)) is None
    assert module._cut_over_contraction(block(5120, 5120, 4096, same=True)) is not None
    monkeypatch.setenv("KERMAC_AMD_NO_CUT", "1")
    assert module._cut_over_contraction(block(100, 100, 100000)) is None


def test_reference_module_name_resolves_to_this_package():
    """Callers of the reference do `import kermac` (examples/cdist.py:2, tests/test_cdist.py:3)."""
    import kermac as by_reference_name
    import kermac.common
    import kermac.module_cache.module_cache
    import kermac_amd.module_cache.module_cache
    assert by_reference_name is kermac
    assert kermac.common is sys.modules["kermac_amd.common"]
    assert sys.modules["kermac.module_cache.module_cache"] is kermac_amd.module_cache.module_cache
    from kermac.common import Majorness
    assert Majorness is kermac.Majorness
    for name in ("cdist", "cdist_grad", "run_kernel", "pre_compile_descriptors", "KernelDescriptor", "InnerOperator",
                 "PowerType", "KernelType", "Symmetry", "ModuleCache", "CudaTimer", "tensor_stats", "TensorStats",
                 "Majorness", "Alignment", "FillMode", "ceil_div", "merge_batch_size", "PyTorchStreamWrapper",
                 "kernel_descriptor_laplace_l1", "kernel_descriptor_laplace_l2", "kernel_descriptor_p_norm",
                 "kernel_descriptor_l1_norm", "kernel_descriptor_l2_norm", "kernel_descriptor_mma"):
        assert hasattr(by_reference_name, name), name


def test_l2_mode_blocks_are_per_thread():
    import threading
    seen = {}
    ready, release = threading.Event(), threading.Event()

    def worker():
        with kermac.l2_mode("gram_bf16"):
            seen["worker_inside"] = kermac.get_l2_mode()
            ready.set()
            release.wait(10)
        seen["worker_after"] = kermac.get_l2_mode()

    thread = threading.Thread(target=worker)
    thread.start()
    assert ready.wait(10)
    assert kermac.get_l2_mode() == kermac.DEFAULT_L2_MODE             # the other thread's block does not leak
    with kermac.l2_mode("gram", trust=0.5):
        assert kermac.get_l2_mode() == "gram"
        plan = _plan_run_kernel(kermac.kernel_descriptor_l2_norm, torch.zeros(4, 64), torch.zeros(4, 64), None, None,
                                None, None, None, None, None, 0, 0, False, require_device=False)
        assert plan.params.flags & _backend.FLAG_L2_GRAM and not plan.params.flags & _backend.FLAG_L2_GRAM_BF16
        assert plan.params.gram_trust == 0.5
        with kermac.l2_mode("direct"):
            assert kermac.get_l2_mode() == "direct"
        assert kermac.get_l2_mode() == "gram"
    release.set()
    thread.join()
    assert seen == {"worker_inside": "gram_bf16", "worker_after": kermac.DEFAULT_L2_MODE}
    assert kermac.get_l2_mode() == kermac.DEFAULT_L2_MODE
    with pytest.raises(ValueError):
        with kermac.l2_mode("fast"):
            pass


def test_cut_decision_for_a_tall_narrow_result():
    """cdist(a[100000, 4096], b[100, 4096]) with the default row-major result reaches the kernel as
    m = 100, n = 100000 (operands exchanged): 782 tiles, so the cut over k is taken; the finishing
    step strides over the rows, so there is no limit of 65535 on n."""
    from kermac_amd import build_a_kernel as module
    plan = _plan_run_kernel(kermac.kernel_descriptor_l1_norm, torch.empty(100000, 4096, device="meta"),
                            torch.empty(100, 4096, device="meta"), torch.empty(100000, 100, device="meta"), None, None,
                            None, None, None, None, 0, 0, False, require_device=False)
    assert plan.swapped and (plan.params.m, plan.params.n) == (100, 100000)
    cut = module._cut_over_contraction(plan.params)
    assert cut is not None and cut[0] * cut[1] >= 4096 and cut[1] % 16 == 0


def test_scratch_memory_is_handed_out_within_the_limit_or_from_the_callers_buffer():
    """kermac_amd/_scratch.py on host memory: the limit counts per outermost operator call, a supplied buffer is
    handed out from its start at 256-byte aligned addresses by every call, what does not fit is refused."""
    import torch
    from kermac_amd import _scratch
    cpu = torch.device("cpu")
    assert _scratch.get_max_scratch_bytes() is None
    with _scratch.operator_call():
        assert _scratch.allocate(1000, cpu).numel() == 1000
    _scratch.set_max_scratch_bytes(4096)
    try:
        with _scratch.operator_call():
            assert _scratch.allocate(3000, cpu) is not None
            with _scratch.operator_call():                       # an operator called by an operator shares the budget
                assert _scratch.allocate(2000, cpu) is None
                assert _scratch.allocate_floats((16, 16), cpu).shape == (16, 16)
            assert _scratch.allocate(100, cpu) is None
        with _scratch.operator_call():                           # the next call starts afresh
            assert _scratch.allocate(4096, cpu) is not None
        _scratch.set_max_scratch_bytes(0)
        with _scratch.operator_call():
            assert _scratch.allocate(1, cpu) is None
    finally:
        _scratch.set_max_scratch_bytes(None)
    buffer = torch.empty(5000, dtype=torch.uint8)
    with _scratch.scratch(buffer):
        for _ in range(2):
            with _scratch.operator_call():
                first = _scratch.allocate(1000, cpu)
                second = _scratch.allocate(2000, cpu)
                assert first.data_ptr() % 256 == 0 and second.data_ptr() % 256 == 0
                assert buffer.data_ptr() <= first.data_ptr() and second.data_ptr() + 2000 <= buffer.data_ptr() + 5000
                assert second.data_ptr() >= first.data_ptr() + 1000
                assert _scratch.allocate(3000, cpu) is None
        with _scratch.operator_call():
            assert _scratch.allocate(100, torch.device("meta")) is None     # another device than the buffer's
    with _scratch.operator_call():
        assert _scratch.allocate(6000, cpu) is not None          # outside the block: torch's allocator again


def test_the_dispatch_table_of_the_design_is_the_generated_one():
    """One source of truth for "which kernel runs when": the thresholds live in csrc/host/dispatch_rules.hpp (read by the
    library's rules, printed by kmc_dispatch_rules) and in the Python layer's module constants; kermac_amd.dispatch renders the
    table from them, and the copy in the design document at the repository root must be that rendering.  The rules themselves
    must flip at the printed numbers."""
    from kermac_amd import dispatch
    known = dispatch.rules()
    table = dispatch.table_markdown()
    design = (ROOT / "DESIGN.md").read_text()
    assert table in design, "the design document's copy of the dispatch table is stale: regenerate it with `python -m kermac_amd.dispatch`"
    header = (ROOT / "include" / "kermac_amd.h").read_text()
    assert "kmc_dispatch_rules" in header and "147456" not in header and "36864" not in header      # pointed to, not restated
    fake = 4096

    def wants_workspace(m, n, k, inner_power, flags, l=1):
        params = _backend.BuildKernelParams()
        params.inner_operator, params.inner_power = 0, inner_power
        params.m, params.n, params.k, params.l = m, n, k, l
        params.a, params.a_ld, params.a_bs = fake, m, m * k
        params.b, params.b_ld, params.b_bs = fake + 4 * m * k * l, n, n * k
        params.c_ld, params.c_bs = m, m * n
        params.flags = flags
        return _backend.gram_workspace_bytes(params) > 0

    wide = _backend.FLAG_L2_GRAM | _backend.FLAG_L2_GRAM_BF16
    side = 256 * 12                                                     # 144 tiles of 256 x 256
    assert known["WIDE_MIN_TILES"] <= 144 < known["WIDE_TILES_FOR_ANY_K"]
    k_needed = -(-known["WIDE_MIN_TILES_TIMES_K"] // 144)
    assert wants_workspace(side, side, k_needed, 2, wide) and not wants_workspace(side, side, k_needed - 1, 2, wide)
    assert not wants_workspace(8192, 8192, known["WIDE_MIN_K"] - 1, 2, wide) and wants_workspace(8192, 8192, known["WIDE_MIN_K"], 2, wide)
    rows = 128 * 46                                                     # 46 x 46 = 2116 tiles of 128 x 128
    assert known["L1_FIXED_MIN_TILES"] <= 2116
    assert wants_workspace(rows, rows, known["L1_FIXED_MIN_K"], 1, _backend.FLAG_L1_FIXED)
    assert not wants_workspace(rows, rows, known["L1_FIXED_MIN_K"] - 1, 1, _backend.FLAG_L1_FIXED)
    assert not wants_workspace(128 * 45, 128 * 45, 512, 1, _backend.FLAG_L1_FIXED) and 45 * 45 < known["L1_FIXED_MIN_TILES"]
