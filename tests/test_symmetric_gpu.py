"""x-against-x matrices: when both operands are the same panel the library computes
only the tiles on and below the diagonal and stores each twice.  The result must be
bit-identical to the full computation (same call with a copy of x as the second
operand, which does not alias and therefore takes the ordinary path), symmetric,
and within tolerance of the oracle; calls that only look similar must not take the
shortcut.  All calls go through the public operators and the C ABI.
"""
import pytest
import torch

import kermac_amd as kermac
from oracle import oracle
from tests.helpers import assert_close_to_truth

pytestmark = pytest.mark.gpu

DESCRIPTORS = {
    "l1": (kermac.kernel_descriptor_l1_norm, {}, ("DIFF", "ABS", "NOOP", "NONE"), {}),
    "l2": (kermac.kernel_descriptor_l2_norm, {}, ("DIFF", "SQUARE", "SQRT", "NONE"), {}),
    "p1.3": (kermac.kernel_descriptor_p_norm, {"p": 1.3}, ("DIFF", "POW", "POW", "NONE"),
             {"p_inner": 1.3, "p_outer": 1.0 / 1.3}),
    "p3": (kermac.kernel_descriptor_p_norm, {"p": 3.0}, ("DIFF", "POW", "POW", "NONE"),
           {"p_inner": 3.0, "p_outer": 1.0 / 3.0}),
    "laplace_l1_reg": (kermac.kernel_descriptor_laplace_l1, {"bandwidth": 9.0, "regularization": 0.5},
                       ("DIFF", "ABS", "NOOP", "LAPLACE"), {"bandwidth": 9.0, "regularization": 0.5}),
    "dot": (kermac.kernel_descriptor_mma, {}, ("DOT", "NOOP", "NOOP", "NONE"), {}),
}


@pytest.fixture(params=["direct", "gram", "gram_bf16"])
def l2_mode(request):
    kermac.set_l2_mode(request.param, min_k=0)
    yield request.param
    kermac.set_l2_mode(kermac.DEFAULT_L2_MODE)


@pytest.mark.parametrize("name", list(DESCRIPTORS))
@pytest.mark.parametrize("rows,K,col_major", [(129, 20, True), (700, 48, True), (515, 33, False), (1024, 64, False)])
def test_self_matrix_equals_the_full_computation(device, name, rows, K, col_major):
    descriptor, kwargs, oracle_descriptor, oracle_kwargs = DESCRIPTORS[name]
    g = torch.Generator().manual_seed(rows + K)
    x = torch.randn(K, rows, generator=g).to(device).t() if col_major else torch.randn(rows, K, generator=g).to(device)
    copy = x.clone(memory_format=torch.preserve_format)          # same values and strides, other memory
    for out_col_major in (True, False):
        store = torch.full((rows, rows + 4), float("nan"), device=device)
        out = store[:, :rows].t() if out_col_major else store[:, :rows]
        got = kermac.run_kernel(descriptor, x, x, out=out, **kwargs)
        full = kermac.run_kernel(descriptor, x, copy, **kwargs)[0]
        assert torch.equal(got, full), f"{name}: shortcut differs from the full computation"
        assert torch.equal(got, got.t()), f"{name}: not symmetric"
        assert torch.isnan(store[:, rows:]).all(), "wrote outside the out view"
    truth = oracle.build_kernel(*oracle_descriptor, x.cpu().contiguous(), x.cpu().contiguous(), **oracle_kwargs)[0]
    fractional = "POW" in oracle_descriptor
    atol = 1e-5 * float(x.norm(dim=1).mean()) ** 2 if name == "dot" else 0.0
    assert_close_to_truth(got, truth, rtol=1e-4 if fractional else 1e-5, atol=atol, what=f"self matrix {name}")


def test_batched_self_matrix_and_matrix_core_mode(device, l2_mode):
    g = torch.Generator().manual_seed(11)
    L, rows, K = 3, 400, 40
    x = torch.randn(L, K, rows, generator=g).to(device).transpose(1, 2)
    bw = torch.tensor([5.0, 9.0, 14.0], device=device)
    got = kermac.run_kernel(kermac.kernel_descriptor_laplace_l2, x, x, bandwidth=bw, regularization=1e-3)
    full = kermac.run_kernel(kermac.kernel_descriptor_laplace_l2, x, x.clone(memory_format=torch.preserve_format),
                             bandwidth=bw, regularization=1e-3)
    assert torch.equal(got, got.transpose(1, 2))
    if l2_mode == "gram_bf16":
        # the six piece products are summed in an order that is not symmetric in a and b, so the
        # full computation is symmetric only up to rounding; the shortcut mirrors one half exactly
        torch.testing.assert_close(got, full, rtol=2e-6, atol=1e-7)
    else:
        assert torch.equal(got, full)
    truth = oracle.build_kernel("DIFF", "SQUARE", "SQRT", "LAPLACE", x.cpu().contiguous(), x.cpu().contiguous(),
                                bandwidth=bw.cpu(), regularization=1e-3)
    assert_close_to_truth(got, truth, rtol=1e-5, atol=1e-7, what=f"batched self matrix, l2 mode {l2_mode}")
    # near-duplicate rows: in matrix-core mode these tiles are recomputed, and mirrored, by the repair launch
    y = torch.randn(300, 24, generator=g).to(device)
    y[150:] = y[:150] + 1e-4 * torch.randn(150, 24, generator=g).to(device)
    d_self = kermac.cdist(y, y, p=2.0)[0]
    d_full = kermac.cdist(y, y.clone(), p=2.0)[0]
    assert torch.equal(d_self, d_self.t())
    if l2_mode == "gram_bf16":
        torch.testing.assert_close(d_self, d_full, rtol=2e-6, atol=1e-7)
    else:
        assert torch.equal(d_self, d_full)
    assert_close_to_truth(d_self, oracle.cdist(y.cpu(), y.cpu(), p=2.0)[0], rtol=1e-5, what="near duplicates")


def test_lookalikes_take_the_ordinary_path(device):
    g = torch.Generator().manual_seed(12)
    rows, K = 300, 16
    x = torch.randn(rows, K, generator=g).to(device)
    # signed inner term: antisymmetric, must not be mirrored
    signed = kermac.KernelDescriptor(kermac.InnerOperator.DIFF, kermac.PowerType.NOOP, kermac.PowerType.NOOP,
                                     kermac.KernelType.NONE)
    got = kermac.run_kernel(signed, x, x)[0]
    truth = (x.double()[:, None] - x.double()[None]).sum(-1)          # sum_k (a[m] - b[n])
    assert_close_to_truth(got, truth, rtol=1e-5, atol=1e-5, what="signed self differences")
    assert torch.equal(got, -got.t())
    # different regularisation offsets: the replaced diagonal is not symmetric
    got = kermac.run_kernel(kermac.kernel_descriptor_laplace_l1, x, x, bandwidth=4.0, regularization=0.25,
                            regularization_offset_x=130, regularization_offset_y=0)[0]
    truth = oracle.run_kernel("DIFF", "ABS", "NOOP", "LAPLACE", x.cpu(), x.cpu(), bandwidth=4.0, regularization=0.25,
                              regularization_offset_x=130, regularization_offset_y=0)[0]
    assert_close_to_truth(got, truth, rtol=1e-5, atol=1e-7, what="offset diagonal")
    assert not torch.equal(got, got.t())
    # same pointer but another extent: rows of one panel against a prefix of it
    got = kermac.cdist(x, x[:140], p=1.0)[0]
    assert_close_to_truth(got, oracle.cdist(x.cpu(), x[:140].cpu(), p=1.0)[0], rtol=1e-5, what="prefix")
    # same pointer, same extent, other leading dimension (every second row of a larger store)
    wide = torch.randn(rows, 2 * K, generator=g).to(device)
    left, both = wide[:, :K], wide.view(2 * rows, K)[:rows]          # both start at the same address
    assert left.data_ptr() == both.data_ptr()
    got = kermac.cdist(left, both, p=1.0)[0]
    assert_close_to_truth(got, oracle.cdist(left.cpu().contiguous(), both.cpu().contiguous(), p=1.0)[0], rtol=1e-5,
                          what="same address, different strides")


def test_switch_off(device, monkeypatch):
    g = torch.Generator().manual_seed(13)
    x = torch.randn(32, 500, generator=g).to(device).t()
    fast = kermac.cdist(x, x, p=1.0)
    monkeypatch.setenv("KERMAC_AMD_NO_SYMMETRY", "1")
    slow = kermac.cdist(x, x, p=1.0)
    assert torch.equal(fast, slow)
