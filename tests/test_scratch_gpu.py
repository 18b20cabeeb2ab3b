"""What the operators allocate beside `out`, and the two controls over it (kermac_amd/_scratch.py): with the limit
at 0 a call allocates nothing -- the reference's contract (README.md:69,135: "aside from `out` ... does not allocate")
-- and inside `kermac.scratch(buffer)` it takes its buffers from the caller's memory and allocates nothing either.
Allocations are counted by torch's allocator statistics around the call.
"""
import pytest
import torch

import kermac_amd as kermac
from tests.helpers import assert_close_to_truth, l1_distances_float64

pytestmark = pytest.mark.gpu


def allocations(device):
    return torch.cuda.memory_stats(device)["allocation.all.allocated"]


def counted(device, fn):
    torch.cuda.synchronize(device)
    before = allocations(device)
    result = fn()
    torch.cuda.synchronize(device)
    return result, allocations(device) - before


@pytest.fixture
def cases(device):
    """Three default-mode calls that take a workspace route when they are given the memory: squared distances,
    the L1 gradient, a Gaussian kernel matrix times coefficients (panels)."""
    g = torch.Generator().manual_seed(31)
    a = torch.randn(512, 4096, generator=g).to(device).t()
    b = torch.randn(512, 4096, generator=g).to(device).t()
    out = torch.empty(4096, 4096, device=device).t()
    kernel = torch.rand(2048, 2048, generator=g).to(device)
    x = (torch.randn(512, 2048, generator=g) / 512 ** 0.5).to(device)
    coefs = torch.randn(16, 2048, generator=g).to(device)
    z = (torch.randn(512, 2048, generator=g) / 512 ** 0.5).to(device)
    grad = torch.empty(1, 16, 512, 2048, device=device)
    coefficients = torch.randn(4096, 32, generator=g).to(device)
    product = torch.empty(4096, 32, device=device)
    gaussian = kermac.KernelDescriptor(kermac.InnerOperator.DIFF, kermac.PowerType.SQUARE, kermac.PowerType.NOOP,
                                       kermac.KernelType.GAUSSIAN)
    calls = {
        "cdist p=2": lambda: kermac.cdist(a, b, out=out, p=2.0),
        "cdist_grad p=1": lambda: kermac.cdist_grad(kernel, x, coefs, z, out=grad, p=1.0),
        "gaussian x coefficients": lambda: kermac.run_kernel(gaussian, a, b, out=product, bandwidth=30.0, coefficients=coefficients),
    }
    for call in calls.values():
        call()                      # kernels loaded, allocator warm
    return calls


def test_default_calls_do_allocate(device, cases):
    for name, call in cases.items():
        _, count = counted(device, call)
        assert count > 0, f"{name}: the default route was expected to take a workspace"


def test_limit_zero_allocates_nothing(device, cases):
    reference = {name: call().clone() for name, call in cases.items()}
    kermac.set_max_scratch_bytes(0)
    try:
        assert kermac.get_max_scratch_bytes() == 0
        for name, call in cases.items():
            result, count = counted(device, call)
            assert count == 0, f"{name}: {count} allocations with the limit at 0"
            # another route (no workspace), the same tolerance: close to the default route's result
            scale = reference[name].abs().mean().item()
            assert (result - reference[name]).abs().max().item() <= 2e-5 * max(scale, 1e-30) * (50 if "grad" in name or "coeff" in name else 1), name
    finally:
        kermac.set_max_scratch_bytes(None)
    assert kermac.get_max_scratch_bytes() is None


def test_supplied_buffer_allocates_nothing_and_takes_the_same_routes(device, cases):
    reference = {name: call().clone() for name, call in cases.items()}
    buffer = torch.empty(3 << 30, dtype=torch.uint8, device=device)
    with kermac.scratch(buffer):
        for name, call in cases.items():
            result, count = counted(device, call)
            assert count == 0, f"{name}: {count} allocations inside scratch(buffer)"
            assert torch.equal(result, reference[name]), f"{name}: the route with the caller's buffer gives other bits"
    # a buffer that is too small for anything: the calls do without, still without allocating
    tiny = torch.empty(1024, dtype=torch.uint8, device=device)
    with kermac.scratch(tiny):
        for name, call in cases.items():
            _, count = counted(device, call)
            assert count == 0, name
    with pytest.raises(TypeError):
        with kermac.scratch(torch.empty(16, device=device)):
            pass


def test_fixed_point_route_and_cut_launches_respect_the_limit(device):
    g = torch.Generator().manual_seed(32)
    a = torch.randn(2048, 700, generator=g).to(device)          # 6 x 6 tiles over k = 2048: cut over k by default
    b = torch.randn(2048, 650, generator=g).to(device)
    a, b = a.t(), b.t()
    out = torch.empty(650, 700, device=device).t()
    kermac.cdist(a, b, out=out, p=1.0)
    _, count = counted(device, lambda: kermac.cdist(a, b, out=out, p=1.0))
    assert count > 0
    kermac.set_max_scratch_bytes(0)
    try:
        _, count = counted(device, lambda: kermac.cdist(a, b, out=out, p=1.0))
        assert count == 0
        assert_close_to_truth(out, l1_distances_float64(a, b), rtol=1e-5, what="uncut launch")
        with kermac.l1_mode("fixed"):
            _, count = counted(device, lambda: kermac.cdist(a, b, out=out, p=1.0))
            assert count == 0
    finally:
        kermac.set_max_scratch_bytes(None)
