"""Seeded random sweeps of the three operators against the CPU oracle (float64
mode): shapes, batch sizes, broadcasting, storage orders, misalignment, padding,
descriptors and hyper-parameters are drawn at random, a few dozen cases per test.
All calls go through the public operators and therefore through the C ABI.

Tolerances as in the other parity tests: 1e-5 where no fractional power is
involved, 1e-4 otherwise; kernel values in [0, 1] get an absolute floor because
exp() turns a relative error of the distance into an absolute one.
"""
import random

import pytest
import torch

import kermac_amd as kermac
from oracle import oracle
from tests.helpers import assert_close_to_truth

pytestmark = pytest.mark.gpu


@pytest.fixture(autouse=True, params=["as launched", "workspace routes"])
def routes(request, monkeypatch):
    """Every sweep twice: as the library launches these small shapes by itself, and with the routes
    that go through a workspace forced onto them (squared differences, their products with
    coefficients panel by panel, and the L1 and L2 gradients on the fp16 matrix instruction, which
    by themselves only take large problems)."""
    if request.param == "workspace routes":
        monkeypatch.setenv("KERMAC_AMD_WIDE_MIN_TILES", "1")
        monkeypatch.setenv("KERMAC_AMD_GRADIENT_F16_MIN_TERMS", "1")
        monkeypatch.setenv("KERMAC_AMD_GRADIENT_L2_MIN_TERMS", "1")
        monkeypatch.setenv("KERMAC_AMD_COEFFICIENT_PANEL_BYTES", "4096")     # products in panels of 256 centres
        kermac.set_l2_mode("gram_bf16", min_k=0)
    yield
    kermac.set_l2_mode(kermac.DEFAULT_L2_MODE)

POWERS = {"NOOP": kermac.PowerType.NOOP, "ABS": kermac.PowerType.ABS, "SQUARE": kermac.PowerType.SQUARE,
          "SQRT": kermac.PowerType.SQRT, "POW": kermac.PowerType.POW}
KERNELS = {"NONE": kermac.KernelType.NONE, "LAPLACE": kermac.KernelType.LAPLACE, "GAUSSIAN": kermac.KernelType.GAUSSIAN}


def random_view(rng, gen, device, L, rows, cols, positive=False):
    """A [L?, rows, cols] fp32 device view with random storage order, padding of the
    leading dimension, misaligned base and, for L == 1, a random choice of 2-D or
    3-D shape.  Returns (device view, identical CPU tensor)."""
    col_major = rng.random() < 0.5
    pad = rng.choice([0, 0, 1, 3, 4])
    shift = rng.choice([0, 0, 1, 2])
    inner, outer = (rows, cols) if col_major else (cols, rows)
    batch = L if L > 1 else rng.choice([0, 1])
    lead = max(batch, 1)
    store = torch.rand if positive else torch.randn
    flat = store(lead * outer * (inner + pad) + shift, generator=gen, dtype=torch.float32)
    cpu = flat[shift:].view(lead, outer, inner + pad)[:, :, :inner]
    dev = flat.to(device)[shift:].view(lead, outer, inner + pad)[:, :, :inner]
    if col_major:
        cpu, dev = cpu.transpose(1, 2), dev.transpose(1, 2)
    if batch == 0:
        cpu, dev = cpu[0], dev[0]
    return dev, cpu.contiguous()


@pytest.mark.parametrize("seed", range(6))
def test_run_kernel_random_descriptors_and_layouts(device, seed):
    rng = random.Random(1000 + seed)
    gen = torch.Generator().manual_seed(2000 + seed)
    for case in range(8):
        L = rng.choice([1, 1, 2, 3])
        M, N, K = rng.randint(1, 290), rng.randint(1, 290), rng.randint(1, 70)
        if L == 1 and rng.random() < 0.3:            # a small result over a long contraction: cut over k
            M, N, K = rng.randint(1, 100), rng.randint(1, 100), rng.randint(512, 2500)
        inner_op = rng.choice(["DIFF", "DIFF", "DIFF", "DOT"])
        inner_pow = rng.choice(["ABS", "SQUARE", "POW", "NOOP"]) if inner_op == "DIFF" else "NOOP"
        outer_pow = rng.choice(["NOOP", "SQRT", "POW", "ABS", "SQUARE"])
        kernel = rng.choice(["NONE", "NONE", "LAPLACE", "GAUSSIAN"])
        if inner_pow == "NOOP":                      # signed sums: keep the outer power defined for negatives
            outer_pow = rng.choice(["NOOP", "ABS", "SQUARE"])
            kernel = "NONE"
        La, Lb = (L, rng.choice([1, L])) if rng.random() < 0.5 else (rng.choice([1, L]), L)
        a, a_cpu = random_view(rng, gen, device, La, M, K)
        b, b_cpu = random_view(rng, gen, device, Lb, N, K)
        kwargs, okwargs = {}, {}
        if inner_pow == "POW":
            p_in = rng.choice([0.5, 0.7, 1.3, 1.5, 2.5, 3.0])
            if rng.random() < 0.4 and L > 1:
                t = torch.tensor([p_in + 0.1 * i for i in range(L)])
                kwargs["inner_p"], okwargs["p_inner"] = t.to(device), t
            else:
                kwargs["inner_p"], okwargs["p_inner"] = p_in, p_in
        if outer_pow == "POW":
            p_out = rng.choice([0.5, 1.0 / 1.3, 2.0])
            kwargs["outer_p"], okwargs["p_outer"] = p_out, p_out
        if kernel != "NONE":
            bw = rng.choice([3.0, 20.0, 150.0])
            reg = rng.choice([0.0, 0.5])
            if rng.random() < 0.4 and L > 1:
                t = torch.tensor([bw * (1 + i) for i in range(L)])
                kwargs["bandwidth"], okwargs["bandwidth"] = t.to(device), t
            else:
                kwargs["bandwidth"], okwargs["bandwidth"] = bw, bw
            kwargs["regularization"], okwargs["regularization"] = reg, reg
            off = (rng.randint(0, 5), rng.randint(0, 5))
            kwargs["regularization_offset_x"], kwargs["regularization_offset_y"] = off
            okwargs["regularization_offset_x"], okwargs["regularization_offset_y"] = off
        descriptor = kermac.KernelDescriptor(getattr(kermac.InnerOperator, inner_op), POWERS[inner_pow],
                                             POWERS[outer_pow], KERNELS[kernel])
        out = None
        if rng.random() < 0.5:                        # caller-supplied result, either storage order, padded
            out, _ = random_view(rng, gen, device, L, M, N)
            if out.dim() == 2:
                out = out.unsqueeze(0)
        what = f"seed {seed} case {case}: {descriptor} L={L} M={M} N={N} K={K} {kwargs.keys()}"
        print(what, flush=True)
        got = kermac.run_kernel(descriptor, a, b, out=out, **kwargs)
        truth = oracle.run_kernel(inner_op, inner_pow, outer_pow, kernel, a_cpu, b_cpu, **okwargs)
        fractional = inner_pow == "POW" or outer_pow == "POW"
        rtol = 1e-4 if fractional else 1e-5
        # signed sums and dot products cancel: measure against the sum of magnitudes
        atol = 1e-7 if kernel != "NONE" else 0.0
        if inner_pow == "NOOP":
            scale = float((a_cpu.abs().sum(-1).mean() + b_cpu.abs().sum(-1).mean())) if inner_op == "DIFF" else \
                float((a_cpu.norm(dim=-1).mean() * b_cpu.norm(dim=-1).mean()))
            atol = 1e-5 * (scale ** (2 if outer_pow == "SQUARE" else 1))
        assert_close_to_truth(got, truth.view(got.shape), rtol=rtol, atol=atol, what=what)


@pytest.mark.parametrize("seed", range(4))
def test_cdist_grad_random_shapes_and_batches(device, seed):
    rng = random.Random(3000 + seed)
    gen = torch.Generator().manual_seed(4000 + seed)
    for case in range(8):
        L = rng.choice([1, 1, 2, 3])
        M, N, K = rng.randint(1, 200), rng.randint(1, 70), rng.randint(1, 90)
        if L == 1 and rng.random() < 0.3:            # few results over a deep contraction: cut over k
            M, N, K = rng.randint(1, 100), rng.randint(1, 40), rng.randint(2048, 4000)
        O = rng.choice([1, 2, 4, 5, 8, 9, 16, 17, 32, 40])
        p = rng.choice([1.0, 2.0, 1.3, 0.7, 3.0])

        def operand(rows, cols, positive=False, batch=None):
            lead = L if batch is None else batch
            pad = rng.choice([0, 0, 1, 4])
            store = (torch.rand if positive else torch.randn)(lead, rows, cols + pad, generator=gen)
            cpu = store[:, :, :cols]
            dev = store.to(device)[:, :, :cols]
            if lead == 1 and rng.random() < 0.5:
                cpu, dev = cpu[0], dev[0]
            return dev, cpu.contiguous()

        a, a_cpu = operand(K, M, positive=True)
        b, b_cpu = operand(N, K, batch=rng.choice([1, L]))
        c, c_cpu = operand(O, K, batch=rng.choice([1, L]))
        d, d_cpu = operand(N, M)
        what = f"seed {seed} case {case}: L={L} M={M} N={N} O={O} K={K} p={p}"
        print(what, flush=True)
        got = kermac.cdist_grad(a, b, c, d, p=p)
        truth = oracle.cdist_grad(a_cpu, b_cpu, c_cpu, d_cpu, p=p)
        rtol = 1e-5 if p in (1.0, 2.0) else 1e-4
        assert_close_to_truth(got, truth, rtol=rtol, atol=rtol * float(truth.abs().mean()) * 10 + 1e-30, what=what)


@pytest.mark.parametrize("seed", range(3))
def test_fused_coefficients_random(device, seed):
    rng = random.Random(5000 + seed)
    gen = torch.Generator().manual_seed(6000 + seed)
    for case in range(6):
        L = rng.choice([1, 2, 3])
        M, N, K = rng.randint(1, 300), rng.randint(1, 700), rng.randint(1, 60)
        O = rng.choice([1, 3, 16, 32, 33, 70])
        name, inner_pow, outer_pow, kernel = rng.choice([
            ("laplace_l1", "ABS", "NOOP", "LAPLACE"), ("laplace_l2", "SQUARE", "SQRT", "LAPLACE"),
            ("gaussian", "SQUARE", "NOOP", "GAUSSIAN"), ("p_norm", "POW", "POW", "LAPLACE")])
        a, a_cpu = random_view(rng, gen, device, rng.choice([1, L]), M, K)
        b, b_cpu = random_view(rng, gen, device, L, N, K)
        coef = torch.randn(L, N, O, generator=gen)
        kwargs, okwargs = {"bandwidth": 12.0}, {"bandwidth": 12.0}
        if inner_pow == "POW":
            kwargs["p"] = 1.4
            okwargs["p_inner"], okwargs["p_outer"] = 1.4, 1.0 / 1.4
        descriptor = kermac.KernelDescriptor(kermac.InnerOperator.DIFF, POWERS[inner_pow], POWERS[outer_pow],
                                             KERNELS[kernel])
        what = f"seed {seed} case {case}: {name} L={L} M={M} N={N} K={K} O={O}"
        print(what, flush=True)
        got = kermac.run_kernel(descriptor, a, b, coefficients=coef.to(device), **kwargs)
        truth = oracle.kernel_times_coefficients("DIFF", inner_pow, outer_pow, kernel, a_cpu, b_cpu, coef, **okwargs)
        # a sum of N signed products of magnitude <= |coef|: error relative to sqrt(N) * typical |coef|
        assert_close_to_truth(got, truth.view(got.shape), rtol=1e-4, atol=2e-5 * (N ** 0.5), what=what)
