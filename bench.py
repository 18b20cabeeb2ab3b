#!/usr/bin/env python3
"""Benchmark of the fused distance hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

One "step" is one ``kermac_amd.cdist`` call on the headline configuration:
a_store[K=1024, M=30000], b_store[K=1024, N=30000] ~ N(0,1) (seed 1), passed as
K-major panels, out_store[N, M] fp32 (3.6 GB), p = 1.0.  Inputs and the output
buffer are resident in HBM before the timed region.  The same data is then timed
for p = 2.0 (the default mode, which puts this problem on the matrix cores, and the
vector-ALU kernel by name) and p = 1.3 (with and without the 1/p epilogue) and reported in
``per_p``; ``other_configs`` holds the gradient and the fused kernel-matrix x coefficients
configurations.  Work is counted as 3 fp32 operations per (m, n, k) -- subtract,
power, accumulate -- i.e. 3*M*N*K = 2.7648e12 per call, against the published
fp32 vector peak of 157.3 TFLOP/s.  The last leg times torch.cdist on the host cores.

Prints ONE JSON line on stdout; progress goes to stderr.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

import torch

M = N = 30000
K = 1024
OPS_PER_CALL = 3.0 * M * N * K
ALGORITHMIC_BYTES = 4.0 * (M * K + N * K + M * N)
PEAK_FP32_VALU_TFLOPS = 157.3        # AMD's published MI355X fp32 vector peak
PEAK_HBM_GBPS = 8000.0

# HBM bytes per p = 1 cdist launch come from the rocprofv3 summary of this kernel under profiles/
# (two --pmc runs, FETCH_SIZE and WRITE_SIZE, each scaled by what the counter reads for a 1 GiB
# copy kernel).  The file ends with "key = value" lines; nothing is pasted here.
TRAFFIC_PROFILE = os.path.join(os.path.dirname(os.path.abspath(__file__)), "profiles",
                               "build_kernel_cdist_p1_30000x30000x1024.txt")


def measured_traffic():
    """(bytes per launch or None, where the figure comes from)."""
    fields = {}
    try:
        with open(TRAFFIC_PROFILE) as handle:
            for text in handle:
                key, sep, value = text.partition("=")
                if sep and key.strip() in ("traffic_bytes_per_launch", "measured_at_commit", "shader_clock_mhz"):
                    fields[key.strip()] = value.strip()
        return float(fields["traffic_bytes_per_launch"]), {
            "file": "profiles/" + os.path.basename(TRAFFIC_PROFILE), "commit": fields.get("measured_at_commit"),
            "shader_clock_mhz": float(fields["shader_clock_mhz"]) if "shader_clock_mhz" in fields else None}
    except (OSError, KeyError, ValueError):
        return None, None


# What the vector ALU issues on registers alone (bench_issue_rates.hip): read from the summary of that program's
# run under profiles/, "key = value" lines at its end; nothing is pasted here.
ISSUE_PROFILE = os.path.join(os.path.dirname(os.path.abspath(__file__)), "profiles", "valu_issue_rates_gfx950.txt")


def issue_rates():
    """{key: float} of the "key = value" lines of the issue-rate summary; {} when the file is missing."""
    rates = {}
    try:
        with open(ISSUE_PROFILE) as handle:
            for text in handle:
                key, sep, value = text.partition("=")
                if sep:
                    try:
                        rates[key.strip()] = float(value)
                    except ValueError:
                        pass
    except OSError:
        pass
    return rates


def log(*args):
    print(*args, file=sys.stderr, flush=True)


def time_cdist(kermac, a, b, out, p, skip_epilogue, steps, warmup):
    """(wall ms per step, mean kernel ms from events on the launch stream)."""
    for _ in range(warmup):
        kermac.cdist(a, b, out=out, p=p, skip_epilogue=skip_epilogue)
    torch.cuda.synchronize()
    starts = [torch.cuda.Event(enable_timing=True) for _ in range(steps)]
    stops = [torch.cuda.Event(enable_timing=True) for _ in range(steps)]
    t0 = time.perf_counter()
    for i in range(steps):
        starts[i].record()
        kermac.cdist(a, b, out=out, p=p, skip_epilogue=skip_epilogue)
        stops[i].record()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3 / steps
    kernel_ms = sum(s.elapsed_time(e) for s, e in zip(starts, stops)) / steps
    return wall_ms, kernel_ms


DEFAULT_SLABS = ((slice(0, 256), slice(0, 2048)), (slice(29900, 30000), slice(29744, 30000)))
# for a matrix of a set against itself: one slab above and one below the diagonal, none on it (0 / 0)
OFF_DIAGONAL_SLABS = ((slice(0, 256), slice(2048, 4096)), (slice(29900, 30000), slice(100, 2148)))


def parity_slab(out, a, b, p, skip_epilogue, slabs=DEFAULT_SLABS):
    """Max relative error of a float64 slab (torch.cdist on the GPU in fp64)."""
    worst = 0.0
    for ms, ns in slabs:
        truth = torch.cdist(a[ms].double(), b[ns].double(), p=p)
        if skip_epilogue:
            truth = truth ** p
        got = out[ms, ns].double()
        worst = max(worst, ((got - truth).abs() / truth.abs()).max().item())
    return worst


def cpu_baseline(a_store_cpu, b_store_cpu, slab=16384):
    """torch.cdist (the oracle of the reference's tests, tests/test_cdist.py:75) on the host cores, on
    bounded slabs of the same workload.  p = 1 (the headline) and p = 2: all of a against the first
    `slab` columns of b, once after a warm-up.  p = 1.3 costs a pow per term: 4096 rows of a against
    2048 columns of b, the median of three runs.  Every figure is scaled to the full problem by the
    ratio of the pair counts and labelled as scaled."""
    a = a_store_cpu.t()
    torch.cdist(a[:2048], b_store_cpu[:, :256].t(), p=1.0)                      # warm the thread pool

    def timed(rows, cols, p, repeats):
        b = b_store_cpu[:, :cols].t()
        seconds = []
        for _ in range(repeats):
            t0 = time.perf_counter()
            torch.cdist(a[:rows], b, p=p)
            seconds.append(time.perf_counter() - t0)
        seconds.sort()
        return seconds[len(seconds) // 2]

    per_p = {}
    for p, rows, cols, repeats in ((1.0, M, slab, 1), (2.0, M, slab, 1), (1.3, 4096, 2048, 3)):
        seconds = timed(rows, cols, p, repeats)
        scale = (M / rows) * (N / cols)
        per_p[str(p)] = {
            "ms_scaled": round(seconds * 1e3 * scale, 1),
            "sample": (f"torch.cdist p={p} fp32: a[{rows},{K}] x b[{cols},{K}] of the same seeded data, "
                       f"{seconds:.2f} s ({'median of ' + str(repeats) if repeats > 1 else 'one run'}), "
                       f"scaled by {scale:.2f} to the full problem"),
        }
        log(f"  p={p}: {seconds:.2f} s on the sample -> {per_p[str(p)]['ms_scaled']:.0f} ms scaled")
    result = {
        "value": per_p["1.0"]["ms_scaled"],
        "unit": "ms",
        "cores": torch.get_num_threads(),
        "kind": "port",
        "sample": per_p["1.0"]["sample"],
        "per_p": per_p,
        "host_cpu_count": os.cpu_count(),
    }
    # The repository's own C restatement (fp32 mode, OpenMP), on a smaller slab.
    try:
        from oracle import oracle
        small = 256
        t0 = time.perf_counter()
        oracle.cdist(a[:8192], b_store_cpu[:, :small].t(), p=1.0, wide=False)
        sec = time.perf_counter() - t0
        result["oracle_c_ms_scaled"] = round(sec * 1e3 * (M / 8192) * (N / small), 1)
    except Exception as exc:  # the baseline is informational; never fail the bench for it
        result["oracle_c_error"] = repr(exc)
    return result


def calibration_copy(device):
    """One plain elementwise kernel that reads 2^30 bytes and writes 2^30 bytes."""
    src = torch.ones(1 << 28, device=device)
    dst = torch.empty_like(src)
    torch.mul(src, 1.0, out=dst)
    torch.cuda.synchronize()


def time_call(fn, steps, warmup):
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    starts = [torch.cuda.Event(enable_timing=True) for _ in range(steps)]
    stops = [torch.cuda.Event(enable_timing=True) for _ in range(steps)]
    t0 = time.perf_counter()
    for i in range(steps):
        starts[i].record()
        fn()
        stops[i].record()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3 / steps
    return wall_ms, sum(s.elapsed_time(e) for s, e in zip(starts, stops)) / steps


PARITY_FAILURES = []        # what exceeded its tolerance; reported in the JSON line, never a silent exit


def check_parity(what, err, tolerance):
    if not err <= tolerance:             # also catches NaN
        PARITY_FAILURES.append({"what": what, "err": err, "tolerance": tolerance})
        log(f"  PARITY FAILURE: {what}: {err:.3e} > {tolerance}")


def side_line(metric, workload, wall_ms, kernel_ms, ops, algorithmic_bytes, bound, peak, extra, args):
    achieved = ops / kernel_ms / 1e9
    return {
        "metric": metric, "value": round(wall_ms, 3), "unit": "ms", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(wall_ms, 3), "higher_is_better": False, "scaling": "weak",
        "vs_baseline": None, "dtype": "f32", "data": "synthetic", "config": {"workload": workload},
        "roofline": {"bound": bound, "achieved": round(achieved, 2), "peak": peak, "unit": "TFLOP/s",
                     "frac": round(achieved / peak, 4), "traffic": None, "ops_per_launch": ops,
                     "hbm_gbps": round(algorithmic_bytes / kernel_ms / 1e6, 1)},
        **extra,
    }


def bench_cdist_grad(kermac, device, args, steps=None, warmup=None):
    """x[K=512,N=8192], centres z[512,8192] ~ N(0,1)/sqrt(512), c[16,8192] ~ N(0,1), kernel-gradient weights
    g[8192,8192] ~ U(0,1), p = 1: in the operator's names a = g [K_ref=8192, M_ref=8192], b = z [N_ref=512, K_ref],
    c [O=16, K_ref], d = x [N_ref, M_ref], out [O, N_ref, M_ref].  Work (2*O + 3) per (m, n, k)."""
    steps, warmup = steps or args.steps, args.warmup if warmup is None else warmup
    torch.manual_seed(3)
    k_ref, m_ref, n_ref, o = 8192, 8192, 512, 16
    a = torch.rand(k_ref, m_ref, device=device)
    b = torch.randn(n_ref, k_ref, device=device) / 512 ** 0.5
    c = torch.randn(o, k_ref, device=device)
    d = torch.randn(n_ref, m_ref, device=device) / 512 ** 0.5
    out = torch.empty(1, o, n_ref, m_ref, device=device)
    if args.calibration_copy:
        calibration_copy(device)
    wall_ms, kernel_ms = time_call(lambda: kermac.cdist_grad(a, b, c, d, out=out, p=1.0), steps, warmup)
    ms, ns = slice(0, 48), slice(0, 16)
    diff = d[ns, ms].double()[:, :, None] - b[ns].double()[:, None, :]
    sign = torch.where(torch.signbit(diff), -1.0, 1.0).double()
    truth = torch.einsum("ok,km,nmk->onm", c.double(), a[:, ms].double(), sign)
    err = ((out[0][:, ns, ms].double() - truth).abs().max() / truth.abs().mean()).item()
    log(f"cdist_grad p=1: {kernel_ms:.2f} ms kernel, slab max abs err / mean |truth| = {err:.2e}")
    check_parity("cdist_grad p=1 (configs[3]) slab, max abs err / mean |truth|", err, 1e-4)
    # The same call on the fp32 kernels (no workspace), timed beside it.
    saved = os.environ.get("KERMAC_AMD_GRADIENT_WORKSPACE")
    os.environ["KERMAC_AMD_GRADIENT_WORKSPACE"] = "0"
    try:
        _, fp32_ms = time_call(lambda: kermac.cdist_grad(a, b, c, d, out=out, p=1.0), max(2, min(steps, 5)), 1)
        fp32_err = ((out[0][:, ns, ms].double() - truth).abs().max() / truth.abs().mean()).item()
    finally:
        if saved is None:
            del os.environ["KERMAC_AMD_GRADIENT_WORKSPACE"]
        else:
            os.environ["KERMAC_AMD_GRADIENT_WORKSPACE"] = saved
    log(f"  on the fp32 matrix-core kernel: {fp32_ms:.2f} ms, slab max abs err / mean |truth| = {fp32_err:.2e}")
    check_parity("cdist_grad p=1 (configs[3], fp32 kernels) slab, max abs err / mean |truth|", fp32_err, 1e-4)
    # Beside it: the same operands with p = 2 (weights d - b instead of their sign), both routes.
    truth_l2 = torch.einsum("ok,km,nmk->onm", c.double(), a[:, ms].double(), diff)
    side = max(2, min(steps, 5))
    _, l2_ms = time_call(lambda: kermac.cdist_grad(a, b, c, d, out=out, p=2.0), side, 1)
    l2_err = ((out[0][:, ns, ms].double() - truth_l2).abs().max() / truth_l2.abs().mean()).item()
    os.environ["KERMAC_AMD_GRADIENT_WORKSPACE"] = "0"
    try:
        _, l2_fp32_ms = time_call(lambda: kermac.cdist_grad(a, b, c, d, out=out, p=2.0), side, 1)
        l2_fp32_err = ((out[0][:, ns, ms].double() - truth_l2).abs().max() / truth_l2.abs().mean()).item()
    finally:
        if saved is None:
            del os.environ["KERMAC_AMD_GRADIENT_WORKSPACE"]
        else:
            os.environ["KERMAC_AMD_GRADIENT_WORKSPACE"] = saved
    log(f"  p=2, same operands: {l2_ms:.2f} ms (slab err {l2_err:.2e}); on the fp32 matrix-core kernel {l2_fp32_ms:.2f} ms ({l2_fp32_err:.2e})")
    check_parity("cdist_grad p=2 slab, max abs err / mean |truth|", l2_err, 1e-4)
    check_parity("cdist_grad p=2 (fp32 kernels) slab, max abs err / mean |truth|", l2_fp32_err, 1e-4)
    # Beside it: 32 outputs, p = 1 (the tile of 16 n x 32 outputs: the sign work is shared by two blocks of outputs).
    c32 = torch.randn(32, k_ref, device=device)
    out32 = torch.empty(1, 32, n_ref, m_ref, device=device)
    truth32 = torch.einsum("ok,km,nmk->onm", c32.double(), a[:, ms].double(), sign)
    _, o32_ms = time_call(lambda: kermac.cdist_grad(a, b, c32, d, out=out32, p=1.0), side, 1)
    o32_err = ((out32[0][:, ns, ms].double() - truth32).abs().max() / truth32.abs().mean()).item()
    os.environ["KERMAC_AMD_GRADIENT_WORKSPACE"] = "0"
    try:
        _, o32_fp32_ms = time_call(lambda: kermac.cdist_grad(a, b, c32, d, out=out32, p=1.0), 2, 1)
    finally:
        if saved is None:
            del os.environ["KERMAC_AMD_GRADIENT_WORKSPACE"]
        else:
            os.environ["KERMAC_AMD_GRADIENT_WORKSPACE"] = saved
    del out32
    log(f"  p=1, 32 outputs: {o32_ms:.2f} ms (slab err {o32_err:.2e}); on the fp32 matrix-core kernel {o32_fp32_ms:.2f} ms")
    check_parity("cdist_grad p=1, 32 outputs, slab, max abs err / mean |truth|", o32_err, 1e-4)
    # Executed matrix work on the default route: three products of fp16 pieces, 2 * O flops each per (m, n, k),
    # against the dense fp16 peak; the sign work on the vector ALU (2.5 instructions per (m, n, k)) is what bounds it.
    ops = 3.0 * 2.0 * o * m_ref * n_ref * k_ref
    nbytes = 4.0 * (k_ref * m_ref + n_ref * k_ref + o * k_ref + n_ref * m_ref + o * n_ref * m_ref)
    return side_line("cdist_grad ms, Laplace-kernel RFM gradient M=8192 N=512 O=16 K=8192 p=1",
                     "cdist_grad p=1.0 fp32: a[8192,8192] U(0,1), b[512,8192], d[512,8192] N(0,1)/sqrt(512), "
                     "c[16,8192] N(0,1), out[16,512,8192] (BASELINE configs[3])",
                     wall_ms, kernel_ms, ops, nbytes, "mfma", 2500.0,
                     {"parity_max_err_over_mean": err, "tolerance": 1e-4,
                      "route": "a and c split once into two fp16 pieces per value, sign of d - b on the pieces, v_mfma_f32_16x16x32_f16",
                      "useful_tflops": round((2.0 * o + 3.0) * m_ref * n_ref * k_ref / kernel_ms / 1e9, 2),
                      "fp32_kernels_same_run": {"ms": round(fp32_ms, 3), "parity_max_err_over_mean": fp32_err,
                                                "frac_of_fp32_mfma_peak": round((2.0 * o + 3.0) * m_ref * n_ref * k_ref / fp32_ms / 1e9 / 157.3, 4)},
                      "p2_same_operands": {"ms": round(l2_ms, 3), "parity_max_err_over_mean": l2_err,
                                           "route": "e = (d - s) (c a) - (c (b - s)) a with s the row means of b: one product of "
                                                    "(o n) x k by k x m from two fp16 pieces per value, v_mfma_f32_32x32x16_f16",
                                           "mfma_tflops": round(3.0 * 2.0 * o * m_ref * n_ref * k_ref / l2_ms / 1e9, 2),
                                           "fp32_kernels_ms": round(l2_fp32_ms, 3), "fp32_kernels_parity_max_err_over_mean": l2_fp32_err},
                      "p1_32_outputs": {"ms": round(o32_ms, 3), "parity_max_err_over_mean": o32_err, "fp32_kernels_ms": round(o32_fp32_ms, 3),
                                        "route": "tiles of 64 m x 16 n x 32 outputs: the signed pieces meet two blocks of 16 outputs"}},
                     args)


def bench_kernel_coef(kermac, device, args, steps=None, warmup=None, with_gaussian=True):
    """batch 4, x[4,K=256,N=16384], centres z[K=256,M=16384] shared by the batch, U(-1,1); exp(-||x-z||_1/10)
    contracted with coeffs[4,16384,32] -> out[4,16384,32]; the 16384 x 16384 matrix is never stored.  Beside
    it, in the same run: the unfused pair it replaces (the kernel matrix written out, then torch.bmm)."""
    steps, warmup = steps or args.steps, args.warmup if warmup is None else warmup
    torch.manual_seed(5)
    L, k, nx, mz, o = 4, 256, 16384, 16384, 32
    x = torch.rand(L, k, nx, device=device) * 2 - 1
    z = torch.rand(k, mz, device=device) * 2 - 1
    coef = torch.randn(L, mz, o, device=device)
    out = torch.empty(L, nx, o, device=device)
    if args.calibration_copy:
        calibration_copy(device)
    call = lambda: kermac.run_kernel(kermac.kernel_descriptor_laplace_l1, x.transpose(1, 2), z.t(), out=out,
                                     bandwidth=10.0, coefficients=coef)
    wall_ms, kernel_ms = time_call(call, steps, warmup)
    rows = slice(0, 64)
    # float64 by blocks of rows (torch.cdist with p = 1 in float64 has returned wrong rows on the GPU for some sizes)
    x64, z64 = x[0, :, rows].t().double(), z.t().double()
    l1 = torch.cat([(x64[i:i + 16, None, :] - z64[None]).abs().sum(-1) for i in range(0, x64.size(0), 16)])
    truth = torch.exp(-l1 / 10.0) @ coef[0].double()
    err = ((out[0, rows].double() - truth).abs().max() / truth.abs().mean()).item()
    log(f"kernel x coefficients: {kernel_ms:.2f} ms kernel, slab max abs err / mean |truth| = {err:.2e}")
    check_parity("fused Laplace kernel matrix x coefficients (configs[4]) slab, max abs err / mean |truth|", err, 1e-4)
    extra = {"parity_max_err_over_mean": err, "tolerance": 1e-4}
    side_steps = max(2, min(steps, 5))
    # The unfused pair: run_kernel writes the 4 x 16384 x 16384 matrix (4.3 GB, m contiguous), torch.bmm contracts it.
    matrix_store = torch.empty(L, mz, nx, device=device)
    unfused_out = torch.empty(L, nx, o, device=device)

    def unfused():
        kermac.run_kernel(kermac.kernel_descriptor_laplace_l1, x.transpose(1, 2), z.t(), out=matrix_store.transpose(1, 2),
                          bandwidth=10.0)
        torch.bmm(matrix_store.transpose(1, 2), coef, out=unfused_out)

    _, unfused_ms = time_call(unfused, side_steps, 1)
    agreement = ((unfused_out - out).abs().max() / out.abs().mean()).item()
    log(f"  unfused kernel matrix + torch.bmm: {unfused_ms:.2f} ms; fused vs unfused max abs / mean = {agreement:.2e}")
    check_parity("fused vs unfused kernel matrix x coefficients, max abs diff / mean", agreement, 1e-4)
    extra["unfused_pair_same_run"] = {"ms": round(unfused_ms, 3), "fused_over_unfused": round(kernel_ms / unfused_ms, 4),
                                      "what": "run_kernel -> 4 x 16384 x 16384 matrix in HBM (4.3 GB), then torch.bmm"}
    del matrix_store, unfused_out
    if with_gaussian:
        # Beside it: the same shape with a Gaussian kernel, vector kernel and opt-in matrix-core kernel.
        gaussian = kermac.KernelDescriptor(kermac.InnerOperator.DIFF, kermac.PowerType.SQUARE, kermac.PowerType.NOOP,
                                           kermac.KernelType.GAUSSIAN)
        call = lambda: kermac.run_kernel(gaussian, x.transpose(1, 2), z.t(), out=out, bandwidth=9.0, coefficients=coef)
        with kermac.l2_mode("direct"):
            _, gaussian_ms = time_call(call, side_steps, 1)
        with kermac.l2_mode("gram"):
            _, gaussian_mfma_ms = time_call(call, side_steps, 1)
        d2 = torch.cdist(x[0, :, rows].t().double(), z.t().double(), p=2.0) ** 2
        truth = torch.exp(-d2 / (2 * 9.0 ** 2)) @ coef[0].double()
        gaussian_err = ((out[0, rows].double() - truth).abs().max() / truth.abs().mean()).item()
        check_parity("gaussian x coefficients (fused, fp32 matrix instruction) slab, max abs err / mean |truth|", gaussian_err, 1e-4)
        out.fill_(float("nan"))
        _, gaussian_panels_ms = time_call(call, side_steps, 1)            # the default mode
        panels_err = ((out[0, rows].double() - truth).abs().max() / truth.abs().mean()).item()
        log(f"gaussian x coefficients: vector {gaussian_ms:.2f} ms, fused on the fp32 matrix instruction {gaussian_mfma_ms:.2f} ms, "
            f"default (panels of the matrix from fp16 pieces, then contracted) {gaussian_panels_ms:.2f} ms; "
            f"slab max abs err / mean |truth| = {gaussian_err:.2e} / {panels_err:.2e}")
        check_parity("gaussian x coefficients (default mode: panels) slab, max abs err / mean |truth|", panels_err, 1e-4)
        extra["gaussian_same_shape"] = {"vector_ms": round(gaussian_ms, 3), "matrix_core_ms": round(gaussian_mfma_ms, 3),
                                        "default_panels_ms": round(gaussian_panels_ms, 3),
                                        "matrix_core_parity_max_err_over_mean": gaussian_err,
                                        "default_panels_parity_max_err_over_mean": panels_err,
                                        "note": "the default l2 mode 'auto' builds the kernel matrix in panels of 4096 centres "
                                                "(1 GiB, reused) on the fp16 matrix instruction and contracts each panel; "
                                                "l2 mode 'gram' is the fused kernel on the fp32 matrix instruction"}
    if with_gaussian:
        # Beside it: the Laplace kernel of the headline with 100 coefficient columns.  The fused kernel holds 64 per
        # walk of the kernel matrix, so the default builds the matrix once per panel and contracts it with all columns.
        coef100 = torch.randn(L, mz, 100, device=device)
        out100 = torch.empty(L, nx, 100, device=device)
        call = lambda: kermac.run_kernel(kermac.kernel_descriptor_laplace_l1, x.transpose(1, 2), z.t(), out=out100,
                                         bandwidth=10.0, coefficients=coef100)
        _, many_ms = time_call(call, 3, 1)
        many_err = ((out100[0, rows].double() - torch.exp(-l1 / 10.0) @ coef100[0].double()).abs().max()
                    / (torch.exp(-l1 / 10.0) @ coef100[0].double()).abs().mean()).item()
        saved = os.environ.get("KERMAC_AMD_COEFFICIENT_PANEL_BYTES")
        os.environ["KERMAC_AMD_COEFFICIENT_PANEL_BYTES"] = "0"
        try:
            _, many_fused_ms = time_call(call, 2, 1)
        finally:
            if saved is None:
                del os.environ["KERMAC_AMD_COEFFICIENT_PANEL_BYTES"]
            else:
                os.environ["KERMAC_AMD_COEFFICIENT_PANEL_BYTES"] = saved
        log(f"laplace x 100 coefficient columns: default (panels of the matrix, then contracted) {many_ms:.2f} ms, "
            f"fused kernel (two walks of the matrix) {many_fused_ms:.2f} ms; slab max abs err / mean |truth| = {many_err:.2e}")
        check_parity("laplace x 100 coefficient columns (panels) slab, max abs err / mean |truth|", many_err, 1e-4)
        extra["laplace_100_columns"] = {"default_panels_ms": round(many_ms, 3), "fused_ms": round(many_fused_ms, 3),
                                        "parity_max_err_over_mean": many_err}
        del coef100, out100
    ops = float(L) * nx * mz * (3 * k + 2 * o)
    nbytes = 4.0 * (L * k * nx + k * mz + 2 * L * nx * o)
    return side_line("fused Laplace kernel matrix x coefficients ms, L=4 N=M=16384 K=256 O=32",
                     "run_kernel(laplace_l1, x[4,16384,256] view, z[16384,256] view, bandwidth=10, "
                     "coefficients[4,16384,32]) -> out[4,16384,32] (BASELINE configs[4])",
                     wall_ms, kernel_ms, ops, nbytes, "valu_fp32", 157.3, extra, args)


def measured_issue_ceiling(p):
    """What the kernel's own instruction mix reaches on registers alone, for launches as long as the benchmark's
    (profiles/valu_issue_rates_gfx950.txt): the time the problem would take at that rate, and the clock it ran at."""
    rates = issue_rates()
    case = {1.0: "p1_rows", 2.0: "p2_rows"}.get(p, "pow_rows")
    per_term = 2 if p in (1.0, 2.0) else 5
    if case + "_lane_ops_per_s" not in rates:
        return None
    return {"source": "profiles/" + os.path.basename(ISSUE_PROFILE), "case": case,
            "lane_ops_per_s": rates[case + "_lane_ops_per_s"], "clock_mhz": rates.get(case + "_clock_mhz"),
            "floor_ms": round(M * N * K * per_term / rates[case + "_lane_ops_per_s"] * 1e3, 2)}


def finish(line):
    """Print the one JSON line; a parity failure is part of it and makes the exit status 1."""
    line["parity_failed"] = PARITY_FAILURES
    print(json.dumps(line), flush=True)
    if PARITY_FAILURES:
        log(f"bench.py: {len(PARITY_FAILURES)} parity failure(s), see 'parity_failed' in the line")
        sys.exit(1)


def p_entry(k_ms, err, rtol, **more):
    """A cdist timing on the vector ALU: the counted 3 fp32 operations per (m, n, k) against the fp32 vector peak."""
    return {"ms": round(k_ms, 3), "tflops_3op": round(OPS_PER_CALL / k_ms / 1e9, 2),
            "pct_fp32_valu_peak": round(OPS_PER_CALL / k_ms / 1e9 / PEAK_FP32_VALU_TFLOPS * 100, 2),
            "parity_max_rel_err": err, "rtol": rtol, **more}


PEAK_MFMA_TFLOPS = {"f16": 2500.0, "bf16": 2500.0, "f32": 157.3}     # dense matrix peaks of the MI355X


def mfma_entry(k_ms, err, rtol, products, operand_type, **more):
    """A timing whose multiply-adds run on the matrix cores: the executed matrix work (2 M N K per piece product)
    against the dense peak of the matrix instruction's operand type."""
    executed = products * 2.0 * M * N * K / k_ms / 1e9
    peak = PEAK_MFMA_TFLOPS[operand_type]
    return {"ms": round(k_ms, 3), "parity_max_rel_err": err, "rtol": rtol,
            "roofline": {"bound": "mfma", "operands": operand_type, "piece_products": products,
                         "achieved": round(executed, 2), "peak": peak, "unit": "TFLOP/s", "frac": round(executed / peak, 4)},
            **more}


def main():
    parser = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    parser.add_argument("--gpus", type=int, default=1)
    parser.add_argument("--steps", type=int, default=10)
    parser.add_argument("--warmup", type=int, default=2)
    parser.add_argument("--skip-cpu", action="store_true", help="skip the host-CPU baseline leg")
    parser.add_argument("--only-p1", action="store_true", help="time only the headline p = 1.0 configuration")
    parser.add_argument("--only-p", type=float, default=None,
                        help="time only cdist with this p as the step (for profiling one kernel: 2.0, 1.3, ...)")
    parser.add_argument("--l2-mode", choices=["auto", "direct", "gram", "gram_bf16"], default=None,
                        help="how squared differences (p = 2) are evaluated in the timed step; default: the library's "
                             "default, 'auto' (matrix cores with repair of ill-conditioned tiles for large problems)")
    parser.add_argument("--l1-mode", choices=["direct", "fixed"], default=None,
                        help="how absolute differences (p = 1) are evaluated in the timed step; default: the library's default, "
                             "'direct' (fp32 on the vector ALU); 'fixed' is the opt-in fixed-point route (for profiling it)")
    parser.add_argument("--workload", choices=["cdist", "cdist_grad", "kernel_coef"], default="cdist",
                        help="cdist (default, the headline metric, with the other two configurations as extra keys); "
                             "cdist_grad = only the Laplace-kernel RFM gradient configuration; kernel_coef = only the "
                             "fused Laplace kernel matrix x coefficients configuration")
    parser.add_argument("--operand-layout", choices=["k_major", "torch"], default="k_major",
                        help="with --only-p1 / --only-p: 'torch' hands over a[M, K], b[N, K], out[M, N] as torch allocates them "
                             "(k and n contiguous) instead of BASELINE's K-major panels; the library then copies the operands "
                             "into K-major panels inside the timed call")
    parser.add_argument("--calibration-copy", action="store_true",
                        help="also run one plain elementwise copy kernel over 1 GiB (read 1 GiB, write 1 GiB), so that "
                             "hardware byte counters collected by a profiler can be scaled against a known transfer")
    args = parser.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        sys.exit("bench.py: this path runs on one GPU only (it shards by giving each GPU its own slab of b "
                 "with no exchange; no multi-GPU figure is produced) -- run with --gpus 1")
    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible; the kernels are gfx950 only and there is no CPU fallback")

    import kermac_amd as kermac

    if args.l2_mode is not None:
        kermac.set_l2_mode(args.l2_mode)
    if args.l1_mode is not None:
        kermac.set_l1_mode(args.l1_mode)
    device = torch.device("cuda:0")
    torch.cuda.set_device(device)
    if args.workload != "cdist":
        finish((bench_cdist_grad if args.workload == "cdist_grad" else bench_kernel_coef)(kermac, device, args))
        return
    log(f"device: {torch.cuda.get_device_name(0)}; allocating {ALGORITHMIC_BYTES / 1e9:.2f} GB")
    torch.manual_seed(1)
    a_store = torch.randn(K, M, device=device)
    b_store = torch.randn(K, N, device=device)
    out_store = torch.empty(N, M, device=device)
    a, b, out = a_store.t(), b_store.t(), out_store.t()      # the operator's [M,K] / [N,K] / [M,N] views

    if args.operand_layout == "torch":
        if not (args.only_p1 or args.only_p is not None):
            sys.exit("bench.py: --operand-layout torch goes with --only-p1 or --only-p (the default run measures BASELINE's layout "
                     "and carries this one as per_p['1.0_torch_layout'])")
        a, b = a.contiguous(), b.contiguous()
        out = out_store.view(-1)[:M * N].view(M, N)

    if args.calibration_copy:
        calibration_copy(device)

    headline_p = 1.0 if args.only_p is None else args.only_p
    headline_rtol = 1e-5 if headline_p in (1.0, 2.0) else 1e-4
    log(f"timing p = {headline_p}" + (" (headline)" if headline_p == 1.0 else ""))
    wall_ms, kernel_ms = time_cdist(kermac, a, b, out, headline_p, False, args.steps, args.warmup)
    err = parity_slab(out, a, b, headline_p, False)
    log(f"  {wall_ms:.2f} ms/step wall, {kernel_ms:.2f} ms kernel, slab max rel err {err:.2e}")
    check_parity(f"cdist p={headline_p} slab max rel err", err, headline_rtol)
    per_p = {str(headline_p): p_entry(kernel_ms, err, headline_rtol)}
    other_configs = {}

    if not args.only_p1 and args.only_p is None:
        side_steps = max(2, min(args.steps, 5))
        for p, skip, rtol, mode in ((2.0, False, 1e-5, None), (2.0, False, 1e-5, "direct"), (1.3, False, 1e-4, None),
                                    (1.3, True, 1e-4, None)):
            label = f"{p}" + ("_skip_epilogue" if skip else "") + (f"_{mode}" if mode else "")
            log(f"timing p = {label}")
            with kermac.l2_mode(mode or kermac.get_l2_mode()):
                _, k_ms = time_cdist(kermac, a, b, out, p, skip, side_steps, 1)
            e = parity_slab(out, a, b, p, skip)
            log(f"  {k_ms:.2f} ms kernel, slab max rel err {e:.2e}")
            check_parity(f"cdist p={label} slab max rel err", e, rtol)
            per_p[label] = p_entry(k_ms, e, rtol)
        if kermac.get_l2_mode() in ("auto", "gram_bf16"):
            # this problem takes the route through the workspace: three products of fp16 pieces
            per_p["2.0"] = mfma_entry(per_p["2.0"]["ms"], per_p["2.0"]["parity_max_rel_err"], 1e-5, 3, "f16")
        per_p["2.0"]["l2_mode"] = kermac.get_l2_mode()
        per_p["2.0"]["note"] = ("default mode 'auto': |a-c|^2 + |b-c|^2 - 2 (a-c).(b-c), c = sample mean, with the cross term on "
                                "the fp16 matrix instruction (both operands split once into two fp16 pieces per value, scaled per "
                                "row, in a workspace; 256 x 256 tiles; three piece products), ill-conditioned 128 x 128 parts "
                                "recomputed by the direct kernel; the vector-ALU kernel is per_p['2.0_direct']")
        # The default mode on data that defeats the matrix-core route: 64 tight clusters far apart (centres N(0, 10^2),
        # noise 1e-3, seed 11), so one pair in 64 is a pair of near-duplicates and every 128 x 128 part holds some.  The
        # route samples pairs before its product kernel and, finding them, leaves everything to the direct kernel.
        log("timing p = 2.0 on clustered data, default mode and direct")
        gen = torch.Generator(device=device).manual_seed(11)
        centres_a = 10.0 * torch.randn(K, 64, device=device, generator=gen)
        centres_b = 10.0 * torch.randn(K, 64, device=device, generator=gen)
        labels_a = torch.randint(0, 64, (M,), device=device, generator=gen)
        ca_store = centres_a[:, labels_a] + 1e-3 * torch.randn(K, M, device=device, generator=gen)
        labels_b = torch.randint(0, 64, (N,), device=device, generator=gen)
        cb_store = centres_a[:, labels_b] + 1e-3 * torch.randn(K, N, device=device, generator=gen)
        del centres_b, centres_a
        ca, cb = ca_store.t(), cb_store.t()
        _, clustered_ms = time_cdist(kermac, ca, cb, out, 2.0, False, side_steps, 1)
        clustered_err = parity_slab(out, ca, cb, 2.0, False)
        with kermac.l2_mode("direct"):
            _, clustered_direct_ms = time_cdist(kermac, ca, cb, out, 2.0, False, side_steps, 1)
            clustered_direct_err = parity_slab(out, ca, cb, 2.0, False)
        log(f"  default {clustered_ms:.2f} ms (slab max rel err {clustered_err:.2e}), direct {clustered_direct_ms:.2f} ms ({clustered_direct_err:.2e})")
        check_parity("cdist p=2.0 clustered data (default mode) slab max rel err", clustered_err, 1e-5)
        check_parity("cdist p=2.0 clustered data (direct) slab max rel err", clustered_direct_err, 1e-5)
        per_p["2.0_clustered"] = {"ms": round(clustered_ms, 3), "direct_ms": round(clustered_direct_ms, 3),
                                  "default_over_direct": round(clustered_ms / clustered_direct_ms, 4),
                                  "parity_max_rel_err": clustered_err, "direct_parity_max_rel_err": clustered_direct_err, "rtol": 1e-5,
                                  "data": "both operands drawn from the same 64 centres N(0, 10^2) per k, plus N(0, 1e-6) noise, seed 11",
                                  "l2_mode": kermac.get_l2_mode()}
        # The same points stored cluster by cluster: the near-duplicates now fill the blocks on the diagonal (one part in
        # 64), the sample sees that they are packed, and the matrix cores keep the call; only those blocks are redone.
        ca_store, cb_store = ca_store[:, labels_a.sort().indices].contiguous(), cb_store[:, labels_b.sort().indices].contiguous()
        ca, cb = ca_store.t(), cb_store.t()
        _, sorted_ms = time_cdist(kermac, ca, cb, out, 2.0, False, side_steps, 1)
        sorted_err = parity_slab(out, ca, cb, 2.0, False)
        with kermac.l2_mode("direct"):
            _, sorted_direct_ms = time_cdist(kermac, ca, cb, out, 2.0, False, side_steps, 1)
        log(f"  stored cluster by cluster: default {sorted_ms:.2f} ms (slab max rel err {sorted_err:.2e}), direct {sorted_direct_ms:.2f} ms")
        check_parity("cdist p=2.0 clustered data stored cluster by cluster (default mode) slab max rel err", sorted_err, 1e-5)
        per_p["2.0_clustered"]["stored_cluster_by_cluster"] = {"ms": round(sorted_ms, 3), "direct_ms": round(sorted_direct_ms, 3),
                                                               "default_over_direct": round(sorted_ms / sorted_direct_ms, 4),
                                                               "parity_max_rel_err": sorted_err, "rtol": 1e-5}
        del ca_store, cb_store, ca, cb, labels_a, labels_b

        # Fractional p costs five instructions per (m, n, k), two of them transcendentals that issue at a quarter
        # of the rate.  issue_floor_ms adds the parts (2 transcendentals + 3 plain instructions per term at the
        # rates each kind reaches alone); isolated_chain_ms is the kernel's own chain (sub, log2, mul, exp2, add)
        # on registers alone: mixing the two kinds costs a fifth on top of the sum of the parts.
        rates = issue_rates()
        needed = ("v_exp_f32_lane_ops_per_s", "v_log_f32_lane_ops_per_s", "v_add_f32_lane_ops_per_s", "pow_rows_lane_ops_per_s")
        if all(key in rates for key in needed):
            floor_ms = M * N * K * (1 / rates["v_exp_f32_lane_ops_per_s"] + 1 / rates["v_log_f32_lane_ops_per_s"]
                                    + 3 / rates["v_add_f32_lane_ops_per_s"]) * 1e3
            chain_ms = M * N * K * 5 / rates["pow_rows_lane_ops_per_s"] * 1e3
            for label in ("1.3", "1.3_skip_epilogue"):
                per_p[label]["issue_floor_ms"] = round(floor_ms, 1)
                per_p[label]["frac_of_issue_ceiling"] = round(floor_ms / per_p[label]["ms"], 4)
                per_p[label]["isolated_chain_ms"] = round(chain_ms, 1)
                per_p[label]["frac_of_isolated_chain"] = round(chain_ms / per_p[label]["ms"], 4)
                per_p[label]["issue_rates_source"] = "profiles/" + os.path.basename(ISSUE_PROFILE)

        # The two matrix-core paths for p = 2 by name (|a|^2 + |b|^2 - 2 a.b on fp32 MFMA, ill-conditioned tiles
        # recomputed directly); same 1e-5 tolerance.  The default 'auto' picks the second for this problem.
        # "gram_bf16": the cross term on the bf16 matrix instruction from three exact bf16 pieces per operand.
        # "gram_bf16" takes the workspace route for a problem of this size (two fp16 pieces, three products); with
        # KERMAC_AMD_L2_WORKSPACE=0 it is the one-step kernel (three bf16 pieces split inside every workgroup, six products).
        for mode, label, products, workspace in (("gram", "2.0_gram_mfma", 1, "1"), ("gram_bf16", "2.0_gram_bf16_mfma", 3, "1"),
                                                 ("gram_bf16", "2.0_gram_bf16_one_step", 6, "0")):
            log(f"timing p = 2.0, l2 mode '{mode}'" + ("" if workspace == "1" else " without a workspace"))
            saved = os.environ.get("KERMAC_AMD_L2_WORKSPACE")
            os.environ["KERMAC_AMD_L2_WORKSPACE"] = workspace
            try:
                with kermac.l2_mode(mode):
                    _, k_ms = time_cdist(kermac, a, b, out, 2.0, False, side_steps, 1)
                    e = parity_slab(out, a, b, 2.0, False)
            finally:
                if saved is None:
                    del os.environ["KERMAC_AMD_L2_WORKSPACE"]
                else:
                    os.environ["KERMAC_AMD_L2_WORKSPACE"] = saved
            log(f"  {k_ms:.2f} ms kernel, slab max rel err {e:.2e}")
            check_parity(f"cdist p=2.0 ({label}) slab max rel err", e, 1e-5)
            per_p[label] = mfma_entry(k_ms, e, 1e-5, products, {1: "f32", 3: "f16", 6: "bf16"}[products], l2_mode=mode)

        # x against x (the kernel matrix of a training set): the library computes the tiles on and
        # below the diagonal only and stores each twice; bit-identical to the full computation.
        log("timing p = 1.0, a against itself")
        _, k_ms = time_cdist(kermac, a, a, out, 1.0, False, side_steps, 1)
        e = parity_slab(out, a, a, 1.0, False, slabs=OFF_DIAGONAL_SLABS)
        log(f"  {k_ms:.2f} ms kernel, slab max rel err {e:.2e}")
        check_parity("cdist p=1.0 (a against itself) slab max rel err", e, 1e-5)
        per_p["1.0_a_against_itself"] = {"ms": round(k_ms, 3), "parity_max_rel_err": e, "rtol": 1e-5,
                                         "note": "symmetric result: half the tiles computed, each stored twice"}
        # The same problem with the operands as torch allocates them and as the reference's own benchmark example does
        # (examples/cdist.py:51-53): a[M, K], b[N, K], out[M, N], k and n contiguous.  The library copies such operands
        # into k-major panels for its fastest direct kernel (the copies are inside the timed region).
        log("timing p = 1.0, operands and result in torch's own layout")
        a_rows, b_rows = a.contiguous(), b.contiguous()
        out_rows = out_store.view(-1)[:M * N].view(M, N)        # [M, N] with n contiguous, over the same memory
        _, k_ms = time_cdist(kermac, a_rows, b_rows, out_rows, 1.0, False, side_steps, 1)
        e = parity_slab(out_rows, a, b, 1.0, False)
        del a_rows, b_rows
        log(f"  {k_ms:.2f} ms kernel, slab max rel err {e:.2e}")
        check_parity("cdist p=1.0 (torch's layout) slab max rel err", e, 1e-5)
        per_p["1.0_torch_layout"] = p_entry(k_ms, e, 1e-5, note="a[M, K], b[N, K], out[M, N] as torch allocates them; the two copies into "
                                                                 "k-major panels (0.15 ms) are part of the call")
        # The opt-in fixed-point route for p = 1 (kermac.l1_mode("fixed")): both operands rounded once to a common
        # 22-bit grid, one v_sad_u32 per term, tiles whose error bound is not met recomputed by the fp32 kernel.
        log("timing p = 1.0, l1 mode 'fixed'")
        with kermac.l1_mode("fixed"):
            _, k_ms = time_cdist(kermac, a, b, out, 1.0, False, side_steps, 1)
            e = parity_slab(out, a, b, 1.0, False)
        log(f"  {k_ms:.2f} ms kernel, slab max rel err {e:.2e}")
        check_parity("cdist p=1.0 (l1 mode 'fixed') slab max rel err", e, 1e-5)
        per_p["1.0_fixed_point"] = p_entry(k_ms, e, 1e-5, l1_mode="fixed",
                                           note="opt-in: sums of |qb - qa| on 32-bit integers (one v_sad_u32 per term where fp32 "
                                                "issues two instructions), operands rounded once to a common power-of-two grid "
                                                "in a workspace, error bound K grid steps per element, elements whose bound "
                                                "exceeds 8e-6 recomputed tile-wise by the fp32 kernel; all launches included")
        rate = issue_rates().get("v_sad_u32_lane_ops_per_s")
        if rate:
            per_p["1.0_fixed_point"]["issue_floor_ms"] = round(M * N * K / rate * 1e3, 2)
            per_p["1.0_fixed_point"]["frac_of_issue_ceiling"] = round(M * N * K / rate * 1e3 / k_ms, 4)

        log("timing p = 2.0, a against itself")
        _, k_ms = time_cdist(kermac, a, a, out, 2.0, False, side_steps, 1)
        e = parity_slab(out, a, a, 2.0, False, slabs=OFF_DIAGONAL_SLABS)
        log(f"  {k_ms:.2f} ms kernel, slab max rel err {e:.2e}")
        check_parity("cdist p=2.0 (a against itself) slab max rel err", e, 1e-5)
        per_p["2.0_a_against_itself"] = {"ms": round(k_ms, 3), "parity_max_rel_err": e, "rtol": 1e-5, "l2_mode": kermac.get_l2_mode(),
                                         "note": "symmetric result on the workspace route: the 256 x 256 tiles on and below the diagonal"}

        # Beside the distances: the same operands through run_kernel with the inner operator DOT (a linear
        # kernel matrix, a @ b.T), on the route through the workspace and on the direct kernel.
        log("timing the sum of products (inner operator DOT)")
        dot = kermac.KernelDescriptor(kermac.InnerOperator.DOT, kermac.PowerType.NOOP, kermac.PowerType.NOOP, kermac.KernelType.NONE)

        def dot_error():
            truth = a[:64].double() @ b[:96].double().t()
            scale = a[:64].abs().double() @ b[:96].abs().double().t()
            return ((out[:64, :96].double() - truth).abs() / scale).max().item()

        _, dot_ms = time_call(lambda: kermac.run_kernel(dot, a, b, out=out), side_steps, 1)
        dot_err = dot_error()
        with kermac.l2_mode("direct"):
            _, dot_direct_ms = time_call(lambda: kermac.run_kernel(dot, a, b, out=out), side_steps, 1)
            dot_direct_err = dot_error()
        log(f"  {dot_ms:.2f} ms kernel (max err / sum |a b| {dot_err:.2e}); direct kernel {dot_direct_ms:.2f} ms ({dot_direct_err:.2e})")
        check_parity("sum of products, max abs err / sum_k |a b|", dot_err, 1e-6)
        check_parity("sum of products (direct kernel), max abs err / sum_k |a b|", dot_direct_err, 1e-6)
        per_p["sum_of_products"] = {"ms": round(dot_ms, 3), "parity_max_err_over_sum_of_absolute_terms": dot_err,
                                    "roofline": mfma_entry(dot_ms, dot_err, 1e-6, 3, "f16")["roofline"],
                                    "direct_kernel_ms": round(dot_direct_ms, 3),
                                    "direct_kernel_parity_max_err_over_sum_of_absolute_terms": dot_direct_err,
                                    "note": "run_kernel with inner operator DOT: two fp16 pieces per value on the 256 x 256 walk; "
                                            "no trust check (nothing cancels in a product)"}

        # The two other configurations of the path, timed in this same run so that the default invocation
        # covers them: each entry is the line `--workload <name>` prints on its own.
        del out_store, out
        torch.cuda.empty_cache()
        for name, fn in (("cdist_grad", bench_cdist_grad), ("kernel_coef", bench_kernel_coef)):
            log(f"other configuration: {name}")
            side = fn(kermac, device, args, steps=side_steps, warmup=1)
            other_configs[name] = {key: side[key] for key in side if key not in ("n_gpus", "higher_is_better", "scaling",
                                                                                  "vs_baseline", "data", "dtype")}
            other_configs[name]["steps"], other_configs[name]["warmup"] = side_steps, 1

    achieved = OPS_PER_CALL / kernel_ms / 1e9
    traffic, traffic_source = (measured_traffic() if headline_p == 1.0 and kermac.get_l1_mode() == "direct" and args.operand_layout == "k_major"
                               else (None, None))
    inner = {1.0: "POW_ABS", 2.0: "POW_SQUARE"}.get(headline_p, "POW_POW")
    headline_kernel = (f"kmc::build_kernel_scalar_b<OP_DIFF,{inner}>" if inner != "POW_POW"
                       else f"kmc::build_kernel<OP_DIFF,{inner},LOAD_COL_VEC,LOAD_COL_VEC>")
    if headline_p == 1.0 and kermac.get_l1_mode() == "fixed":
        headline_kernel = "kmc::l1_fixed_kernel (l1 mode fixed)"
    if headline_p == 2.0 and kermac.get_l2_mode() != "direct":
        headline_kernel = "kmc::gram_f16_wide / kmc::gram_bf16_l2_kernel / kmc::gram_l2_kernel (l2 mode %s)" % kermac.get_l2_mode()
    line = {
        "metric": "cdist ms and % fp32-VALU peak at M=N=30000,K=1024 for p=1/1.3/2",
        "value": round(wall_ms, 3),
        "unit": "ms",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(wall_ms, 3),
        "higher_is_better": False,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": (f"cdist p={headline_p} fp32, a[K=1024,M=30000] b[K=1024,N=30000] K-major N(0,1) seed 1, "
                                "out[N=30000,M=30000] with epilogue, no batch (BASELINE configs[1])" if args.operand_layout == "k_major" else
                                f"cdist p={headline_p} fp32, a[M=30000,K=1024] b[N=30000,K=1024] out[M=30000,N=30000] as torch allocates "
                                "them, N(0,1) seed 1, with epilogue, no batch (BASELINE configs[1] in the other storage order)"),
                   "M": M, "N": N, "K": K, "p": headline_p},
        "per_p": per_p,
        "roofline": {
            "bound": "valu_fp32",
            "kernel": headline_kernel,
            "achieved": round(achieved, 2),
            "peak": PEAK_FP32_VALU_TFLOPS,
            "unit": "TFLOP/s",
            "frac": round(achieved / PEAK_FP32_VALU_TFLOPS, 4),
            "traffic": traffic,
            "traffic_source": traffic_source,
            "ops_per_launch": OPS_PER_CALL,
            "counting": "3 fp32 ops per (m,n,k); the kernel issues 2 VALU instructions per (m,n,k), so its "
                        "instruction-issue ceiling is 1.5 x 78.6 = 117.9 TFLOP/s in this unit at 2.4 GHz",
            "frac_of_issue_ceiling": round(achieved / 117.9, 4),
            "measured_issue_rate": measured_issue_ceiling(headline_p),
            "clock": {"nominal_mhz_in_peak": 2400,
                      "shader_mhz_under_this_kernel": (traffic_source or {}).get("shader_clock_mhz"),
                      "how": "GRBM_GUI_ACTIVE / kernel duration in the profile named by traffic_source; "
                             "the board sustains less than the nominal clock under this load"},
            "hbm_gbps": round(ALGORITHMIC_BYTES / kernel_ms / 1e6, 1),
            "hbm_frac": round(ALGORITHMIC_BYTES / kernel_ms / 1e6 / PEAK_HBM_GBPS, 4),
        },
    }
    if other_configs:
        line["other_configs"] = other_configs
    if not args.skip_cpu:
        log("host CPU baseline (torch.cdist on slabs)")
        line["cpu_baseline"] = cpu_baseline(a_store.cpu(), b_store.cpu())
    finish(line)


if __name__ == "__main__":
    main()
