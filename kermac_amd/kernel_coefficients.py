"""Fused kernel matrix x coefficients: ``run_kernel(..., coefficients=...)``.

The reference's ``run_kernel`` always writes the full ``[L, M, N]`` matrix
(src/kermac/build_a_kernel.py:259,378-392); contracting it with coefficients is
left to the caller.  This operator produces
``out[l, m, o] = sum_n kernelmatrix[l, m, n] * coefficients[l, n, o]`` without the
matrix ever reaching memory, with exactly the per-element semantics of
``run_kernel`` (outer power, epsilon mask, kernel function, regularised diagonal).
"""
from __future__ import annotations

import functools
from typing import Optional

import torch

from . import _backend
from .common import launch_cuts_enabled, merge_batch_size
from .module_cache.module_cache import ModuleCache, kernel_coefficients_function_name


class _CoefPlan:
    __slots__ = ("params", "out", "keepalive", "L", "M", "N", "K", "O")


def _plan_run_kernel_coefficients(
    kernel_descriptor, a, b, coefficients, out, p, inner_p, outer_p, bandwidth, epsilon, regularization,
    regularization_offset_x, regularization_offset_y, require_device=True,
) -> _CoefPlan:
    from .build_a_kernel import _plan_run_kernel

    if not isinstance(coefficients, torch.Tensor):
        raise TypeError("coefficients must be a PyTorch tensor")
    if coefficients.dtype != torch.float32:
        raise TypeError("coefficients must have dtype torch.float32")
    if out is not None and not isinstance(out, torch.Tensor):
        raise TypeError("out must be a PyTorch tensor if provided")
    if out is not None and out.dtype != torch.float32:
        raise TypeError("out must have dtype torch.float32")
    if coefficients.dim() not in (2, 3):
        raise ValueError("coefficients must be 2-dimensional or 3-dimensional with a batch mode")
    if out is not None and out.dim() not in (2, 3):
        raise ValueError("out must be 2-dimensional or 3-dimensional with a batch mode")

    # Validate a / b / hyper-parameters exactly like run_kernel does.  The kernel
    # matrix itself is never allocated; coefficients and out join the batch merge.
    base = _plan_run_kernel(
        kernel_descriptor, a, b, None, p, inner_p, outer_p, bandwidth, epsilon, regularization,
        regularization_offset_x, regularization_offset_y, False, require_device=require_device, allocate_out=False)
    L = base.L
    L = merge_batch_size("coefficients", L, coefficients, expected_dims=2, can_be_none=False)
    L = merge_batch_size("out", L, out, expected_dims=2, can_be_none=True)
    M, N, K = base.M, base.N, base.K
    device = a.device
    if require_device and not coefficients.is_cuda:
        raise ValueError("coefficients must be on a CUDA device")
    if coefficients.device != device:
        raise ValueError(f"coefficients must be on the same CUDA device as inputs: got {coefficients.device}")
    if coefficients.size(-2) != N:
        raise ValueError(f"coefficients must have shape (N={N}, O), got {tuple(coefficients.shape[-2:])}")
    O = coefficients.size(-1)
    if coefficients.stride(-1) != 1 and O > 1:
        raise ValueError("coefficients must have stride 1 in last dimension")
    if out is not None:
        if require_device and not out.is_cuda:
            raise ValueError("out must be on a CUDA device")
        if out.device != device:
            raise ValueError(f"out must be on the same CUDA device as inputs: got {out.device}, expected {device}")
        if tuple(out.shape[-2:]) != (M, O):
            raise ValueError(f"out must have shape (M={M}, O={O}), got {tuple(out.shape[-2:])}")
        L_out = out.size(0) if out.dim() == 3 else 1
        if L_out != L:
            raise ValueError(f"out must have batch dimension (L={L}), got {L_out}")
        if out.stride(-1) != 1 and O > 1:
            raise ValueError("out must have stride 1 in last dimension")
    else:
        # every element is written by the kernel (zeros when N = 0), so no fill is needed
        out = torch.empty((L, M, O), dtype=torch.float32, device=device)

    def batch_stride(t):
        return t.stride(0) if t.dim() == 3 and t.size(0) != 1 else 0

    params = _backend.KernelCoefficientsParams()
    params.kernel = base.params
    params.kernel.l = L
    params.o = O
    params.coef, params.coef_ld, params.coef_bs = coefficients.data_ptr(), coefficients.stride(-2), batch_stride(coefficients)
    params.out, params.out_ld, params.out_bs = out.data_ptr(), out.stride(-2), batch_stride(out)

    plan = _CoefPlan()
    plan.params, plan.out = params, out
    plan.keepalive = base.keepalive + [coefficients, out]
    plan.L, plan.M, plan.N, plan.K, plan.O = L, M, N, K, O
    return plan


def run_kernel_coefficients(
    kernel_descriptor, a, b, coefficients, out: Optional[torch.Tensor] = None, p=None, inner_p=None, outer_p=None,
    bandwidth=None, epsilon=None, regularization=None, regularization_offset_x: int = 0,
    regularization_offset_y: int = 0, debug=False, _may_split=True,
):
    """``out[l, m, o] = sum_n run_kernel(descriptor, a, b, ...)[l, m, n] * coefficients[l, n, o]``.

    ``a`` is ``[L?, M, K]``, ``b`` is ``[L?, N, K]`` (row- or column-major),
    ``coefficients`` is ``[L?, N, O]`` and ``out`` ``[L?, M, O]``, both with the last
    dimension contiguous.  Returns ``out`` (allocated ``[L, M, O]`` when None).
    """
    from .build_a_kernel import _current_stream_for

    plan = _plan_run_kernel_coefficients(
        kernel_descriptor, a, b, coefficients, out, p, inner_p, outer_p, bandwidth, epsilon, regularization,
        regularization_offset_x, regularization_offset_y)
    split = _split_over_centres(plan, a, b, coefficients, regularization) if _may_split else None
    if split is not None:
        _run_split_over_centres(split, plan, kernel_descriptor, a, b, coefficients, p, inner_p, outer_p, bandwidth,
                                epsilon, debug)
        return plan.out
    stream = _current_stream_for(a.device)
    params = plan.params
    kernel = params.kernel
    if _backend.kernel_times_coefficients_has_variant(kernel.inner_operator, kernel.inner_power):
        if debug:
            print(f"(Kermac Debug) Launching ahead-of-time fused coefficient kernel for {kernel_descriptor!r}")
        _backend.kernel_times_coefficients(params, stream)
    else:
        load_a, load_b = _backend.build_kernel_load_modes(kernel)
        name = kernel_coefficients_function_name(kernel.inner_operator, kernel.inner_power, load_a, load_b)
        function = ModuleCache(debug).get_function(a.device, name, debug=debug)
        if debug:
            print(f"(Kermac Debug) Launching kernel: {name}")
        _backend.kernel_times_coefficients_jit(function, params, stream)
    return plan.out


# A workgroup of the fused kernel owns 128 rows of ``a`` and walks every centre, so a
# launch has ceil(M / 128) x L x ceil(O / 64) long-running workgroups, of which 512 run at
# a time (two per CU).  Few rows against many centres (prediction for a small batch of
# points) would leave most of the chip idle, and a count just above a multiple of 512
# leaves it idle for most of the last round.  Such an unbatched call is cut over the
# centres: slices of ``b`` and ``coefficients`` become the batch of one launch (``a``
# broadcasts), each slice writes its own partial result, and the partial results are summed
# in a fixed order.
_SPLIT_CONCURRENT_WORKGROUPS = 512
_SPLIT_MIN_CENTRES = 128
_SPLIT_WORKGROUP_OVERHEAD = 64           # start-up and store of a workgroup, in centres walked
_SPLIT_MAX_PARTIAL_BYTES = 256 << 20
_SPLIT_WORTH = 0.92                      # cut only for at least 8 % less modelled time (448 workgroups: 10 % modelled, 14 % measured)


def _split_over_centres(plan, a, b, coefficients, regularization):
    """(slices, rows per slice, leftover rows), or None when the call is launched as it is."""
    if plan.L != 1:
        return None                      # the batch index of the launch is taken by the caller's batches
    if regularization is not None and not (isinstance(regularization, (int, float)) and regularization == 0):
        return None                      # the regularised diagonal is addressed by the global centre index
    if plan.M == 0 or plan.O == 0 or plan.N < 2 * _SPLIT_MIN_CENTRES or not launch_cuts_enabled():
        return None
    return _choose_split(plan.M, plan.N, plan.O)


@functools.lru_cache(maxsize=256)
def _choose_split(M, N, O):
    workgroups = -(-M // 128) * max(1, -(-O // 64))

    def rounds(count):
        return -(-count // _SPLIT_CONCURRENT_WORKGROUPS)

    # Modelled time of a launch: centres walked per workgroup (plus its fixed cost) times rounds of
    # workgroups.  Slices are a whole number of tiles each, so a 16-byte aligned operand stays
    # aligned in every slice; the rows that remain go into a second launch.
    unsplit = (N + _SPLIT_WORKGROUP_OVERHEAD) * rounds(workgroups)
    most = min(N // _SPLIT_MIN_CENTRES, _SPLIT_MAX_PARTIAL_BYTES // (4 * M * O) - 1,
               max(16, _SPLIT_CONCURRENT_WORKGROUPS // workgroups))
    best = None
    for slices in range(2, most + 1):
        for rows in (N // slices // 128 * 128, -(-N // slices // 128) * 128):
            if rows < _SPLIT_MIN_CENTRES:
                continue
            full = N // rows
            leftover = N - full * rows
            cost = (rows + _SPLIT_WORKGROUP_OVERHEAD) * rounds(full * workgroups)
            if leftover:
                cost += (leftover + _SPLIT_WORKGROUP_OVERHEAD) * rounds(workgroups)
            if full >= 2 and (best is None or cost < best[0]):
                best = (cost, full, rows, leftover)
    if best is None or best[0] > _SPLIT_WORTH * unsplit:
        return None
    return best[1:]


def _run_split_over_centres(split, plan, kernel_descriptor, a, b, coefficients, p, inner_p, outer_p, bandwidth, epsilon,
                            debug):
    full, rows, leftover = split
    a2, b2, c2 = (t[0] if t.dim() == 3 else t for t in (a, b, coefficients))
    M, K, O = plan.M, plan.K, plan.O
    partial = torch.empty((full + (1 if leftover else 0), M, O), dtype=torch.float32, device=a.device)
    b_slices = b2.as_strided((full, rows, K), (rows * b2.stride(0), b2.stride(0), b2.stride(1)), b2.storage_offset())
    c_slices = c2.as_strided((full, rows, O), (rows * c2.stride(0), c2.stride(0), c2.stride(1)), c2.storage_offset())
    hyper = dict(p=p, inner_p=inner_p, outer_p=outer_p, bandwidth=bandwidth, epsilon=epsilon, debug=debug,
                 _may_split=False)
    run_kernel_coefficients(kernel_descriptor, a2, b_slices, c_slices, partial[:full], **hyper)
    if leftover:
        run_kernel_coefficients(kernel_descriptor, a2, b2[full * rows:], c2[full * rows:], partial[full:], **hyper)
    target = plan.out[0] if plan.out.dim() == 3 else plan.out
    if target.is_contiguous():
        torch.sum(partial, dim=0, out=target)
    else:
        # the order in which torch adds the slices depends on the layout of the result: a strided
        # `out` gets the bits of a contiguous one
        target.copy_(torch.sum(partial, dim=0))
