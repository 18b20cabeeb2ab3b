"""``cdist``: p-norm distance matrix on the fused gfx950 kernel.

Same signature as the reference's ``kermac.cdist`` (src/kermac/cdist.py:9-17).
"""
from __future__ import annotations

import torch

from .build_a_kernel import (PowerType, kernel_descriptor_l1_norm, kernel_descriptor_l2_norm,
                             kernel_descriptor_p_norm, run_kernel)


def cdist(
    a: torch.Tensor,
    b: torch.Tensor,
    out: torch.Tensor = None,
    p: float = 2.0,
    skip_epilogue: bool = False,
    try_to_align: bool = False,
    debug=False,
):
    """Pairwise p-norm distances, ``torch.cdist`` semantics.

    In storage terms (``a_store[K,M]``, ``b_store[K,N]``, ``out_store[N,M]`` passed
    as ``.T`` views) this computes::

        out_store[n, m] = (sum_k |b_store[k, n] - a_store[k, m]| ** p) ** (1 / p)

    and with ``skip_epilogue`` the sum without the final ``1/p`` power.

    Args:
        a: ``[L?, M, K]`` fp32 on the GPU, row- or column-major.
        b: ``[L?, N, K]`` fp32 on the GPU.
        out: optional ``[L?, M, N]`` fp32 result, written in place and returned.
        p: norm order; 1.0 and 2.0 take paths without transcendental functions,
            3.0 and 4.0 too, 0.5 and 1.5 need one square root per term; any other
            value costs a log2 and an exp2 per term.
        skip_epilogue: return ``sum_k |b - a|**p``.
        try_to_align: accepted for compatibility; aligned operands always use
            128-bit accesses.
        debug: print what is launched.

    Raises:
        TypeError: non-tensor inputs or a dtype other than fp32.
        ValueError: bad shapes, strides, batch sizes or devices.

    Unlike the reference (cdist.py:65,75), ``skip_epilogue`` does not modify the
    shared predefined descriptors, and it works for fractional p.
    """
    if p == 1.0:
        # |x|^1 summed is already the 1-norm: there is no epilogue to skip.
        return run_kernel(kernel_descriptor_l1_norm, a, b, out=out, try_to_align=try_to_align, debug=debug)
    if p == 2.0:
        descriptor = kernel_descriptor_l2_norm
        if skip_epilogue:
            descriptor = descriptor._replace(outer_power=PowerType.NOOP)
        return run_kernel(descriptor, a, b, out=out, try_to_align=try_to_align, debug=debug)
    if skip_epilogue:
        descriptor = kernel_descriptor_p_norm._replace(outer_power=PowerType.NOOP)
        return run_kernel(descriptor, a, b, out=out, inner_p=float(p), try_to_align=try_to_align, debug=debug)
    return run_kernel(kernel_descriptor_p_norm, a, b, out=out, p=float(p), try_to_align=try_to_align, debug=debug)
