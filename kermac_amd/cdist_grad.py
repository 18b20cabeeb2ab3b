"""``cdist_grad``: fused kernel-gradient contraction (AGOP / RFM gradient).

Same signature as the reference's ``kermac.cdist_grad``
(src/kermac/cdist_grad.py:10-18).
"""
from __future__ import annotations

import os
from typing import Union

import numpy as np
import torch

from . import _backend
from . import _scratch
from .build_a_kernel import _current_stream_for
from .common import launch_cuts_enabled, merge_batch_size, tensor_stats

_NORM_L1, _NORM_L2, _NORM_P = 0, 1, 2


class _GradPlan:
    __slots__ = ("params", "out", "keepalive", "L", "M", "N", "O", "K")


def _plan_cdist_grad(a, b, c, d, out, p, require_device=True) -> _GradPlan:
    """Validation and parameter marshalling of ``cdist_grad``
    (reference: cdist_grad.py:62-235), without the launch."""
    if not all(isinstance(x, torch.Tensor) for x in (a, b, c, d)):
        raise TypeError("All inputs must be PyTorch tensors")
    if out is not None and not isinstance(out, torch.Tensor):
        raise TypeError("out must be a PyTorch tensor if provided")
    if not all(x.dtype == torch.float32 for x in (a, b, c, d)):
        raise TypeError("All inputs must have dtype torch.float32")
    if out is not None and out.dtype != torch.float32:
        raise TypeError("out must have dtype torch.float32")
    if not all(x.dim() in (2, 3) for x in (a, b, c, d)):
        raise ValueError("All inputs must be 2-dimensional or 3-dimensional with a batch mode")
    if out is not None and out.dim() not in (3, 4):
        raise ValueError("out must be 3-dimensional or 4-dimensional with a batch mode")
    if require_device:
        if not all(x.is_cuda for x in (a, b, c, d)):
            raise ValueError("All inputs must be on a CUDA device")
        if out is not None and not out.is_cuda:
            raise ValueError("out must be on a CUDA device")
    device = a.device
    if not all(x.device == device for x in (a, b, c, d)):
        raise ValueError(f"All inputs must be on the same CUDA device: got {[x.device for x in (a, b, c, d)]}")
    if out is not None and out.device != device:
        raise ValueError(f"out must be on the same CUDA device as inputs: got {out.device}, expected {device}")

    if isinstance(p, int) and not isinstance(p, bool):
        p = float(p)

    stats_a, stats_b, stats_c, stats_d = tensor_stats(a), tensor_stats(b), tensor_stats(c), tensor_stats(d)
    _, K, M = stats_a.shape
    _, N, K_b = stats_b.shape
    _, O, K_c = stats_c.shape
    _, N_d, M_d = stats_d.shape

    L = 1
    L = merge_batch_size("p", L, p, expected_dims=0, can_be_none=False)
    L = merge_batch_size("a", L, a, expected_dims=2, can_be_none=False)
    L = merge_batch_size("b", L, b, expected_dims=2, can_be_none=False)
    L = merge_batch_size("c", L, c, expected_dims=2, can_be_none=False)
    L = merge_batch_size("d", L, d, expected_dims=2, can_be_none=False)
    L = merge_batch_size("out", L, out, expected_dims=3, can_be_none=True)

    if (N, K_b) != (N, K):
        raise ValueError(f"Expected shape {(N, K)} for b, got {(N, K_b)}")
    if (O, K_c) != (O, K):
        raise ValueError(f"Expected shape {(O, K)} for c, got {(O, K_c)}")
    if (N_d, M_d) != (N, M):
        raise ValueError(f"Expected shape {(N, M)} for d, got {(N_d, M_d)}")
    if out is not None:
        if L == 1:
            if tuple(out.shape) not in ((O, N, M), (1, O, N, M)):
                raise ValueError(f"Expected shape {(O, N, M)} or {(L, O, N, M)} for out, got {tuple(out.shape)}")
        elif tuple(out.shape) != (L, O, N, M):
            raise ValueError(f"Expected shape {(L, O, N, M)} for out, got {tuple(out.shape)}")

    for name, x in (("a", a), ("b", b), ("c", c), ("d", d)):
        if x.stride(-1) != 1:
            raise ValueError(f"{name} must have stride 1 in last dimension")
    if out is not None and out.stride(-1) != 1:
        raise ValueError("out must have stride 1 in last dimension")

    if isinstance(p, float):
        p_ptr, p_bs, p_value, p_keep = 0, 0, float(np.float32(p)), None
        scalar_p = p_value
    else:
        if not isinstance(p, torch.Tensor):
            raise TypeError("`p` must be a float or a torch.Tensor")
        if p.dtype != torch.float32:
            raise TypeError("`p` tensor must have dtype torch.float32")
        if require_device and (not p.is_cuda or p.device != device):
            raise ValueError("`p` tensor must be on the same CUDA device as inputs")
        if p.numel() != 1 and p.numel() != L:
            raise ValueError(f"`p` tensor has {p.numel()} elements but the batch size is {L}")
        p_ptr, p_value, p_keep = p.data_ptr(), 0.0, p
        p_bs = 0 if p.numel() == 1 else p.stride(0)
        # One device-to-host read, as in the reference (cdist_grad.py:181-190), to
        # pick the transcendental-free kernels for p = 1 and p = 2.
        scalar_p = p.item() if p.numel() == 1 else None

    if scalar_p == 1.0:
        norm_type = _NORM_L1
    elif scalar_p == 2.0:
        norm_type = _NORM_L2
    else:
        norm_type = _NORM_P

    if out is None:
        # every element is written by the kernel, so no fill is needed
        out = torch.empty((L, O, N, M), dtype=torch.float32, device=device)

    params = _backend.NormGradientParams()
    params.norm_type = norm_type
    params.flags = 0
    params.m, params.n, params.o, params.k, params.l = M, N, O, K, L
    params.a, params.a_ld, params.a_bs = a.data_ptr(), stats_a.leading_dimension_stride, stats_a.batch_stride
    params.b, params.b_ld, params.b_bs = b.data_ptr(), stats_b.leading_dimension_stride, stats_b.batch_stride
    params.c, params.c_ld, params.c_bs = c.data_ptr(), stats_c.leading_dimension_stride, stats_c.batch_stride
    params.d, params.d_ld, params.d_bs = d.data_ptr(), stats_d.leading_dimension_stride, stats_d.batch_stride
    params.e = out.data_ptr()
    params.e_ld_n = out.stride(-2)
    params.e_ld_o = out.stride(-3)
    params.e_bs = 0 if (L == 1 or out.dim() == 3) else out.stride(-4)
    params.p, params.p_bs, params.p_value = p_ptr, p_bs, p_value

    plan = _GradPlan()
    plan.params, plan.out, plan.keepalive = params, out, [a, b, c, d, out, p_keep]
    plan.L, plan.M, plan.N, plan.O, plan.K = L, M, N, O, K
    return plan


@_scratch.operator
def cdist_grad(
    a: torch.Tensor,           # [K,M]   m contiguous   kernel_matrix
    b: torch.Tensor,           # [N,K]   k contiguous   x
    c: torch.Tensor,           # [O,K]   k contiguous   coefs
    d: torch.Tensor,           # [N,M]   m contiguous   z
    out: torch.Tensor = None,  # [O,N,M] m contiguous   grad
    p: Union[float, torch.Tensor] = 2.0,
    debug=False,
    _may_split=True,
):
    """Gradient of the p-norm kernel contracted with coefficients::

        out[o, n, m] = sum_k c[o, k] * a[k, m] * sign(d[n, m] - b[n, k]) * |d[n, m] - b[n, k]| ** (p - 1)

    ``sign`` is ``copysign(1, x)`` (so ``sign(0) = 1``); for ``p = 2`` the weight is
    simply the difference.  Every tensor may carry a leading batch dimension of 1
    or L.  Returns ``out`` (allocated ``[L, O, N, M]`` when None; every element is written).

    Raises:
        TypeError: non-tensor inputs or a dtype other than fp32.
        ValueError: bad shapes, strides, batch sizes or devices.
    """
    plan = _plan_cdist_grad(a, b, c, d, out, p)
    split = _split_over_contraction(plan) if _may_split else None
    if split is not None and _run_split_over_contraction(split, plan, a, b, c, d, p, debug):
        return plan.out
    stream = _current_stream_for(a.device)
    if debug:
        print(f"(Kermac Debug) Launching kernel: norm_kernel_gradient<{('L1', 'L2', 'P')[plan.params.norm_type]}>")
    workspace = _attach_workspace(plan.params, a.device)
    _backend.norm_kernel_gradient(plan.params, stream)
    del workspace           # the launches are queued: the allocator hands the memory on in stream order
    return plan.out


def _attach_workspace(params, device):
    """Large L1 and L2 gradients run on the fp16 matrix instruction through a workspace (include/
    kermac_amd.h, kmc_norm_gradient_params::workspace.  L1: a and c split once into two fp16 pieces
    per value, the sign of d - b put on the pieces of a.  L2: the sum factors into
    (d - s) (c a) - (c (b - s)) a, one product of pieces); the library says how much it wants for
    this call, 0 when it would not use one.  KERMAC_AMD_GRADIENT_WORKSPACE=0 keeps every call on
    the fp32 kernels."""
    if os.environ.get("KERMAC_AMD_GRADIENT_WORKSPACE", "1") in ("", "0"):
        return None
    needed = _backend.norm_gradient_workspace_bytes(params)
    if needed == 0:
        return None
    workspace = _scratch.allocate(needed, device)
    if workspace is None:
        return None             # no room for it, or the caller's limit: the fp32 kernels need none
    params.workspace, params.workspace_bytes = workspace.data_ptr(), needed
    return workspace


# A workgroup owns 64 (m) x 32 or 16 (n) results and walks the whole contraction index k,
# so few samples and features against many centres (M = 2000, N = 100, K = 10000) launch a
# hundred workgroups on 256 CUs, and a few hundred workgroups, all started together, leave
# the CUs unevenly loaded (256 workgroups at O = 16: 65 TFLOP/s where 4096 reach 120).  Such
# an unbatched call is cut over k: slices of a, b and c become the batch of one launch
# through strided views (d broadcasts), every slice writes a partial result, and the
# partial results are summed in a fixed order.  Measured at N = 128, K = 4096, cut in 8:
# O = 16, M = 2048: 65 -> 96 TFLOP/s; O = 1, M = 4096: 24 -> 60; nothing from 1536
# workgroups on.
_SPLIT_BELOW_WORKGROUPS = 1536
_SPLIT_TARGET_WORKGROUPS = 3072
_SPLIT_MIN_DEPTH = 512                      # from 512 workgroups on: 1024, and 2048 for the matrix-core kernels
_SPLIT_MAX_SLICES = 24
_SPLIT_MAX_PARTIAL_BYTES = 512 << 20


def _split_over_contraction(plan):
    """(slices, k per slice, leftover k), or None when the call is launched as it is."""
    if plan.L != 1 or plan.M == 0 or plan.N == 0 or plan.O == 0 or not launch_cuts_enabled():
        return None
    M, N, O, K = plan.M, plan.N, plan.O, plan.K
    n_tile = 32 if O <= 8 else 16
    workgroups = -(-M // 64) * -(-N // n_tile) * max(1, -(-O // 32))
    min_depth = _SPLIT_MIN_DEPTH * (1 if workgroups < 512 else 2 if O <= 8 else 4)
    if workgroups >= _SPLIT_BELOW_WORKGROUPS or K < 2 * min_depth:
        return None
    slices = min(max(2, round(_SPLIT_TARGET_WORKGROUPS / workgroups)), K // min_depth, _SPLIT_MAX_SLICES,
                 _SPLIT_MAX_PARTIAL_BYTES // (4 * O * N * M) - 1)
    if slices < 2:
        return None
    depth = K // slices // 64 * 64       # whole K slices of the kernels; 16-byte alignment survives
    slices = K // depth
    return slices, depth, K - slices * depth


def _run_split_over_contraction(split, plan, a, b, c, d, p, debug):
    slices, depth, leftover = split
    a2, b2, c2, d2 = (t[0] if t.dim() == 3 else t for t in (a, b, c, d))
    M, N, O = plan.M, plan.N, plan.O
    partial = _scratch.allocate_floats((slices + (1 if leftover else 0), O, N, M), a.device)
    target = plan.out[0] if plan.out.dim() == 4 else plan.out
    # the order in which torch adds the slices depends on the layout of the result: a strided `out` gets the
    # bits of a contiguous one, through a buffer of its own
    staged = None if target.is_contiguous() or partial is None else _scratch.allocate_floats((O, N, M), a.device)
    if partial is None or (staged is None and not target.is_contiguous()):
        return False            # no memory for the partial results: the call goes out as it is
    a_slices = a2.as_strided((slices, depth, M), (depth * a2.stride(0), a2.stride(0), a2.stride(1)), a2.storage_offset())
    b_slices = b2.as_strided((slices, N, depth), (depth * b2.stride(1), b2.stride(0), b2.stride(1)), b2.storage_offset())
    c_slices = c2.as_strided((slices, O, depth), (depth * c2.stride(1), c2.stride(0), c2.stride(1)), c2.storage_offset())
    cdist_grad(a_slices, b_slices, c_slices, d2, out=partial[:slices], p=p, debug=debug, _may_split=False)
    if leftover:
        done = slices * depth
        cdist_grad(a2[done:], b2[:, done:], c2[:, done:], d2, out=partial[slices:], p=p, debug=debug, _may_split=False)
    if staged is None:
        torch.sum(partial, dim=0, out=target)
    else:
        torch.sum(partial, dim=0, out=staged)
        target.copy_(staged)
    return True
