"""Kernel descriptors and the fused kernel-matrix builder ``run_kernel``.

Same public surface as the reference's ``src/kermac/build_a_kernel.py``:
``InnerOperator``, ``PowerType``, ``KernelType``, ``Symmetry``,
``KernelDescriptor``, the six predefined descriptors,
``pre_compile_descriptors`` and ``run_kernel`` with the same positional order,
defaults, return value and exception types.  The work is done by the gfx950
kernels in ``csrc/kernels/build_kernel.hpp`` through the C ABI.

View convention (torch.cdist's): ``a`` is ``[L?, M, K]``, ``b`` is ``[L?, N, K]``,
``out`` is ``[L?, M, N]``.  The fast path is the "K-major panel" storage
``a_store[K, M]``, ``b_store[K, N]``, ``out_store[N, M]`` passed as ``.T`` views.
"""
from __future__ import annotations

import contextlib
import functools
import os
import threading
from enum import Enum, auto
from itertools import product
from typing import Any, List, Optional, Union

import numpy as np
import torch

from . import _backend
from . import _scratch
from .common import (Alignment, Majorness, PyTorchStreamWrapper, TensorStats, ceil_div, launch_cuts_enabled,
                     merge_batch_size, tensor_stats)
from .module_cache.module_cache import ModuleCache, build_kernel_function_name


class InnerOperator(Enum):
    DIFF = auto()
    DOT = auto()


class PowerType(Enum):
    NOOP = auto()
    ABS = auto()
    SQUARE = auto()
    SQRT = auto()
    POW = auto()


class KernelType(Enum):
    NONE = auto()
    LAPLACE = auto()
    GAUSSIAN = auto()


class Symmetry(Enum):
    NonSymmetric = auto()
    Symmetric = auto()


# Enum member -> C-ABI value (include/kermac_amd.h).
_INNER_OPERATOR_ABI = {InnerOperator.DIFF: 0, InnerOperator.DOT: 1}
_POWER_TYPE_ABI = {PowerType.NOOP: 0, PowerType.ABS: 1, PowerType.SQUARE: 2, PowerType.SQRT: 3, PowerType.POW: 4}
_KERNEL_TYPE_ABI = {KernelType.NONE: 0, KernelType.LAPLACE: 1, KernelType.GAUSSIAN: 2}
_MAJORNESS_ABI = {Majorness.COL_MAJOR: _backend.COL_MAJOR, Majorness.ROW_MAJOR: _backend.ROW_MAJOR}
# (majorness, alignment) -> device loader variant (csrc/kernels/device_common.hpp LoadMode).
_LOAD_MODE = {
    (Majorness.COL_MAJOR, Alignment.ALIGN_4): 0,
    (Majorness.COL_MAJOR, Alignment.ALIGN_1): 1,
    (Majorness.ROW_MAJOR, Alignment.ALIGN_4): 2,
    (Majorness.ROW_MAJOR, Alignment.ALIGN_1): 3,
}


class KernelDescriptor:
    """What the fused kernel computes per output element
    (reference: build_a_kernel.py:39-71):

    ``kernel_type( outer_power( sum_k inner_power( a[m,k] (-|*) b[n,k] ) ) )``
    """

    def __init__(self, inner_operator, inner_power, outer_power, kernel_type):
        self._inner_operator = inner_operator
        self._inner_power = inner_power
        self._outer_power = outer_power
        self._kernel_type = kernel_type

    def _replace(self, **fields) -> "KernelDescriptor":
        current = dict(inner_operator=self._inner_operator, inner_power=self._inner_power,
                       outer_power=self._outer_power, kernel_type=self._kernel_type)
        current.update(fields)
        return KernelDescriptor(**current)

    def _render_function_name(self, majorness_A, majorness_B, align_A, align_B):
        """Template-id of the device function for this descriptor and operand
        layout.  Outer power and kernel type are run-time arguments of the gfx950
        kernel, so they are not part of the name (one binary serves them all)."""
        return build_kernel_function_name(
            _INNER_OPERATOR_ABI[self._inner_operator],
            _POWER_TYPE_ABI[self._inner_power],
            _LOAD_MODE[(majorness_A, align_A)],
            _LOAD_MODE[(majorness_B, align_B)],
        )

    def __repr__(self):
        return (f"KernelDescriptor({self._inner_operator.name}, {self._inner_power.name}, "
                f"{self._outer_power.name}, {self._kernel_type.name})")


kernel_descriptor_laplace_l1 = KernelDescriptor(
    inner_operator=InnerOperator.DIFF, inner_power=PowerType.ABS,
    outer_power=PowerType.NOOP, kernel_type=KernelType.LAPLACE)

kernel_descriptor_laplace_l2 = KernelDescriptor(
    inner_operator=InnerOperator.DIFF, inner_power=PowerType.SQUARE,
    outer_power=PowerType.SQRT, kernel_type=KernelType.LAPLACE)

kernel_descriptor_p_norm = KernelDescriptor(
    inner_operator=InnerOperator.DIFF, inner_power=PowerType.POW,
    outer_power=PowerType.POW, kernel_type=KernelType.NONE)

kernel_descriptor_l1_norm = KernelDescriptor(
    inner_operator=InnerOperator.DIFF, inner_power=PowerType.ABS,
    outer_power=PowerType.NOOP, kernel_type=KernelType.NONE)

kernel_descriptor_l2_norm = KernelDescriptor(
    inner_operator=InnerOperator.DIFF, inner_power=PowerType.SQUARE,
    outer_power=PowerType.SQRT, kernel_type=KernelType.NONE)

kernel_descriptor_mma = KernelDescriptor(
    inner_operator=InnerOperator.DOT, inner_power=PowerType.NOOP,
    outer_power=PowerType.NOOP, kernel_type=KernelType.NONE)


def pre_compile_descriptors(device, descriptors: List[Any], try_to_align=False, debug=False):
    """Make every operand-layout variant of ``descriptors`` ready before the
    first call (reference: build_a_kernel.py:121-156).

    Variants that ship ahead-of-time compiled in the library need nothing; the
    others are compiled with hiprtc in one program and stored in the on-disk
    kernel cache.  ``try_to_align`` adds the 16-byte-aligned loader variants,
    as in the reference.
    """
    layouts = [(Majorness.ROW_MAJOR, Alignment.ALIGN_1), (Majorness.COL_MAJOR, Alignment.ALIGN_1)]
    if try_to_align:
        if debug:
            print("(Kermac Debug) Because `try_to_align` is set, generating full matrix of alignment conditions")
        layouts += [(Majorness.COL_MAJOR, Alignment.ALIGN_4), (Majorness.ROW_MAJOR, Alignment.ALIGN_4)]

    function_names = []
    for descriptor in descriptors:
        op = _INNER_OPERATOR_ABI[descriptor._inner_operator]
        power = _POWER_TYPE_ABI[descriptor._inner_power]
        if _backend.build_kernel_has_variant(op, power):
            if debug:
                print(f"(Kermac Debug) {descriptor!r} is compiled ahead of time")
            continue
        for (majorness_A, align_A), (majorness_B, align_B) in product(layouts, layouts):
            name = descriptor._render_function_name(majorness_A, majorness_B, align_A, align_B)
            if name not in function_names:
                function_names.append(name)
    if function_names:
        ModuleCache(debug).compile_and_cache_functions(device=device, function_names=function_names, debug=debug)


def _hyper_parameter(name, value, L, device, require_device):
    """Normalise a scalar hyper-parameter to (pointer, batch stride, by-value, keepalive).

    A Python number is passed by value in the parameter block (no device
    allocation, no host-to-device copy).  A tensor must be fp32 on ``device``
    with 0 dimensions, or 1 dimension of length 1 or L; it is read in place.
    """
    if value is None:
        return 0, 0, 0.0, None
    if isinstance(value, (float, int)) and not isinstance(value, bool):
        return 0, 0, float(np.float32(value)), None
    if not isinstance(value, torch.Tensor):
        raise TypeError(f"`{name}` must be a float or a torch.Tensor")
    if value.dtype != torch.float32:
        raise TypeError(f"`{name}` tensor must have dtype torch.float32")
    if require_device and (not value.is_cuda or value.device != device):
        raise ValueError(f"`{name}` tensor must be on the same CUDA device as inputs")
    if value.dim() > 1:
        raise ValueError(f"`{name}` tensor must have 0 or 1 dimensions, got {value.dim()}")
    if value.numel() == 1:
        return value.data_ptr(), 0, 0.0, value
    if value.numel() != L:
        raise ValueError(f"`{name}` tensor has {value.numel()} elements but the batch size is {L}")
    return value.data_ptr(), value.stride(0), 0.0, value


# How DIFF + SQUARE descriptors (L2 norm, Laplace-L2, Gaussian) are evaluated.
#   "direct": subtract, square, accumulate on the vector ALU (the reference's arithmetic).
#   "gram":   |a|^2 + |b|^2 - 2 a.b with the cross term on the matrix cores, and the
#             direct kernel re-run on every 128 x 128 tile where cancellation makes
#             that untrustworthy (any element below trust * (|a|^2 + |b|^2)).
#   "gram_bf16": the same with the cross term on the (13 x faster) bf16 matrix
#             instruction, each fp32 operand split into three bf16 pieces; same
#             accuracy, same trust rule.  run_kernel only (the fused coefficient
#             product uses the fp32 matrix instruction in both gram modes).
#   Contractions shorter than `min_k` stay on the direct kernel in every mode: such
#   launches are bound by the result stores, and the direct kernel has the cheaper
#   epilogue and no repair launch (M = N = 30000, K = 16: 1.2 ms against 2.4 .. 2.6 ms).
_L2_DEFAULT_MIN_K = 64
_L2_AUTO_MIN_TERMS = 5e8          # "auto", coefficient products: a bound of L * M * N * K terms in their rules
_L2_MODES = ("direct", "gram", "gram_bf16", "auto")
# The process-wide setting, and per host thread what `l2_mode(...)` blocks have put on top
# of it: two threads can evaluate squared differences in different modes at the same time.
DEFAULT_L2_MODE = os.environ.get("KERMAC_AMD_L2_MODE", "auto")      # what the process starts with
_l2_process = {"mode": DEFAULT_L2_MODE, "trust": None, "min_k": _L2_DEFAULT_MIN_K}
if _l2_process["mode"] not in _L2_MODES:
    raise ValueError(f"KERMAC_AMD_L2_MODE must be one of {_L2_MODES}, got {_l2_process['mode']!r}")
_l2_thread = threading.local()


def _l2_setting(mode, trust, min_k):
    if mode not in _L2_MODES:
        raise ValueError(f"l2 mode must be 'direct', 'gram', 'gram_bf16' or 'auto', got {mode!r}")
    if trust is not None and not trust > 0.0:
        raise ValueError("trust must be positive")
    if min_k is not None and min_k < 0:
        raise ValueError("min_k must not be negative")
    return {"mode": mode, "trust": trust, "min_k": _L2_DEFAULT_MIN_K if min_k is None else int(min_k)}


def _l2_current():
    stack = getattr(_l2_thread, "stack", None)
    return stack[-1] if stack else _l2_process


def set_l2_mode(mode: str, trust: Optional[float] = None, min_k: Optional[int] = None) -> None:
    """Choose, for the whole process, how squared-difference descriptors (L2 norm, Laplace-L2, Gaussian) are
    evaluated.  A thread inside an ``l2_mode(...)`` block keeps the mode of its block.

    ``"auto"`` (the default; ``KERMAC_AMD_L2_MODE`` sets what the process starts with): by shape -- large
        problems through a workspace on the fp16 matrix instruction (two fp16 pieces per value, three piece
        products), mid-size ones on the one-step matrix-core kernels, short contractions (K < ``min_k``) and
        small ones on the direct kernel; every matrix-core route checks its result against
        ``trust * (|a|^2 + |b|^2)`` and has the direct kernel recompute what fails.  The arithmetic differs from
        the reference's fp32 subtract-square-accumulate; the stated tolerance (1e-5 relative to the float64
        truth) is the same.
    ``"direct"``: the reference's arithmetic everywhere (fp32 on the vector ALU).
    ``"gram"``: ``|a|^2 + |b|^2 - 2 a.b`` with the cross term on the fp32 matrix instruction.
    ``"gram_bf16"``: the cross term from 16-bit pieces (the workspace route where the library takes it, else
        three bf16 pieces split inside the kernel).

    ``trust`` (matrix-core routes) is the fraction of ``|a|^2 + |b|^2`` below which a squared distance is recomputed
    directly.  The default, ``max(0.25, sqrt(K) * 2**-24 / 8e-6)``, keeps the relative error of a trusted squared
    distance below about 8e-6 on the one-step kernels.  The workspace route stops the rule at 0.5 (it would pass 1
    near K = 18000 and send everything to the direct kernel, whose own fp32 sum over so many terms is no better): for
    K above about 4500 the error of a trusted squared distance there is bounded by ``sqrt(K) * 2**-24 / 0.5``, 1.1e-5 at
    K = 8192 (5e-6 on the distance itself), and both kernels' measured errors stay below 1e-5 of the distance up to
    K = 200000.
    ``min_k`` (default 64): contractions shorter than this use the direct kernel, which is the faster one there.
    """
    _l2_process.update(_l2_setting(mode, trust, min_k))


@contextlib.contextmanager
def l2_mode(mode: str, trust: Optional[float] = None, min_k: Optional[int] = None):
    """``with kermac.l2_mode("gram"): ...`` evaluates squared-difference descriptors in
    ``mode`` for the calls the current host thread makes inside the block; other threads
    and the process-wide setting (``set_l2_mode``) are not affected.  Arguments as for
    ``set_l2_mode``; blocks nest."""
    setting = _l2_setting(mode, trust, min_k)
    stack = getattr(_l2_thread, "stack", None)
    if stack is None:
        stack = _l2_thread.stack = []
    stack.append(setting)
    try:
        yield
    finally:
        stack.pop()


def get_l2_mode() -> str:
    return _l2_current()["mode"]


def _gram_trust(K: int, setting) -> float:
    if setting["trust"] is not None:
        return float(setting["trust"])
    return max(0.25, (K ** 0.5) * 2.0 ** -24 / 8e-6)


# How DIFF + ABS descriptors (L1 norm, Laplace-L1) are evaluated.
#   "direct": subtract, add |x| on the vector ALU in fp32 (the reference's arithmetic).  The default.
#   "fixed":  large stored matrices on 32-bit fixed point: both operands rounded once to a common
#             power-of-two grid (in a workspace allocated per call, as large as the operands), the
#             sums of |qb - qa| on one integer instruction per term, exactly; an element whose distance
#             is so small against the grid step that the rounding of the operands could show
#             (relative error bound above `tolerance`, 8e-6 unless given) has its 128 x 128 tile
#             recomputed by the direct kernel.  About 0.85 of the direct kernel's time at
#             M = N = 30000, K = 1024, and closer to the exact sums on spread-out data.
_L1_MODES = ("direct", "fixed")
DEFAULT_L1_MODE = os.environ.get("KERMAC_AMD_L1_MODE", "direct")
_l1_process = {"mode": DEFAULT_L1_MODE, "tolerance": None}
if _l1_process["mode"] not in _L1_MODES:
    raise ValueError(f"KERMAC_AMD_L1_MODE must be one of {_L1_MODES}, got {_l1_process['mode']!r}")
_l1_thread = threading.local()


def _l1_setting(mode, tolerance):
    if mode not in _L1_MODES:
        raise ValueError(f"l1 mode must be 'direct' or 'fixed', got {mode!r}")
    if tolerance is not None and not 0.0 < tolerance < 1.0:
        raise ValueError("tolerance must lie between 0 and 1")
    return {"mode": mode, "tolerance": tolerance}


def _l1_current():
    stack = getattr(_l1_thread, "stack", None)
    return stack[-1] if stack else _l1_process


def set_l1_mode(mode: str, tolerance: Optional[float] = None) -> None:
    """Choose, for the whole process, how sums of absolute differences (``cdist(p=1)``, the L1-norm and
    Laplace-L1 descriptors) are evaluated: ``"direct"`` (default; fp32 on the vector ALU, the
    reference's arithmetic) or ``"fixed"`` (large stored matrices on 32-bit fixed point with one
    integer instruction per term; elements whose relative error bound exceeds ``tolerance``, 8e-6
    by default, are recomputed by the direct kernel tile by tile).  A thread inside an
    ``l1_mode(...)`` block keeps the mode of its block."""
    _l1_process.update(_l1_setting(mode, tolerance))


@contextlib.contextmanager
def l1_mode(mode: str, tolerance: Optional[float] = None):
    """``with kermac.l1_mode("fixed"): ...`` for the calls the current host thread makes inside the
    block; arguments as for ``set_l1_mode``; blocks nest."""
    setting = _l1_setting(mode, tolerance)
    stack = getattr(_l1_thread, "stack", None)
    if stack is None:
        stack = _l1_thread.stack = []
    stack.append(setting)
    try:
        yield
    finally:
        stack.pop()


def get_l1_mode() -> str:
    return _l1_current()["mode"]


class _LaunchPlan:
    """Everything needed to launch: the C parameter block, the tensor that will
    be returned, and references that keep device memory alive until launch."""

    __slots__ = ("params", "out", "keepalive", "swapped", "L", "M", "N", "K", "l2_auto")


def _plan_run_kernel(
    kernel_descriptor, a, b, out, p, inner_p, outer_p, bandwidth, epsilon, regularization,
    regularization_offset_x, regularization_offset_y, try_to_align, require_device=True, allocate_out=True,
) -> _LaunchPlan:
    """Validation, batch merge, layout analysis and parameter marshalling of
    ``run_kernel`` (reference: build_a_kernel.py:174-390), without the launch."""
    d = kernel_descriptor
    # Descriptor / hyper-parameter consistency (reference: :174-199).
    if d._inner_power is PowerType.POW:
        if p is None and inner_p is None:
            raise ValueError("'inner_power' 'PowerType' is 'Pow' but 'p' and 'inner_p' is not set")
    elif p is not None or inner_p is not None:
        raise ValueError("'inner_power' 'PowerType' is not 'Pow' but 'p' or 'inner_p' is set")
    if d._outer_power is PowerType.POW:
        if p is None and outer_p is None:
            raise ValueError("'outer_power' 'PowerType' is 'Pow' but 'p' and 'outer_p' is not set")
    elif p is not None or outer_p is not None:
        raise ValueError("'outer_power' 'PowerType' is not 'Pow' but 'p' or 'outer_p' is set")
    if d._kernel_type is KernelType.NONE:
        if bandwidth is not None or epsilon is not None or regularization is not None:
            raise ValueError("'KernelType' is 'None' but 'bandwidth' or 'epsilon' or 'regularization' is set")
    elif bandwidth is None:
        raise ValueError("'KernelType' is not 'None' but 'bandwidth' is not set")
    if p is not None and inner_p is not None:
        raise ValueError("'p' is not 'None' but 'inner_p' is also not 'None")
    if p is not None and outer_p is not None:
        raise ValueError("'p' is not 'None' but 'outer_p' is also not 'None")

    def as_float(x):
        return float(x) if isinstance(x, int) and not isinstance(x, bool) else x

    p, inner_p, outer_p = as_float(p), as_float(inner_p), as_float(outer_p)
    bandwidth, regularization = as_float(bandwidth), as_float(regularization)

    # Batch size: every operand's batch is 1 or the common L (reference: :203-211).
    L = 1
    L = merge_batch_size("p", L, p, expected_dims=0, can_be_none=True)
    L = merge_batch_size("inner_p", L, inner_p, expected_dims=0, can_be_none=True)
    L = merge_batch_size("outer_p", L, outer_p, expected_dims=0, can_be_none=True)
    L = merge_batch_size("bandwidth", L, bandwidth, expected_dims=0, can_be_none=True)
    L = merge_batch_size("regularization", L, regularization, expected_dims=0, can_be_none=True)
    if not isinstance(a, torch.Tensor) or not isinstance(b, torch.Tensor):
        raise TypeError("a and b must be PyTorch tensors")
    if out is not None and not isinstance(out, torch.Tensor):
        raise TypeError("out must be a PyTorch tensor if provided")
    L = merge_batch_size("a", L, a, expected_dims=2, can_be_none=False)
    L = merge_batch_size("b", L, b, expected_dims=2, can_be_none=False)
    L = merge_batch_size("out", L, out, expected_dims=2, can_be_none=True)

    if a.dtype != torch.float32 or b.dtype != torch.float32:
        raise TypeError("a and b must have dtype torch.float32")
    if out is not None and out.dtype != torch.float32:
        raise TypeError("out must have dtype torch.float32")
    if require_device:
        if not a.is_cuda or not b.is_cuda:
            raise ValueError("a and b must be on a CUDA device")
        if out is not None and not out.is_cuda:
            raise ValueError("out must be on a CUDA device")
    device = a.device
    if b.device != device:
        raise ValueError(f"All inputs must be on the same CUDA device: got {[x.device for x in (a, b)]}")
    if out is not None and out.device != device:
        raise ValueError(f"out must be on the same CUDA device as inputs: got {out.device}, expected {device}")

    stats_a, stats_b = tensor_stats(a), tensor_stats(b)
    _, M, K_a = stats_a.shape
    _, N, K_b = stats_b.shape
    if K_a != K_b:
        raise ValueError(f"K dimensions must match: got {K_a} for a and {K_b} for b")
    K = K_a

    if out is not None:
        stats_c = tensor_stats(out)
        L_c, M_c, N_c = stats_c.shape
        if (M_c, N_c) != (M, N):
            raise ValueError(f"out must have shape (M={M}, N={N}), got {(M_c, N_c)}")
        if L_c != L and L != 1:
            raise ValueError(f"out must have batch dimension (L={L}), got {(L_c)}")
    elif allocate_out:
        # every element is written by the kernel (also for K = 0), so no fill is needed; the
        # reference allocates zeros (build_a_kernel.py:259), which costs 0.6 ms at 30000 x 30000
        out = torch.empty((L, M, N), dtype=torch.float32, device=device)
        stats_c = tensor_stats(out)
    else:
        stats_c = None

    keepalive = [a, b, out]

    # Hyper-parameters.  `p` sets inner = p and outer = 1/p, both rounded to fp32
    # the way the reference's device-side division does (reference: :281-290).
    if p is not None:
        if isinstance(p, float):
            inner_p = float(np.float32(p))
            outer_p = float(np.float32(1.0) / np.float32(p)) if p != 0.0 else float("inf")
        else:
            if not isinstance(p, torch.Tensor):
                raise TypeError("`p` must be a float or a torch.Tensor")
            if p.dtype != torch.float32:
                raise TypeError("`p` tensor must have dtype torch.float32")
            if require_device and (not p.is_cuda or p.device != device):
                raise ValueError("`p` tensor must be on the same CUDA device as inputs")
            inner_p = p.contiguous()
            outer_p = 1.0 / inner_p
    pi_ptr, pi_bs, pi_val, pi_keep = _hyper_parameter("inner_p", inner_p, L, device, require_device)
    po_ptr, po_bs, po_val, po_keep = _hyper_parameter("outer_p", outer_p, L, device, require_device)
    bw_ptr, bw_bs, bw_val, bw_keep = _hyper_parameter("bandwidth", bandwidth, L, device, require_device)
    rg_ptr, rg_bs, rg_val, rg_keep = _hyper_parameter("regularization", regularization, L, device, require_device)
    keepalive += [pi_keep, po_keep, bw_keep, rg_keep]

    # The kernel writes C with m contiguous.  A row-major out is the transpose of
    # that, so swap the operands (reference: :323-336).  The reference swaps neither the
    # regularisation offsets nor the sign of a signed inner term, so there the result
    # depends on the layout of `out`.  Here it does not: every layout gives what the
    # reference returns for `out=None` (a row-major result, the case all of its users
    # see): the inner difference is a[m] - b[n] and the regularised elements are those
    # with offset_x + n == offset_y + m.  The kernel itself computes B - A and tests
    # offset_x + (row of A) == offset_y + (row of B), so the swapped launch passes
    # through as it is and the unswapped one exchanges the offsets and negates.
    swapped = stats_c is not None and stats_c.majorness is Majorness.ROW_MAJOR
    off_x, off_y = int(regularization_offset_x), int(regularization_offset_y)
    if swapped:
        M, N = N, M
        a, b = b, a
        stats_a, stats_b = stats_b, stats_a
    else:
        off_x, off_y = off_y, off_x

    params = _backend.BuildKernelParams()
    params.inner_operator = _INNER_OPERATOR_ABI[d._inner_operator]
    params.inner_power = _POWER_TYPE_ABI[d._inner_power]
    params.outer_power = _POWER_TYPE_ABI[d._outer_power]
    params.kernel_type = _KERNEL_TYPE_ABI[d._kernel_type]
    params.a_majorness = _MAJORNESS_ABI[stats_a.majorness]
    params.b_majorness = _MAJORNESS_ABI[stats_b.majorness]
    params.flags = 0 if swapped else _backend.FLAG_NEGATE_DIFF
    if os.environ.get("KERMAC_AMD_NO_SYMMETRY", "0") not in ("", "0"):
        # the library computes x-against-x matrices from the tiles on and below the diagonal
        # (bit-identical result, about half the time); this keeps it to the full computation
        params.flags |= _backend.FLAG_NO_SYMMETRY
    l2 = _l2_current()
    l2_auto = False
    if (l2["mode"] != "direct" and d._inner_operator is InnerOperator.DIFF
            and d._inner_power is PowerType.SQUARE and K >= l2["min_k"]):
        # "auto": a candidate for the matrix cores from min_k on; run_kernel decides for a stored matrix
        # (_auto_matrix_core_flags), run_kernel_coefficients for the coefficient product (no out matrix
        # here), whose fused kernel has a matrix-core variant too
        l2_auto = l2["mode"] == "auto"
        params.flags |= _backend.FLAG_L2_GRAM
        if l2["mode"] == "gram_bf16" or (l2_auto and stats_c is not None):
            params.flags |= _backend.FLAG_L2_GRAM_BF16
        params.gram_trust = _gram_trust(K, l2)
    elif (l2["mode"] in ("auto", "gram_bf16") and d._inner_operator is InnerOperator.DOT
            and d._inner_power is PowerType.NOOP and K >= l2["min_k"] and stats_c is not None):
        # sums of products (linear and polynomial kernels): large ones on the fp16 matrix instruction from two
        # fp16 pieces per value, when the library has a use for the workspace that run_kernel offers it
        l2_auto = l2["mode"] == "auto"
        params.flags |= _backend.FLAG_DOT_PIECES
    l1 = _l1_current()
    if (l1["mode"] == "fixed" and d._inner_operator is InnerOperator.DIFF and d._inner_power is PowerType.ABS
            and stats_c is not None):
        # sums of absolute differences: large stored matrices on fixed point, when the library has a
        # use for the workspace that run_kernel offers it
        params.flags |= _backend.FLAG_L1_FIXED
        if os.environ.get("KERMAC_AMD_L1_FIXED_ANY_SIZE", "0") not in ("", "0"):
            params.flags |= _backend.FLAG_GRAM_WORKSPACE_ANY_SIZE      # tests send small shapes down the route
        if l1["tolerance"] is not None:
            params.gram_trust = float(l1["tolerance"])
    params.m, params.n, params.k, params.l = M, N, K, L
    params.a, params.a_ld, params.a_bs = a.data_ptr(), stats_a.leading_dimension_stride, stats_a.batch_stride
    params.b, params.b_ld, params.b_bs = b.data_ptr(), stats_b.leading_dimension_stride, stats_b.batch_stride
    if stats_c is not None:
        params.c, params.c_ld, params.c_bs = out.data_ptr(), stats_c.leading_dimension_stride, stats_c.batch_stride
    params.p_inner, params.p_inner_bs, params.p_inner_value = pi_ptr, pi_bs, pi_val
    params.p_outer, params.p_outer_bs, params.p_outer_value = po_ptr, po_bs, po_val
    params.bandwidth, params.bandwidth_bs, params.bandwidth_value = bw_ptr, bw_bs, bw_val
    params.regularization, params.regularization_bs, params.regularization_value = rg_ptr, rg_bs, rg_val
    params.regularization_offset_x, params.regularization_offset_y = off_x, off_y
    params.epsilon = 1e-5 if epsilon is None else float(epsilon)

    plan = _LaunchPlan()
    plan.params, plan.out, plan.keepalive, plan.swapped = params, out, keepalive, swapped
    plan.L, plan.M, plan.N, plan.K = L, M, N, K
    plan.l2_auto = l2_auto
    return plan


_raw_current_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _current_stream_for(device: torch.device) -> int:
    """The hipStream_t of torch's current stream, which must be on the tensors' device
    (reference: build_a_kernel.py:314-321).  The raw-handle accessor saves the construction of
    a Stream object on every call; a launch costs about 10 microseconds of host time."""
    current = torch.cuda.current_device()
    index = current if device.index is None else device.index
    if current != index:
        raise ValueError(f"cuda stream must be on the same device as the tensors: got cuda:{current}, expected {device}")
    if _raw_current_stream is not None:
        return _raw_current_stream(index)
    return PyTorchStreamWrapper(torch.cuda.current_stream()).handle


@_scratch.operator
def run_kernel(
    kernel_descriptor: KernelDescriptor,
    a: torch.Tensor,
    b: torch.Tensor,
    out: torch.Tensor = None,
    p: Optional[Union[float, torch.Tensor]] = None,
    inner_p: Optional[Union[float, torch.Tensor]] = None,
    outer_p: Optional[Union[float, torch.Tensor]] = None,
    bandwidth: Optional[Union[float, torch.Tensor]] = None,
    epsilon: Optional[float] = None,
    regularization: Optional[Union[float, torch.Tensor]] = None,
    regularization_offset_x: int = 0,
    regularization_offset_y: int = 0,
    try_to_align: bool = False,
    debug=False,
    coefficients: Optional[torch.Tensor] = None,
):
    """Fused pairwise kernel matrix (reference: build_a_kernel.py:158-394).

    ``out[l, m, n] = kernel_type(outer_power(sum_k inner_power(a[l,m,k] (-|*) b[l,n,k])))``
    followed, for Laplace/Gaussian kernels with a non-zero ``regularization``,
    by replacing every element with ``offset_x + n == offset_y + m`` by
    ``1 + regularization``.  ``a``, ``b``, ``out`` and the hyper-parameter
    tensors may each carry a leading batch dimension of 1 or L; a missing batch
    broadcasts.  Returns ``out`` (allocated ``[L, M, N]`` when None).

    The sign of the difference (it matters for the inner powers NOOP and SQRT only)
    and the side each offset belongs to are those of the reference's result for
    ``out=None``; the reference gives the mirrored convention when it is handed a
    column-major ``out`` (it swaps the operands but not the offsets or the sign,
    build_a_kernel.py:323-336), here the result is the same for every layout of ``out``.

    ``try_to_align`` is accepted for signature compatibility: 128-bit accesses
    are used whenever pointer, leading dimension and batch stride allow them.

    ``coefficients`` (an addition to the reference's signature): a ``[L?, N, O]``
    tensor with the ``O`` columns contiguous (any number of them).  When given, the kernel matrix is
    contracted with it on the fly and ``out`` is ``[L?, M, O]``:
    ``out[l, m, o] = sum_n kernelmatrix[l, m, n] * coefficients[l, n, o]``; the
    M x N matrix is never written to memory.
    """
    if coefficients is not None:
        from .kernel_coefficients import run_kernel_coefficients
        return run_kernel_coefficients(
            kernel_descriptor, a, b, coefficients, out=out, p=p, inner_p=inner_p, outer_p=outer_p,
            bandwidth=bandwidth, epsilon=epsilon, regularization=regularization,
            regularization_offset_x=regularization_offset_x, regularization_offset_y=regularization_offset_y,
            debug=debug)

    plan = _plan_run_kernel(
        kernel_descriptor, a, b, out, p, inner_p, outer_p, bandwidth, epsilon, regularization,
        regularization_offset_x, regularization_offset_y, try_to_align)
    stream = _current_stream_for(a.device)
    params = plan.params

    def launch(block):
        if _backend.build_kernel_has_variant(block.inner_operator, block.inner_power):
            if debug:
                print(f"(Kermac Debug) Launching ahead-of-time kernel for {kernel_descriptor!r}")
            _backend.build_kernel(block, stream)
        else:
            load_a, load_b = _backend.build_kernel_load_modes(block)
            function_name = build_kernel_function_name(block.inner_operator, block.inner_power, load_a, load_b)
            function = ModuleCache(debug).get_function(a.device, function_name, debug=debug)
            if debug:
                print(f"(Kermac Debug) Launching kernel: {function_name}")
            _backend.build_kernel_jit(function, block, stream)

    matrix_core = _backend.FLAG_L2_GRAM | _backend.FLAG_L2_GRAM_BF16 | _backend.FLAG_DOT_PIECES
    if plan.l2_auto and params.flags & matrix_core:
        asked = params.flags & matrix_core
        params.flags &= ~matrix_core
        params.flags |= _auto_matrix_core_flags(params, asked)
    if params.flags & _backend.FLAG_DOT_PIECES:
        # products have no matrix-core kernel beside the route through the workspace: a call the
        # library has no use for a workspace for is an ordinary call of the direct kernel
        workspace = _attach_gram_workspace(params, a.device)
        if workspace is None:
            params.flags &= ~_backend.FLAG_DOT_PIECES
        plan.keepalive.append(workspace)
    if params.flags & _backend.FLAG_L1_FIXED:
        # the fixed-point route exists only through a workspace: without one (a problem too small
        # for the library to want one, no memory) the call is an ordinary one of the direct kernel
        workspace = _attach_gram_workspace(params, a.device, switch="KERMAC_AMD_L1_WORKSPACE")
        if workspace is None:
            params.flags &= ~_backend.FLAG_L1_FIXED
        plan.keepalive.append(workspace)
    cut = _cut_over_contraction(params)
    if params.flags & (_backend.FLAG_L2_GRAM | _backend.FLAG_L2_GRAM_BF16):
        plan.keepalive.append(_attach_gram_centre(params, stream, a.device))
        plan.keepalive.append(_attach_gram_workspace(params, a.device))
    elif (cut is None and not params.flags & (_backend.FLAG_DOT_PIECES | _backend.FLAG_L1_FIXED)
            and params.inner_operator == _backend.OP_DIFF
            and (params.inner_power in (_backend.POW_ABS, _backend.POW_SQUARE)
                 or (params.inner_power == _backend.POW_POW and not params.p_inner and params.p_inner_value in (3.0, 4.0)
                     and not params.flags & _backend.FLAG_GENERIC_POWER))):
        # absolute differences and their squares, cubes and fourth powers on the direct kernel: large problems whose operands its fastest
        # variant cannot take as they are (k contiguous, as torch allocates them; K or N not multiples of 16) run
        # on copies that it can, when the library wants room for them (include/kermac_amd.h, KMC_FLAG_DIRECT_PANELS)
        any_size = os.environ.get("KERMAC_AMD_DIRECT_PANELS_ANY_SIZE", "0") not in ("", "0")     # tests send small shapes down the route
        # (the library decides; a call far below its size rule is not worth the question: small calls are bound by the host)
        if any_size or -(-params.m // 256) * -(-params.n // 64) >= _direct_panels_min_tiles():
            params.flags |= _backend.FLAG_DIRECT_PANELS
            if any_size:
                params.flags |= _backend.FLAG_GRAM_WORKSPACE_ANY_SIZE
            workspace = _attach_gram_workspace(params, a.device, switch="KERMAC_AMD_DIRECT_PANELS")
            if workspace is None:
                params.flags &= ~(_backend.FLAG_DIRECT_PANELS | _backend.FLAG_GRAM_WORKSPACE_ANY_SIZE)
            plan.keepalive.append(workspace)
    if cut is None:
        launch(params)
    else:
        _run_cut_over_contraction(cut, params, launch, stream, a.device)
    return plan.out


@functools.lru_cache(maxsize=1)
def _direct_panels_min_tiles() -> int:
    """The smallest count of 256 x 64 tiles per batch entry for which the library copies operands for its direct kernel."""
    return int(_backend.dispatch_rules()["DIRECT_PANELS_MIN_TILES"])


def _attach_gram_centre(params, stream, device):
    """Matrix-core launches subtract a point near the data from both operands while staging them
    (include/kermac_amd.h, gram_centre): the mean of a sample of the rows of the first operand,
    computed by the library into a small buffer allocated here.  KERMAC_AMD_L2_CENTRE=0 keeps the
    operands as they are."""
    if os.environ.get("KERMAC_AMD_L2_CENTRE", "1") in ("", "0") or params.m == 0 or params.k == 0 or params.l == 0:
        return None
    # per batch entry: the centre padded to a multiple of 64 floats, a flag (subtract or not: the
    # library leaves it out when the centre is negligible against the spread) and the variances
    width = 2 * (-(-params.k // _backend.CENTRE_PAD) * _backend.CENTRE_PAD) + _backend.CENTRE_PAD
    batches = params.l if params.a_bs != 0 else 1
    centre = _scratch.allocate_floats((batches, width), device)
    if centre is None:
        return None
    _backend.sample_mean(params.a, params.a_majorness, params.m, params.k, params.a_ld, params.a_bs, batches,
                         centre.data_ptr(), width, stream)
    params.gram_centre, params.gram_centre_bs = centre.data_ptr(), (width if batches > 1 else 0)
    return centre


# The l2 mode "auto", from sweeps of the public call over shapes, batches and storage orders
# (microseconds, direct / matrix cores):
#   * the route through a workspace wherever the library takes it (kmc_gram_workspace_bytes: large
#     problems from K = 64 on; 10000 x 10000 x 96 413 / 304, 4096 x 4096 x 4096 2400 cut / 530, 4096 x 4096 x 20000
#     12500 / 2300), sums of products nowhere else (they have no one-step kernel);
#   * the one-step kernels from K = 128 on (128 x 128 x 200 65 / 37, 8 x 256 x 256 x 512 141 / 54, 2000 x 2000 x 200
#     71 / 52; at K = 128 over ten shapes, k contiguous: 512 x 512 40 / 31, 1000 x 30000 165 / 127, 32 x 256 x 256 41 / 32,
#     4096 x 4096 90 / 86, 2000 x 2000 44 / 46, 2500 x 2500 50 / 59, the one that loses more than a tenth; with the rows
#     contiguous 2000 x 2000 45 / 36, 5000 x 5000 146 / 116; at K = 96 the direct kernel is ahead, 0.73 .. 0.97, but for
#     few rows against many: 1000 x 30000 x 96 130 / 115), unless the direct path would cut the call over k and the grid is
#     below 192 tiles (1024 x 1024 x 32768: 1400 cut / 10000; 1500 x 1500 x 3072 312 cut / 408), or the
#     contraction is so long that they trust nothing they compute (K > 18000: every tile would be redone);
#   * of the one-step kernels the fp32 one for K >= 384 on 128 to 768 tiles (2000 x 2000 x 784 fp32 135 / split 171,
#     8 x 1000 x 1000 x 3072 634 / 855), the split one otherwise (K = 200: 47 .. 55 / 37 .. 44; 4096 x 4096 x 512 212 / 161;
#     8 x 256 x 256 x 512, 32 tiles, 69 / 55), and for a single row of 128 tiles or more (4 x 100 x 50000
#     x 784 fp32 558 / split 857, at K = 256 252 / 340);
#   * the numbers above are for operands with k contiguous, as torch allocates them.  With the rows contiguous
#     (the kernels' own order) the split kernel stages faster: it is taken instead of the fp32 one (2500 x 2500 x 1024
#     fp32 198 / split 137), and uncut from 128 tiles on.
_AUTO_ONE_STEP_MIN_K = 128
_AUTO_FP32_MIN_K = 384
_AUTO_FP32_MIN_TILES = 128
_AUTO_FP32_MAX_TILES = 768
# ... and only for batch entries of 32 tiles and more: on batches of small entries the split kernel is far ahead
# (8 x 512 x 512 x 1024, k contiguous: fp32 108 / split 69 us; 32 x 256 x 256 x 3072 280 / 163; 8 x 700 x 700 x 1024 216 / 228)
_AUTO_FP32_MIN_TILES_PER_ENTRY = 32
# A call that the direct path would cut over k stays there below this many tiles: the matrix cores run it uncut.
# With k contiguous the one-step kernels stage more slowly and need more tiles to be ahead (1500 x 1500, 144 tiles:
# direct, cut / fp32 at K = 784 107 / 130 us, at K = 3072 312 / 408; 500 x 5000, 160 tiles, 125 / 121 and 343 / 396;
# 2000 x 2000, 256 tiles, 157 / 130 and 493 / 408; with the rows contiguous 1536 x 1536 x 4096 380 / 250).
_AUTO_UNCUT_MIN_TILES = 128
_AUTO_UNCUT_MIN_TILES_K_CONTIGUOUS = 192


def _auto_matrix_core_flags(params, asked):
    """Which of the matrix-core flags `asked` (those the descriptor allows) this call gets in the l2 mode "auto"."""
    if _workspace_route_applies(params, asked):
        return asked
    # operands with the rows contiguous (m or n, the kernels' own order) stage faster in the split kernel
    rows_contiguous = params.a_majorness == _backend.COL_MAJOR and params.b_majorness == _backend.COL_MAJOR
    if not asked & _backend.FLAG_L2_GRAM or params.k < _AUTO_ONE_STEP_MIN_K or params.gram_trust >= 1.0:
        return 0
    tiles = -(-params.m // 128) * -(-params.n // 128)
    if tiles < (_AUTO_UNCUT_MIN_TILES if rows_contiguous else _AUTO_UNCUT_MIN_TILES_K_CONTIGUOUS):
        kept = params.flags
        params.flags &= ~asked                  # the question is what the direct path would do
        try:
            if _cut_over_contraction(params) is not None:
                return 0
        finally:
            params.flags = kept
    if not rows_contiguous:
        if (params.k >= _AUTO_FP32_MIN_K and _AUTO_FP32_MIN_TILES <= tiles * params.l <= _AUTO_FP32_MAX_TILES
                and tiles >= _AUTO_FP32_MIN_TILES_PER_ENTRY):
            return _backend.FLAG_L2_GRAM
        if min(params.m, params.n) <= 128 and tiles * params.l >= _AUTO_FP32_MIN_TILES:      # one long row of tiles
            return _backend.FLAG_L2_GRAM
    return asked


def _workspace_route_applies(params, flags):
    """Whether kmc_build_kernel would take this call through a workspace, given these matrix-core flags."""
    if os.environ.get("KERMAC_AMD_L2_WORKSPACE", "1") in ("", "0"):
        return False
    kept = params.flags
    params.flags |= flags
    try:
        return _backend.gram_workspace_bytes(params) > 0
    finally:
        params.flags = kept


# The sample that the library takes in front of a one-step matrix-core kernel when it is handed KMC_SAMPLE_BYTES of
# workspace is one more launch, 5 to 8 us on the stream.  On data whose near-duplicates sit in every tile it saves the
# matrix cores' work (4096 x 4096 x 512: 441 -> 362 us where the direct kernel takes 319; 2048 x 2048 x 1024 374 -> 300
# against 193, the repair launch being the direct kernel uncut), on every other call it is a tax: 38 -> 46 us at
# 1024 x 1024 x 256.  From 4e9 terms on the tax is below a tenth.
_L2_SAMPLE_MIN_TERMS = 4_000_000_000


def _attach_gram_workspace(params, device, switch="KERMAC_AMD_L2_WORKSPACE"):
    """Large squared-difference problems in the split-bf16 mode go through a workspace (include/
    kermac_amd.h, gram_workspace: both operands split once into fp16 pieces, then 256 x 256 tiles);
    the library says how much it wants for this call, 0 when it would not use one.
    KERMAC_AMD_L2_WORKSPACE=0 keeps every call on the one-step kernel."""
    if os.environ.get(switch, "1") in ("", "0"):
        return None
    if os.environ.get("KERMAC_AMD_L2_PROBE", "1") in ("", "0"):
        params.flags |= _backend.FLAG_NO_PROBE      # no sample of the result in front of the matrix-core kernel
    needed = _backend.gram_workspace_bytes(params)
    if (needed == 0 and (params.flags & (_backend.FLAG_L2_GRAM | _backend.FLAG_L2_GRAM_BF16)) and not (params.flags & _backend.FLAG_NO_PROBE)
            and params.m * params.n * params.k * params.l >= _L2_SAMPLE_MIN_TERMS):
        needed = _backend.SAMPLE_BYTES              # a one-step kernel: room for the sample that is taken in front of it
    if needed == 0:
        return None
    workspace = _scratch.allocate(needed, device)
    if workspace is None:
        return None             # no room for it, or the caller's limit: the one-step kernel needs none
    params.gram_workspace, params.gram_workspace_bytes = workspace.data_ptr(), needed
    return workspace


# A workgroup owns one 128 x 128 tile of the result and walks the whole contraction index, so
# a small result over a long contraction (100 x 100 over k = 100000 is one tile) leaves the
# chip idle, and a few hundred tiles are a few workgroups per CU, all started together: the
# CUs that got one more set the time, and a CU works through such a single round at 0.73 of
# the rate it reaches on a long queue (576 tiles at K = 4096 run at 62 TFLOP/s, 1024 at 90).  Such an
# unbatched call is cut over k: ranges of k become the batch of one launch that stores plain
# sums (no outer power, no kernel function) into a buffer, and a second, element-wise kernel
# adds the partial sums in range order and applies the epilogue.  The number of ranges comes
# from a model of the launch time fitted to sweeps of M = N = 512 ... 5760, K = 1024 ... 16384.
_CUT_BELOW_TILES = 2048
_CUT_MIN_K = 512
_CUT_MIN_DEPTH = 128
_CUT_RANGES = (2, 3, 4, 5, 6, 8, 10, 12, 16, 20, 24, 32, 48, 64, 96, 128, 192, 256, 384, 512, 768)
_CUT_WORTH = 0.9                # cut only for at least 10 % less modelled time
_CUT_MAX_PARTIAL_BYTES = 512 << 20


def _launch_ms(workgroups, depth):
    """Modelled time of `workgroups` tiles that walk `depth` terms each, in milliseconds."""
    per_cu = workgroups / 256
    if per_cu <= 1:
        return (depth + 128) / 3900             # one wave per SIMD: latency bound
    if per_cu <= 3:
        return -(-workgroups // 256) * (depth + 128) / 7300      # one round
    return (per_cu + 1.92) * (depth + 40) / 10000                # rounds that the dispatcher balances


@functools.lru_cache(maxsize=256)
def _choose_cut(tiles, K, mirrored, plane_bytes):
    # A mirrored launch of so few tiles has one workgroup per tile of the triangle (no empty
    # ones); its workgroups store every tile twice.
    unsplit = _launch_ms(tiles, K)
    best = None
    seen = 0
    for wanted in _CUT_RANGES:
        depth = -(-K // (16 * wanted)) * 16
        if depth < _CUT_MIN_DEPTH:
            break
        ranges = -(-K // depth)
        if ranges < 2 or ranges == seen or ranges * plane_bytes > _CUT_MAX_PARTIAL_BYTES:
            continue
        seen = ranges
        workgroups = ranges * tiles
        cost = (_launch_ms(workgroups, depth)
                + 2.1e-5 * workgroups * (2 if mirrored else 1) + 0.01)      # partial sums stored and added, second launch
        if best is None or cost < best[0]:
            best = (cost, ranges, depth)
    if best is None or best[0] > _CUT_WORTH * unsplit:
        return None
    return best[1:]


def _cut_over_contraction(params):
    """(ranges of k, k per range), or None when the launch goes out as it is."""
    if params.l != 1 or params.flags & (_backend.FLAG_L2_GRAM | _backend.FLAG_L2_GRAM_BF16 | _backend.FLAG_DOT_PIECES
                                        | _backend.FLAG_L1_FIXED):
        return None
    tiles = -(-params.m // 128) * -(-params.n // 128)
    if tiles == 0 or params.k < _CUT_MIN_K or not launch_cuts_enabled():
        return None
    mirrored = (params.a == params.b and params.m == params.n and params.a_ld == params.b_ld
                and params.a_majorness == params.b_majorness and not params.flags & _backend.FLAG_NO_SYMMETRY)
    if mirrored:
        side = -(-params.m // 128)
        tiles = side * (side + 1) // 2      # the kernel computes one triangle and mirrors it
    if tiles >= _CUT_BELOW_TILES:
        return None
    return _choose_cut(tiles, params.k, bool(mirrored), 4 * -(-params.m // 4) * 4 * params.n)


def _run_cut_over_contraction(cut, params, launch, stream, device):
    slices, depth = cut
    ld = -(-params.m // 4) * 4
    plane = ld * params.n
    partial = _scratch.allocate_floats((slices * plane,), device)
    if partial is None:
        launch(params)          # no memory for the partial sums: the launch goes out as it is
        return

    def k_stride(majorness, leading):
        return leading if majorness == _backend.COL_MAJOR else 1

    ranges = _backend.BuildKernelParams.from_buffer_copy(params)
    ranges.outer_power, ranges.kernel_type = _POWER_TYPE_ABI[PowerType.NOOP], _KERNEL_TYPE_ABI[KernelType.NONE]
    ranges.k, ranges.l, ranges.k_total = depth, slices, params.k      # the last range is what is left of k
    ranges.a_bs = depth * k_stride(params.a_majorness, params.a_ld)
    ranges.b_bs = depth * k_stride(params.b_majorness, params.b_ld)
    ranges.c, ranges.c_ld, ranges.c_bs = partial.data_ptr(), ld, plane
    launch(ranges)
    _backend.build_kernel_finish(params, partial.data_ptr(), ld, 0, plane, slices, stream)
