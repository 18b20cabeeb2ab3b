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
import os
from typing import Optional

import torch

from . import _backend
from . import _scratch
from .common import launch_cuts_enabled, merge_batch_size
from .module_cache.module_cache import ModuleCache, build_kernel_function_name, kernel_coefficients_function_name


class _CoefPlan:
    __slots__ = ("params", "out", "keepalive", "L", "M", "N", "K", "O", "l2_auto")


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
    plan.l2_auto = base.l2_auto
    return plan


@_scratch.operator
def run_kernel_coefficients(
    kernel_descriptor, a, b, coefficients, out: Optional[torch.Tensor] = None, p=None, inner_p=None, outer_p=None,
    bandwidth=None, epsilon=None, regularization=None, regularization_offset_x: int = 0,
    regularization_offset_y: int = 0, debug=False,
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
    stream = _current_stream_for(a.device)
    params = plan.params
    kernel = params.kernel
    aot = _backend.kernel_times_coefficients_has_variant(kernel.inner_operator, kernel.inner_power)
    matrix_core = bool(kernel.flags & _backend.FLAG_L2_GRAM)
    if matrix_core:
        from .build_a_kernel import _attach_gram_centre
        panels = _panel_shape(plan, _backend.FLAG_L2_GRAM_BF16) if aot else None
        if panels is None and plan.l2_auto and not _auto_fused_on_matrix_cores(plan):
            kernel.flags &= ~(_backend.FLAG_L2_GRAM | _backend.FLAG_L2_GRAM_BF16)
            matrix_core = False
        else:
            plan.keepalive.append(_attach_gram_centre(kernel, stream, a.device))
            if panels is not None and _run_in_panels(plan, panels, stream, a.device, debug):
                return plan.out
    elif _products_in_panels(plan) and _backend.build_kernel_has_variant(kernel.inner_operator, kernel.inner_power):
        panels = _panel_shape(plan, _backend.FLAG_DOT_PIECES)
        if panels is not None and _run_in_panels(plan, panels, stream, a.device, debug):
            return plan.out
    if plan.O > _FUSED_COLUMNS_PER_WALK and float(plan.L) * plan.M * plan.N >= _MANY_COLUMNS_MIN_ELEMENTS:
        # any descriptor, compiled ahead of time or at run time: the fused kernel would walk the matrix once per 64 columns
        panels = _panel_shape(plan, 0)
        if panels is not None and _run_in_panels(plan, panels, stream, a.device, debug):
            return plan.out
    ranges = _centre_ranges(plan, three_resident=aot and not matrix_core and plan.O <= 32)
    partial = None
    if ranges > 1:
        # every range of centres writes its own partial product; they are added below in range order
        partial = _partial_products(ranges, plan, a.device)       # refused: the centres stay one range
    if partial is not None:
        params.out, params.out_ld, params.out_bs = partial[0].data_ptr(), plan.O, plan.M * plan.O
        params.n_ranges, params.out_range_stride = ranges, plan.L * plan.M * plan.O
    if aot:
        if debug:
            print(f"(Kermac Debug) Launching ahead-of-time fused coefficient kernel for {kernel_descriptor!r}"
                  + (f", centres in {ranges} ranges" if ranges > 1 else ""))
        _backend.kernel_times_coefficients(params, stream)
    else:
        load_a, load_b = _backend.build_kernel_load_modes(kernel)
        name = kernel_coefficients_function_name(kernel.inner_operator, kernel.inner_power, load_a, load_b)
        function = ModuleCache(debug).get_function(a.device, name, debug=debug)
        if debug:
            print(f"(Kermac Debug) Launching kernel: {name}")
        _backend.kernel_times_coefficients_jit(function, params, stream)
    if partial is not None:
        _sum_partials(partial, plan.out)
    return plan.out


def _partial_products(parts, plan, device):
    """(buffer [parts, L, M, O], staging buffer or None) for partial products that are added into `plan.out`; None
    when the memory for them is refused (the caller then does without partial products)."""
    partial = _scratch.allocate_floats((parts, plan.L, plan.M, plan.O), device)
    if partial is None:
        return None
    target = plan.out if plan.out.dim() == 3 else plan.out.unsqueeze(0)
    if target.is_contiguous():
        return partial, None
    # the order in which torch adds the ranges depends on the layout of the result: a strided `out` gets the
    # bits of a contiguous one, through a buffer of its own
    staged = _scratch.allocate_floats((plan.L, plan.M, plan.O), device)
    return None if staged is None else (partial, staged)


# Squared differences and sums of products on the matrix cores: the route of kmc_build_kernel through a workspace
# (operands split once into fp16 pieces, 256 x 256 tiles) builds the kernel matrix several times
# faster than the fused kernel walks it, so a large product is taken panel by panel instead: the
# kernel matrix of all rows against a few thousand centres is written into a buffer that is
# reused, and kmc_matrix_times_coefficients contracts it with the coefficients of those centres.
# The full matrix never exists; the panel (1 GiB unless KERMAC_AMD_COEFFICIENT_PANEL_BYTES says
# otherwise, 0 switches the route off) does.  Measured, fused kernel -> panels: L = 4,
# M = N = 16384, O = 32 at K = 256 7.7 -> 4.7 ms, at K = 1024 22.6 -> 8.4 ms; M = N = 30000,
# K = 1024, O = 16 18.6 -> 7.1 ms; M = 10000, N = 100000, K = 784, O = 10 16.6 -> 8.0 ms; M = 20000,
# N = 50000, K = 3072, O = 10 56.8 -> 17.8 ms.  The partial products of the panels (and of the
# ranges a panel is cut into when the rows alone do not fill the chip) are added in a fixed order.
#
# The same two steps serve every descriptor (also those compiled at run time) when there are more
# than 64 coefficient columns: the fused
# kernel holds at most 64 per walk of the kernel matrix and walks it ceil(O / 64) times, while a panel
# built once by kmc_build_kernel (whatever kernel this descriptor and l2 mode launch for a stored
# matrix) is contracted with all columns at 4 bytes of traffic per element.  Laplace kernel on L1
# distances, L = 4, M = N = 16384, K = 256: O = 65 .. 128 22.1 -> 11.8 .. 12.0 ms, O = 256 44.0 -> 14.6 ms,
# O = 1000 176 -> 18.7 ms (the panels contracted from fp16 pieces, below); p = 1.3 norm, M = 1000, N = 20000, K = 784, O = 300: 15.1 -> 3.2 ms.
_PANEL_BYTES = 1 << 30
_FUSED_COLUMNS_PER_WALK = 64
_MANY_COLUMNS_MIN_ELEMENTS = 1e6        # below, the three launches cost what the second walk does (500 x 500, O = 100: 54 against 41 us)
_PANEL_MAX_PARTIAL_BYTES = 512 << 20


def _panel_splits(M, O, L, rows):
    """Ranges of centres per panel for kmc_matrix_times_coefficients: a workgroup per CU, and sums
    of at most 4096 rows per workgroup."""
    workgroups = -(-M // 128) * -(-O // 32) * L
    splits = 1 if workgroups >= 256 else min(-(-256 // workgroups), max(1, rows // 512))
    return min(max(splits, -(-rows // 4096)), max(1, 65535 // L))


def _products_in_panels(plan):
    """Sums of products (linear and polynomial kernels) have the same route, in the l2 modes "auto" and
    "gram_bf16" (_panel_shape decides which problems take it)."""
    from .build_a_kernel import _l2_current

    kernel = plan.params.kernel
    if kernel.inner_operator != _backend.OP_DOT or kernel.inner_power != _backend.POW_NOOP:
        return False
    l2 = _l2_current()
    return l2["mode"] in ("auto", "gram_bf16") and plan.K >= l2["min_k"]


# The matrix-core variant of the fused kernel holds 32 coefficient columns per workgroup where the
# direct one holds up to 64: with more than 32 columns it computes every distance once more often
# than the direct kernel and loses what the matrix instruction gains (O = 40: 1.3 .. 1.5 times
# slower at K = 128 and 256, level at K = 784 and beyond), unless the problem is so small that
# the additional workgroups find idle CUs (500 x 500 x 256: 71 us against 98).  With at most 32
# columns it is ahead from K = 192 on at any size (500 x 500 x 256: 71 us against 96), from 5e8
# terms on also at K = 128; at K = 64 the direct kernel is ahead everywhere (10000 x 10000: 393
# us against 479).
_AUTO_FUSED_MIN_K = 128
_AUTO_FUSED_ANY_SIZE_MIN_K = 192
_AUTO_FUSED_MAX_COLUMNS = 32
_AUTO_FUSED_SMALL_ELEMENTS = 4e6


def _auto_fused_on_matrix_cores(plan):
    """l2 mode "auto", a product that stays with the fused kernel: its matrix-core variant or the direct one."""
    from .build_a_kernel import _L2_AUTO_MIN_TERMS

    elements = float(plan.L) * plan.M * plan.N
    if plan.K < _AUTO_FUSED_MIN_K:
        return False
    if plan.O > _AUTO_FUSED_MAX_COLUMNS:
        return plan.K >= _AUTO_FUSED_ANY_SIZE_MIN_K and elements <= _AUTO_FUSED_SMALL_ELEMENTS
    return plan.K >= _AUTO_FUSED_ANY_SIZE_MIN_K or elements * plan.K >= _L2_AUTO_MIN_TERMS


# The rule of kmc_gram_workspace_bytes weighs the route through a workspace against the one-step kernels
# of a stored matrix.  Here the alternative is the fused kernel, which walks the matrix several times
# more slowly, so in "auto" squared differences are taken in panels (KMC_FLAG_GRAM_WORKSPACE_ANY_SIZE) also
# for (fused kernel / panels, the faster of the fused variants):
#   - long contractions of any number of tiles (K = 3072: 4 tiles 1.4, 16 tiles 1.35, 64 tiles 1.3 .. 1.4,
#     with O = 40 1.4 .. 2.0; K = 784: 0.95 .. 1.05);
#   - from 192 tiles on at K >= 256 whatever the storage order (256 tiles 1.06 .. 1.24, 316 tiles 1.3;
#     64 tiles 0.6);
#   - more than 32 coefficient columns, where both fused variants pay for them, from K = 784 and 64 tiles
#     on (64 tiles 1.3, 100 x 50000 1.2 .. 1.3, K = 3072 1.5 .. 2.0), even with most of the tiles padding.
# The first two need 60 % of the tiles' area used (100 rows against 50000 centres, O = 32: 0.8 .. 0.95).
# Contractions below 128 stay with the fused kernel (K = 64: 0.83 .. 1.1 at any size).
_AUTO_PANEL_MIN_K = 128
_AUTO_PANEL_LONG_K = 1536
_AUTO_PANEL_MID_K, _AUTO_PANEL_MID_TILES = 256, 192
_AUTO_PANEL_WIDE_K, _AUTO_PANEL_WIDE_TILES = 784, 64
_AUTO_PANEL_MIN_USED = 0.6


def _auto_panels_of_any_size(plan):
    tiles_m, tiles_n = -(-plan.M // 256), -(-plan.N // 256)
    tiles = tiles_m * tiles_n * plan.L
    used = plan.M * plan.N / (65536.0 * tiles_m * tiles_n)
    if plan.O > _AUTO_FUSED_MAX_COLUMNS and plan.K >= _AUTO_PANEL_WIDE_K and tiles >= _AUTO_PANEL_WIDE_TILES:
        return True
    if used < _AUTO_PANEL_MIN_USED:
        return False
    return plan.K >= _AUTO_PANEL_LONG_K or (plan.K >= _AUTO_PANEL_MID_K and tiles >= _AUTO_PANEL_MID_TILES)


# Sums of products: the fused kernel walks them more slowly than squared differences (it has no matrix-core
# variant), so panels pay earlier (fused kernel / panels): any number of tiles from K = 784 on (500 x 500: 1.4 at
# K = 784, 2.1 at K = 3072), and with more than 32 coefficient columns any contraction from 1e7 elements on
# (4096 x 4096 x 64 1.2, 4 x 4096 x 4096 x 64 1.55, 1000 x 20000 x 128 1.6; 2000 x 2000 x 64 0.54), both with 60 % of
# the tiles' area used;
# few rows against many centres stay fused with up to 32 columns even where the library would take the route
# (100 x 50000 x 256: 0.74, x 784: 0.86).
_AUTO_PRODUCT_PANEL_ANY_TILES_K = 784
_AUTO_PRODUCT_PANEL_MIN_ELEMENTS = 1e7


def _auto_product_panels(plan, library_takes_them):
    """l2 mode "auto", sums of products: None (fused kernel), False (panels as the library's rule has them) or
    True (panels of any size)."""
    tiles_m, tiles_n = -(-plan.M // 256), -(-plan.N // 256)
    used = plan.M * plan.N / (65536.0 * tiles_m * tiles_n)
    many_columns = plan.O > _AUTO_FUSED_MAX_COLUMNS
    if used < _AUTO_PANEL_MIN_USED and not many_columns:
        return None
    if library_takes_them:
        return False
    if used < _AUTO_PANEL_MIN_USED:
        return None
    if plan.K >= _AUTO_PRODUCT_PANEL_ANY_TILES_K:
        return True
    return True if many_columns and float(plan.L) * plan.M * plan.N >= _AUTO_PRODUCT_PANEL_MIN_ELEMENTS else None


def _panel_shape(plan, route):
    """(rows, panels, ld, splits, flags) of the product panel by panel (above); None when this problem
    stays with the fused kernel.  `route`: the flag of kmc_build_kernel's route through a workspace
    for this descriptor; `flags`: what the calls for the panels add to the caller's.  No device call."""
    from .build_a_kernel import _l2_current

    budget = int(os.environ.get("KERMAC_AMD_COEFFICIENT_PANEL_BYTES", _PANEL_BYTES))
    L, M, N, O = plan.L, plan.M, plan.N, plan.O
    if budget <= 0 or 0 in (L, M, N, O, plan.K):
        return None
    # l2 mode "gram" asks for the fp32 matrix instruction; the panels of a route are built from fp16 pieces
    mode = _l2_current()["mode"]
    if route and mode not in ("auto", "gram_bf16"):
        return None
    if route == _backend.FLAG_L2_GRAM_BF16 and mode == "auto" and plan.K < _AUTO_PANEL_MIN_K:
        return None
    ld = -(-M // 4) * 4                                          # rows of the panel start on 16 bytes
    rows = min(N, max(256, budget // (4 * L * ld) // 256 * 256))
    panels = -(-N // rows)
    rows = min(N, -(-(-(-N // panels)) // 256) * 256)             # panels of equal size, whole tiles
    panels = -(-N // rows)
    block = _backend.BuildKernelParams.from_buffer_copy(plan.params.kernel)
    block.flags |= route
    block.n, block.c, block.c_ld, block.c_bs = rows, 256, ld, rows * ld      # c: any address, for the query
    if route:
        taken = _backend.gram_workspace_bytes(block) > 0       # by the library's rule, made for stored matrices
        if mode != "auto":
            any_size = None if not taken else False
        elif route == _backend.FLAG_DOT_PIECES:
            any_size = _auto_product_panels(plan, taken)
        else:
            any_size = False if taken else (True if _auto_panels_of_any_size(plan) else None)
        if any_size is None:
            return None
        if any_size:
            route |= _backend.FLAG_GRAM_WORKSPACE_ANY_SIZE
            block.flags |= route
            if _backend.gram_workspace_bytes(block) == 0:
                return None
    splits = _panel_splits(M, O, L, rows)
    if panels * splits > 1 and 4 * panels * splits * L * M * O > _PANEL_MAX_PARTIAL_BYTES:
        splits = 0              # too many partial products to keep: every panel is added to the result as it comes
    return rows, panels, ld, splits, route


def _run_in_panels(plan, shape, stream, device, debug):
    """The product in the panels of `shape` (_panel_shape); False when memory for them is missing."""
    from .build_a_kernel import _attach_gram_workspace

    rows, panels, ld, splits, route = shape
    L, M, N, O = plan.L, plan.M, plan.N, plan.O
    parts = panels * splits                                      # 0: no partial products, the panels accumulate
    params = plan.params
    block = _backend.BuildKernelParams.from_buffer_copy(params.kernel)
    block.flags |= route
    block.n, block.c_ld, block.c_bs = rows, ld, rows * ld
    panel = _scratch.allocate_floats((L * rows * ld,), device)
    if panel is None:
        return False
    product = _contraction_by_pieces(plan, rows, ld, panel, device)
    partial = None
    if parts > 1 and product is None:
        partial = _partial_products(parts, plan, device)
        if partial is None:
            return False
    block.c = panel.data_ptr()
    workspace = _attach_gram_workspace(block, device) if route else None
    if route and workspace is None:
        return False
    if debug:
        print(f"(Kermac Debug) Kernel matrix x coefficients in {panels} panels of {rows} centres, "
              + ("contracted from fp16 pieces" if product is not None else
                 f"{splits} partial products each" if splits else "added to the result one after the other"))
    row_major_b = block.b_majorness == _backend.ROW_MAJOR
    contraction = _backend.MatrixCoefficientsParams()
    contraction.m, contraction.o, contraction.l = M, O, L
    contraction.matrix, contraction.matrix_ld = panel.data_ptr(), ld
    contraction.coef_ld, contraction.coef_bs = params.coef_ld, params.coef_bs
    if partial is None:
        contraction.out, contraction.out_ld, contraction.out_bs = params.out, params.out_ld, params.out_bs
    else:
        contraction.out_ld, contraction.out_bs = O, M * O
        contraction.n_splits, contraction.out_split_stride = splits, L * M * O
    first_b, first_offset = params.kernel.b, params.kernel.regularization_offset_y
    function = None
    if not _backend.build_kernel_has_variant(block.inner_operator, block.inner_power):
        # a descriptor compiled at run time; the panels start at multiples of 256 rows of b, so all of them
        # take the loader variant of the first
        load_a, load_b = _backend.build_kernel_load_modes(block)
        name = build_kernel_function_name(block.inner_operator, block.inner_power, load_a, load_b)
        function = ModuleCache(debug).get_function(device, name, debug=debug)
    for index in range(panels):
        n0 = index * rows
        count = min(rows, N - n0)
        block.n, block.c_bs = count, count * ld
        block.b = first_b + 4 * n0 * (block.b_ld if row_major_b else 1)
        block.regularization_offset_y = first_offset + n0
        if function is None:
            _backend.build_kernel(block, stream)
        else:
            _backend.build_kernel_jit(function, block, stream)
        if route:
            block.flags |= _backend.FLAG_GRAM_A_KEPT             # the rows are the same for every panel: split once
        if product is not None:
            # out[m, o] (+)= sum_n panel[n, m] coef[n, o] as a product of fp16 pieces (below)
            pieces, sums, _ = product
            pieces.k, pieces.b_bs = count, count * ld
            pieces.a = params.coef + 4 * n0 * params.coef_ld
            if index == 0:
                pieces.c, pieces.c_ld, pieces.c_bs = params.out, params.out_ld, params.out_bs
            else:
                pieces.c, pieces.c_ld, pieces.c_bs = sums.data_ptr(), O, M * O
            _backend.build_kernel(pieces, stream)
            if index:
                target = plan.out if plan.out.dim() == 3 else plan.out.unsqueeze(0)
                target.add_(sums)
            continue
        contraction.n, contraction.matrix_bs = count, count * ld
        contraction.coef = params.coef + 4 * n0 * params.coef_ld
        if partial is not None:
            contraction.out = partial[0].data_ptr() + 4 * index * splits * L * M * O
        else:
            contraction.accumulate = 1 if index else 0
        _backend.matrix_times_coefficients(contraction, stream)
    if partial is not None:
        _sum_partials(partial, plan.out)
    plan.keepalive += [panel, partial, workspace, product]
    return True


# Hundreds of coefficient columns: kmc_matrix_times_coefficients multiplies on the fp32 matrix instruction and is
# bound by it from about 128 columns on (O = 1000 above: 20 of 31 ms).  The contraction of a panel is itself a
# sum of products, out[m, o] = sum_n panel[n, m] coef[n, o], with both operands stored the way kmc_build_kernel reads
# them (m and o contiguous), so from _PIECES_MIN_COLUMNS columns on it runs on kmc_build_kernel's route for sums of
# products (KMC_FLAG_DOT_PIECES: two fp16 pieces per value, scale per row m and o, error below 3 * 2^-22 sum_n |k c|)
# into the result for the first panel and into a buffer that is added to the result for the others.  Gaussian
# kernel, fp32 contraction -> pieces: L = 4, M = N = 16384, K = 256 at O = 256 9.6 -> 8.1 ms, O = 512 15.6 -> 9.4,
# O = 1000 25.5 -> 12.0; M = 10000, N = 100000, K = 784, O = 1000 28.5 -> 17.2 ms.  The split of a panel costs what
# its fp32 contraction with 64 columns does, and the product runs in tiles of 256 x 256 over (o, m): not below 256
# columns (O = 128: 6.7 -> 7.8 ms) nor below 128 tiles over the batch (M = 10000, O = 256, 40 tiles: 12.3 -> 16.1 ms;
# M = 2000, O = 1000, 32 tiles: 1.2 -> 2.0 ms).  KERMAC_AMD_COEFFICIENT_PIECES_MIN_COLUMNS replaces both conditions
# by a number of columns (tests send small shapes this way with 1).
_PIECES_MIN_COLUMNS = 256
_PIECES_MIN_TILES = 128


def _contraction_by_pieces_pays(L, M, O):
    forced = os.environ.get("KERMAC_AMD_COEFFICIENT_PIECES_MIN_COLUMNS")
    if forced is not None:
        return O >= int(forced)
    return O >= _PIECES_MIN_COLUMNS and -(-O // 256) * -(-M // 256) * L >= _PIECES_MIN_TILES


def _contraction_by_pieces(plan, rows, ld, panel, device):
    """(parameter block, buffer for the sums of a panel, workspace) of the contraction as a product of fp16
    pieces; None when kmc_matrix_times_coefficients contracts the panels."""
    from .build_a_kernel import _attach_gram_workspace

    L, M, N, O = plan.L, plan.M, plan.N, plan.O
    if not _contraction_by_pieces_pays(L, M, O):
        return None
    params = plan.params
    block = _backend.BuildKernelParams()
    block.inner_operator, block.inner_power, block.outer_power, block.kernel_type = _backend.OP_DOT, _backend.POW_NOOP, 0, 0
    block.a_majorness = block.b_majorness = _backend.COL_MAJOR
    block.flags = _backend.FLAG_DOT_PIECES | _backend.FLAG_GRAM_WORKSPACE_ANY_SIZE
    # the product the library sees: rows o of the coefficients against rows m of the panel, contraction over n;
    # its result C(o, m) at c[o + m c_ld] is out[m, o]
    block.m, block.n, block.k, block.l = O, M, min(rows, N), L
    block.a, block.a_ld, block.a_bs = params.coef, params.coef_ld, params.coef_bs
    block.b, block.b_ld, block.b_bs = panel.data_ptr(), ld, min(rows, N) * ld
    block.c, block.c_ld, block.c_bs = params.out, params.out_ld, params.out_bs
    block.epsilon = 0.0
    workspace = _attach_gram_workspace(block, device)
    if workspace is None:
        return None
    sums = _scratch.allocate_floats((L, M, O), device) if N > rows else None
    if N > rows and sums is None:
        return None
    return block, sums, workspace


def _sum_partials(buffers, out):
    partial, staged = buffers
    target = out if out.dim() == 3 else out.unsqueeze(0)
    if staged is None:
        torch.sum(partial, dim=0, out=target)
    else:
        torch.sum(partial, dim=0, out=staged)
        target.copy_(staged)


# A workgroup of the fused kernel owns 128 rows of ``a`` (one batch entry, one chunk of up to 64
# coefficient columns) and walks every centre, so a launch has ceil(M / 128) x L x ceil(O / 64)
# long-running workgroups, three to a CU (two for the 64-column and matrix-core variants).  Few rows
# against many centres (prediction for a small batch of points) would leave most of the chip idle;
# a batch that fills two places per CU (L = 4, M = 16384: 512 workgroups) leaves a third of the
# places empty; and a few long workgroups per CU, all started together, finish unevenly.  The
# kernel therefore takes the centres in ranges (``n_ranges`` of the C parameter block): every range
# is walked by workgroups of its own into a partial product of its own, and the partial products
# are added in range order.  Measured at L = 4, M = N = 16384, K = 256, O = 32: 10.4 ms uncut,
# 10.0 ms in 6 ranges, 9.6 ms in 12 to 43, 9.7 ms in 64 (the kernel matrix written out and
# multiplied by torch.bmm: 10.0 ms).  The number of ranges comes from the model of the launch time
# that the pairwise kernel uses for its cut over k (same K walk, same three regimes).
_SPLIT_MAX_PARTIAL_BYTES = 256 << 20
_SPLIT_WORTH = 0.95                           # cut only for at least 5 % less modelled time
_TILE_OVERHEAD_K = 24                         # coefficient staging and contraction of one tile, in k-steps


def _centre_ranges(plan, three_resident):
    """How many ranges the centres are cut into (1: the launch goes out as it is)."""
    if plan.M == 0 or plan.O == 0 or plan.L == 0 or plan.N <= 128 or not launch_cuts_enabled():
        return 1
    workgroups = -(-plan.M // 128) * plan.L * max(1, -(-plan.O // 64))
    return _choose_ranges(workgroups, -(-plan.N // 128), plan.K, 3 if three_resident else 2,
                          4 * plan.L * plan.M * plan.O)


def _launch_ms(workgroups, depth, resident):
    """Modelled time of `workgroups` workgroups that walk `depth` k-steps each, in milliseconds."""
    per_cu = workgroups / 256
    if per_cu <= 1:
        return (depth + 128) / 3900                               # one wave per SIMD: latency bound
    slower = 1.0 if resident == 3 else 1.0 / 0.912                # two resident workgroups deliver 0.91 of three
    if per_cu <= resident:
        return -(-workgroups // 256) * (depth + 128) / 7300 * slower     # one round, all started together
    return (per_cu + 1.92) * (depth + 40) / 10000 * slower       # rounds that the dispatcher balances


@functools.lru_cache(maxsize=512)
def _choose_ranges(workgroups, tiles, K, resident, product_bytes):
    per_tile = K + _TILE_OVERHEAD_K
    unsplit = _launch_ms(workgroups, tiles * per_tile, resident)
    best = (unsplit, 1)
    most = min(tiles, _SPLIT_MAX_PARTIAL_BYTES // max(product_bytes, 1))
    seen = tiles
    for ranges in range(2, most + 1):
        walk = -(-tiles // ranges)
        if walk == seen:
            continue                      # the same tiles per range as one range fewer: only more empty ranges
        seen = walk
        used = -(-tiles // walk)
        count = workgroups * used
        cost = _launch_ms(count, walk * per_tile, resident) + 2.1e-5 * count + 0.01     # partial products, second launch
        if cost < best[0]:
            best = (cost, used)
    return best[1] if best[0] <= _SPLIT_WORTH * unsplit else 1
