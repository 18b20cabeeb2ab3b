"""ctypes wrapper of the CPU oracle (oracle/kermac_oracle.c).

TEST INFRASTRUCTURE ONLY.  Nothing under ``kermac_amd/`` imports this module;
it is used by ``tests/``, by ``__graft_entry__.smoke()`` and by the CPU
baseline leg of ``bench.py`` to check (never to produce) results.

All functions take CPU fp32 ``torch`` tensors with arbitrary strides, using the
same view conventions as the operators they check, and return new tensors.
``wide=True`` (default) evaluates in double precision; ``wide=False`` follows the
reference's fp32 operation order.
"""
from __future__ import annotations

import ctypes
import subprocess
from ctypes import POINTER, c_float, c_int, c_int64
from pathlib import Path

import torch

ORACLE_DIR = Path(__file__).resolve().parent
SOURCE = ORACLE_DIR / "kermac_oracle.c"
LIBRARY = ORACLE_DIR / "libkermac_oracle.so"

OP = {"DIFF": 0, "DOT": 1}
POWER = {"NOOP": 0, "ABS": 1, "SQUARE": 2, "SQRT": 3, "POW": 4}
KERNEL = {"NONE": 0, "LAPLACE": 1, "GAUSSIAN": 2}
NORM = {"L1": 0, "L2": 1, "P": 2}


def build(force: bool = False) -> Path:
    """Compile the C restatement with gcc (OpenMP) into oracle/libkermac_oracle.so."""
    if force or not LIBRARY.exists() or LIBRARY.stat().st_mtime < SOURCE.stat().st_mtime:
        subprocess.run(
            ["gcc", "-O2", "-fopenmp", "-std=c99", "-shared", "-fPIC", "-o", str(LIBRARY), str(SOURCE), "-lm"],
            check=True,
        )
    return LIBRARY


_lib = None


def _library():
    global _lib
    if _lib is None:
        build()
        _lib = ctypes.CDLL(str(LIBRARY))
    return _lib


def _fptr(t):
    return ctypes.cast(t.data_ptr(), POINTER(c_float)) if t is not None else None


def _batched(t: torch.Tensor, dims: int):
    """(tensor, batch stride): a tensor with `dims` dimensions broadcasts."""
    if t.dim() == dims:
        return t, 0
    return t, (0 if t.size(0) == 1 else t.stride(0))


def _hyper(value, L):
    """float / tensor / None -> (cpu tensor or None, stride)."""
    if value is None:
        return None, 0
    if not isinstance(value, torch.Tensor):
        value = torch.tensor(float(value), dtype=torch.float32)
    value = value.detach().to("cpu", torch.float32).contiguous()
    return value, (0 if value.numel() == 1 else 1)


def _common_batch(*pairs):
    L = 1
    for t, dims in pairs:
        if t is not None and isinstance(t, torch.Tensor) and t.dim() == dims + 1:
            L = max(L, t.size(0))
    return L


def build_kernel(inner_operator, inner_power, outer_power, kernel_type, a, b,
                 p_inner=None, p_outer=None, bandwidth=None, regularization=None,
                 regularization_offset_x=0, regularization_offset_y=0, epsilon=1e-5, wide=True):
    """out[L, M, N] for a [L?, M, K], b [L?, N, K] (see kmo_build_kernel)."""
    assert a.dtype == torch.float32 and b.dtype == torch.float32 and not a.is_cuda and not b.is_cuda
    L = _common_batch((a, 2), (b, 2), (p_inner, 0), (p_outer, 0), (bandwidth, 0), (regularization, 0))
    M, K = a.shape[-2:]
    N = b.shape[-2]
    assert b.shape[-1] == K
    out = torch.empty((L, M, N), dtype=torch.float32)
    a, a_sl = _batched(a, 2)
    b, b_sl = _batched(b, 2)
    pi, pi_s = _hyper(p_inner, L)
    po, po_s = _hyper(p_outer, L)
    bw, bw_s = _hyper(bandwidth, L)
    rg, rg_s = _hyper(regularization, L)
    _library().kmo_build_kernel(
        c_int(OP[inner_operator]), c_int(POWER[inner_power]), c_int(POWER[outer_power]), c_int(KERNEL[kernel_type]),
        c_int(M), c_int(N), c_int(K), c_int(L),
        _fptr(a), c_int64(a.stride(-2)), c_int64(a.stride(-1)), c_int64(a_sl),
        _fptr(b), c_int64(b.stride(-2)), c_int64(b.stride(-1)), c_int64(b_sl),
        _fptr(out), c_int64(out.stride(1)), c_int64(out.stride(2)), c_int64(out.stride(0)),
        _fptr(pi), c_int64(pi_s), _fptr(po), c_int64(po_s), _fptr(bw), c_int64(bw_s), _fptr(rg), c_int64(rg_s),
        c_int(regularization_offset_x), c_int(regularization_offset_y), c_float(epsilon), c_int(1 if wide else 0))
    return out


def run_kernel(inner_operator, inner_power, outer_power, kernel_type, a, b, **kw):
    """out[L, M, N] as the reference's ``run_kernel`` returns it for ``out=None``
    (src/kermac/build_a_kernel.py:259 allocates a row-major ``[L, M, N]``; :323-336 then
    swap the operands, but neither the regularisation offsets nor the sign of the
    difference, before the kernel of ``build_kernel`` runs and writes the transpose):
    the inner difference is ``a[m] - b[n]`` and the regularised elements are those with
    ``offset_x + n == offset_y + m``.  For the inner powers that ignore the sign and
    with equal offsets this is ``build_kernel(a, b)`` itself."""
    return build_kernel(inner_operator, inner_power, outer_power, kernel_type, b, a, **kw).transpose(-1, -2)


def run_kernel_coefficients(inner_operator, inner_power, outer_power, kernel_type, a, b, coef,
                            regularization_offset_x=0, regularization_offset_y=0, **kw):
    """out[L, M, O] = run_kernel(...)[L, M, N] @ coef[L?, N, O] without the matrix, in the
    convention of ``run_kernel`` above: negating both operands turns the kernel's b - a
    into a - b (and leaves products unchanged), and the offsets change sides."""
    return kernel_times_coefficients(inner_operator, inner_power, outer_power, kernel_type, -a, -b, coef,
                                     regularization_offset_x=regularization_offset_y,
                                     regularization_offset_y=regularization_offset_x, **kw)


def cdist(a, b, p=2.0, skip_epilogue=False, wide=True):
    """What kermac.cdist documents: (sum_k |b - a|^p)^(1/p), or the bare sum."""
    if p == 1.0:
        return build_kernel("DIFF", "ABS", "NOOP", "NONE", a, b, wide=wide)
    if p == 2.0:
        return build_kernel("DIFF", "SQUARE", "NOOP" if skip_epilogue else "SQRT", "NONE", a, b, wide=wide)
    p32 = torch.tensor(p, dtype=torch.float32)
    if skip_epilogue:
        return build_kernel("DIFF", "POW", "NOOP", "NONE", a, b, p_inner=p32, wide=wide)
    return build_kernel("DIFF", "POW", "POW", "NONE", a, b, p_inner=p32, p_outer=1.0 / p32, wide=wide)


def norm_kernel_gradient(norm_type, a, b, c, d, p=None, wide=True):
    """out[L, O, N, M] for a [L?, K, M], b [L?, N, K], c [L?, O, K], d [L?, N, M]."""
    for t in (a, b, c, d):
        assert t.dtype == torch.float32 and not t.is_cuda
    L = _common_batch((a, 2), (b, 2), (c, 2), (d, 2), (p, 0))
    K, M = a.shape[-2:]
    N = b.shape[-2]
    O = c.shape[-2]
    out = torch.empty((L, O, N, M), dtype=torch.float32)
    a, a_sl = _batched(a, 2)
    b, b_sl = _batched(b, 2)
    c, c_sl = _batched(c, 2)
    d, d_sl = _batched(d, 2)
    pt, p_s = _hyper(p, L)
    _library().kmo_norm_kernel_gradient(
        c_int(NORM[norm_type]), c_int(M), c_int(N), c_int(O), c_int(K), c_int(L),
        _fptr(a), c_int64(a.stride(-2)), c_int64(a.stride(-1)), c_int64(a_sl),
        _fptr(b), c_int64(b.stride(-2)), c_int64(b.stride(-1)), c_int64(b_sl),
        _fptr(c), c_int64(c.stride(-2)), c_int64(c.stride(-1)), c_int64(c_sl),
        _fptr(d), c_int64(d.stride(-2)), c_int64(d.stride(-1)), c_int64(d_sl),
        _fptr(out), c_int64(out.stride(1)), c_int64(out.stride(2)), c_int64(out.stride(3)), c_int64(out.stride(0)),
        _fptr(pt), c_int64(p_s), c_int(1 if wide else 0))
    return out


def cdist_grad(a, b, c, d, p=2.0, wide=True):
    if not isinstance(p, torch.Tensor):
        if p == 1.0:
            return norm_kernel_gradient("L1", a, b, c, d, wide=wide)
        if p == 2.0:
            return norm_kernel_gradient("L2", a, b, c, d, wide=wide)
    return norm_kernel_gradient("P", a, b, c, d, p=p, wide=wide)


def kernel_times_coefficients(inner_operator, inner_power, outer_power, kernel_type, a, b, coef,
                              p_inner=None, p_outer=None, bandwidth=None, regularization=None,
                              regularization_offset_x=0, regularization_offset_y=0, epsilon=1e-5, wide=True):
    """out[L, M, O] = kernelmatrix[L, M, N] @ coef[L?, N, O] without the matrix."""
    L = _common_batch((a, 2), (b, 2), (coef, 2), (p_inner, 0), (p_outer, 0), (bandwidth, 0), (regularization, 0))
    M, K = a.shape[-2:]
    N = b.shape[-2]
    O = coef.shape[-1]
    assert O <= 256
    out = torch.empty((L, M, O), dtype=torch.float32)
    a, a_sl = _batched(a, 2)
    b, b_sl = _batched(b, 2)
    coef, w_sl = _batched(coef, 2)
    pi, pi_s = _hyper(p_inner, L)
    po, po_s = _hyper(p_outer, L)
    bw, bw_s = _hyper(bandwidth, L)
    rg, rg_s = _hyper(regularization, L)
    _library().kmo_kernel_times_coefficients(
        c_int(OP[inner_operator]), c_int(POWER[inner_power]), c_int(POWER[outer_power]), c_int(KERNEL[kernel_type]),
        c_int(M), c_int(N), c_int(K), c_int(O), c_int(L),
        _fptr(a), c_int64(a.stride(-2)), c_int64(a.stride(-1)), c_int64(a_sl),
        _fptr(b), c_int64(b.stride(-2)), c_int64(b.stride(-1)), c_int64(b_sl),
        _fptr(coef), c_int64(coef.stride(-2)), c_int64(coef.stride(-1)), c_int64(w_sl),
        _fptr(out), c_int64(out.stride(1)), c_int64(out.stride(2)), c_int64(out.stride(0)),
        _fptr(pi), c_int64(pi_s), _fptr(po), c_int64(po_s), _fptr(bw), c_int64(bw_s), _fptr(rg), c_int64(rg_s),
        c_int(regularization_offset_x), c_int(regularization_offset_y), c_float(epsilon), c_int(1 if wide else 0))
    return out
