"""ctypes binding of libkermac_amd.so (the C ABI declared in include/kermac_amd.h).

There is no fallback: if the library has not been built, or a call fails, the
operators raise.  Nothing here touches torch; callers pass raw device pointers
and the stream handle.
"""
from __future__ import annotations

import ctypes
import os
import threading
from ctypes import POINTER, Structure, byref, c_char_p, c_float, c_int32, c_int64, c_size_t, c_void_p
from pathlib import Path
from typing import List, Optional, Sequence, Tuple

# KERMAC_AMD_LIBRARY points at another build of the same ABI (e.g. an experimental one).
LIB_PATH = Path(os.environ.get("KERMAC_AMD_LIBRARY") or Path(__file__).resolve().parent / "_lib" / "libkermac_amd.so")

ABI_VERSION = 2

# enum kmc_status
OK = 0
ERR_INVALID_ARGUMENT = 1
ERR_UNSUPPORTED_VARIANT = 2
ERR_WRONG_DEVICE = 3
ERR_JIT = 4

# enum kmc_majorness
COL_MAJOR = 0
ROW_MAJOR = 1

# enum kmc_inner_operator, enum kmc_power_type (the values the Python mirror tests for)
OP_DIFF = 0
OP_DOT = 1
POW_NOOP = 0
POW_ABS = 1
POW_SQUARE = 2
POW_POW = 4

FLAG_FORCE_SCALAR_ACCESS = 1
FLAG_NEGATE_DIFF = 2
FLAG_L2_GRAM = 4
FLAG_GENERIC_POWER = 8
FLAG_NO_SYMMETRY = 16
FLAG_L2_GRAM_BF16 = 32
FLAG_GRAM_A_KEPT = 64
FLAG_DOT_PIECES = 128
FLAG_GRAM_WORKSPACE_ANY_SIZE = 256
FLAG_L1_FIXED = 512
FLAG_NO_PROBE = 1024
FLAG_DIRECT_PANELS = 2048
SAMPLE_BYTES = 1024             # KMC_SAMPLE_BYTES: what the sample in front of a matrix-core launch takes of the workspace

_float_p = c_void_p  # device pointers are passed as integers


class BuildKernelParams(Structure):
    """struct kmc_build_kernel_params"""
    _fields_ = [
        ("inner_operator", c_int32), ("inner_power", c_int32), ("outer_power", c_int32), ("kernel_type", c_int32),
        ("a_majorness", c_int32), ("b_majorness", c_int32), ("flags", c_int32),
        ("m", c_int32), ("n", c_int32), ("k", c_int32), ("l", c_int32),
        ("a", _float_p), ("a_ld", c_int64), ("a_bs", c_int64),
        ("b", _float_p), ("b_ld", c_int64), ("b_bs", c_int64),
        ("c", _float_p), ("c_ld", c_int64), ("c_bs", c_int64),
        ("p_inner", _float_p), ("p_inner_bs", c_int64), ("p_inner_value", c_float),
        ("p_outer", _float_p), ("p_outer_bs", c_int64), ("p_outer_value", c_float),
        ("bandwidth", _float_p), ("bandwidth_bs", c_int64), ("bandwidth_value", c_float),
        ("regularization", _float_p), ("regularization_bs", c_int64), ("regularization_value", c_float),
        ("regularization_offset_x", c_int32), ("regularization_offset_y", c_int32),
        ("epsilon", c_float),
        ("gram_trust", c_float),
        ("k_total", c_int32),
        ("gram_centre", _float_p), ("gram_centre_bs", c_int64),
        ("gram_workspace", c_void_p), ("gram_workspace_bytes", c_int64),
    ]


class NormGradientParams(Structure):
    """struct kmc_norm_gradient_params"""
    _fields_ = [
        ("norm_type", c_int32), ("flags", c_int32),
        ("m", c_int32), ("n", c_int32), ("o", c_int32), ("k", c_int32), ("l", c_int32),
        ("a", _float_p), ("a_ld", c_int64), ("a_bs", c_int64),
        ("b", _float_p), ("b_ld", c_int64), ("b_bs", c_int64),
        ("c", _float_p), ("c_ld", c_int64), ("c_bs", c_int64),
        ("d", _float_p), ("d_ld", c_int64), ("d_bs", c_int64),
        ("e", _float_p), ("e_ld_n", c_int64), ("e_ld_o", c_int64), ("e_bs", c_int64),
        ("p", _float_p), ("p_bs", c_int64), ("p_value", c_float),
        ("workspace", c_void_p), ("workspace_bytes", c_int64),
    ]


class KernelCoefficientsParams(Structure):
    """struct kmc_kernel_coefficients_params"""
    _fields_ = [
        ("kernel", BuildKernelParams),
        ("o", c_int32),
        ("coef", _float_p), ("coef_ld", c_int64), ("coef_bs", c_int64),
        ("out", _float_p), ("out_ld", c_int64), ("out_bs", c_int64),
        ("n_ranges", c_int32), ("out_range_stride", c_int64),
    ]


class MatrixCoefficientsParams(Structure):
    """struct kmc_matrix_coefficients_params"""
    _fields_ = [
        ("m", c_int32), ("n", c_int32), ("o", c_int32), ("l", c_int32),
        ("matrix", _float_p), ("matrix_ld", c_int64), ("matrix_bs", c_int64),
        ("coef", _float_p), ("coef_ld", c_int64), ("coef_bs", c_int64),
        ("out", _float_p), ("out_ld", c_int64), ("out_bs", c_int64),
        ("accumulate", c_int32),
        ("n_splits", c_int32), ("out_split_stride", c_int64),
    ]


# Every exported symbol of include/kermac_amd.h: name -> (restype, argtypes).
SIGNATURES = {
    "kmc_abi_version": (ctypes.c_int, []),
    "kmc_last_error": (c_char_p, []),
    "kmc_device_arch": (ctypes.c_int, [ctypes.c_int, c_char_p, c_size_t]),
    "kmc_dispatch_rules": (ctypes.c_int, [c_char_p, c_size_t]),
    "kmc_build_kernel_has_variant": (ctypes.c_int, [c_int32, c_int32]),
    "kmc_build_kernel": (ctypes.c_int, [POINTER(BuildKernelParams), c_void_p]),
    "kmc_build_kernel_jit": (ctypes.c_int, [c_void_p, POINTER(BuildKernelParams), c_void_p]),
    "kmc_build_kernel_finish": (ctypes.c_int, [POINTER(BuildKernelParams), c_void_p, c_int64, c_int64, c_int64, c_int32,
                                               c_void_p]),
    "kmc_build_kernel_cut_static": (ctypes.c_int, [POINTER(BuildKernelParams), c_int32, c_void_p]),
    "kmc_sample_mean": (ctypes.c_int, [c_void_p, c_int32, c_int32, c_int32, c_int64, c_int64, c_int32, c_void_p, c_int64,
                                       c_void_p]),
    "kmc_gram_workspace_bytes": (ctypes.c_int, [POINTER(BuildKernelParams), POINTER(c_int64)]),
    "kmc_build_kernel_load_modes": (ctypes.c_int, [POINTER(BuildKernelParams), POINTER(c_int32), POINTER(c_int32)]),
    "kmc_norm_kernel_gradient": (ctypes.c_int, [POINTER(NormGradientParams), c_void_p]),
    "kmc_norm_gradient_workspace_bytes": (ctypes.c_int, [POINTER(NormGradientParams), POINTER(c_int64)]),
    "kmc_kernel_times_coefficients": (ctypes.c_int, [POINTER(KernelCoefficientsParams), c_void_p]),
    "kmc_matrix_times_coefficients": (ctypes.c_int, [POINTER(MatrixCoefficientsParams), c_void_p]),
    "kmc_kernel_times_coefficients_has_variant": (ctypes.c_int, [c_int32, c_int32]),
    "kmc_kernel_times_coefficients_jit": (ctypes.c_int, [c_void_p, POINTER(KernelCoefficientsParams), c_void_p]),
    "kmc_jit_compile": (ctypes.c_int, [
        c_char_p, c_char_p,
        ctypes.c_int, POINTER(c_char_p), POINTER(c_char_p),
        ctypes.c_int, POINTER(c_char_p),
        ctypes.c_int, POINTER(c_char_p),
        POINTER(c_void_p), POINTER(c_size_t), POINTER(c_void_p),
    ]),
    "kmc_jit_free": (None, [c_void_p]),
    "kmc_module_load": (ctypes.c_int, [c_void_p, c_size_t, POINTER(c_void_p)]),
    "kmc_module_get_function": (ctypes.c_int, [c_void_p, c_char_p, POINTER(c_void_p)]),
    "kmc_module_unload": (ctypes.c_int, [c_void_p]),
}


class BackendError(RuntimeError):
    """A C-ABI call returned a non-zero status."""

    def __init__(self, status: int, message: str):
        super().__init__(f"libkermac_amd status {status}: {message}")
        self.status = status


class WrongDeviceError(BackendError, ValueError):
    """The current device is not a gfx950.  Also a ValueError, like the reference's
    rejection of an unsupported compute capability (src/kermac/module_cache/module_cache.py:166-167)."""


_lib = None
_lib_lock = threading.Lock()


def library() -> ctypes.CDLL:
    """Load the shared library once; raise if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    with _lib_lock:
        if _lib is None:
            if not LIB_PATH.exists():
                raise RuntimeError(
                    f"{LIB_PATH} is missing: build it with `python -m kermac_amd._build` "
                    "(needs hipcc); there is no fallback implementation"
                )
            lib = ctypes.CDLL(str(LIB_PATH))
            for name, (restype, argtypes) in SIGNATURES.items():
                fn = getattr(lib, name)
                fn.restype = restype
                fn.argtypes = argtypes
            version = lib.kmc_abi_version()
            if version != ABI_VERSION:
                raise RuntimeError(f"{LIB_PATH} has ABI version {version}, this package needs {ABI_VERSION}")
            _lib = lib
    return _lib


def last_error() -> str:
    return library().kmc_last_error().decode("utf-8", "replace")


def check(status: int) -> None:
    if status == ERR_WRONG_DEVICE:
        raise WrongDeviceError(status, last_error())
    if status != OK:
        raise BackendError(status, last_error())


def build_kernel(params: BuildKernelParams, stream: int) -> None:
    check(library().kmc_build_kernel(byref(params), c_void_p(stream)))


def build_kernel_finish(params: BuildKernelParams, partials: int, partial_ld: int, partial_bs: int, partial_slice: int,
                        slices: int, stream: int) -> None:
    check(library().kmc_build_kernel_finish(byref(params), c_void_p(partials), partial_ld, partial_bs, partial_slice,
                                            slices, c_void_p(stream)))


STATIC_SCRATCH_BYTES = 64 << 20


def build_kernel_cut_static(params: BuildKernelParams, ranges: int, stream: int) -> None:
    """The cut over k with the partial sums in the library's static device array: allocates nothing."""
    check(library().kmc_build_kernel_cut_static(byref(params), ranges, c_void_p(stream)))


CENTRE_PAD = 64


def sample_mean(x: int, majorness: int, rows: int, k: int, ld: int, bs: int, l: int, mean: int, mean_bs: int,
                stream: int) -> None:
    check(library().kmc_sample_mean(c_void_p(x), majorness, rows, k, ld, bs, l, c_void_p(mean), mean_bs, c_void_p(stream)))


def gram_workspace_bytes(params: BuildKernelParams) -> int:
    """Bytes of gram_workspace that kmc_build_kernel would use for these parameters (0: none)."""
    needed = c_int64(0)
    check(library().kmc_gram_workspace_bytes(byref(params), byref(needed)))
    return needed.value


def build_kernel_jit(function: int, params: BuildKernelParams, stream: int) -> None:
    check(library().kmc_build_kernel_jit(c_void_p(function), byref(params), c_void_p(stream)))


def build_kernel_has_variant(inner_operator: int, inner_power: int) -> bool:
    return bool(library().kmc_build_kernel_has_variant(inner_operator, inner_power))


def build_kernel_load_modes(params: BuildKernelParams) -> Tuple[int, int]:
    la, lb = c_int32(0), c_int32(0)
    check(library().kmc_build_kernel_load_modes(byref(params), byref(la), byref(lb)))
    return la.value, lb.value


def norm_gradient_workspace_bytes(params: NormGradientParams) -> int:
    """Bytes of workspace that kmc_norm_kernel_gradient would use for these parameters (0: none)."""
    needed = c_int64(0)
    check(library().kmc_norm_gradient_workspace_bytes(byref(params), byref(needed)))
    return needed.value


def norm_kernel_gradient(params: NormGradientParams, stream: int) -> None:
    check(library().kmc_norm_kernel_gradient(byref(params), c_void_p(stream)))


def kernel_times_coefficients(params: KernelCoefficientsParams, stream: int) -> None:
    check(library().kmc_kernel_times_coefficients(byref(params), c_void_p(stream)))


def kernel_times_coefficients_jit(function: int, params: KernelCoefficientsParams, stream: int) -> None:
    check(library().kmc_kernel_times_coefficients_jit(c_void_p(function), byref(params), c_void_p(stream)))


def matrix_times_coefficients(params: MatrixCoefficientsParams, stream: int) -> None:
    check(library().kmc_matrix_times_coefficients(byref(params), c_void_p(stream)))


def kernel_times_coefficients_has_variant(inner_operator: int, inner_power: int) -> bool:
    return bool(library().kmc_kernel_times_coefficients_has_variant(inner_operator, inner_power))


def dispatch_rules() -> dict:
    """The library's table of thresholds for its routes through a workspace: {name: integer}."""
    buf = ctypes.create_string_buffer(4096)
    check(library().kmc_dispatch_rules(buf, 4096))
    rules = {}
    for text in buf.value.decode().splitlines():
        name, _, value = text.partition("=")
        rules[name.strip()] = int(value)
    return rules


def device_arch(device: int) -> str:
    buf = ctypes.create_string_buffer(256)
    check(library().kmc_device_arch(device, buf, 256))
    return buf.value.decode()


def jit_compile(
    source: str,
    source_name: str,
    headers: Sequence[Tuple[str, str]],
    options: Sequence[str],
    name_expressions: Sequence[str],
) -> Tuple[bytes, List[str]]:
    """hiprtc-compile ``source``; returns (code object, lowered names)."""
    lib = library()
    n_headers = len(headers)
    header_names = (c_char_p * max(n_headers, 1))(*[h[0].encode() for h in headers])
    header_sources = (c_char_p * max(n_headers, 1))(*[h[1].encode() for h in headers])
    opts = (c_char_p * max(len(options), 1))(*[o.encode() for o in options])
    names = (c_char_p * max(len(name_expressions), 1))(*[n.encode() for n in name_expressions])
    lowered = (c_void_p * max(len(name_expressions), 1))()
    code = c_void_p()
    size = c_size_t()
    check(lib.kmc_jit_compile(
        source.encode(), source_name.encode(),
        n_headers, header_sources, header_names,
        len(options), opts,
        len(name_expressions), names,
        byref(code), byref(size), lowered,
    ))
    try:
        blob = ctypes.string_at(code.value, size.value)
        lowered_names = [ctypes.string_at(lowered[i]).decode() for i in range(len(name_expressions))]
    finally:
        lib.kmc_jit_free(code)
        for i in range(len(name_expressions)):
            if lowered[i]:
                lib.kmc_jit_free(lowered[i])
    return blob, lowered_names


def module_load(code: bytes) -> int:
    handle = c_void_p()
    check(library().kmc_module_load(code, len(code), byref(handle)))
    return handle.value


def module_get_function(module: int, lowered_name: str) -> int:
    fn = c_void_p()
    check(library().kmc_module_get_function(c_void_p(module), lowered_name.encode(), byref(fn)))
    return fn.value


def module_unload(module: int) -> None:
    check(library().kmc_module_unload(c_void_p(module)))
