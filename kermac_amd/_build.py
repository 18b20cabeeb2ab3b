"""Ahead-of-time build of libkermac_amd.so (hipcc, gfx950 only).

Run as ``python -m kermac_amd._build`` or through ``__graft_entry__.build()``.
The object files and the library stay inside the package directory so that the
library travels with the source tree; nothing is installed elsewhere.
"""
from __future__ import annotations

import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

PACKAGE_DIR = Path(__file__).resolve().parent
CSRC = PACKAGE_DIR / "csrc"
OBJ_DIR = PACKAGE_DIR / "_obj"
LIB_DIR = PACKAGE_DIR / "_lib"
LIB_PATH = LIB_DIR / "libkermac_amd.so"

ARCH = "gfx950"

# Compiler flags for every translation unit.  Packed-fp32 code generation is
# switched off on purpose (the last three words are one clang target feature).
HIPCC_FLAGS = [
    f"--offload-arch={ARCH}",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-x", "hip",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]

# (inner operator, inner power) pairs compiled ahead of time; must match
# csrc/host/launcher_table.cpp.
# (0, 5) .. (0, 8) are the special exponents 0.5, 1.5, 3, 4 the library substitutes for (0, 4).
AOT_BUILD_KERNEL_VARIANTS = [(0, 0), (0, 1), (0, 2), (0, 4), (0, 5), (0, 6), (0, 7), (0, 8), (1, 0)]

# Pairs compiled ahead of time for the fused kernel-matrix x coefficients kernel.
AOT_COEFFICIENT_VARIANTS = [(0, 1), (0, 2), (0, 4)]

HOST_SOURCES = [
    "host/runtime.cpp",
    "host/build_kernel_launch.cpp",
    "host/launcher_table.cpp",
    "host/norm_gradient_launch.cpp",
    "host/kernel_coefficients_launch.cpp",
]


# Device translation units without per-variant defines.
EXTRA_DEVICE_SOURCES = ["kernels/norm_gradient_inst.hip", "kernels/gram_kernel_inst.hip",
                        "kernels/gram_coefficients_inst.hip", "kernels/gram_bf16_kernel_inst.hip",
                        "kernels/finish_partials.hip", "kernels/cut_static_scratch.hip", "kernels/sample_mean.hip", "kernels/gram_probe.hip",
                        "kernels/gram_f16_wide_inst.hip", "kernels/norm_gradient_f16_inst.hip",
                        "kernels/matrix_times_coefficients.hip", "kernels/l1_fixed_inst.hip", "kernels/panel_copy.hip"]


def _hipcc() -> str:
    found = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(found):
        raise RuntimeError("hipcc not found; the library can only be built in a ROCm image")
    return found


def _jobs():
    jobs = []
    for rel in HOST_SOURCES:
        src = CSRC / rel
        jobs.append((src, OBJ_DIR / (src.stem + ".o"), []))
    inst = CSRC / "kernels" / "build_kernel_inst.hip"
    for op, pw in AOT_BUILD_KERNEL_VARIANTS:
        jobs.append((inst, OBJ_DIR / f"build_kernel_inst_{op}_{pw}.o", [f"-DKMC_INNER_OP={op}", f"-DKMC_INNER_POW={pw}"]))
    inst = CSRC / "kernels" / "kernel_coefficients_inst.hip"
    for op, pw in AOT_COEFFICIENT_VARIANTS:
        jobs.append((inst, OBJ_DIR / f"kernel_coefficients_inst_{op}_{pw}.o",
                     [f"-DKMC_INNER_OP={op}", f"-DKMC_INNER_POW={pw}"]))
    for rel in EXTRA_DEVICE_SOURCES:
        src = CSRC / rel
        jobs.append((src, OBJ_DIR / (src.stem + ".o"), []))
    return jobs


def _newest_source_mtime() -> float:
    newest = 0.0
    for path in list(CSRC.rglob("*")) + [Path(__file__), PACKAGE_DIR.parent / "include" / "kermac_amd.h"]:
        if path.is_file():
            newest = max(newest, path.stat().st_mtime)
    return newest


def build(force: bool = True, verbose: bool = False, workers: int | None = None,
          extra_flags: list | None = None, lib_path: Path | None = None) -> Path:
    """Compile every translation unit and link the shared library.

    force=False skips objects that are newer than every source file (used while
    developing); the default always recompiles.
    """
    hipcc = _hipcc()
    extra_flags = list(extra_flags or [])
    lib_path = Path(lib_path) if lib_path else LIB_PATH
    if extra_flags:
        force = True            # objects of a differently-flagged build must not be reused
    OBJ_DIR.mkdir(exist_ok=True)
    LIB_DIR.mkdir(exist_ok=True)
    newest = _newest_source_mtime()

    def compile_one(job):
        src, obj, defines = job
        if not force and obj.exists() and obj.stat().st_mtime > newest:
            return obj
        cmd = [hipcc, *HIPCC_FLAGS, *extra_flags, *defines, "-c", str(src), "-o", str(obj)]
        if verbose:
            print(" ".join(cmd), flush=True)
        proc = subprocess.run(cmd, capture_output=True, text=True)
        if proc.returncode != 0:
            raise RuntimeError(f"hipcc failed for {src.name} {defines}:\n{proc.stdout}\n{proc.stderr}")
        return obj

    workers = workers or min(8, os.cpu_count() or 1)
    with ThreadPoolExecutor(max_workers=workers) as pool:
        objects = list(pool.map(compile_one, _jobs()))

    lib_path.parent.mkdir(parents=True, exist_ok=True)
    tmp = lib_path.with_suffix(".so.tmp")
    cmd = [hipcc, f"--offload-arch={ARCH}", "-shared", "-fPIC", "-o", str(tmp), *map(str, objects), "-lhiprtc"]
    if verbose:
        print(" ".join(cmd), flush=True)
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"link failed:\n{proc.stdout}\n{proc.stderr}")
    os.replace(tmp, lib_path)
    if lib_path == LIB_PATH:
        build_c_example(verbose=verbose)
    if extra_flags:
        for _, obj, _ in _jobs():       # leave no differently-flagged objects behind
            obj.unlink(missing_ok=True)
    return lib_path


def build_c_example(verbose: bool = False) -> Path:
    """Build the stand-alone program of examples/ next to the library: c_abi_cdist uses nothing but
    the C ABI and is linked against the library with an rpath relative to the binary."""
    examples = PACKAGE_DIR.parent / "examples"
    target = LIB_DIR / "c_abi_cdist"
    cmd = [_hipcc(), f"--offload-arch={ARCH}", "-O2", "-std=c++17", f"-I{PACKAGE_DIR.parent / 'include'}",
           str(examples / "c_abi_cdist.cpp"), f"-L{LIB_DIR}", "-lkermac_amd", "-Wl,-rpath,$ORIGIN", "-o", str(target)]
    if verbose:
        print(" ".join(cmd), flush=True)
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"building {cmd[-1]} failed:\n{proc.stdout}\n{proc.stderr}")
    return target


if __name__ == "__main__":
    # python -m kermac_amd._build [--incremental] [-v] [--define NAME[=VALUE]]... [--output PATH]
    # --define / --output build a variant of the library elsewhere (the measurement switches of the kernel headers,
    # e.g. --define NGF_ABLATE_NO_SIGN --output /tmp/no_sign/libkermac_amd.so; KERMAC_AMD_LIBRARY=PATH then loads it)
    arguments = sys.argv[1:]
    defines, output = [], None
    while "--define" in arguments:
        at = arguments.index("--define")
        defines.append("-D" + arguments[at + 1])
        del arguments[at:at + 2]
    if "--output" in arguments:
        at = arguments.index("--output")
        output = Path(arguments[at + 1])
        del arguments[at:at + 2]
    path = build(force="--incremental" not in arguments, verbose="-v" in arguments, extra_flags=defines, lib_path=output)
    print(path)
