"""Run-time compilation (hiprtc) with a persistent on-disk cache.

Takes the place of the reference's NVRTC + LMDB ``ModuleCache``
(src/kermac/module_cache/module_cache.py:110-239): a process-wide, lock-guarded
singleton that maps ``(device, function name)`` to a loaded device function,
compiling through hiprtc on a miss and keeping code objects on disk keyed by
(package, version, HIP version, arch, flags, function name).
"""
from __future__ import annotations

import hashlib
import threading
from typing import Dict, List, Sequence, Tuple

import torch

from .. import _backend
from .code_object_store import CodeObjectStore, FunctionKey
from .paths import cache_root, get_kernel_source_dir, get_package_name, get_package_version

ARCH = "gfx950"

# hiprtc options; the last four words switch packed-fp32 code generation off,
# the same way the ahead-of-time build does.
JIT_OPTIONS = [
    f"--offload-arch={ARCH}",
    "-O3",
    "-std=c++17",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]

_INNER_OPERATOR_NAMES = ["kmc::OP_DIFF", "kmc::OP_DOT"]
_POWER_NAMES = ["kmc::POW_NOOP", "kmc::POW_ABS", "kmc::POW_SQUARE", "kmc::POW_SQRT", "kmc::POW_POW"]
_LOAD_MODE_NAMES = ["kmc::LOAD_COL_VEC", "kmc::LOAD_COL_SCALAR", "kmc::LOAD_ROW_VEC", "kmc::LOAD_ROW_SCALAR"]

JIT_TRANSLATION_UNIT = '#include "kernel_coefficients.hpp"\n'
JIT_HEADERS = ["device_common.hpp", "build_kernel.hpp", "kernel_coefficients.hpp"]


def build_kernel_function_name(inner_operator: int, inner_power: int, load_a: int, load_b: int) -> str:
    """Template-id (a hiprtc name expression) of one kernel instantiation."""
    return (f"kmc::build_kernel<{_INNER_OPERATOR_NAMES[inner_operator]},{_POWER_NAMES[inner_power]},"
            f"{_LOAD_MODE_NAMES[load_a]},{_LOAD_MODE_NAMES[load_b]}>")


def kernel_coefficients_function_name(inner_operator: int, inner_power: int, load_a: int, load_b: int) -> str:
    """Template-id of one fused kernel-matrix x coefficients instantiation."""
    return (f"kmc::kernel_times_coefficients<{_INNER_OPERATOR_NAMES[inner_operator]},{_POWER_NAMES[inner_power]},"
            f"{_LOAD_MODE_NAMES[load_a]},{_LOAD_MODE_NAMES[load_b]}>")


def _read_headers() -> List[Tuple[str, str]]:
    directory = get_kernel_source_dir()
    return [(name, (directory / name).read_text()) for name in JIT_HEADERS]


def hash_kernel_sources() -> str:
    """sha256 over the device headers, in a fixed order
    (reference: module_cache/common.py:15-36)."""
    hasher = hashlib.sha256()
    for name, text in _read_headers():
        hasher.update(name.encode())
        hasher.update(text.encode())
    return hasher.hexdigest()


def compile_functions(function_names: Sequence[str], debug: bool = False) -> Tuple[bytes, List[str]]:
    """Compile all ``function_names`` in ONE hiprtc program; returns the code
    object and the lowered (mangled) names, in order
    (reference: module_cache.py:13-51)."""
    if debug:
        for name in function_names:
            print(f"(Kermac Debug) Compiling ({ARCH}): {name}")
    return _backend.jit_compile(JIT_TRANSLATION_UNIT, "kermac_amd_jit.hip", _read_headers(), JIT_OPTIONS,
                                list(function_names))


class Singleton(type):
    _instances: Dict[type, object] = {}
    _lock = threading.Lock()

    def __call__(cls, *args, **kwargs):
        with cls._lock:
            if cls not in cls._instances:
                cls._instances[cls] = super().__call__(*args, **kwargs)
        return cls._instances[cls]


class ModuleCache(metaclass=Singleton):
    """(device, function name) -> loaded device function, compiled on demand."""

    def __init__(self, debug=False):
        self._loaded_modules: Dict[Tuple[int, str], int] = {}
        self._loaded_kernel_functions: Dict[Tuple[int, str], int] = {}
        self._lock = threading.Lock()
        root = cache_root()
        if debug:
            print(f"(Kermac Debug) Using kernel cache at: {root.resolve()}")
        source_hash = hash_kernel_sources()
        if debug:
            print(f"(Kermac Debug) Combined hash of device source files: {source_hash}")
        self._store = CodeObjectStore(root, source_hash, debug=debug)
        self._toolchain_version = str(torch.version.hip)

    def _key(self, function_name: str) -> FunctionKey:
        return FunctionKey(
            package_name=get_package_name(),
            package_version=get_package_version(),
            toolchain_version=self._toolchain_version,
            arch=ARCH,
            flags=" ".join(JIT_OPTIONS),
            function_name=function_name,
        )

    def compile_and_cache_functions(self, device, function_names: List[str], debug=False) -> bool:
        """Compile whatever of ``function_names`` is not in the store yet, in one
        program (reference: module_cache.py:53-108, 149-162).  Needs no GPU."""
        missing = [name for name in function_names if self._store.get_function_mapping(self._key(name)) is None]
        if not missing:
            if debug:
                print(f"(Kermac Debug) Nothing needs to compile ({ARCH})")
            return True
        code, lowered = compile_functions(missing, debug=debug)
        code_hash = self._store.put_code(code)
        for name, lowered_name in zip(missing, lowered):
            self._store.put_function_mapping(self._key(name), lowered_name, code_hash)
        if debug:
            print("(Kermac Debug) Stored all mappings")
        return True

    def get_function(self, device, function_name: str, debug=False) -> int:
        """Device function handle (a ``hipFunction_t`` as int) for
        ``function_name`` on ``device`` (reference: module_cache.py:164-239)."""
        device = torch.device(device)
        device_id = device.index if device.index is not None else torch.cuda.current_device()
        memo_key = (device_id, function_name)
        with self._lock:
            function = self._loaded_kernel_functions.get(memo_key)
            if function is not None:
                if debug:
                    print(f"(Kermac Debug) Loaded function found for (device:{device_id}, function:{function_name})")
                return function
            arch = _backend.device_arch(device_id)
            if not arch.startswith(ARCH):
                raise ValueError(f"Invalid device architecture {arch}: these kernels require {ARCH} (MI355X)")
            key = self._key(function_name)
            mapping = self._store.get_function_mapping(key)
            if mapping is None:
                if debug:
                    print(f"(Kermac Debug) Mapping does not exist for {key}")
                self.compile_and_cache_functions(device, [function_name], debug=debug)
                mapping = self._store.get_function_mapping(key)
                if mapping is None:
                    raise RuntimeError(f"kernel cache lost the entry for {function_name} right after compiling it")
            lowered_name, code_hash = mapping
            module_key = (device_id, code_hash)
            module = self._loaded_modules.get(module_key)
            if module is None:
                code = self._store.get_code(code_hash)
                if code is None:
                    # the stored file vanished or failed its hash check (the store has dropped it):
                    # compile again; other functions of the lost program follow when they are asked for
                    if debug:
                        print(f"(Kermac Debug) Code object {code_hash} is unusable, compiling {function_name} again")
                    self.compile_and_cache_functions(device, [function_name], debug=debug)
                    mapping = self._store.get_function_mapping(key)
                    if mapping is None:
                        raise RuntimeError(f"kernel cache lost the entry for {function_name} right after compiling it")
                    lowered_name, code_hash = mapping
                    module_key = (device_id, code_hash)
                    code = self._store.get_code(code_hash)
                    if code is None:
                        raise RuntimeError(f"kernel cache has no code object {code_hash}")
                with torch.cuda.device(device_id):
                    module = _backend.module_load(code)
                self._loaded_modules[module_key] = module
            function = _backend.module_get_function(module, lowered_name)
            self._loaded_kernel_functions[memo_key] = function
            return function
