"""kermac_amd: kermac's fused distance hot path on MI355X (gfx950).

``import kermac_amd as kermac`` gives the reference's names:
``cdist``, ``cdist_grad``, ``run_kernel``, ``pre_compile_descriptors``,
``KernelDescriptor``, the enums, the predefined descriptors, ``ModuleCache``
and the helpers of ``common``.
"""
from .common import (Alignment, CudaTimer, FillMode, Majorness, PyTorchStreamWrapper, TensorStats, ceil_div,
                     merge_batch_size, tensor_stats)
from .module_cache.module_cache import ModuleCache
from .build_a_kernel import (InnerOperator, KernelDescriptor, KernelType, PowerType, Symmetry,
                             kernel_descriptor_l1_norm, kernel_descriptor_l2_norm, kernel_descriptor_laplace_l1,
                             kernel_descriptor_laplace_l2, kernel_descriptor_mma, kernel_descriptor_p_norm,
                             pre_compile_descriptors, run_kernel, set_l2_mode, get_l2_mode, l2_mode, DEFAULT_L2_MODE,
                             set_l1_mode, get_l1_mode, l1_mode, DEFAULT_L1_MODE)
from .cdist import cdist
from ._scratch import scratch, set_max_scratch_bytes, get_max_scratch_bytes
from .cdist_grad import cdist_grad

__version__ = "0.1.0"

__all__ = [
    "cdist", "cdist_grad", "KernelDescriptor", "run_kernel", "PowerType", "InnerOperator", "KernelType",
    "Symmetry", "kernel_descriptor_laplace_l1", "kernel_descriptor_laplace_l2", "kernel_descriptor_p_norm",
    "kernel_descriptor_l1_norm", "kernel_descriptor_l2_norm", "kernel_descriptor_mma",
    "pre_compile_descriptors", "ModuleCache", "CudaTimer", "PyTorchStreamWrapper", "TensorStats",
    "tensor_stats", "Majorness", "Alignment", "FillMode", "ceil_div", "merge_batch_size",
    "set_l2_mode", "get_l2_mode", "l2_mode", "DEFAULT_L2_MODE",
    "set_l1_mode", "get_l1_mode", "l1_mode", "DEFAULT_L1_MODE",
    "scratch", "set_max_scratch_bytes", "get_max_scratch_bytes",
]
