#!/usr/bin/env python3
"""Batched and broadcast hyper-parameters: one launch evaluates several kernels
on shared data, and the regularised diagonal can be placed for sub-blocks of a
larger symmetric kernel matrix with the offsets."""
import sys
from pathlib import Path

import torch

sys.path.insert(0, str(Path(__file__).resolve().parents[1]))
import kermac  # noqa: E402

device = torch.device("cuda")
data = torch.randn(10000, 6, device=device)

laplace_l2 = kermac.KernelDescriptor(kermac.InnerOperator.DIFF, kermac.PowerType.SQUARE, kermac.PowerType.SQRT,
                                     kermac.KernelType.LAPLACE)
out = kermac.run_kernel(laplace_l2, data, data, bandwidth=torch.tensor([10.0, 20.0], device=device),
                        regularization=10.0, regularization_offset_x=3, regularization_offset_y=1)
print(out.shape)            # [2, 10000, 10000]: one kernel matrix per bandwidth
print(out[:, :5, :5])       # elements [m, n] with 3 + n == 1 + m hold 1 + 10 (as in the reference for out=None)

laplace_p = kermac.KernelDescriptor(kermac.InnerOperator.DIFF, kermac.PowerType.POW, kermac.PowerType.POW,
                                    kermac.KernelType.LAPLACE)
out = kermac.run_kernel(laplace_p, data, data, p=torch.tensor([0.5, 0.6, 0.7, 2.0], device=device),
                        bandwidth=torch.tensor(10.0, device=device),
                        regularization=torch.tensor([1e-3, 1e-2, 1e-1, 1.0], device=device))
print(out.shape)            # [4, 10000, 10000]: one (p, regularisation) pair per batch
print(out[:, :3, :3])
