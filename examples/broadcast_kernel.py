#!/usr/bin/env python3
"""Batched and broadcast hyper-parameters: one launch evaluates several kernels
on shared data, and the regularised diagonal can be placed for sub-blocks of a
larger symmetric kernel matrix with the offsets."""
import argparse
import sys
from pathlib import Path

import torch

sys.path.insert(0, str(Path(__file__).resolve().parents[1]))
import kermac  # noqa: E402

parser = argparse.ArgumentParser(description=__doc__)
parser.add_argument("-n", type=int, default=10000, help="points (the reference's script has 10000)")
parser.add_argument("-k", type=int, default=6, help="features per point (the reference's script has 6)")
args = parser.parse_args()

device = torch.device("cuda")
torch.manual_seed(0)
data = torch.randn(args.n, args.k, device=device)

laplace_l2 = kermac.KernelDescriptor(kermac.InnerOperator.DIFF, kermac.PowerType.SQUARE, kermac.PowerType.SQRT,
                                     kermac.KernelType.LAPLACE)
out = kermac.run_kernel(laplace_l2, data, data, bandwidth=torch.tensor([10.0, 20.0], device=device),
                        regularization=10.0, regularization_offset_x=3, regularization_offset_y=1)
print(tuple(out.shape))     # [2, n, n]: one kernel matrix per bandwidth
print(out[:, :5, :5])       # elements [m, n] with 3 + n == 1 + m hold 1 + 10 (as in the reference for out=None)
shifted = torch.diagonal(out, offset=-2, dim1=1, dim2=2)
print(f"elements [n + 2, n] that hold 1 + regularization = 11: {int((shifted == 11.0).sum())} of {shifted.numel()}; "
      f"elsewhere: {int((out == 11.0).sum()) - int((shifted == 11.0).sum())}")

laplace_p = kermac.KernelDescriptor(kermac.InnerOperator.DIFF, kermac.PowerType.POW, kermac.PowerType.POW,
                                    kermac.KernelType.LAPLACE)
out = kermac.run_kernel(laplace_p, data, data, p=torch.tensor([0.5, 0.6, 0.7, 2.0], device=device),
                        bandwidth=torch.tensor(10.0, device=device),
                        regularization=torch.tensor([1e-3, 1e-2, 1e-1, 1.0], device=device))
print(tuple(out.shape))     # [4, n, n]: one (p, regularisation) pair per batch
print(out[:, :3, :3])
diagonal = torch.diagonal(out, dim1=1, dim2=2)
expected = 1.0 + torch.tensor([1e-3, 1e-2, 1e-1, 1.0], device=device)[:, None]
print(f"largest deviation of the diagonals from 1 + regularization: {(diagonal - expected).abs().max().item():.3e}")
