#!/usr/bin/env python3
"""Tour of run_kernel: predefined and custom descriptors, hyper-parameter
batching, and the fused kernel-matrix x coefficients contraction.

    python examples/build_a_kernel.py -m 4000 -n 3000 -k 64
"""
import argparse
import sys
from pathlib import Path

import torch

sys.path.insert(0, str(Path(__file__).resolve().parents[1]))
import kermac  # noqa: E402


def main():
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("-m", "--M", type=int, default=4000)
    ap.add_argument("-n", "--N", type=int, default=3000)
    ap.add_argument("-k", "--K", type=int, default=64)
    ap.add_argument("-a", "--try_align", action="store_true", help="accepted for compatibility (alignment is automatic)")
    ap.add_argument("-d", "--debug", action="store_true")
    ap.add_argument("-s", "--skip_torch", action="store_true", help="run the kernels without the torch comparisons")
    args = ap.parse_args()
    device = torch.device("cuda")
    a = torch.randn(args.M, args.K, device=device)
    b = torch.randn(args.N, args.K, device=device)
    out = torch.zeros(args.M, args.N, device=device)

    # a descriptor that is not compiled ahead of time: hiprtc builds it once, the
    # code object is cached on disk
    sqrt_sum = kermac.KernelDescriptor(kermac.InnerOperator.DOT, kermac.PowerType.SQRT, kermac.PowerType.NOOP,
                                       kermac.KernelType.NONE)
    gaussian_p = kermac.KernelDescriptor(kermac.InnerOperator.DIFF, kermac.PowerType.POW, kermac.PowerType.POW,
                                         kermac.KernelType.GAUSSIAN)
    kermac.pre_compile_descriptors(device, [kermac.kernel_descriptor_l1_norm, sqrt_sum, gaussian_p], debug=args.debug)

    def show(title, value, expected):
        """`expected` is a function so that --skip_torch really skips the torch side."""
        if args.skip_torch:
            print(f"{title:42s} result {tuple(value.shape)}")
            return
        truth = expected()
        err = (value - truth).abs().max().item()
        print(f"{title:42s} max abs difference to torch {err:.2e}   relative to max |torch| {err / truth.abs().max().item():.2e}")

    def d1():
        return torch.cdist(a, b, p=1.0)

    def d2():
        return torch.cdist(a, b, p=2.0)

    align = dict(try_to_align=args.try_align)
    show("laplace, L2 distance, bandwidth 10",
         kermac.run_kernel(kermac.kernel_descriptor_laplace_l2, a, b, out=out, bandwidth=10.0, epsilon=1e-5, **align),
         lambda: torch.exp(-d2() / 10.0))
    show("laplace, L1 distance, bandwidth 10",
         kermac.run_kernel(kermac.kernel_descriptor_laplace_l1, a, b, out=out, bandwidth=10.0, **align),
         lambda: torch.exp(-d1() / 10.0))
    show("L1 norm", kermac.run_kernel(kermac.kernel_descriptor_l1_norm, a, b, out=out, **align), d1)
    show("L2 norm", kermac.run_kernel(kermac.kernel_descriptor_l2_norm, a, b, out=out, **align), d2)
    # the Gaussian function is applied to whatever the outer power yields: here the 1.3-norm itself
    show("gaussian of the 1.3-norm, bandwidth 10",
         kermac.run_kernel(gaussian_p, a, b, out=out, inner_p=1.3, outer_p=1.0 / 1.3, bandwidth=10.0, **align),
         lambda: torch.exp(-torch.cdist(a, b, p=1.3) / 200.0))
    show("plain a @ b.T", kermac.run_kernel(kermac.kernel_descriptor_mma, a, b, out=out, **align), lambda: a @ b.T)
    if args.M * args.N * args.K < 2e9:
        show("sum_k sqrt(a b) (run-time compiled)", kermac.run_kernel(sqrt_sum, a.abs(), b.abs(), out=out, **align),
             lambda: (a.abs()[:, None, :] * b.abs()[None, :, :]).sqrt().sum(-1))

    # per-batch hyper-parameters: 4 kernels in one launch
    p = torch.tensor([0.5, 1.0, 1.5, 2.0], device=device)
    batched = kermac.run_kernel(kermac.kernel_descriptor_p_norm, a, b, p=p)
    show("4 p-norms in one launch", batched, lambda: torch.stack([torch.cdist(a, b, p=float(x)) for x in p]))

    # fused contraction: the M x N kernel matrix is never stored
    coef = torch.randn(args.N, 8, device=device)
    fused = kermac.run_kernel(kermac.kernel_descriptor_laplace_l1, a, b, bandwidth=10.0, coefficients=coef)
    show("laplace-L1 kernel matrix @ coefficients", fused[0], lambda: torch.exp(-d1() / 10.0) @ coef)


if __name__ == "__main__":
    main()
