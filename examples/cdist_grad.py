#!/usr/bin/env python3
"""kermac.cdist_grad on an AGOP / RFM-shaped problem, timed and checked.

Same switches as the reference's examples/cdist_grad.py:

    python examples/cdist_grad.py -m 10000 -n 768 -o 16 -k 10000 -l 2 -p 2.0 --warmup 1 --iters 1

a = kernel matrix [L, K, M], b = x [L, N, K], c = coefficients [L, O, K], d = z [L, N, M],
out = gradient [L, O, N, M]; K is the contracted (centres) dimension.  For p = 2 the
whole result is compared with the two-einsum identity the reference's own test uses; for
every p a slab is compared with a float64 sum over the centres.
"""
import argparse
import sys
from pathlib import Path

import torch

sys.path.insert(0, str(Path(__file__).resolve().parents[1]))
import kermac  # noqa: E402


def parse_args():
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("-m", "--M", type=int, default=10000, help="points z the gradient is taken at")
    ap.add_argument("-n", "--N", type=int, default=768, help="coordinates per point")
    ap.add_argument("-o", "--O", type=int, default=16, help="output channels of the coefficients")
    ap.add_argument("-k", "--K", type=int, default=10000, help="centres x (the contracted dimension)")
    ap.add_argument("-l", "--L", type=int, default=2, help="batches")
    ap.add_argument("-p", "--p", type=float, default=2.0, help="norm order")
    ap.add_argument("-d", "--debug", action="store_true", help="print what is launched")
    ap.add_argument("--skip_torch_einsum", action="store_true", help="do not run the einsum composition (p = 2)")
    ap.add_argument("--skip_numeric_compare", action="store_true", help="do not compare results")
    ap.add_argument("--warmup", type=int, default=1)
    ap.add_argument("--iters", type=int, default=1)
    return ap.parse_args()


def einsum_gradient_l2(coefs, kernel_matrix, x, z):
    """p = 2: sum_k c[o,k] a[k,m] (z[n,m] - x[n,k]) as two contractions."""
    return (torch.einsum("lok,lkm,lnm->lonm", coefs, kernel_matrix, z)
            - torch.einsum("lok,lkm,lnk->lonm", coefs, kernel_matrix, x))


def slab_truth(a, b, c, d, p, ms, ns):
    """float64 sum over the centres for out[:, :, ns, ms] of the last batch."""
    diff = d[-1, ns, ms].double()[:, :, None] - b[-1, ns].double()[:, None, :]              # [n, m, k]
    sign = torch.where(torch.signbit(diff), -1.0, 1.0).double()                             # copysign(1, x)
    weight = sign * diff.abs() ** (p - 1.0) if p != 1.0 else sign
    return torch.einsum("ok,km,nmk->onm", c[-1].double(), a[-1][:, ms].double(), weight)


def main():
    args = parse_args()
    M, N, O, K, L, p = args.M, args.N, args.O, args.K, args.L, args.p
    device = torch.device("cuda")
    timer = kermac.CudaTimer()
    p_tensor = torch.full((1,), p, dtype=torch.float32, device=device)      # as the reference passes it
    a = torch.randn(L, K, M, device=device)
    b = torch.randn(L, N, K, device=device)
    c = torch.randn(L, O, K, device=device)
    d = torch.randn(L, N, M, device=device)
    out = torch.zeros(L, O, N, M, device=device)

    print(f"Warmup {args.warmup} iterations of kermac.cdist_grad")
    for _ in range(args.warmup):
        kermac.cdist_grad(a, b, c, d, out=out, p=p_tensor, debug=args.debug)
    torch.cuda.synchronize()
    timer.start()
    for _ in range(args.iters):
        result = kermac.cdist_grad(a, b, c, d, out=out, p=p_tensor, debug=args.debug)
    ms = timer.stop() / args.iters
    print(f"Running {args.iters} iterations of p-norm-gradient={p} with size ({L},{K},{M}) by ({L},{N},{K}) by "
          f"({L},{O},{K}) by ({L},{N},{M}) => ({L},{O},{N},{M})")
    print(f"\tkermac.cdist_grad \t\t{ms:.3f} ms / iteration\t"
          f"{(2 * O + 3) * float(L) * M * N * K / ms / 1e9:.1f} TFLOP/s ((2 O + 3) ops per m,n,k)")

    if not args.skip_numeric_compare:
        ms_, ns_ = slice(0, min(M, 24)), slice(0, min(N, 12))
        truth = slab_truth(a, b, c, d, p, ms_, ns_)
        err = (result[-1][:, ns_, ms_].double() - truth).abs().max().item() / truth.abs().mean().item()
        print(f"\tfloat64 slab check: max abs error / mean |truth| = {err:.3e}")
    if p != 2.0:
        print("Cannot compare timing or results to the torch einsum composition unless p=2.0")
        return
    if args.skip_torch_einsum:
        return
    timer.start()
    for _ in range(args.iters):
        expected = einsum_gradient_l2(c, a, b, d)
    print(f"\ttorch-einsum-cdist_grad\t\t{timer.stop() / args.iters:.3f} ms / iteration")
    if not args.skip_numeric_compare:
        diff = (result - expected).abs()
        print("\nTensor Comparison:")
        print(f"\tRoot Mean Squared Error:\t{diff.pow(2).mean().sqrt().item():.6e}")
        print(f"\tMax Absolute Error:\t\t{diff.max().item():.6e}")
        print(f"\tMean Absolute Error:\t\t{diff.mean().item():.6e}")


if __name__ == "__main__":
    main()
