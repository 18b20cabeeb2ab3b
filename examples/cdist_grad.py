#!/usr/bin/env python3
"""kermac_amd.cdist_grad on an AGOP / RFM-shaped problem, checked against einsum.

    python examples/cdist_grad.py -m 10000 -n 768 -o 16 -k 10000 -p 2.0

a = kernel matrix [K, M], b = x [N, K], c = coefficients [O, K], d = z [N, M],
out = gradient [O, N, M]; K is the contracted (centres) dimension.
"""
import argparse
import sys
from pathlib import Path

import torch

sys.path.insert(0, str(Path(__file__).resolve().parents[1]))
import kermac_amd as kermac  # noqa: E402


def main():
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("-m", "--M", type=int, default=10000)
    ap.add_argument("-n", "--N", type=int, default=768)
    ap.add_argument("-o", "--O", type=int, default=16)
    ap.add_argument("-k", "--K", type=int, default=10000)
    ap.add_argument("-p", "--p", type=float, default=2.0)
    ap.add_argument("-d", "--debug", action="store_true")
    ap.add_argument("--iters", type=int, default=5)
    ap.add_argument("--skip_torch", action="store_true")
    args = ap.parse_args()
    device = torch.device("cuda")
    M, N, O, K = args.M, args.N, args.O, args.K
    a = torch.randn(K, M, device=device)
    b = torch.randn(N, K, device=device)
    c = torch.randn(O, K, device=device)
    d = torch.randn(N, M, device=device)
    out = torch.zeros(O, N, M, device=device)
    timer = kermac.CudaTimer()
    kermac.cdist_grad(a, b, c, d, out=out, p=args.p, debug=args.debug)
    torch.cuda.synchronize()
    timer.start()
    for _ in range(args.iters):
        kermac.cdist_grad(a, b, c, d, out=out, p=args.p)
    ms = timer.stop() / args.iters
    print(f"kermac_amd.cdist_grad p={args.p}\t{ms:.3f} ms\t{(2 * O + 3) * M * N * K / ms / 1e9:.1f} TFLOP/s")
    if args.skip_torch or args.p != 2.0:
        return
    # p = 2 separates into two einsums (the identity the reference's test uses)
    timer.start()
    expected = torch.einsum("ok,km,nm->onm", c, a, d) - torch.einsum("ok,km,nk->onm", c, a, b)
    print(f"torch.einsum\t\t\t{timer.stop():.3f} ms")
    diff = (out - expected).abs()
    print(f"RMSE {diff.pow(2).mean().sqrt().item():.3e}   max abs {diff.max().item():.3e}")


if __name__ == "__main__":
    main()
