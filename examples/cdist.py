#!/usr/bin/env python3
"""Time kermac.cdist against torch.cdist on one MI355X.

Same switches as the reference's examples/cdist.py, so its README table can be
reproduced one-for-one:

    python examples/cdist.py -m 30000 -n 30000 -k 1024 -l 1 -p 1.0 -t nnn --iters 10

-t takes three characters for (a, b, out): 'n' = that tensor is stored K-major /
column-major ("panel" layout, the fast path), 't' = torch's default row-major.
"""
import argparse
import sys
from pathlib import Path

import torch

sys.path.insert(0, str(Path(__file__).resolve().parents[1]))
import kermac  # noqa: E402


def parse_args():
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("-m", "--M", type=int, default=10000, help="rows of the output (points in a)")
    ap.add_argument("-n", "--N", type=int, default=10000, help="columns of the output (points in b)")
    ap.add_argument("-k", "--K", type=int, default=1024, help="dimension of the points")
    ap.add_argument("-l", "--L", type=int, default=2, help="number of batches")
    ap.add_argument("-p", "--p", type=float, default=1.0, help="norm order")
    ap.add_argument("-s", "--skip_epilogue", action="store_true", help="return the sum without the 1/p power")
    ap.add_argument("-a", "--try_align", action="store_true", help="accepted for compatibility (alignment is automatic)")
    ap.add_argument("-d", "--debug", action="store_true", help="print what is launched")
    ap.add_argument("-t", "--transposes", type=str, default=None, help="three of 'n'/'t' for a, b, out")
    ap.add_argument("--l2_mode", choices=["auto", "direct", "gram", "gram_bf16"], default="auto", help="evaluation of p = 2 (see set_l2_mode)")
    ap.add_argument("--skip_numeric_compare", action="store_true", help="do not compare with torch.cdist")
    ap.add_argument("--skip_torch", action="store_true", help="do not run torch.cdist at all")
    ap.add_argument("--warmup", type=int, default=2)
    ap.add_argument("--iters", type=int, default=10)
    args = ap.parse_args()
    layout = args.transposes or "ttt"
    if len(layout) != 3 or any(c not in "nt" for c in layout):
        ap.error("--transposes needs three characters out of 'n' and 't'")
    return args, [c == "n" for c in layout]


def operand(L, rows, cols, col_major, device):
    if col_major:
        return torch.randn(L, cols, rows, device=device).permute(0, 2, 1)
    return torch.randn(L, rows, cols, device=device)


def main():
    args, (a_col, b_col, c_col) = parse_args()
    device = torch.device("cuda")
    kermac.set_l2_mode(args.l2_mode)
    timer = kermac.CudaTimer()
    a = operand(args.L, args.M, args.K, a_col, device)
    b = operand(args.L, args.N, args.K, b_col, device)
    out = operand(args.L, args.M, args.N, c_col, device)

    def run():
        return kermac.cdist(a, b, out=out, p=args.p, skip_epilogue=args.skip_epilogue, try_to_align=args.try_align,
                            debug=args.debug)

    for _ in range(args.warmup):
        run()
    torch.cuda.synchronize()
    timer.start()
    for _ in range(args.iters):
        result = run()
    ms = timer.stop() / args.iters
    ops = 3.0 * args.L * args.M * args.N * args.K
    print(f"p={args.p} ({args.L},{args.M},{args.K}) x ({args.L},{args.N},{args.K})")
    print(f"\tkermac.cdist\t\t{ms:.3f} ms / iteration\t{ops / ms / 1e9:.1f} TFLOP/s (3 ops per m,n,k)")
    if args.skip_torch:
        return
    for _ in range(args.warmup):
        torch.cdist(a, b, p=args.p)
    torch.cuda.synchronize()
    timer.start()
    for _ in range(args.iters):
        reference = torch.cdist(a, b, p=args.p)
    t_ms = timer.stop() / args.iters
    print(f"\ttorch.cdist\t\t{t_ms:.3f} ms / iteration\t({t_ms / ms:.1f}x)")
    if args.skip_numeric_compare:
        return
    if args.skip_epilogue:
        reference = reference ** args.p
    diff = (result - reference).abs()
    print(f"\tvs torch.cdist (fp32): RMSE {diff.pow(2).mean().sqrt().item():.3e}   max abs {diff.max().item():.3e}   "
          f"mean abs {diff.mean().item():.3e}")
    # float64 truth on a slab of the last batch, for both implementations
    l, ms, ns = args.L - 1, slice(0, min(512, args.M)), slice(0, min(512, args.N))
    truth = torch.cdist(a[l, ms].double(), b[l, ns].double(), p=args.p)
    if args.skip_epilogue:
        truth = truth ** args.p
    for name, value in (("kermac", result), ("torch fp32", reference)):
        rel = ((value[l, ms, ns].double() - truth).abs() / truth.abs().clamp_min(1e-30)).max().item()
        print(f"\t{name} vs float64 torch.cdist on a 512 x 512 slab: max rel err {rel:.3e}")


if __name__ == "__main__":
    main()
