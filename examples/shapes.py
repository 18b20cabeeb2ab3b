"""Times the three operators on shapes away from the benchmark configuration: small results over
long contractions, batches of small problems, few rows against many centres, gradients with few
outputs or a deep contraction.  Prints milliseconds and TFLOP/s in the units of the benchmark
(3 operations per (m, n, k) for the pairwise kernels, (2 O + 3) per (m, n, k) for the gradient).

    python examples/shapes.py            # everything
    python examples/shapes.py cdist      # one group: cdist, self, grad or fused
"""
import sys
from pathlib import Path

import torch

sys.path.insert(0, str(Path(__file__).resolve().parents[1]))
import kermac_amd as kermac  # noqa: E402


def timeit(fn, iters=5):
    fn()
    torch.cuda.synchronize()
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    start.record()
    for _ in range(iters):
        fn()
    stop.record()
    torch.cuda.synchronize()
    return start.elapsed_time(stop) / iters


def cdist_shapes(device):
    print("cdist, K-major panels: L, M, N, K -> p = 1 / p = 2")
    shapes = [(1, 30000, 30000, 1024), (1, 4096, 4096, 1024), (1, 2048, 2048, 1024), (1, 1024, 1024, 4096),
              (1, 100, 100, 100000), (1, 512, 512, 16384), (1, 128, 1000000, 64), (1, 1000, 100000, 512),
              (1, 30000, 30000, 16), (64, 512, 512, 256), (1000, 128, 128, 128), (1, 3000, 2900, 2048),
              (1, 3072, 3072, 1000), (1, 2304, 2304, 16384)]
    for L, M, N, K in shapes:
        a = torch.randn(L, K, M, device=device).transpose(1, 2)
        b = torch.randn(L, K, N, device=device).transpose(1, 2)
        out = torch.empty(L, N, M, device=device).transpose(1, 2)
        cells = []
        for p in (1.0, 2.0):
            ms = timeit(lambda: kermac.cdist(a, b, out=out, p=p))
            cells.append(f"{ms:8.3f} ms {3.0 * L * M * N * K / ms / 1e9:6.1f} TFLOP/s")
        print(f"  {L:5d} {M:6d} {N:8d} {K:7d}   " + "   ".join(cells), flush=True)
        del a, b, out


def self_shapes(device):
    print("cdist of a set against itself (one triangle of tiles computed, mirrored): M, K -> p = 1 / p = 2")
    for M, K in ((30000, 1024), (8192, 1024), (4096, 4096), (3072, 1024), (1536, 4096)):
        x = torch.randn(K, M, device=device).t()
        out = torch.empty(M, M, device=device).t()
        cells = []
        for p in (1.0, 2.0):
            ms = timeit(lambda: kermac.cdist(x, x, out=out, p=p))
            cells.append(f"{ms:8.3f} ms {3.0 * M * M * K / ms / 1e9:6.1f} TFLOP/s of the full matrix")
        print(f"  {M:6d} {K:6d}   " + "   ".join(cells), flush=True)
        del x, out


def grad_shapes(device):
    print("cdist_grad: K (contraction), M, N, O -> p = 1 / p = 1.3")
    shapes = [(8192, 8192, 512, 16), (8192, 8192, 512, 1), (8192, 8192, 512, 5), (8192, 8192, 512, 17),
              (8192, 8192, 512, 48), (10000, 2000, 100, 1), (100000, 1000, 64, 1), (8192, 8192, 16, 16),
              (4096, 16384, 784, 10)]
    for K, M, N, O in shapes:
        a = torch.rand(K, M, device=device)
        b = torch.randn(N, K, device=device)
        c = torch.randn(O, K, device=device)
        d = torch.randn(N, M, device=device)
        out = torch.empty(1, O, N, M, device=device)
        cells = []
        for p in (1.0, 1.3):
            ms = timeit(lambda: kermac.cdist_grad(a, b, c, d, out=out, p=p))
            cells.append(f"{ms:8.3f} ms {(2 * O + 3) * M * N * K / ms / 1e9:6.1f} TFLOP/s")
        print(f"  {K:7d} {M:6d} {N:5d} {O:3d}   " + "   ".join(cells), flush=True)
        del a, b, c, d, out


def fused_shapes(device):
    print("run_kernel(laplace_l1, ..., coefficients=...): L, rows M, centres N, K, O")
    shapes = [(4, 16384, 16384, 256, 32), (1, 65536, 16384, 256, 32), (1, 100000, 16384, 256, 32),
              (1, 16384, 16384, 256, 64), (1, 16384, 16384, 256, 100), (1, 1000, 100000, 512, 1),
              (1, 128, 100000, 256, 10), (1, 4096, 65536, 256, 32)]
    for L, M, N, K, O in shapes:
        x = (torch.rand(L, K, M, device=device) * 2 - 1).transpose(1, 2)
        z = (torch.rand(K, N, device=device) * 2 - 1).t()
        coef = torch.randn(L, N, O, device=device)
        out = torch.empty(L, M, O, device=device)
        if L == 1:
            x, coef, out = x[0], coef[0], out[0]
        ms = timeit(lambda: kermac.run_kernel(kermac.kernel_descriptor_laplace_l1, x, z, out=out, bandwidth=10.0,
                                              coefficients=coef), iters=3)
        print(f"  {L:2d} {M:7d} {N:7d} {K:4d} {O:4d}   {ms:8.3f} ms {L * M * N * (3.0 * K + 2 * O) / ms / 1e9:6.1f} TFLOP/s",
              flush=True)
        del x, z, coef, out


if __name__ == "__main__":
    if not torch.cuda.is_available():
        sys.exit("examples/shapes.py needs a GPU")
    groups = {"cdist": cdist_shapes, "self": self_shapes, "grad": grad_shapes, "fused": fused_shapes}
    chosen = sys.argv[1:] or list(groups)
    for name in chosen:
        if name not in groups:
            sys.exit(f"unknown group {name!r}; choose from {', '.join(groups)}")
        groups[name](torch.device("cuda:0"))
