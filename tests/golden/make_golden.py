"""Writes tests/golden/hot_path_vectors.npz: small seeded inputs and the
expected outputs of every operator on the hot path.

The expectations come from torch / numpy in float64 -- torch.cdist is the
oracle of the reference's own tests (tests/test_cdist.py:75), and the gradient
expectation for p = 2 is the einsum identity of tests/test_cdist_grad.py:43-49 --
never from this repository's kernels or CPU oracle, and not from the reference
package (which needs CUDA-only dependencies and is not importable here).

Run from the repository root:  python tests/golden/make_golden.py
"""
from pathlib import Path

import numpy as np
import torch

OUT = Path(__file__).resolve().parent / "hot_path_vectors.npz"


def main():
    g = torch.Generator().manual_seed(20240607)
    L, M, N, K, O = 2, 37, 29, 19, 5
    a = torch.randn(L, M, K, generator=g, dtype=torch.float32)
    b = torch.randn(L, N, K, generator=g, dtype=torch.float32)
    a64, b64 = a.double(), b.double()
    vec = {"a": a.numpy(), "b": b.numpy()}

    # cdist, torch.cdist semantics, with and without the 1/p epilogue.
    for p in (1.0, 1.3, 2.0, 0.5, 3.0):
        d = torch.cdist(a64, b64, p=p)
        vec[f"cdist_p{p}"] = d.numpy()
        vec[f"cdist_p{p}_skip"] = (d ** p).numpy()

    # Kernel functions on top of the distances (bandwidth 3, default epsilon 1e-5).
    bw = 3.0
    d1 = torch.cdist(a64, b64, p=1.0)
    d2 = torch.cdist(a64, b64, p=2.0)
    vec["laplace_l1_bw3"] = torch.exp(-d1 / bw).numpy()
    vec["laplace_l2_bw3"] = torch.exp(-d2 / bw).numpy()
    vec["gaussian_sq_bw3"] = torch.exp(-(d2 ** 2) / (2 * bw * bw)).numpy()   # DIFF, SQUARE, NOOP, GAUSSIAN
    vec["dot"] = (a64 @ b64.transpose(-1, -2)).numpy()

    # Symmetric case with exact zeros on the diagonal: epsilon mask and regularisation.
    x = a[0]
    dxx = torch.cdist(x.double(), x.double(), p=1.0)
    kxx = torch.exp(-dxx / bw)
    reg = 0.25
    kxx_reg = kxx.clone()
    kxx_reg[torch.arange(M), torch.arange(M)] = 1.0 + reg
    vec["laplace_l1_self_bw3_reg0.25"] = kxx_reg.numpy()
    # offset_x = 3, offset_y = 1: elements with 3 + m == 1 + n are replaced.
    kxx_off = kxx.clone()
    for m in range(M):
        n = m + 2
        if n < M:
            kxx_off[m, n] = 1.0 + reg
    vec["laplace_l1_self_bw3_reg0.25_off3_1"] = kxx_off.numpy()

    # Gradient: a[K,M] kernel matrix, b[N,K] x, c[O,K] coefficients, d[N,M] z.
    Kg, Mg, Ng = 23, 31, 11
    ga = torch.rand(L, Kg, Mg, generator=g, dtype=torch.float32)
    gb = torch.randn(L, Ng, Kg, generator=g, dtype=torch.float32)
    gc = torch.randn(L, O, Kg, generator=g, dtype=torch.float32)
    gd = torch.randn(L, Ng, Mg, generator=g, dtype=torch.float32)
    vec.update({"grad_a": ga.numpy(), "grad_b": gb.numpy(), "grad_c": gc.numpy(), "grad_d": gd.numpy()})
    A, B, C, D = ga.double(), gb.double(), gc.double(), gd.double()
    # p = 2: the separable einsum form the reference test uses.
    left = torch.einsum("lok,lkm,lnm->lonm", C, A, D)
    right = torch.einsum("lok,lkm,lnk->lonm", C, A, B)
    vec["grad_p2.0"] = (left - right).numpy()
    # general p: brute force over the full [L, N, M, K] difference tensor.
    diff = D[:, :, :, None] - B[:, :, None, :]             # l n m k
    sign = torch.where(torch.signbit(diff), -torch.ones_like(diff), torch.ones_like(diff))
    for p in (1.0, 1.3, 3.0):
        weight = sign * diff.abs() ** (p - 1.0)
        vec[f"grad_p{p}"] = torch.einsum("lok,lkm,lnmk->lonm", C, A, weight).numpy()

    # Kernel matrix x coefficients (Laplace-L1, bandwidth 3).
    coef = torch.randn(L, N, O, generator=g, dtype=torch.float32)
    vec["coef"] = coef.numpy()
    vec["laplace_l1_bw3_times_coef"] = (torch.exp(-d1 / bw) @ coef.double()).numpy()

    np.savez_compressed(OUT, **vec)
    print(f"wrote {OUT} ({OUT.stat().st_size} bytes, {len(vec)} arrays)")


if __name__ == "__main__":
    main()
