"""Shared helpers for the parity tests."""
import torch


def assert_close_to_truth(got: torch.Tensor, truth: torch.Tensor, rtol: float, atol: float = 0.0, what: str = ""):
    """|got - truth| <= rtol * |truth| + atol element-wise, with a useful message."""
    got = got.detach().to("cpu", torch.float64)
    truth = truth.detach().to("cpu", torch.float64)
    assert got.shape == truth.shape, f"{what}: shape {tuple(got.shape)} vs {tuple(truth.shape)}"
    err = (got - truth).abs()
    bound = rtol * truth.abs() + atol
    bad = err > bound
    if bad.any() or torch.isnan(got).any() != torch.isnan(truth).any():
        idx = torch.nonzero(bad)[0].tolist() if bad.any() else None
        rel = (err / truth.abs().clamp_min(1e-300)).max().item()
        raise AssertionError(
            f"{what}: {int(bad.sum())} of {bad.numel()} elements outside rtol={rtol} atol={atol}; "
            f"max abs err {err.max().item():.3e}, max rel err {rel:.3e}, first bad index {idx}")


def make_operand(L, rows, K, col_major, device, generator, batch=True, dist="randn"):
    """A [L, rows, K] (or [rows, K]) fp32 view that is row- or column-major."""
    shape = (L, K, rows) if col_major else (L, rows, K)
    if not batch:
        shape = shape[1:]
    fn = torch.randn if dist == "randn" else torch.rand
    t = fn(shape, generator=generator, dtype=torch.float32).to(device)
    if col_major:
        t = t.transpose(-1, -2)
    return t


def l1_distances_float64(a: torch.Tensor, b: torch.Tensor, block: int = 16) -> torch.Tensor:
    """sum_k |a[m, k] - b[n, k]| in float64, by blocks of rows of a, on the device of the operands
    (torch.cdist with p = 1 in float64 has returned wrong rows on the GPU for some sizes)."""
    a, b = a.double(), b.double()
    return torch.cat([(a[i:i + block, None, :] - b[None]).abs().sum(-1) for i in range(0, a.size(0), block)])
