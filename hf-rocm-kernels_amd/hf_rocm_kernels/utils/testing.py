from typing import Optional, Tuple

import torch
from torch import Tensor


def compare_x_with_ref(x: Tensor, ref: Tensor, name: Optional[str] = None) -> Tuple[float, float, int]:
    """Max absolute difference, max relative difference (over ref != 0) and number of differing elements
    (same metrics as the reference's utils/testing.py:5-51).  Prints a short report when `name` is given."""
    if x.shape != ref.shape:
        raise ValueError(f"Cannot compare tensor of shape {x.shape} with reference of shape {ref.shape} (name: {name}).")
    xf, rf = x.float(), ref.float()
    delta = (rf - xf).abs()
    max_delta = delta.max().item() if delta.numel() else 0.0
    rel = delta.div(rf)[rf != 0]
    max_rel = rel.max().item() if rel.numel() else float("inf")
    changed = int(delta.not_equal(0).sum().item())
    if name is not None:
        if max_delta == 0:
            print(f"All good for {name}")
        else:
            print(f"{name}: max abs {max_delta:.6g}, max rel {max_rel:.6g}, mean abs {delta.mean().item():.6g}, "
                  f"{changed}/{delta.numel()} differ, NaNs x/ref {int(x.isnan().sum())}/{int(ref.isnan().sum())}")
    return max_delta, max_rel, changed


def compare_x_and_ref_to_precise(x: Tensor, ref: Tensor, precise: Tensor) -> Tuple[float, ...]:
    """Errors of `x` and of `ref` against a higher-precision result, and where `x` is the worse of the two
    (reference: utils/testing.py:54-80).  Returns (max err x, max err ref, mean err x, mean err ref,
    % of elements where x is worse, max and mean of x's error over those elements)."""
    if x.shape != ref.shape or x.shape != precise.shape:
        raise ValueError(f"Shapes differ: {x.shape}, {ref.shape}, {precise.shape}")
    dx = (precise.float() - x.float()).abs()
    dr = (precise.float() - ref.float()).abs()
    worse = dx > dr
    return (dx.max().item(), dr.max().item(), dx.mean().item(), dr.mean().item(),
            worse.float().mean().item() * 100, (dx * worse).max().item(), (dx * worse).mean().item())


def allclose_report(x: Tensor, ref: Tensor, rtol: float, atol: float) -> Tuple[bool, float, int]:
    """|x - ref| <= atol + rtol*|ref| elementwise; returns (ok, worst excess, number of violations)."""
    xf, rf = x.float(), ref.float()
    excess = (xf - rf).abs() - (atol + rtol * rf.abs())
    bad = int((excess > 0).sum().item())
    return bad == 0, (excess.max().item() if excess.numel() else 0.0), bad
