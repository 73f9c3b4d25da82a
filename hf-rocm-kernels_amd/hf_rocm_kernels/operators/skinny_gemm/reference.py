"""Torch reference of the FP8 skinny GEMM, for callers who want to check the kernel on their own data.

Counterpart of the reference package's operators/skinny_gemm/reference.py:8-25, which calls
`torch._scaled_mm`; here the arithmetic is spelled out (dequantise, fp32 matmul, scale, one rounding) so that it
runs on any device torch supports for float8_e4m3fn.  The operators never call it.
"""
from typing import Optional

import torch
from torch import Tensor


def reference_skinny_gemm(
    skinny_a: Tensor,
    b: Tensor,
    scale_a: Tensor,
    scale_b: Tensor,
    out_dtype: torch.dtype = torch.bfloat16,
    output: Optional[Tensor] = None,
) -> Tensor:
    """((skinny_a * scale_a) @ (b * scale_b)) accumulated in fp32 and rounded once to `out_dtype`; added to
    `output` first when one is given.  scale_a has 1 or m elements, scale_b 1 or n."""
    acc = (skinny_a.float() * scale_a.float().reshape(-1, 1)) @ (b.float() * scale_b.float().reshape(1, -1))
    if output is not None:
        return (acc + output.float()).to(output.dtype)
    return acc.to(out_dtype)
