"""Torch references of the residual-RMSNorm operator (counterparts of the reference package's
operators/residual_rms/reference.py:7-72), for callers who want to check the kernel.  The operators never call them."""
from typing import Optional, Tuple

import torch
from torch import Tensor

from hf_rocm_kernels.utils.fp8 import fp8_quantize


def reference_rms(x: Tensor, eps: float) -> Tensor:
    """x / sqrt(mean(x^2) + eps) over the last dimension, in fp32."""
    x = x.to(torch.float32)
    return x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + eps)


def reference_residual_rms(
    input: Tensor,
    residual: Tensor,
    weight: Tensor,
    epsilon: float,
    scale_tensor: Optional[Tensor],
    next_buffer: Optional[Tensor] = None,
) -> Tuple[Tensor, Tensor, Optional[Tensor]]:
    """The op as a chain of torch calls with a 16-bit rounding after each: add, normalise (fp32, rounded to the
    weight dtype), multiply by the weight, then quantise to float8_e4m3fn when a scale is given.
    Returns (output, input + residual, scale); does not modify `residual`."""
    summed = input + residual
    normed = weight * reference_rms(summed, epsilon).to(weight.dtype)
    if scale_tensor is None:
        return normed, summed, None
    out, scale_tensor = fp8_quantize(normed, scale_tensor)
    if next_buffer is not None:
        next_buffer.zero_()
    return out, summed, scale_tensor


def precise_residual_rms(
    input: Tensor,
    residual: Tensor,
    weight: Tensor,
    epsilon: float,
    scale_tensor: Optional[Tensor],
    next_buffer: Optional[Tensor] = None,
) -> Tuple[Tensor, Tensor]:
    """The same in float64 up to the final quantisation (the sum is not rounded to 16 bits either): the yardstick
    both the kernel and `reference_residual_rms` are measured against.  Returns (output, float64 sum)."""
    summed = input.double() + residual.double()
    normed = weight.double() * summed * torch.rsqrt(summed.pow(2).mean(-1, keepdim=True) + epsilon)
    if scale_tensor is None:
        return normed, summed
    out, _ = fp8_quantize(normed, scale_tensor)
    if next_buffer is not None:
        next_buffer.zero_()
    return out, summed
