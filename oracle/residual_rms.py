"""Oracle of the residual-RMSNorm op.  Test infrastructure only (see __init__.py)."""
from typing import Optional, Tuple

import torch

from . import fp8


def reference_rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    """x * rsqrt(mean(x^2) + eps) in fp32 (hf_rocm_kernels/operators/residual_rms/reference.py:69-72)."""
    x = x.to(torch.float32)
    variance = x.pow(2).mean(-1, keepdim=True)
    return x * torch.rsqrt(variance + eps)


def reference_residual_rms(input: torch.Tensor, residual: torch.Tensor, weight: torch.Tensor, epsilon: float,
                           scale_tensor: Optional[torch.Tensor], next_buffer: Optional[torch.Tensor] = None
                           ) -> Tuple[torch.Tensor, torch.Tensor, Optional[torch.Tensor]]:
    """Order of operations of reference.py:7-36: 16-bit add -> fp32 rms -> cast to the weight dtype -> * weight
    (16-bit multiply) -> fp8_quantize; zero the next buffer.  Accepts float16 or bfloat16 (the reference asserts
    float16).  Does not modify its arguments; returns (output, new residual, scale)."""
    assert input.dtype in (torch.float16, torch.bfloat16) and residual.dtype == input.dtype
    summed = input + residual
    normed = reference_rms(summed, epsilon)
    if weight.dtype in (torch.float16, torch.bfloat16):
        normed = normed.to(weight.dtype)
    normed = weight * normed
    if scale_tensor is not None:
        out, scale_tensor = fp8.fp8_quantize(normed, scale_tensor)
        if next_buffer is not None:
            next_buffer.fill_(0)
    else:
        out = normed
    return out, summed, scale_tensor


def precise_residual_rms(input: torch.Tensor, residual: torch.Tensor, weight: torch.Tensor, epsilon: float,
                         scale_tensor: Optional[torch.Tensor], next_buffer: Optional[torch.Tensor] = None
                         ) -> Tuple[torch.Tensor, torch.Tensor]:
    """Everything in float64 up to the final quantisation (reference.py:39-66).  As there, the sum itself is
    not rounded to 16 bits.  Returns (output, float64 residual)."""
    x = input.to(torch.float64) + residual.to(torch.float64)
    variance = x.pow(2).mean(-1, keepdim=True)
    normed = x * torch.rsqrt(variance + epsilon)
    normed = weight.to(torch.float64) * normed
    if scale_tensor is not None:
        out, _ = fp8.fp8_quantize(normed, scale_tensor)
        if next_buffer is not None:
            next_buffer.fill_(0)
    else:
        out = normed
    return out, x


def precise_residual_rms_dynamic(input: torch.Tensor, residual: torch.Tensor, weight: torch.Tensor, epsilon: float
                                 ) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
    """Per-row dynamic quantisation of the normalised row (no reference counterpart; the reference's
    operators/residual_rms/reference.py:7-36 quantises with one static scale): the residual is the 16-bit sum as in
    `reference_residual_rms`, y = weight * z * rsqrt(mean(z^2) + eps) in float64, scale[row] = amax|y| / 448 rounded to
    float32, output = e4m3fn(y / scale).  Returns (output fp8, new residual (16-bit), scales fp32 [rows], y float64).
    Pinned by the textbook formula and by what the scaling fixes: every non-zero row of the output has a code of
    magnitude 448, and output * scale reproduces y to within half an fp8 step."""
    z = (input.float() + residual.float()).to(input.dtype)
    x = z.to(torch.float64)
    y = weight.to(torch.float64) * x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + epsilon)
    scales = fp8.amax_scale(y, dim=1)
    out, _ = fp8.fp8_quantize(y, scales)
    return out, z, scales.reshape(-1), y
