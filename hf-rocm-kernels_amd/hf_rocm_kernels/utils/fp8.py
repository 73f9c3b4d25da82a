from typing import Tuple

import torch
from torch import Tensor

FP8_DTYPE = torch.float8_e4m3fn
FP8_MAX = 448.0


def fp8_quantize(x_full_precision: Tensor, scale: Tensor) -> Tuple[Tensor, Tensor]:
    """Quantize `x / scale` to OCP float8_e4m3fn, saturating at +-448, round to nearest even.

    Same recipe as the reference's fp8_quantize (hf_rocm_kernels/utils/fp8.py:6-29) up to the cast; the
    reference then re-labels the bits as e4m3fnuz (removing -0, which is NaN there) and returns 2*scale because
    an fnuz value is half the fn value on the same bits.  gfx950 computes in e4m3fn, so the bits stay as they
    are and the scale comes back unchanged.  `scale` may be a scalar tensor or broadcast against `x`
    (per-row [m,1] or per-channel [n,1]).
    """
    x_quantized = (x_full_precision.float() * scale.reciprocal()).clamp(min=-FP8_MAX, max=FP8_MAX)
    return x_quantized.to(FP8_DTYPE), scale


def amax_scale(x: Tensor, dim=None) -> Tensor:
    """scale = amax/448 over the whole tensor (dim=None) or per slice along `dim` (kept), never zero."""
    x = x.float().abs()
    amax = x.amax() if dim is None else x.amax(dim=dim, keepdim=True)
    return (amax / FP8_MAX).clamp_min(torch.finfo(torch.float32).tiny).to(torch.float32)
