from typing import Optional, Tuple

import torch
from torch import Tensor

from ...utils.fp8 import amax_scale, fp8_quantize


def reference_quantize_fp8(x: Tensor, scale_tensor: Optional[Tensor] = None) -> Tuple[Tensor, Tensor]:
    """Torch form of `quantize_fp8`: the reference's fp8_quantize recipe (hf_rocm_kernels/utils/fp8.py:6-29, OCP
    flavour) with the given scale, or with one scale per row, amax/448."""
    if scale_tensor is None:
        scale_tensor = amax_scale(x, dim=1)
    q, _ = fp8_quantize(x, scale_tensor)
    return q, scale_tensor.reshape(-1)
