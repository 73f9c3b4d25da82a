from typing import Optional, Tuple

import torch
from torch import Tensor

import hf_rocm_kernels._HFRK_C  # noqa: F401  (registers torch.ops._HFRK_C)


def quantize_fp8(x: Tensor, scale_tensor: Optional[Tensor] = None) -> Tuple[Tensor, Tensor]:
    """Quantise a 16-bit activation block to float8_e4m3fn in one kernel.

    The reference quantises on the caller's side with torch ops (hf_rocm_kernels/utils/fp8.py:6-29: divide, clamp,
    cast); this is that recipe as one launch, and additionally per token.
    Args:
        - x: a (rows, cols) float16/bfloat16 tensor in row-major format, cols % 8 == 0 and cols <= 32768
        - scale_tensor: one float32 (static scale: output = x / scale, saturating at +-448), or None for one dynamic
          scale per row, amax/448
    Outputs:
        - the float8_e4m3fn tensor, and the scale(s): `scale_tensor` itself, or a float32 (rows,) tensor ready to be
          the GEMM's per-token `scale_a`
    """
    assert x.dim() == 2 and x.is_contiguous(), f"Expected a contiguous 2-D tensor but got {x.shape = } {x.stride() = }"
    assert x.dtype in (torch.float16, torch.bfloat16), f"Expected {x.dtype = } to be torch.float16 or torch.bfloat16"
    assert x.device.type == "cuda", f"Expected a device tensor but got {x.device = }"
    rows, cols = x.shape
    assert cols % 8 == 0 and cols <= 32768, f"Expected cols % 8 == 0 and cols <= 32768: {x.shape = }"
    output = torch.empty(size=(rows, cols), dtype=torch.float8_e4m3fn, device=x.device)
    if scale_tensor is not None:
        assert scale_tensor.numel() == 1 and scale_tensor.dtype == torch.float32, "Expected scale_tensor to be one float32"
        assert scale_tensor.device == x.device, f"Expected {scale_tensor.device = } to be {x.device}"
        torch.ops._HFRK_C.quantize_fp8(x, scale_tensor, output, scale_tensor)
        return output, scale_tensor
    scales = torch.empty(size=(rows,), dtype=torch.float32, device=x.device)
    torch.ops._HFRK_C.quantize_fp8(x, None, output, scales)
    return output, scales
