from .wrapped import quantize_fp8
from .reference import reference_quantize_fp8

__all__ = ["quantize_fp8", "reference_quantize_fp8"]
