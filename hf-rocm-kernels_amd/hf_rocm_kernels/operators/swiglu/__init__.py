from .wrapped import swiglu, swiglu_dynamic
from .data import generate_swiglu_data

__all__ = ["swiglu", "swiglu_dynamic", "generate_swiglu_data"]
