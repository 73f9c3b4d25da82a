from .wrapped import swiglu, swiglu_dynamic
from .reference import reference_swiglu
from .data import generate_swiglu_data

__all__ = ["swiglu", "swiglu_dynamic", "reference_swiglu", "generate_swiglu_data"]
