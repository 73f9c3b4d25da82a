from .wrapped import swiglu
from .data import generate_swiglu_data

__all__ = ["swiglu", "generate_swiglu_data"]
