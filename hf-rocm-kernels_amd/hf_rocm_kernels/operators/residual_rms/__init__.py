from .wrapped import residual_rms
from .data import generate_residual_rms_data

__all__ = ["residual_rms", "generate_residual_rms_data"]
