from .wrapped import residual_rms, residual_rms_dynamic
from .data import generate_residual_rms_data

__all__ = ["residual_rms", "residual_rms_dynamic", "generate_residual_rms_data"]
