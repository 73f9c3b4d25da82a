from .wrapped import residual_rms, residual_rms_dynamic
from .reference import reference_residual_rms, precise_residual_rms
from .data import generate_residual_rms_data

__all__ = ["residual_rms", "residual_rms_dynamic", "reference_residual_rms", "generate_residual_rms_data",
           "precise_residual_rms"]
