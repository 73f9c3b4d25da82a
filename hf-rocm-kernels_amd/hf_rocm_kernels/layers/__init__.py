from .fp8_linear import Fp8Linear, apply_fp8_linear, convert_linear_layers

__all__ = ["Fp8Linear", "apply_fp8_linear", "convert_linear_layers"]
