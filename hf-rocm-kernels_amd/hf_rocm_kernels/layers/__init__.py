from .fp8_linear import Fp8Linear, apply_fp8_linear

__all__ = ["Fp8Linear", "apply_fp8_linear"]
