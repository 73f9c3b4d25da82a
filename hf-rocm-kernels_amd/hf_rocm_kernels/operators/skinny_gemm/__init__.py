from .wrapped import rms_prologue_available, skinny_gemm, skinny_gemm_add, skinny_gemm_rms, skinny_gemm_scaled, skinny_gemm_swiglu
from .reference import reference_skinny_gemm
from .data import generate_skinny_gemm_data, generate_llama_gemm_data

__all__ = ["skinny_gemm", "skinny_gemm_scaled", "skinny_gemm_add", "skinny_gemm_swiglu", "skinny_gemm_rms", "rms_prologue_available",
           "reference_skinny_gemm",
           "generate_skinny_gemm_data", "generate_llama_gemm_data"]
