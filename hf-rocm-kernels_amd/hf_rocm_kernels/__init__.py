"""MI355X (gfx950) implementation of the `hf_rocm_kernels` operator surface.

Same names as the reference package (hf_rocm_kernels/__init__.py:1-6): four operators backed by
`torch.ops._HFRK_C`, which forwards to the C ABI of `libhfrk_gfx950.so` (include/hfrk_gfx950.h).
Importing this package loads both shared objects and fails if either is missing: there is no fallback path.
"""
from .operators.increment import increment
from .operators.residual_rms import residual_rms, residual_rms_dynamic
from .operators.swiglu import swiglu, swiglu_dynamic
from .operators.skinny_gemm import skinny_gemm, skinny_gemm_add, skinny_gemm_rms, skinny_gemm_scaled, skinny_gemm_swiglu
from .operators.quantize import quantize_fp8

from . import _fake_kernels  # noqa: F401  (shape-only implementations, so the operators can be traced)
from . import plan_table

plan_table.load_from_environment()  # HFRK_PLAN_TABLE=<json>: tuned GEMM decompositions, if the deployment has a table

__all__ = ["increment", "residual_rms", "swiglu", "skinny_gemm", "skinny_gemm_scaled", "skinny_gemm_add",
           "skinny_gemm_swiglu", "skinny_gemm_rms", "residual_rms_dynamic", "swiglu_dynamic", "quantize_fp8"]
