"""Oracle of the decoder MLP sub-block: the four reference functions chained in the order of
hf_rocm_kernels/combined_ops/llama_mlp.py:7-60.  Test infrastructure only (see __init__.py).

The reference has no test and no fixture for this chain (and its own function raises TypeError as written), so
beyond the parity of the four parts the wiring below is "parity unpinned"."""
from typing import Tuple

import torch

from .residual_rms import precise_residual_rms, reference_residual_rms
from .skinny_gemm import reference_skinny_gemm
from .swiglu import reference_swiglu


def reference_llama_mlp(attn_output: torch.Tensor, residual: torch.Tensor, rms_weight: torch.Tensor, rms_epsilon: float,
                        gate_up_weight: torch.Tensor, gate_up_input_scale: torch.Tensor,
                        gate_up_output_scale: torch.Tensor, down_weight: torch.Tensor, down_input_scale: torch.Tensor,
                        down_output_scale: torch.Tensor, add_residual: bool = False,
                        exact_norm: bool = False) -> Tuple[torch.Tensor, torch.Tensor]:
    """rms(attn_output + residual) -> fp8 -> gate_up GEMM -> swiglu -> fp8 -> down GEMM [-> + residual].
    `*_output_scale` is activation scale x weight scale, applied to the GEMM result as one factor.

    exact_norm=False normalises with the reference's torch function (16-bit roundings before the fp8 cast,
    operators/residual_rms/reference.py:20-27); exact_norm=True with float64 arithmetic on the 16-bit sum and a
    single rounding to fp8, which is what the reference's vectorised kernel approximates in fp32
    (csrc/op_src/residual_rms/residual_rms_vectorized.cu:124-135) and what the kernel here is held to."""
    one = torch.ones((), dtype=torch.float32)
    dtype = attn_output.dtype
    normalized, new_residual, _ = reference_residual_rms(attn_output, residual, rms_weight, rms_epsilon, gate_up_input_scale)
    if exact_norm:
        normalized, _ = precise_residual_rms(new_residual, torch.zeros_like(new_residual), rms_weight, rms_epsilon,
                                             gate_up_input_scale)
    gate_up = reference_skinny_gemm(normalized, gate_up_weight, gate_up_output_scale, one, out_dtype=dtype)
    act = reference_swiglu(gate_up, down_input_scale)
    base = new_residual if add_residual else None
    out = reference_skinny_gemm(act, down_weight, down_output_scale, one, output=base, out_dtype=dtype)
    return out, new_residual
