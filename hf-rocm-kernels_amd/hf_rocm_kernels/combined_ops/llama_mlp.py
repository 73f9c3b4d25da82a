from typing import Optional, Tuple

import torch
from torch import Tensor

from hf_rocm_kernels import residual_rms, skinny_gemm, skinny_gemm_add, skinny_gemm_rms, skinny_gemm_scaled, skinny_gemm_swiglu, swiglu


def llama_mlp_combined_ops(
    attn_output: Tensor,
    residual: Tensor,
    rms_weight: Tensor,
    rms_epsilon: float,
    gate_up_weight: Tensor,
    gate_up_input_scale: Tensor,
    gate_up_output_scale: Tensor,
    down_weight: Tensor,
    down_input_scale: Tensor,
    down_output_scale: Tensor,
    gate_up_gemm_hp: Tuple[Optional[int], Optional[int]] = (None, None),
    down_gemm_hp: Tuple[Optional[int], Optional[int]] = (None, None),
    add_residual: bool = False,
    fused: bool = False,
    rms_prologue: bool = False,
) -> Tuple[Tensor, Tensor]:
    """Decoder MLP sub-block as four launches on one stream (reference: combined_ops/llama_mlp.py:7-60):
    residual RMSNorm -> fp8, gate_up GEMM, SwiGLU -> fp8, down GEMM.

    - attn_output, residual: (m, hidden) 16-bit; residual <- attn_output + residual in place
    - gate_up_weight: (hidden, 2*inter) fp8, col-major; down_weight: (inter, hidden) fp8, col-major
    - *_input_scale: the activation quantisation scale of each GEMM; *_output_scale: activation scale x weight scale
    - gate_up_gemm_hp / down_gemm_hp: accepted for signature compatibility; the library plans each GEMM itself
      (the reference forwards them as split_k / b_lanes keywords its skinny_gemm does not take)
    - add_residual: the down projection accumulates onto a copy of the updated residual instead of zeros, so
      the first output is the block's output hidden state (residual + mlp) rounded once

    - fused: three launches instead of four (plus a copy): the SwiGLU runs as the epilogue of the gate_up GEMM,
      nothing is zeroed beforehand (the GEMMs overwrite), and with add_residual the down projection reads the
      residual as its addend instead of accumulating onto a copy.  Same arithmetic, same roundings.

    - rms_prologue (with fused): two launches where the library has the prologue (up to 8 rows, hidden 4096 or 8192,
      row-major gate_up weight): the RMSNorm runs inside the gate_up GEMM, in every workgroup.  Same bits as the three
      launches, but the summed residual is returned as a new tensor and `residual` is left as it was (every workgroup of
      the fused launch reads the old residual, so it cannot be updated in place).

    RMSNorm and SwiGLU zero the buffer the following GEMM accumulates into, as in the reference.
    Returns (mlp_output, residual)."""
    del gate_up_gemm_hp, down_gemm_hp
    if fused and rms_prologue:
        swiglu_out, residual = skinny_gemm_rms(attn_output, residual, rms_weight, rms_epsilon, gate_up_input_scale, gate_up_weight,
                                               gate_up_output_scale, None, None, out_scale=down_input_scale)
        if add_residual:
            mlp_output = skinny_gemm_add(swiglu_out, down_weight, down_output_scale, None, base=residual)
        else:
            mlp_output = torch.empty(size=(attn_output.size(0), down_weight.size(1)), dtype=attn_output.dtype,
                                     device=attn_output.device)
            skinny_gemm_scaled(swiglu_out, down_weight, down_output_scale,
                               torch.ones(1, device=attn_output.device), output=mlp_output)
        return mlp_output, residual
    if fused:
        normalized, residual = residual_rms(input=attn_output, residual=residual, weight=rms_weight, epsilon=rms_epsilon,
                                            scale_tensor=gate_up_input_scale)
        swiglu_out = skinny_gemm_swiglu(normalized, gate_up_weight, gate_up_output_scale, None, down_input_scale,
                                        intermediate_dtype=attn_output.dtype)
        if add_residual:
            mlp_output = skinny_gemm_add(swiglu_out, down_weight, down_output_scale, None, base=residual)
        else:
            mlp_output = torch.empty(size=(attn_output.size(0), down_weight.size(1)), dtype=attn_output.dtype,
                                     device=attn_output.device)
            skinny_gemm_scaled(swiglu_out, down_weight, down_output_scale,
                               torch.ones(1, device=attn_output.device), output=mlp_output)
        return mlp_output, residual
    m = attn_output.size(0)
    dtype = attn_output.dtype

    # RMS norm (zeroes the gate_up GEMM's accumulator)
    gate_up_proj = torch.empty(size=(m, gate_up_weight.size(1)), dtype=dtype, device=attn_output.device)
    normalized, residual = residual_rms(
        input=attn_output,
        residual=residual,
        weight=rms_weight,
        epsilon=rms_epsilon,
        scale_tensor=gate_up_input_scale,
        next_buffer=gate_up_proj,
    )

    # Gate + up projection
    skinny_gemm(skinny_a=normalized, b=gate_up_weight, scale_tensor=gate_up_output_scale, output=gate_up_proj)

    # Swiglu (zeroes the down GEMM's accumulator unless it starts from the residual)
    if add_residual:
        mlp_output = residual.clone()
        swiglu_out = swiglu(gate_up_proj=gate_up_proj, scale_tensor=down_input_scale)
    else:
        mlp_output = torch.empty(size=(m, down_weight.size(1)), dtype=dtype, device=attn_output.device)
        swiglu_out = swiglu(gate_up_proj=gate_up_proj, scale_tensor=down_input_scale, next_buffer=mlp_output)

    # Down projection
    skinny_gemm(skinny_a=swiglu_out, b=down_weight, scale_tensor=down_output_scale, output=mlp_output)
    return mlp_output, residual


class LlamaMlpGraph:
    """The decoder MLP sub-block captured once into a HIP graph: one host call per token step instead of three or four
    operator launches (the reference times its kernels inside graphs, operators/skinny_gemm/benchmarking_fn.py:62-92,
    but ships no captured block).

    The graph reads `attn_output` and `residual` from buffers owned by this object: write the step's inputs with
    `copy_` (or pass them to `__call__`, which does) and read the results from `mlp_output` / `residual`, which are
    overwritten by every replay.  Weights and scales are the tensors given here; replace their contents in place if
    they change.  Capturing needs the library's workspace to exist, so one eager run happens first."""

    def __init__(self, rows: int, hidden: int, rms_weight: Tensor, rms_epsilon: float, gate_up_weight, gate_up_input_scale: Tensor,
                 gate_up_output_scale: Tensor, down_weight, down_input_scale: Tensor, down_output_scale: Tensor,
                 dtype: torch.dtype = torch.bfloat16, add_residual: bool = True, fused: bool = True):
        device = rms_weight.device
        self.attn_output = torch.zeros((rows, hidden), dtype=dtype, device=device)
        self.residual = torch.zeros((rows, hidden), dtype=dtype, device=device)
        args = (rms_weight, rms_epsilon, gate_up_weight, gate_up_input_scale, gate_up_output_scale, down_weight,
                down_input_scale, down_output_scale)
        kwargs = dict(add_residual=add_residual, fused=fused)
        self._stream = torch.cuda.Stream(device)
        with torch.cuda.stream(self._stream):
            llama_mlp_combined_ops(self.attn_output, self.residual, *args, **kwargs)  # eager: workspace, code objects
            self.residual.zero_()
            torch.cuda.synchronize(device)
            self.graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(self.graph, stream=self._stream):
                self.mlp_output, residual_out = llama_mlp_combined_ops(self.attn_output, self.residual, *args, **kwargs)
        assert residual_out.data_ptr() == self.residual.data_ptr()  # updated in place
        torch.cuda.synchronize(device)

    def __call__(self, attn_output: Tensor, residual: Tensor) -> Tuple[Tensor, Tensor]:
        """Copy the inputs in, replay, return (mlp_output, residual) -- views of this object's buffers."""
        self.attn_output.copy_(attn_output)
        self.residual.copy_(residual)
        self.graph.replay()
        return self.mlp_output, self.residual
