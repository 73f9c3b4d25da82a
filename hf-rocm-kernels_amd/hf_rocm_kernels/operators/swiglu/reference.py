"""Torch reference of the SwiGLU operator (counterpart of the reference package's operators/swiglu/reference.py:7-27),
for callers who want to check the kernel.  The operators never call it."""
from typing import Optional

import torch
from torch import Tensor

from hf_rocm_kernels.utils.fp8 import fp8_quantize


def reference_swiglu(gate_up_proj: Tensor, scale_tensor: Tensor, next_buffer: Optional[Tensor] = None) -> Tensor:
    """silu(gate) * up in fp32 (gate = first half of the columns, up = second half), divided by the scale and
    quantised to float8_e4m3fn."""
    cols = gate_up_proj.size(-1) // 2
    gate, up = gate_up_proj[..., :cols].float(), gate_up_proj[..., cols:].float()
    out, _ = fp8_quantize(torch.nn.functional.silu(gate) * up, scale_tensor)
    if next_buffer is not None:
        next_buffer.zero_()
    return out
