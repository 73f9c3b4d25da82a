"""Oracle of the SwiGLU op.  Test infrastructure only (see __init__.py)."""
from typing import Optional, Tuple

import torch

from . import fp8


def reference_swiglu(gate_up_proj: torch.Tensor, scale_tensor: torch.Tensor,
                     next_buffer: Optional[torch.Tensor] = None) -> torch.Tensor:
    """silu(gate) * up in fp32, then fp8_quantize (hf_rocm_kernels/operators/swiglu/reference.py:7-27):
    gate = columns [0, n), up = columns [n, 2n) of each row.  float16 or bfloat16 input."""
    assert gate_up_proj.dtype in (torch.float16, torch.bfloat16)
    gu = gate_up_proj.view(-1, 2, gate_up_proj.size(1) // 2).float()
    out = torch.nn.functional.silu(gu[:, 0]) * gu[:, 1]
    q, _ = fp8.fp8_quantize(out, scale_tensor)
    if next_buffer is not None:
        next_buffer.fill_(0)
    return q


def swiglu_fp32(gate_up_proj: torch.Tensor) -> torch.Tensor:
    """The unquantised fp32 value silu(gate) * up, for tolerance checks in real units."""
    gu = gate_up_proj.view(-1, 2, gate_up_proj.size(1) // 2).float()
    return torch.nn.functional.silu(gu[:, 0]) * gu[:, 1]


def precise_swiglu_dynamic(gate_up_proj: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """silu(gate) * up in float64, per-row scale amax/448 (float32), e4m3fn(y / scale).  No reference counterpart
    (operators/swiglu/reference.py:7-27 divides by one static scale).  Returns (output fp8, scales [rows], y)."""
    gu = gate_up_proj.view(-1, 2, gate_up_proj.size(1) // 2).to(torch.float64)
    y = torch.nn.functional.silu(gu[:, 0]) * gu[:, 1]
    scales = fp8.amax_scale(y, dim=1)
    out, _ = fp8.fp8_quantize(y, scales)
    return out, scales.reshape(-1), y
