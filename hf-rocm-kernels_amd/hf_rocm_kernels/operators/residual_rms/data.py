from typing import Optional, Tuple

import torch
from torch import Tensor


def generate_residual_rms_data(
    rows: int, cols: int, buffer_cols: int = 0, dtype: torch.dtype = torch.float16, seed: Optional[int] = None,
    device: str = "cuda", io_dtype: Optional[torch.dtype] = None, llama_weight: bool = False,
) -> Tuple[Tensor, Tensor, Tensor, float, Optional[Tensor], Optional[Tensor]]:
    """Random inputs with the reference's recipe (operators/residual_rms/reference.py:75-91): input, residual
    and weight ~ N(0,1), epsilon in [1e-5, 2e-5), a scale in [1, 3) when `dtype` is an fp8 dtype (else None) and
    an uninitialised (rows, buffer_cols) buffer (None when buffer_cols is 0).  `io_dtype` is the 16-bit dtype of
    the tensors (float16 unless given); `llama_weight` draws the weight ~ 1 + N(0, 0.1) instead.  Drawn on the
    CPU from a seeded generator, then moved to `device`."""
    gen = torch.Generator(device="cpu")
    if seed is not None:
        gen.manual_seed(seed)
    else:
        gen.seed()
    if io_dtype is None:
        io_dtype = dtype if dtype in (torch.float16, torch.bfloat16) else torch.float16
    input = torch.randn(size=(rows, cols), generator=gen, dtype=torch.float32).to(io_dtype)
    residual = torch.randn(size=(rows, cols), generator=gen, dtype=torch.float32).to(io_dtype)
    weights = torch.randn(size=(cols,), generator=gen, dtype=torch.float32)
    if llama_weight:
        weights = weights.mul(0.1).add(1.0)
    weights = weights.to(io_dtype)
    epsilon = torch.rand(size=(1,), generator=gen).add(1).mul(1e-5).item()
    if dtype in (torch.float8_e4m3fn, torch.float8_e4m3fnuz):
        scale_tensor = torch.rand(size=(1,), generator=gen, dtype=torch.float32).mul(2).add(1).to(device)
    else:
        scale_tensor = None
    next_buffer = None if buffer_cols == 0 else torch.full((rows, buffer_cols), 7.0, dtype=io_dtype).to(device)
    return input.to(device), residual.to(device), weights.to(device), epsilon, scale_tensor, next_buffer
