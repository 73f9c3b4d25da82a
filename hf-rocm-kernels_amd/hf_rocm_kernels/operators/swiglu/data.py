from typing import Optional, Tuple

import torch
from torch import Tensor


def generate_swiglu_data(
    rows: int, hidden_dim: int, buffer_cols: int = 0, seed: Optional[int] = None, device: str = "cuda",
    io_dtype: torch.dtype = torch.float16,
) -> Tuple[Tensor, Tensor, Optional[Tensor]]:
    """Random inputs with the reference's recipe (operators/swiglu/reference.py:30-41): gate_up ~ N(0,1) of shape
    (rows, 2*hidden_dim), a scale in [1, 3) and a (rows, buffer_cols) buffer filled with a non-zero value (None
    when buffer_cols is 0).  Drawn on the CPU from a seeded generator, then moved to `device`."""
    gen = torch.Generator(device="cpu")
    if seed is not None:
        gen.manual_seed(seed)
    else:
        gen.seed()
    gate_up_proj = torch.randn(size=(rows, 2 * hidden_dim), generator=gen, dtype=torch.float32).to(io_dtype)
    scale_tensor = torch.rand(size=(1,), generator=gen, dtype=torch.float32).mul(2).add(1)
    next_buffer = None if buffer_cols == 0 else torch.full((rows, buffer_cols), 7.0, dtype=io_dtype).to(device)
    return gate_up_proj.to(device), scale_tensor.to(device), next_buffer
