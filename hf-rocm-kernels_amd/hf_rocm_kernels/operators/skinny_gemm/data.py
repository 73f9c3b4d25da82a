from typing import Optional, Tuple

import torch
from torch import Tensor

from hf_rocm_kernels.utils.fp8 import amax_scale, fp8_quantize


def _generator(seed: Optional[int]) -> torch.Generator:
    gen = torch.Generator(device="cpu")
    if seed is not None:
        gen.manual_seed(seed)
    else:
        gen.seed()
    return gen


def generate_skinny_gemm_data(
    m: int, n: int, k: int, seed: Optional[int] = None, device: str = "cuda", out_dtype: torch.dtype = torch.bfloat16,
) -> Tuple[Tensor, Tensor, Tensor, Tensor]:
    """Random inputs with the reference's recipe (operators/skinny_gemm/reference.py:28-46): one scale in [1, 3),
    A ~ N(0,1) of shape (m, k) and B ~ N(0,1) of shape (n, k), both divided by the scale and quantised, B
    returned transposed, plus a zeroed (m, n) output.  Drawn on the CPU from a seeded generator, so the same
    seed gives the same bits on any device."""
    gen = _generator(seed)
    scale_tensor = torch.rand(size=(1,), generator=gen, dtype=torch.float32).mul(2).add(1)
    skinny_a = fp8_quantize(torch.randn(size=(m, k), generator=gen, dtype=torch.float32), scale_tensor)[0]
    b = fp8_quantize(torch.randn(size=(n, k), generator=gen, dtype=torch.float32), scale_tensor)[0]
    output = torch.zeros(size=(m, n), dtype=out_dtype)
    return skinny_a.to(device), b.to(device).t(), scale_tensor.to(device), output.to(device)


def generate_llama_gemm_data(
    m: int, n: int, k: int, seed: Optional[int] = None, device: str = "cuda", per_token: bool = False,
    per_channel: bool = False, outlier_rows: Tuple[int, ...] = (), weight_std: float = 0.02,
) -> Tuple[Tensor, Tensor, Tensor, Tensor]:
    """Decode-time linear-layer inputs: activations ~ N(0,1) rounded to bfloat16, weights ~ N(0, weight_std),
    each quantised to float8_e4m3fn with scale = amax/448 -- one scale per tensor, or per activation row
    (`per_token`) / per output channel (`per_channel`).  Rows listed in `outlier_rows` are multiplied by 20
    before quantisation.  Returns (A_fp8 [m,k], W_fp8.t() [k,n], scale_a [1 or m], scale_w [1 or n])."""
    gen = _generator(seed)
    a = torch.randn(size=(m, k), generator=gen, dtype=torch.float32).to(torch.bfloat16).float()
    for r in outlier_rows:
        a[r] *= 20.0
    w = torch.randn(size=(n, k), generator=gen, dtype=torch.float32).mul(weight_std)
    scale_a = amax_scale(a, dim=1 if per_token else None)
    scale_w = amax_scale(w, dim=1 if per_channel else None)
    a_q = fp8_quantize(a, scale_a)[0]
    w_q = fp8_quantize(w, scale_w)[0]
    return a_q.to(device), w_q.to(device).t(), scale_a.reshape(-1).to(device), scale_w.reshape(-1).to(device)
