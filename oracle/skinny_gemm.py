"""Oracle of the FP8 skinny GEMM.  Test infrastructure only (see __init__.py).

The reference's own oracle is `torch._scaled_mm(a, b, scale_a, scale_b, out_dtype=float16)`
(hf_rocm_kernels/operators/skinny_gemm/reference.py:8-25, called from tests/test_skinny_gemm.py:16-17), i.e.
"dequantise, multiply-accumulate in fp32, scale, round to 16 bits" executed by hipBLASLt -- a dependency that is
not part of the reference tree (torch 2.5.1+rocm6.2 in its uv.lock) and that cannot run fnuz inputs on a CPU.
This file restates that arithmetic in plain torch on the CPU, with OCP e4m3fn operands.
"""
from typing import Optional

import numpy as np
import torch

from . import fp8


def reference_skinny_gemm(skinny_a: torch.Tensor, b: torch.Tensor, scale_a: torch.Tensor, scale_b: torch.Tensor,
                          output: Optional[torch.Tensor] = None, out_dtype: torch.dtype = torch.bfloat16) -> torch.Tensor:
    """out = output + ((A_fp8 * scale_a) @ (B_fp8 * scale_b)) in fp32, rounded once to `out_dtype`.

    skinny_a [m,k] fp8, b [k,n] fp8 (a transposed [n,k] weight), scale_a scalar or [m] / [m,1], scale_b scalar or
    [n].  Same call shape as the reference function (reference.py:8-25); `output` plays the role of its
    pre-zeroed (or bias-holding) accumulator."""
    a32 = skinny_a.float() * scale_a.float().reshape(-1, 1)
    b32 = b.float() * scale_b.float().reshape(1, -1)
    acc = a32 @ b32
    if output is not None:
        acc = acc + output.float()
        out_dtype = output.dtype
    return acc.to(out_dtype)


def exact_skinny_gemm(skinny_a: torch.Tensor, b: torch.Tensor, scale_a: torch.Tensor, scale_b: torch.Tensor,
                      output: Optional[torch.Tensor] = None) -> torch.Tensor:
    """The same product with no rounding before the result: float64 [m,n].

    Every e4m3fn value is an integer multiple of 2^-9 below 2^18 * 2^-9, so products are multiples of 2^-18 below
    2^36 * 2^-18 and a sum of up to 2^15 of them stays below 2^51 * 2^-18: float64 accumulates it exactly in any
    order.  The scales are applied in float64 afterwards."""
    a64 = torch.from_numpy(fp8.decode(skinny_a)).reshape(skinny_a.shape)
    b64 = torch.from_numpy(fp8.decode(b.t().contiguous())).reshape(b.shape[1], b.shape[0]).t()
    assert skinny_a.shape[1] <= 2 ** 15
    acc = a64 @ b64
    acc = acc * scale_a.double().reshape(-1, 1) * scale_b.double().reshape(1, -1)
    if output is not None:
        acc = acc + output.double()
    return acc


def ulp16(ref: torch.Tensor, dtype: torch.dtype) -> torch.Tensor:
    """One unit in the last place of `dtype` (bfloat16 or float16) at |ref|, as float64."""
    mant, min_exp = (8, -126) if dtype == torch.bfloat16 else (11, -14)
    e = torch.floor(torch.log2(ref.double().abs().clamp_min(2.0 ** min_exp)))
    return torch.pow(2.0, e - (mant - 1))


def error_bound(skinny_a, b, scale_a, scale_b, dtype: torch.dtype, exact: torch.Tensor) -> torch.Tensor:
    """Largest |result - exact| an fp32-accumulating implementation with one final rounding may show:
    one ulp of the 16-bit result (its rounding, with room for a boundary flip) + 2^-16 * sum_k |a_k b_k| scaled
    (fp32 accumulation in any order over K <= 2^15 terms stays far below this; losing or misplacing a K chunk
    does not, its effect is of the order of the result)."""
    abs_a = skinny_a.float().abs().to(torch.float8_e4m3fn)
    abs_b = b.float().abs().to(torch.float8_e4m3fn)
    abs_sum = exact_skinny_gemm(abs_a, abs_b, scale_a.abs(), scale_b.abs())
    return ulp16(exact, dtype) + abs_sum * 2.0 ** -16


def int_dot_products(skinny_a: torch.Tensor, b: torch.Tensor) -> np.ndarray:
    """sum_k A[i,k]*B[k,j] as exact integers in units of 2^-18 (int64 [m,n]); slow, for small shapes."""
    ai = np.rint(fp8.decode(skinny_a) * 512.0).astype(np.int64)
    bi = np.rint(fp8.decode(b.t().contiguous()) * 512.0).astype(np.int64)  # [n,k]
    return ai @ bi.T


def generate_skinny_gemm_data(m: int, n: int, k: int, seed: Optional[int] = None, out_dtype=torch.bfloat16):
    """CPU twin of the package's generator (same seeded draws, same recipe as reference.py:28-46):
    returns (skinny_a, b, scale_tensor, zero output)."""
    gen = torch.Generator(device="cpu")
    if seed is not None:
        gen.manual_seed(seed)
    scale_tensor = torch.rand(size=(1,), generator=gen, dtype=torch.float32).mul(2).add(1)
    skinny_a = fp8.fp8_quantize(torch.randn(size=(m, k), generator=gen, dtype=torch.float32), scale_tensor)[0]
    b = fp8.fp8_quantize(torch.randn(size=(n, k), generator=gen, dtype=torch.float32), scale_tensor)[0].t()
    return skinny_a, b, scale_tensor, torch.zeros(size=(m, n), dtype=out_dtype)
