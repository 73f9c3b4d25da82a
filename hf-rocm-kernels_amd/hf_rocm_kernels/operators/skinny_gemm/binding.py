import torch
from torch import Tensor

import hf_rocm_kernels._HFRK_C  # noqa: F401  (registers torch.ops._HFRK_C)


def _skinny_gemm(
    A: Tensor,
    B: Tensor,
    scale_tensor: Tensor,
    D: Tensor,
    split_k: int,
    A_producers: int,
    B_producers: int,
    consumers: int,
    a_lanes: int,
    b_lanes: int,
    qsize: int,
    op_m: int,
    ops: int,
) -> int:
    """Same argument order as the reference's binding (operators/skinny_gemm/binding.py:7-28)."""
    return torch.ops._HFRK_C.skinny_gemm_tb(
        A, B, D, scale_tensor,
        split_k,
        A_producers, B_producers, consumers,
        a_lanes, b_lanes, qsize,
        op_m, ops,
    )


def _skinny_gemm_scaled(A: Tensor, B: Tensor, D: Tensor, scale_a: Tensor, scale_b: Tensor, accumulate: bool) -> int:
    return torch.ops._HFRK_C.skinny_gemm_scaled(A, B, D, scale_a, scale_b, accumulate)


def _skinny_gemm_fused(A: Tensor, B: Tensor, D: Tensor, base, scale_a: Tensor, scale_b: Tensor, out_scale, epilogue: int,
                       intermediate_dtype: int) -> int:
    return torch.ops._HFRK_C.skinny_gemm_fused(A, B, D, base, scale_a, scale_b, out_scale, epilogue, intermediate_dtype)


def _skinny_gemm_packed(A: Tensor, B_packed: Tensor, n: int, D: Tensor, base, scale_a: Tensor, scale_b, out_scale, epilogue: int,
                        intermediate_dtype: int) -> int:
    return torch.ops._HFRK_C.skinny_gemm_packed(A, B_packed, n, D, base, scale_a, scale_b, out_scale, epilogue, intermediate_dtype)


def _skinny_gemm_checked(A: Tensor, B: Tensor, packed: bool, n: int, D: Tensor, base, scale_a: Tensor, scale_b, out_scale,
                         epilogue: int, intermediate_dtype: int) -> None:
    """The fused GEMM as an operator that raises instead of returning its status (traceable: it returns nothing)."""
    torch.ops._HFRK_C.skinny_gemm_checked(A, B, packed, n, D, base, scale_a, scale_b, out_scale, epilogue, intermediate_dtype)
