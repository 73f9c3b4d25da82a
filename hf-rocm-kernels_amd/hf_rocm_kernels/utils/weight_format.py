"""Weight load format for the skinny GEMM: pack once when a model is loaded, stream contiguously per token.

No counterpart in the reference, whose kernel reads the row-major weight through an LDS ring
(csrc/op_src/skinny_gemm/producers/n_full_tiles.cu:4-127) and whose fp8 tensors are e4m3fn bits viewed as
e4m3fnuz with a doubled scale (hf_rocm_kernels/utils/fp8.py:17-29).  Here:

  pack_weight(weight)        [n, k] float8_e4m3fn (or float8_e4m3fnuz, re-encoded on the way) -> PackedWeight
  pack_weight(weight, scales) the same with the n per-output-channel scales behind the bytes: one allocation per layer
  unpack_weight(packed)      back to a row-major [n, k] float8_e4m3fn tensor
  reencode_fnuz(tensor)      float8_e4m3fnuz -> float8_e4m3fn with the same values (scales unchanged)
  fnuz_bits_as_ocp(q, scale) zero-copy alternative for tensors written by the reference's fp8_quantize

A PackedWeight goes wherever the GEMM wrappers take `b`: skinny_gemm, skinny_gemm_scaled, skinny_gemm_add,
skinny_gemm_swiglu and llama_mlp_combined_ops.  Results are bit-identical to the row-major weight's.
"""
from typing import Optional, Tuple

import torch
from torch import Tensor

import hf_rocm_kernels._HFRK_C  # noqa: F401  (registers torch.ops._HFRK_C)

from .. import _capi
from .fp8 import FP8_DTYPE

_BYTE_DTYPES = (torch.uint8, torch.float8_e4m3fn, torch.float8_e4m3fnuz)


class PackedWeight:
    """A [n, k] fp8 weight in the packed load format (16-row x 256-byte chunks in matrix-core operand order).

    Quacks like the `[k, n]` column-major view the GEMM wrappers expect (`shape`, `size`, `stride`, `dtype`,
    `device`), so their argument checks apply unchanged; `data` is the flat float8_e4m3fn buffer.  A buffer made
    with scales is longer by 4 bytes per padded row; `scales` is then the float32 view of its n per-channel scales:
    pass it as `scale_b` (`skinny_gemm_scaled` and the linear layer do so when given none).  In every other wrapper an
    omitted `scale_b` means 1, as for a row-major weight, so that one call gives one result in both layouts."""

    def __init__(self, data: Tensor, n: int, k: int):
        assert data.dim() == 1 and data.is_contiguous() and data.dtype == FP8_DTYPE, "data must be a flat float8_e4m3fn tensor"
        plain = packed_weight_bytes(n, k)
        assert data.numel() in (plain, packed_weight_bytes(n, k, scaled=True)), f"{data.numel()} bytes do not hold a packed [{n}, {k}] weight"
        self.data, self.n, self.k = data, int(n), int(k)
        self.scales: Optional[Tensor] = None if data.numel() == plain else data[plain:].view(torch.float32)[:n]

    @property
    def shape(self) -> Tuple[int, int]:
        return (self.k, self.n)

    def size(self, dim=None):
        return self.shape if dim is None else self.shape[dim]

    def dim(self) -> int:
        return 2

    def stride(self, dim=None):
        strides = (1, self.k)
        return strides if dim is None else strides[dim]

    @property
    def dtype(self) -> torch.dtype:
        return self.data.dtype

    @property
    def device(self) -> torch.device:
        return self.data.device

    def __repr__(self) -> str:
        return f"PackedWeight(n={self.n}, k={self.k}, device={self.device})"


def packed_weight_bytes(n: int, k: int, scaled: bool = False) -> int:
    """Size of the packed buffer of a [n, k] weight: rows padded to a multiple of 16 (k must be a multiple of 256);
    scaled: with one float32 scale per padded row behind the bytes."""
    lib = _capi.load()
    size = lib.hfrk_packed_weight_bytes_scaled(int(n), int(k)) if scaled else lib.hfrk_packed_weight_bytes(int(n), int(k))
    if size == 0:
        raise ValueError(f"a [{n}, {k}] weight cannot be packed: sizes must be positive and k a multiple of 256")
    return size


def pack_weight(weight: Tensor, scales: Optional[Tensor] = None) -> PackedWeight:
    """Pack a row-major [n, k] weight (an nn.Linear weight; rows may be strided, k contiguous).
    float8_e4m3fnuz input is re-encoded to float8_e4m3fn values on the way (see reencode_fnuz); uint8 is taken as
    float8_e4m3fn bits.  scales: the weight's n float32 per-output-channel scales, stored behind the packed bytes."""
    assert weight.dim() == 2 and weight.stride(1) == 1, f"Expected a [n, k] weight with unit stride along k but got {weight.stride() = }"
    assert weight.dtype in _BYTE_DTYPES, f"Expected a one-byte dtype but got {weight.dtype = }"
    assert weight.device.type == "cuda", f"Expected a device tensor but got {weight.device = }"
    n, k = weight.shape
    data = torch.empty(packed_weight_bytes(n, k, scaled=scales is not None), dtype=FP8_DTYPE, device=weight.device)
    src_format = _capi.WEIGHT_E4M3FNUZ if weight.dtype == torch.float8_e4m3fnuz else _capi.WEIGHT_E4M3FN
    if scales is None:
        torch.ops._HFRK_C.pack_weight(weight, data, src_format)
    else:
        assert scales.dtype == torch.float32 and scales.numel() == n, f"Expected {n} float32 scales but got {scales.shape = }, {scales.dtype = }"
        torch.ops._HFRK_C.pack_weight_scaled(weight, scales.reshape(-1).contiguous(), data, src_format)
    return PackedWeight(data, n, k)


def unpack_weight(packed: PackedWeight) -> Tensor:
    """The row-major [n, k] float8_e4m3fn weight a PackedWeight was made from (use `.t()` for the GEMM's view)."""
    out = torch.empty((packed.n, packed.k), dtype=FP8_DTYPE, device=packed.device)
    torch.ops._HFRK_C.unpack_weight(packed.data, out)
    return out


def reencode_fnuz(tensor: Tensor) -> Tensor:
    """float8_e4m3fnuz -> float8_e4m3fn, same values, same shape; scales stay as they are.
    Exact except for magnitudes below 2^-6, which round (to nearest even) onto fn's subnormal grid of 2^-9; the
    fnuz NaN becomes the fn NaN."""
    assert tensor.dtype == torch.float8_e4m3fnuz, f"Expected {tensor.dtype = } to be torch.float8_e4m3fnuz"
    assert tensor.device.type == "cuda", f"Expected a device tensor but got {tensor.device = }"
    src = tensor.contiguous()
    out = torch.empty(src.shape, dtype=FP8_DTYPE, device=src.device)
    torch.ops._HFRK_C.reencode_fnuz(src, out)
    return out


def fnuz_bits_as_ocp(quantized: Tensor, scale: Tensor) -> Tuple[Tensor, Tensor]:
    """Zero-copy conversion of what the reference's fp8_quantize returns (utils/fp8.py:17-29: fn bits labelled fnuz,
    -0 cleared, scale doubled): the same bits read as float8_e4m3fn are twice the fnuz value, so the scale is
    halved.  Only valid when no element is fnuz NaN (0x80) or +-240 (0x7f / 0xff, NaN as fn) -- true for every
    tensor that function writes; checked here (one device reduction and a host read)."""
    assert quantized.dtype == torch.float8_e4m3fnuz, f"Expected {quantized.dtype = } to be torch.float8_e4m3fnuz"
    bits = quantized.view(torch.uint8)
    bad = ((bits == 0x80) | ((bits & 0x7F) == 0x7F)).any()
    if bool(bad):
        raise ValueError("the tensor holds fnuz NaN or +-240, which have no float8_e4m3fn code on the same bits: use reencode_fnuz")
    return quantized.view(FP8_DTYPE), scale * 0.5
