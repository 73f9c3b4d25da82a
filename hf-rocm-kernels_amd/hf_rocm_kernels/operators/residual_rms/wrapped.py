from typing import Optional, Tuple

import torch
from torch import Tensor

from .binding import _residual_rms

_IO_DTYPES = (torch.bfloat16, torch.float16)


def residual_rms_checks(
    input: Tensor,
    residual: Tensor,
    weight: Tensor,
    scale_tensor: Optional[Tensor],
    epsilon: float,
    next_buffer: Tensor,
) -> None:
    """Same assertions as the reference (operators/residual_rms/wrapped.py:11-36) plus the dtype checks the
    reference leaves to its kernel."""
    # Check shapes
    assert input.dim() == 2, f"Expected input to have 2 dimensions but got {input.dim() = } instead."
    assert residual.shape == input.shape, \
        f"Expected input and residual to have same shape but got {input.shape = } and {residual.shape = }"
    assert weight.shape == (input.size(1), ), \
        f"Expected weight to have shape {(input.size(1), ) = } but got {weight.shape = }"
    # Check dtypes
    assert input.dtype in _IO_DTYPES, f"Expected {input.dtype = } to be torch.bfloat16 or torch.float16"
    assert residual.dtype == input.dtype, f"Expected {residual.dtype = } to be {input.dtype}"
    assert weight.dtype == input.dtype, f"Expected {weight.dtype = } to be {input.dtype}"
    # Check devices
    device = input.device
    assert device.type == "cuda", f"Expected input.device to be of type cuda, but got {device.type = } instead."
    assert residual.device == device, f"Expected {residual.device = } to be the same as {input.device = }"
    assert weight.device == device, f"Expected {weight.device = } to be the same as {input.device = }"
    if scale_tensor is not None:
        assert scale_tensor.device == device, f"Expected {scale_tensor.device = } to be the same as {input.device = }"
        assert scale_tensor.numel() == 1, f"Expected {scale_tensor.numel() = } to be 1."
    assert next_buffer.device == device, f"Expected {next_buffer.device = } to be the same as {input.device = }"
    # Check layouts
    assert input.is_contiguous(), f"Expected input to be contiguous but got {input.stride() = }"
    assert residual.is_contiguous(), f"Expected residual to be contiguous but got {residual.stride() = }"
    # Check scalars
    assert epsilon > 0, f"Expected RMS epsilon to be > 0 to avoid division by zero, but got {epsilon = }"


def infer_num_threads(rows: int, num_threads: int) -> int:
    """0 lets the launcher size the workgroup from the row length (one or two 16-byte pieces per thread); an
    explicit value is rounded up to whole 64-lane wavefronts.  The reference instead interpolates a table of
    thread counts by number of rows (wrapped.py:59-75); its error case is kept."""
    if num_threads < 0 or num_threads > 1024:
        raise ValueError(f"{num_threads = } is not between 0 and 1024")
    return ((num_threads + 63) // 64) * 64


def residual_rms(
    input: Tensor,
    residual: Tensor,
    weight: Tensor,
    epsilon: float,
    scale_tensor: Optional[Tensor] = None,
    next_buffer: Optional[Tensor] = None,
    num_threads: int = 0,
    force_scalar: bool = False,
) -> Tuple[Tensor, Tensor]:
    """Fused residual connection, RMS normalisation and conversion to fp8.  The residual argument is modified
    inplace (residual <- input + residual).
    Args (reference: operators/residual_rms/wrapped.py:77-124):
        - input, residual: 16-bit (bfloat16 or float16) tensors of shape (rows, cols) in row-major format
        - weight: a tensor of shape (cols, ) of the same dtype, the weight of the RMS norm
        - epsilon: the small epsilon used inside the RMS norm to avoid division by zero
        - scale_tensor: a fp32 one-item tensor to divide the output of the RMS norm by before conversion to
            float8_e4m3fn.  If None, the output keeps the input dtype
        - next_buffer: an optional 16-bit tensor of shape (rows, .) to set to zero
        - num_threads: threads per row; 0 lets the launcher choose
    Outputs:
        - the normalised tensor of shape (rows, cols), float8_e4m3fn or the input dtype
        - the residual modified in place
    """
    if next_buffer is None:
        next_buffer = torch.empty(size=(input.size(0), 0), device=input.device, dtype=input.dtype)
    residual_rms_checks(input, residual, weight, scale_tensor, epsilon, next_buffer)
    num_threads = infer_num_threads(input.size(0), num_threads)

    if scale_tensor is not None:
        output = torch.empty(size=input.shape, dtype=torch.float8_e4m3fn, device=input.device)
    else:
        output = torch.empty(size=input.shape, dtype=input.dtype, device=input.device)
        scale_tensor = torch.empty(size=(0,), dtype=torch.float32, device=input.device)  # schema wants a Tensor
    _residual_rms(
        input=input,
        residual=residual,
        weight=weight,
        scale_tensor=scale_tensor,
        epsilon=epsilon,
        output=output,
        next_buffer=next_buffer,
        num_threads=num_threads,
        force_scalar=force_scalar,
    )
    return output, residual


def residual_rms_dynamic(
    input: Tensor,
    residual: Tensor,
    weight: Tensor,
    epsilon: float,
    next_buffer: Optional[Tensor] = None,
) -> Tuple[Tensor, Tensor, Tensor]:
    """residual <- input + residual, RMS normalisation, and per-row dynamic quantisation to float8_e4m3fn: every row
    gets its own scale amax/448, so no activation scale has to be known in advance.
    Returns (output fp8 (rows, cols), residual, scales fp32 (rows,)); `scales` is the GEMM's per-token `scale_a`.
    Rows must be 16-byte aligned (cols % 8 == 0) and at most 32768 wide."""
    if next_buffer is None:
        next_buffer = torch.empty(size=(input.size(0), 0), device=input.device, dtype=input.dtype)
    residual_rms_checks(input, residual, weight, None, epsilon, next_buffer)
    assert input.size(1) % 8 == 0 and input.size(1) <= 32768, f"Expected cols % 8 == 0 and cols <= 32768: {input.shape = }"
    output = torch.empty(size=input.shape, dtype=torch.float8_e4m3fn, device=input.device)
    scales = torch.empty(size=(input.size(0),), dtype=torch.float32, device=input.device)
    torch.ops._HFRK_C.residual_rms_dynamic(input, residual, weight, epsilon, output, scales, next_buffer)
    return output, residual, scales
