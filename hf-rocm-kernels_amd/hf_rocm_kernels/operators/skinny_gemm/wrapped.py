from typing import Dict, Optional, Tuple

import torch
from torch import Tensor

from ... import _capi
from ...utils.weight_format import PackedWeight
from .binding import _skinny_gemm, _skinny_gemm_checked, _skinny_gemm_fused, _skinny_gemm_packed, _skinny_gemm_scaled

_OUT_DTYPES = (torch.bfloat16, torch.float16)


def skinny_gemm_checks(
    skinny_a: Tensor,
    b: Tensor,
    scale_tensor: Tensor,
    output: Tensor,
) -> None:
    """Same assertions as the reference (operators/skinny_gemm/wrapped.py:9-35), with the dtypes of this build:
    float8_e4m3fn operands (gfx950 is OCP fp8, not fnuz) and a bfloat16 or float16 output."""
    # Check shapes
    assert skinny_a.dim() == 2, f"Expected skinny_a to have 2 dimensions but got {skinny_a.dim() = } instead."
    assert skinny_a.size(1) == b.size(0), f"Expected {skinny_a.size(1) = } and {b.size(0) = } to be the same."
    assert scale_tensor.numel() == 1, f"Expected {scale_tensor.numel() = } to be 1."
    assert output.shape == (skinny_a.size(0), b.size(1)), (
        f"{output.shape} does not match with {skinny_a.shape = } and {b.shape =}")
    # Check layouts
    assert skinny_a.is_contiguous(), f"Expected skinny_a to be contiguous but got {skinny_a.stride() = }"
    assert b.stride(0) == 1, f"Expected b to be column-major but got {b.stride() = }"
    assert output.is_contiguous(), f"Expected output to be contiguous but got {output.stride() = }"
    # Check dtypes
    assert skinny_a.dtype == torch.float8_e4m3fn, f"Expected {skinny_a.dtype = } to be torch.float8_e4m3fn"
    assert b.dtype == torch.float8_e4m3fn, f"Expected {b.dtype = } to be torch.float8_e4m3fn"
    assert scale_tensor.dtype == torch.float32, f"Expected {scale_tensor.dtype = } to be torch.float32"
    assert output.dtype in _OUT_DTYPES, f"Expected {output.dtype = } to be torch.bfloat16 or torch.float16"
    # Check devices
    device = skinny_a.device
    assert device.type == "cuda", f"Expected input.device to be of type cuda, but got {device.type = } instead."
    assert b.device == device, f"Expected {b.device = } to be the same as {device = }"
    assert scale_tensor.device == device, f"Expected {scale_tensor.device = } to be the same as {device = }"
    assert output.device == device, f"Expected {output.device = } to be the same as {device = }"


def infer_skinny_gemm_m_params(m: int) -> Tuple[int, int]:
    """(a_lanes, op_m) exactly as the reference derives them from m (wrapped.py:37-40)."""
    a_lanes = 2 if m > 16 else 1
    op_m = 16 if m > 8 else 8
    return a_lanes, op_m


@torch.compiler.assume_constant_result
def _planned_k_slabs(m: int, n: int, k: int) -> int:
    """K slabs per row panel in the library's plan for the shape: a host-only call into the C library, a constant
    of the shape to a tracer (which cannot follow a ctypes call)."""
    if k % 256 and m > 32:  # no single plan: the library runs two launches of up to 32 rows
        return (k + 255) // 256
    return int(_capi.plan(m, n, k).slabs)


def infer_skinny_gemm_params(skinny_a: Tensor, b: Tensor) -> Dict[str, int]:
    """The nine integers of the op schema.

    The reference looks them up in a table tuned for four shapes on 304 CUs (wrapped.py:42-102).  Here the
    decomposition is chosen by the library's planner (`hfrk_skinny_gemm_plan`, one persistent workgroup per CU
    of 256, stream-K over (row panel, K slab) units); the integers only have to pass the launcher's validation,
    so they are the reference's defaults, with `split_k` reporting the planner's K slabs per panel."""
    m, k = skinny_a.shape
    n = b.shape[1]
    a_lanes, op_m = infer_skinny_gemm_m_params(m)
    ops = 4 if op_m == 8 else 8
    if k % 256 and k % 16 == 0:
        # a row that ends inside a 256-byte chunk: name the reference's narrowest tile that divides k, (512/op_m)*ops =
        # 128 or 64 (skinny_gemm_caller.cu:33-48), so that the launcher's validation passes where the reference's would
        op_m, ops = (16, 4) if k % 128 == 0 else (32, 4)
    b_lanes = min(4, max(1, n // (256 * 16)))
    qsize = 3
    return {"A_producers": 3, "B_producers": min(6, qsize * b_lanes), "consumers": 3,
            "a_lanes": a_lanes, "b_lanes": b_lanes,
            "qsize": qsize, "op_m": op_m, "ops": ops, "split_k": _planned_k_slabs(m, n, k)}


def _raise_on_status(status: int, what: str) -> None:
    if status != _capi.SUCCESS:
        raise RuntimeError(f"{what} rejected the call with status {status}: {_capi.status_string(status)}")


def _fused(skinny_a: Tensor, b, output: Tensor, base: Optional[Tensor], scale_a: Tensor, scale_b: Optional[Tensor],
           out_scale: Optional[Tensor], epilogue: int, intermediate_dtype: int) -> None:
    """One launch of the fused GEMM on a row-major view or a PackedWeight; raises on a non-zero status."""
    if torch.compiler.is_compiling():  # an operator that returns its status cannot stay inside a traced graph
        packed = isinstance(b, PackedWeight)
        _skinny_gemm_checked(skinny_a, b.data if packed else b, packed, b.n if packed else b.size(1), output, base, scale_a,
                             scale_b, out_scale, epilogue, intermediate_dtype)
    elif isinstance(b, PackedWeight):
        status = _skinny_gemm_packed(skinny_a, b.data, b.n, output, base, scale_a, scale_b, out_scale, epilogue, intermediate_dtype)
        _raise_on_status(status, "skinny_gemm_packed")
    else:
        status = _skinny_gemm_fused(skinny_a, b, output, base, scale_a, scale_b, out_scale, epilogue, intermediate_dtype)
        _raise_on_status(status, "skinny_gemm_fused")


def skinny_gemm(
    skinny_a: Tensor,
    b: Tensor,
    scale_tensor: Tensor,
    output: Optional[Tensor] = None,
) -> Tensor:
    """FP8 skinny GEMM: output += scale * skinny_a @ b, fp32 accumulation, one rounding.
    Args (reference: operators/skinny_gemm/wrapped.py:104-128):
        - skinny_a: a float8_e4m3fn tensor of shape (m, k) in row-major format, m <= 64
        - b: a float8_e4m3fn tensor of shape (k, n) in col-major format (an nn.Linear weight [n, k], transposed),
          or the PackedWeight made from that weight (utils/weight_format.py), here and in the variants below
        - scale_tensor: a fp32 one-item tensor, the product of the two quantisation scales
        - output: an optional (m, n) bfloat16/float16 tensor that is accumulated into: zero-initialised, or
          holding a bias or residual.  Allocated as float16 zeros when omitted, like the reference's (wrapped.py:119).
    Outputs:
        the (m, n) output tensor.
    Unlike the reference, a launcher status other than 0 raises instead of leaving the output untouched.
    """
    if output is None:
        output = torch.zeros(size=(skinny_a.size(0), b.size(1)), dtype=torch.float16, device=skinny_a.device)
    skinny_gemm_checks(skinny_a, b, scale_tensor, output)
    if isinstance(b, PackedWeight) or torch.compiler.is_compiling():  # the 13-argument op takes the row-major view only
        _fused(skinny_a, b, output, output, scale_tensor.view(-1), None, None, _capi.EPILOGUE_NONE, 0)
        return output
    kwargs = infer_skinny_gemm_params(skinny_a, b)
    status = _skinny_gemm(A=skinny_a, B=b, scale_tensor=scale_tensor, D=output, **kwargs)
    _raise_on_status(status, "skinny_gemm_tb")
    return output


def skinny_gemm_scaled(
    skinny_a: Tensor,
    b: Tensor,
    scale_a: Tensor,
    scale_b: Optional[Tensor],
    output: Optional[Tensor] = None,
    accumulate: bool = False,
) -> Tensor:
    """Per-token x per-output-channel variant: output[i, j] (+)= scale_a[i] * scale_b[j] * (skinny_a @ b)[i, j].
    `scale_a` has 1 or m float32 elements, `scale_b` 1 or n; `scale_b` None stands for `b.scales`, the scales a
    PackedWeight carries (`pack_weight(weight, scales)`), and is an error for any other weight.  With accumulate=False
    the output is overwritten.
    This variant has no counterpart in the reference; an omitted output is allocated as bfloat16 (the serving dtype of the
    Llama-3 checkpoints it is used with), unlike `skinny_gemm`, which keeps the reference's float16."""
    m, n = skinny_a.size(0), b.size(1)
    if output is None:
        output = torch.empty(size=(m, n), dtype=torch.bfloat16, device=skinny_a.device)
        accumulate = False
    skinny_gemm_checks(skinny_a, b, scale_a.reshape(-1)[:1], output)
    assert scale_a.numel() in (1, m) and scale_a.dtype == torch.float32, f"Expected 1 or {m} float32 in scale_a"
    if scale_b is None:
        assert isinstance(b, PackedWeight) and b.scales is not None, "scale_b may be omitted only for a PackedWeight that carries its scales"
        scale_b = b.scales  # a float32 view of the packed buffer's tail: passed like any other per-channel scale
    assert scale_b.numel() in (1, n) and scale_b.dtype == torch.float32, f"Expected 1 or {n} float32 in scale_b"
    if isinstance(b, PackedWeight) or torch.compiler.is_compiling():
        _fused(skinny_a, b, output, output if accumulate else None, scale_a.contiguous().view(-1),
               scale_b.contiguous().view(-1), None, _capi.EPILOGUE_NONE, 0)
        return output
    status = _skinny_gemm_scaled(skinny_a, b, output, scale_a.contiguous().view(-1), scale_b.contiguous().view(-1),
                                 accumulate)
    _raise_on_status(status, "skinny_gemm_scaled")
    return output


class _ShapeOnly:
    """Stands in for the (m, n) 16-bit tensor the fused op never materialises, for `skinny_gemm_checks`."""

    def __init__(self, m: int, n: int, dtype: torch.dtype, device: torch.device):
        self.shape, self.dtype, self.device = (m, n), dtype, device

    def is_contiguous(self) -> bool:
        return True

    def stride(self) -> Tuple[int, int]:
        return (self.shape[1], 1)


def _scale_vectors(skinny_a: Tensor, b: Tensor, scale_a: Tensor, scale_b: Optional[Tensor]) -> Tuple[Tensor, Optional[Tensor]]:
    m, n = skinny_a.size(0), b.size(1)
    assert scale_a.numel() in (1, m) and scale_a.dtype == torch.float32, f"Expected 1 or {m} float32 in scale_a"
    if scale_b is None:  # one combined scale in scale_a: the weight's side of it is 1, whatever the weight's layout
        return scale_a.contiguous().view(-1), None
    assert scale_b.numel() in (1, n) and scale_b.dtype == torch.float32, f"Expected 1 or {n} float32 in scale_b"
    return scale_a.contiguous().view(-1), scale_b.contiguous().view(-1)


def skinny_gemm_add(
    skinny_a: Tensor,
    b: Tensor,
    scale_a: Tensor,
    scale_b: Optional[Tensor],
    base: Tensor,
    output: Optional[Tensor] = None,
) -> Tensor:
    """output[i, j] = base[i, j] + scale_a[i] * scale_b[j] * (skinny_a @ b)[i, j], summed in fp32 and rounded once
    (`scale_b` None = 1 in either weight layout; pass `b.scales` to apply the scales a PackedWeight carries).
    `base` has the output's shape and dtype (a residual stream, a bias broadcast beforehand); it is only read, so
    the residual add after a projection costs no extra launch and no copy."""
    m, n = skinny_a.size(0), b.size(1)
    if output is None:
        output = torch.empty(size=(m, n), dtype=base.dtype, device=skinny_a.device)
    skinny_gemm_checks(skinny_a, b, scale_a.reshape(-1)[:1], output)
    assert base.shape == output.shape and base.dtype == output.dtype and base.is_contiguous(), (
        f"Expected base to be contiguous with {output.shape = } and {output.dtype = }")
    sa, sb = _scale_vectors(skinny_a, b, scale_a, scale_b)
    _fused(skinny_a, b, output, base, sa, sb, None, _capi.EPILOGUE_NONE, 0)
    return output


def skinny_gemm_swiglu(
    skinny_a: Tensor,
    gate_up_weight: Tensor,
    scale_a: Tensor,
    scale_b: Optional[Tensor],
    out_scale: Tensor,
    output: Optional[Tensor] = None,
    intermediate_dtype: torch.dtype = torch.bfloat16,
) -> Tensor:
    """gate_up projection and SwiGLU in one launch: with [gate | up] = scale_a * scale_b * (skinny_a @ gate_up_weight)
    rounded to `intermediate_dtype`, returns float8_e4m3fn(silu(gate) * up / out_scale) of shape (m, n/2) -- what
    `skinny_gemm` followed by `swiglu` produces, without the (m, n) intermediate and the second launch.
    One launch for n % 32 == 0 and m <= 16, m <= 64 on k = 2048 / 4096, or m <= 32 on row-major weights of at least 1024 output
    columns (`hfrk_skinny_gemm_fused`'s conditions); other shapes run the two kernels."""
    m, n = skinny_a.size(0), gate_up_weight.size(1)
    assert n % 2 == 0, f"Expected an even number of gate_up columns but got {n}"
    assert intermediate_dtype in _OUT_DTYPES, f"Expected one of {_OUT_DTYPES} but got {intermediate_dtype = }"
    assert out_scale.numel() == 1 and out_scale.dtype == torch.float32, "Expected out_scale to be one float32"

    def two_launches() -> Tensor:
        from ..swiglu import swiglu
        gate_up = skinny_gemm_scaled(skinny_a, gate_up_weight, scale_a,
                                     scale_b if scale_b is not None else torch.ones(1, device=skinny_a.device),
                                     output=torch.empty((m, n), dtype=intermediate_dtype, device=skinny_a.device))
        result = swiglu(gate_up_proj=gate_up, scale_tensor=out_scale)
        if output is None:
            return result
        output.copy_(result)
        return output

    k = skinny_a.size(1)
    if n % 32 != 0 or (m > 32 and k not in (2048, 4096)):
        return two_launches()
    # 17..32 rows on other k: one launch where the library's row-split kernel takes the shape (row-major weights whose
    # output columns deal out over the workgroups), which its status says -- and where it is the faster way: measured on
    # k = 8192 at 20 / 32 rows, 16384 columns 25.8 / 26.5 us fused against 26.0 / 26.1 in two launches, 28672 columns 44.0 /
    # 46.4 against 40.7 / 41.0, 57344 columns 78.3 / 84.4 against 77.3 / 78.0 (above 16 rows the workgroup kernel is the
    # faster GEMM on large weights, by more than the SwiGLU launch costs)
    maybe = m > 16 and k not in (2048, 4096)
    if maybe and (isinstance(gate_up_weight, PackedWeight) or torch.compiler.is_compiling() or n * k > (128 << 20)):
        return two_launches()
    if output is None:
        output = torch.empty(size=(m, n // 2), dtype=torch.float8_e4m3fn, device=skinny_a.device)
    assert output.shape == (m, n // 2) and output.dtype == torch.float8_e4m3fn and output.is_contiguous(), (
        f"Expected a contiguous float8_e4m3fn output of shape {(m, n // 2)}")
    skinny_gemm_checks(skinny_a, gate_up_weight, scale_a.reshape(-1)[:1],
                       _ShapeOnly(m, n, intermediate_dtype, skinny_a.device))
    sa, sb = _scale_vectors(skinny_a, gate_up_weight, scale_a, scale_b)
    dtype_tag = _capi.BF16 if intermediate_dtype == torch.bfloat16 else _capi.F16
    if maybe:
        status = _skinny_gemm_fused(skinny_a, gate_up_weight, output, None, sa, sb, out_scale, _capi.EPILOGUE_SWIGLU, dtype_tag)
        if status == _capi.BAD_SHAPE:
            return two_launches()
        _raise_on_status(status, "skinny_gemm_fused")
        return output
    _fused(skinny_a, gate_up_weight, output, None, sa, sb, out_scale, _capi.EPILOGUE_SWIGLU, dtype_tag)
    return output


def rms_prologue_available(m: int, n_rows: int, k: int, b, swiglu: bool = False) -> bool:
    """Whether `skinny_gemm_rms` runs as one launch: the RMSNorm prologue exists in the row-split kernel -- row-major
    weights, up to 8 rows, k = 4096 or 8192, and weight rows (output columns with SwiGLU: `n_rows` then counts those)
    that deal out evenly over the workgroups.  The library decides (`hfrk_skinny_gemm_rms_plan`, the function its fused
    entry point plans with)."""
    if isinstance(b, PackedWeight) or torch.compiler.is_compiling():
        return False
    if swiglu:
        return _capi.rms_plan(m, 2 * n_rows, k, _capi.EPILOGUE_SWIGLU) is not None
    return _capi.rms_plan(m, n_rows, k) is not None


def skinny_gemm_rms(
    input: Tensor,
    residual: Tensor,
    rms_weight: Tensor,
    epsilon: float,
    act_scale: Tensor,
    b: Tensor,
    scale: Tensor,
    scale_b: Optional[Tensor] = None,
    base: Optional[Tensor] = None,
    out_scale: Optional[Tensor] = None,
    output: Optional[Tensor] = None,
    residual_out: Optional[Tensor] = None,
) -> Tuple[Tensor, Tensor]:
    """Residual RMSNorm and the projection that consumes it, in one launch where the prologue exists
    (`rms_prologue_available`), else as `residual_rms` followed by the GEMM -- same bits either way:
        residual_out = input + residual                                  (16-bit add)
        a            = float8_e4m3fn(rmsnorm(residual_out) * rms_weight / act_scale)
        output       = base + scale * scale_b * (a @ b)                  (out_scale None), or
        output       = float8_e4m3fn(silu(gate) * up / out_scale)        (out_scale given: b is a gate_up weight)
    `scale` is one float32 (activation scale x weight scale), `scale_b` optionally one per output channel.
    Unlike `residual_rms`, which updates `residual` in place, the sum goes to `residual_out` (allocated if None; it
    must not alias `input` or `residual`): every workgroup of the fused launch reads the old residual.
    Returns (output, residual_out).  No counterpart in the reference, which launches the two kernels
    (combined_ops/llama_mlp.py:23-41)."""
    m, k = input.shape
    n = b.size(1)
    swiglu = out_scale is not None
    dtype = input.dtype
    if output is None:
        output = torch.empty((m, n // 2), dtype=torch.float8_e4m3fn, device=input.device) if swiglu else \
            torch.empty((m, n), dtype=dtype, device=input.device)
    def two_launches(res: Tensor) -> Tuple[Tensor, Tensor]:
        from ..residual_rms import residual_rms
        res.copy_(residual)
        normalized, res = residual_rms(input=input, residual=res, weight=rms_weight, epsilon=epsilon, scale_tensor=act_scale)
        if swiglu:
            skinny_gemm_swiglu(normalized, b, scale, scale_b, out_scale, output=output, intermediate_dtype=dtype)
        elif base is not None:
            skinny_gemm_add(normalized, b, scale, scale_b, base, output=output)
        else:
            skinny_gemm_scaled(normalized, b, scale, scale_b if scale_b is not None else torch.ones(1, device=input.device), output=output)
        return output, res

    if residual_out is None:
        residual_out = torch.empty_like(residual)
    assert residual_out.data_ptr() not in (input.data_ptr(), residual.data_ptr()), "residual_out must not alias input or residual"
    if not rms_prologue_available(m, n // 2 if swiglu else n, k, b, swiglu):
        return two_launches(residual_out)
    assert scale.numel() == 1 and scale.dtype == torch.float32, "Expected scale to be one float32"
    status = torch.ops._HFRK_C.skinny_gemm_rms_fused(
        input, residual, residual_out, rms_weight, float(epsilon), act_scale, b, output, base, scale.reshape(-1),
        None if scale_b is None else scale_b.contiguous().view(-1), out_scale,
        _capi.EPILOGUE_SWIGLU if swiglu else _capi.EPILOGUE_NONE, _capi.BF16 if dtype == torch.bfloat16 else _capi.F16)
    if status == _capi.BAD_SHAPE:  # the library has no prologue for this shape after all (its own planner decides)
        return two_launches(residual_out)
    _raise_on_status(status, "skinny_gemm_rms_fused")
    return output, residual_out
