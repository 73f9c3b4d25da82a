"""Linear-layer front end of the FP8 skinny GEMM: what a serving stack binds in place of its fp8 linear method.

The reference points to its vLLM integration for this (README.md:95-97); the hook there replaces the fp8 linear
apply function for decode-sized batches.  This module is that hook without the vLLM dependency: a function with the
usual (input, weight, weight_scale, input_scale, bias) signature, and an nn.Module that owns a quantised weight.

Decode batches (up to 64 tokens) run as: one quantisation kernel (skipped when the caller already holds fp8
activations and their scales, e.g. from `residual_rms_dynamic` / `swiglu_dynamic`) and one GEMM with the scales, the
bias or residual folded into its epilogue.  Larger batches are cut into pieces of 64 rows; a prefill-sized batch
belongs on a GEMM library and is only handled here so that the layer is always correct.
"""
from typing import Optional, Sequence, Tuple, Union

import torch
from torch import Tensor

from .. import _capi
from ..operators.quantize import quantize_fp8
from ..operators.skinny_gemm import skinny_gemm_add, skinny_gemm_scaled
from ..utils.fp8 import amax_scale, fp8_quantize
from ..utils.weight_format import PackedWeight, pack_weight

Weight = Union[Tensor, PackedWeight]


def _weight_view(weight: Weight) -> Weight:
    """[n, k] row-major fp8 (an nn.Linear weight) -> the [k, n] view the GEMM takes; a PackedWeight passes through."""
    return weight if isinstance(weight, PackedWeight) else weight.t()


def apply_fp8_linear(
    input: Tensor,
    weight: Weight,
    weight_scale: Optional[Tensor],
    input_scale: Optional[Tensor] = None,
    bias: Optional[Tensor] = None,
    residual: Optional[Tensor] = None,
    out_dtype: Optional[torch.dtype] = None,
) -> Tensor:
    """y = input @ dequant(weight).T (+ bias) (+ residual), computed in FP8 with fp32 accumulation.

    - input: (..., k) float16/bfloat16 activations, quantised here -- with `input_scale` (one float32: static) or,
      when it is None, dynamically per token -- or a float8_e4m3fn tensor already quantised, `input_scale` then being
      its scale(s): one float32 or one per token
    - weight: (n, k) float8_e4m3fn row-major, or its PackedWeight; weight_scale: one float32 or one per output channel,
      or None for a PackedWeight that carries its scales
    - bias: (n,) in the output dtype; residual: (..., n) in the output dtype, added in the GEMM's epilogue (fp32 sum
      with the product, one rounding).  Given both, the bias is added to the residual first (one 16-bit add).
    - out_dtype: float16/bfloat16; defaults to the input's (bfloat16 for an fp8 input)
    """
    k = input.shape[-1]
    lead = input.shape[:-1]
    x = input.reshape(-1, k)
    if x.dtype == torch.float8_e4m3fn:
        assert input_scale is not None, "an fp8 input needs its scale(s)"
        q, sa = x.contiguous(), input_scale.reshape(-1)
        out_dtype = out_dtype or torch.bfloat16
    else:
        out_dtype = out_dtype or x.dtype
        q, sa = quantize_fp8(x.contiguous(), input_scale)
        sa = sa.reshape(-1)
    w = _weight_view(weight)
    n = w.size(1)
    if weight_scale is None:
        assert isinstance(w, PackedWeight) and w.scales is not None, "a weight without scales of its own needs weight_scale"
        sb = w.scales  # the per-channel scales stored behind the packed bytes, passed explicitly
    else:
        sb = weight_scale.reshape(-1)
    m = q.size(0)
    base = None
    if residual is not None:
        base = residual.reshape(m, n)
        if bias is not None:
            base = base + bias
        base = base.contiguous()
    elif bias is not None:
        base = bias.to(out_dtype).expand(m, n).contiguous()
    out = torch.empty((m, n), dtype=out_dtype, device=q.device)
    for r0 in range(0, m, _capi.GEMM_MAX_M):
        r1 = min(m, r0 + _capi.GEMM_MAX_M)
        sa_part = sa if sa.numel() == 1 else sa[r0:r1]
        if base is None:
            skinny_gemm_scaled(q[r0:r1], w, sa_part, sb, output=out[r0:r1])
        else:
            skinny_gemm_add(q[r0:r1], w, sa_part, sb, base[r0:r1], output=out[r0:r1])
    return out.reshape(*lead, n)


class Fp8Linear(torch.nn.Module):
    """nn.Linear with an FP8 weight: per-output-channel (default) or per-tensor weight scale, dynamic per-token or
    static activation scale, optional packed load format.  Inference only.

    The tensors are registered buffers (`weight_data`, `weight_scale`, `bias`, `input_scale`), so the layer moves with
    `.to()` and round-trips through `state_dict()` / `load_state_dict()`; `weight_data` is the (n, k) fp8 weight or,
    packed, the flat buffer of its PackedWeight (its rank tells which).  A packed weight with per-channel scales keeps
    them in that same buffer (one allocation per layer) and `weight_scale` is None."""

    def __init__(self, weight: Weight, weight_scale: Optional[Tensor], bias: Optional[Tensor] = None,
                 input_scale: Optional[Tensor] = None):
        super().__init__()
        self.packed = isinstance(weight, PackedWeight)
        assert weight_scale is not None or (self.packed and weight.scales is not None), "a weight without scales of its own needs weight_scale"
        self.out_features, self.in_features = (weight.n, weight.k) if self.packed else tuple(weight.shape)
        self.register_buffer("weight_data", weight.data if self.packed else weight)
        self.register_buffer("weight_scale", weight_scale)
        self.register_buffer("bias", bias)
        self.register_buffer("input_scale", input_scale)
        self._refresh()
        self.register_load_state_dict_post_hook(lambda module, incompatible_keys: module._refresh())

    def _refresh(self) -> None:
        """The operand handed to the GEMM wrappers: the (n, k) tensor, or a PackedWeight over the current buffer."""
        self.packed = self.weight_data.dim() == 1
        self._operand = PackedWeight(self.weight_data, self.out_features, self.in_features) if self.packed else self.weight_data

    _QUANTISED = ("weight_data", "weight_scale", "input_scale")

    def _apply(self, fn, *args, **kwargs):
        """Device moves reach every buffer; dtype casts (`.half()`, `.to(torch.bfloat16)`) reach the bias only: the fp8
        weight and the float32 scales are what the GEMM takes and keep their dtypes."""
        before = {name: getattr(self, name) for name in self._QUANTISED}
        module = super()._apply(fn, *args, **kwargs)
        for name, old in before.items():
            new = getattr(self, name)
            if old is not None and new is not None and new.dtype != old.dtype:
                self._buffers[name] = old.to(new.device)
        self._refresh()
        return module

    @property
    def weight(self) -> Weight:
        return self._operand

    @classmethod
    def from_float(cls, linear: torch.nn.Linear, per_channel: bool = True, packed: bool = False,
                   input_scale: Optional[Tensor] = None) -> "Fp8Linear":
        """Quantise an nn.Linear's weight (scale = amax/448 per output channel or per tensor).  Packing runs on the
        GPU: `packed=True` needs the layer there."""
        w = linear.weight.detach()
        scale = amax_scale(w, dim=1 if per_channel else None)
        q, _ = fp8_quantize(w, scale)
        scale = scale.reshape(-1).contiguous()
        bias = None if linear.bias is None else linear.bias.detach().clone()
        if packed and per_channel:
            return cls(pack_weight(q, scale), None, bias, input_scale)
        return cls(pack_weight(q) if packed else q, scale, bias, input_scale)

    def forward(self, input: Tensor, input_scale: Optional[Tensor] = None, residual: Optional[Tensor] = None) -> Tensor:
        """`input` 16-bit (quantised here) or fp8 with `input_scale`; `residual` is added in the GEMM's epilogue."""
        scale = input_scale if input_scale is not None else self.input_scale
        return apply_fp8_linear(input, self._operand, self.weight_scale, scale, self.bias, residual)

    def extra_repr(self) -> str:
        kind = "packed" if self.packed else "row-major"
        return f"in_features={self.in_features}, out_features={self.out_features}, weight={kind}, bias={self.bias is not None}"


def convert_linear_layers(module: torch.nn.Module, per_channel: bool = True, packed: bool = False,
                          skip: Sequence[str] = ()) -> int:
    """Replace, in place and recursively, every nn.Linear under `module` that the FP8 path can take (in_features a
    multiple of 16 -- of 256 for packed weights -- and at most 32768, 16-bit weight) by an Fp8Linear quantised from it; returns how many were replaced.
    skip: layers whose dotted name ends with one of these strings stay as they are (e.g. ("lm_head",)).
    The counterpart, without the serving stack, of switching a model's linear method (reference README.md:95-97)."""
    replaced = 0

    def visit(parent: torch.nn.Module, prefix: str) -> None:
        nonlocal replaced
        for name, child in list(parent.named_children()):
            full = f"{prefix}.{name}" if prefix else name
            if isinstance(child, torch.nn.Linear):
                # the activation quantiser reads a row of at most 32768 values in one pass
                usable = (child.in_features % (256 if packed else 16) == 0 and child.in_features <= 32768
                          and child.weight.dtype in (torch.float16, torch.bfloat16))
                if usable and not any(full.endswith(suffix) for suffix in skip):
                    setattr(parent, name, Fp8Linear.from_float(child, per_channel=per_channel, packed=packed))
                    replaced += 1
            else:
                visit(child, full)

    visit(module, "")
    return replaced
