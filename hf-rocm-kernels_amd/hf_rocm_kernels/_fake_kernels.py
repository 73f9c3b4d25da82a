"""Shape-only ("fake") implementations of the `_HFRK_C` operators, for tracing.

The reference registers its operators on the CUDA dispatch key only (csrc/torch_bindings.cpp:20-41), so they cannot
be traced with fake tensors.  Every operator here writes into tensors the caller passes (`Tensor!` in the schema)
and returns nothing or a status integer, so the fake implementation has nothing to compute: it returns None, or 0
for the GEMM entry points (the status of a call whose arguments the real implementation accepts).  With these
registered torch can trace through the operators; the mutations are functionalised by torch from the schema.
A tracer cannot keep an operator that returns an integer inside a graph, so while torch is compiling the GEMM
wrappers call `skinny_gemm_checked`, which raises on a non-zero status instead of returning it; with that,
`torch.compile(..., fullgraph=True)` takes the whole MLP block as one graph.  Nothing here runs when an operator
is called on real tensors.
"""
import torch

import hf_rocm_kernels._HFRK_C  # noqa: F401  (registers torch.ops._HFRK_C)

_RETURNS_NOTHING = ("increment", "residual_rms", "swiglu", "pack_weight", "pack_weight_scaled", "unpack_weight", "reencode_fnuz",
                    "residual_rms_dynamic", "swiglu_dynamic", "quantize_fp8", "skinny_gemm_checked")
_RETURNS_STATUS = ("skinny_gemm_tb", "skinny_gemm_scaled", "skinny_gemm_fused", "skinny_gemm_packed", "skinny_gemm_rms_fused")


def _nothing(*args, **kwargs) -> None:
    return None


def _success(*args, **kwargs) -> int:
    return 0


def register() -> None:
    for name in _RETURNS_NOTHING:
        torch.library.register_fake(f"_HFRK_C::{name}", _nothing)
    for name in _RETURNS_STATUS:
        torch.library.register_fake(f"_HFRK_C::{name}", _success)


register()
