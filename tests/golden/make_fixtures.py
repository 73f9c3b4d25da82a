"""Writes the small committed fixtures under tests/golden/ from this repository's own oracle.

The reference holds no golden vectors, known-answer tests or fixture files for this path (its tests draw random
data on the GPU at run time), so these are regression anchors made by the oracle once it was pinned by the checks
in tests/test_oracle_*.py: FP8 operand bytes in, expected bf16 bits and exact integer dot products out.
Run from the repository root:  python tests/golden/make_fixtures.py
"""
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

from oracle import c_oracle, fp8  # noqa: E402
from oracle import residual_rms as orr  # noqa: E402
from oracle import skinny_gemm as og  # noqa: E402
from oracle import swiglu as osw  # noqa: E402


def gemm_case(name, m, n, k, seed, per_token=False, per_channel=False):
    g = torch.Generator().manual_seed(seed)
    act = torch.randn(m, k, generator=g).to(torch.bfloat16).float()
    w = torch.randn(n, k, generator=g) * 0.02
    sa = fp8.amax_scale(act, dim=1 if per_token else None).reshape(-1)
    sw = fp8.amax_scale(w, dim=1 if per_channel else None).reshape(-1)
    a8 = fp8.fp8_quantize(act, sa.reshape(-1, 1) if per_token else sa)[0]
    w8 = fp8.fp8_quantize(w, sw.reshape(-1, 1) if per_channel else sw)[0]
    out = og.reference_skinny_gemm(a8, w8.t(), sa, sw)
    a_codes, w_codes = a8.view(torch.uint8).numpy(), w8.view(torch.uint8).numpy()
    np.savez_compressed(os.path.join(HERE, f"gemm_{name}.npz"), a_codes=a_codes, w_codes=w_codes,
                        scale_a=sa.numpy(), scale_w=sw.numpy(), out_bf16_bits=out.view(torch.int16).numpy(),
                        int_dots=c_oracle.gemm_int(a_codes, w_codes))


def rms_case(name, rows, cols, seed, dtype):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(rows, cols, generator=g).to(dtype)
    r = torch.randn(rows, cols, generator=g).to(dtype)
    w = (1 + 0.1 * torch.randn(cols, generator=g)).to(dtype)
    scale = torch.tensor([0.011], dtype=torch.float32)
    q, res, _ = orr.reference_residual_rms(x, r, w, 1e-5, scale)
    h, _, _ = orr.reference_residual_rms(x, r, w, 1e-5, None)
    np.savez_compressed(os.path.join(HERE, f"rms_{name}.npz"), input_bits=x.view(torch.int16).numpy(),
                        residual_bits=r.view(torch.int16).numpy(), weight_bits=w.view(torch.int16).numpy(),
                        scale=scale.numpy(), eps=np.float32(1e-5), out_fp8=q.view(torch.uint8).numpy(),
                        out16_bits=h.view(torch.int16).numpy(), new_residual_bits=res.view(torch.int16).numpy())


def swiglu_case(name, rows, cols, seed, dtype):
    g = torch.Generator().manual_seed(seed)
    gu = torch.randn(rows, 2 * cols, generator=g).to(dtype)
    scale = torch.tensor([0.013], dtype=torch.float32)
    q = osw.reference_swiglu(gu, scale)
    np.savez_compressed(os.path.join(HERE, f"swiglu_{name}.npz"), gate_up_bits=gu.view(torch.int16).numpy(),
                        scale=scale.numpy(), out_fp8=q.view(torch.uint8).numpy())


if __name__ == "__main__":
    gemm_case("m8_n256_k512", 8, 256, 512, 1)
    gemm_case("m3_n48_k256", 3, 48, 256, 2)
    gemm_case("m17_n130_k1024_rowcol", 17, 130, 1024, 3, per_token=True, per_channel=True)
    rms_case("bf16_4x512", 4, 512, 4, torch.bfloat16)
    rms_case("f16_3x24", 3, 24, 5, torch.float16)
    swiglu_case("bf16_4x256", 4, 256, 6, torch.bfloat16)
    swiglu_case("f16_3x24", 3, 24, 7, torch.float16)
    print("fixtures written to", HERE)
