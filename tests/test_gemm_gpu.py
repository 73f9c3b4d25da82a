"""GPU parity of the FP8 skinny GEMM against the CPU oracle, through the C ABI and through torch.ops._HFRK_C.

Tolerances: the result must be within rtol 1e-2 / atol 1e-2 of the fp32 reference path in bfloat16 (the bar
this build is given).  The sharper check is against the exactly computed product (exact dot products scaled in
float64): |got - exact| <= 1 ulp of the 16-bit output (its single rounding, with slack for a rounding-boundary
flip) + 2^-16 * sum_k |a_k b_k| (fp32 accumulation error, far above what K <= 28672 random terms produce but far
below the effect of a lost or misplaced K chunk, which is of the order of the result itself).
"""
import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu


def _oracle():
    from oracle import skinny_gemm as og
    return og


def _ulp16(ref: torch.Tensor, dtype) -> torch.Tensor:
    """size of one unit in the last place of `dtype` at |ref| (float64 tensor)."""
    mant = 8 if dtype == torch.bfloat16 else 11
    min_exp = -126 if dtype == torch.bfloat16 else -14
    e = torch.floor(torch.log2(ref.abs().clamp_min(2.0 ** min_exp)))
    return torch.pow(2.0, e - (mant - 1))


def check_against_oracle(out, a, b, sa, sb, base=None, rtol=1e-2, atol=1e-2):
    og = _oracle()
    a_c, b_c = a.cpu(), b.cpu()
    sa_c, sb_c = sa.cpu(), sb.cpu()
    base_c = None if base is None else base.cpu()
    ref32 = og.reference_skinny_gemm(a_c, b_c, sa_c, sb_c, output=base_c, out_dtype=out.dtype)
    exact = og.exact_skinny_gemm(a_c, b_c, sa_c, sb_c, output=base_c)
    got = out.cpu()
    assert not got.isnan().any()
    err32 = (got.float() - ref32.float()).abs()
    tol = atol + rtol * ref32.float().abs()
    assert (err32 <= tol).all(), f"max excess over rtol/atol: {(err32 - tol).max().item()}"
    err_exact = (got.double() - exact).abs()
    one = torch.ones(1, dtype=torch.float64)
    abs_sum = og.exact_skinny_gemm(a_c.float().abs().to(torch.float8_e4m3fn), b_c.float().abs().to(torch.float8_e4m3fn),
                                   sa_c.abs(), sb_c.abs())
    bound = _ulp16(exact, out.dtype) + abs_sum * 2.0 ** -16
    worst = (err_exact / bound).max().item()
    assert worst <= 1.0, f"error is {worst} x the bound (1 ulp + 2^-16 sum|a b|) from the exact product"


def run_ex(a, b, sa, sb, out, accumulate, plan=None):
    from hf_rocm_kernels import _capi
    lib = _capi.load()
    m, k = a.shape
    n = b.shape[1]
    d_dtype = _capi.BF16 if out.dtype == torch.bfloat16 else _capi.F16
    status = lib.hfrk_skinny_gemm_ex(
        a.data_ptr(), b.data_ptr(), out.data_ptr(), sa.data_ptr(), 0 if sa.numel() == 1 else 1,
        sb.data_ptr(), 0 if sb.numel() == 1 else 1, m, n, k, b.stride(1), d_dtype, int(accumulate),
        None if plan is None else ctypes.byref(plan), torch.cuda.current_stream().cuda_stream)
    _capi.check(status, "hfrk_skinny_gemm_ex")
    torch.cuda.synchronize()
    return out


def all_plans(m, n, k):
    """every decomposition the kernel family offers for this shape, as GemmPlan structs"""
    from hf_rocm_kernels import _capi
    mt = (m + 15) // 16
    plans = []
    for wn in (1, 2, 4, 8):
        wk = 8 // wn
        for ch in (1, 2):
            ks = 256 * wk * ch
            if k % ks:
                continue
            lds = 8 * 4096 + 2 * 16 * mt * ks + 16
            if lds > 160 * 1024:
                continue
            panels = (n + 16 * wn - 1) // (16 * wn)
            slabs = k // ks
            units = panels * slabs
            for grid in sorted({min(256, units), min(200, units), min(7, units)}):
                p = _capi.GemmPlan(mt, wn, wk, ch, grid, panels, slabs, lds)
                plans.append(p)
    return plans


@pytest.mark.parametrize("m", [1, 3, 8, 16, 17, 32, 33, 64])
@pytest.mark.parametrize("n,k", [(128, 256), (1024, 1024), (4096, 4096), (6144, 4096), (4096, 14336), (1000, 512), (50, 256)])
def test_default_plan_matches_oracle(m, n, k):
    from hf_rocm_kernels.operators.skinny_gemm import generate_llama_gemm_data
    a, b, sa, sw = generate_llama_gemm_data(m, n, k, seed=m * 131 + n + k)
    out = torch.empty((m, n), dtype=torch.bfloat16, device="cuda")
    run_ex(a, b, sa, sw, out, accumulate=False)
    check_against_oracle(out, a, b, sa, sw)


@pytest.mark.parametrize("m,n,k", [(8, 512, 2048), (16, 1040, 4096), (33, 256, 1024), (64, 6144, 4096), (5, 4096, 14336)])
def test_every_plan_gives_the_same_answer(m, n, k):
    from hf_rocm_kernels.operators.skinny_gemm import generate_llama_gemm_data
    a, b, sa, sw = generate_llama_gemm_data(m, n, k, seed=7)
    plans = all_plans(m, n, k)
    assert plans
    for p in plans:
        out = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device="cuda")
        run_ex(a, b, sa, sw, out, accumulate=False, plan=p)
        try:
            check_against_oracle(out, a, b, sa, sw)
        except AssertionError as e:
            raise AssertionError(f"plan {p.as_dict()}: {e}")
