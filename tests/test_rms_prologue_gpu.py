"""GPU tests of the residual RMSNorm as the GEMM's prologue (`hfrk_skinny_gemm_rms_fused`, `skinny_gemm_rms`,
`llama_mlp_combined_ops(fused=True, rms_prologue=True)`).  The prologue uses the stand-alone kernel's per-piece functions and
its order of sums, and the GEMM part is the row-split kernel under the same plan: the one launch must give, bit for bit,
what `residual_rms` followed by the GEMM gives -- which the other GPU tests hold against the oracle stage by stage
(reference chain: hf_rocm_kernels/combined_ops/llama_mlp.py:23-41)."""
import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu


def _inputs(m, n, k, dtype, seed):
    from hf_rocm_kernels.utils.fp8 import amax_scale, fp8_quantize
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(m, k, generator=g).to(dtype).cuda()
    res = torch.randn(m, k, generator=g).to(dtype).cuda()
    w_norm = (1 + 0.1 * torch.randn(k, generator=g)).to(dtype).cuda()
    w = torch.randn(n, k, generator=g) * 0.02
    sw = amax_scale(w)
    w8 = fp8_quantize(w, sw)[0].cuda().t()
    act_scale = torch.tensor([6.0 / 448]).cuda()
    return x, res, w_norm, w8, act_scale, (act_scale * sw.cuda()).reshape(1)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("m,n,k", [(1, 6144, 4096), (4, 4096, 4096), (8, 28672, 4096), (3, 10240, 8192), (8, 8192, 8192), (5, 3584, 4096), (4, 4098, 4096)])
def test_plain_projection_with_the_norm_as_prologue(m, n, k, dtype):
    from hf_rocm_kernels import residual_rms, skinny_gemm_add, skinny_gemm_rms, skinny_gemm_scaled
    from hf_rocm_kernels.operators.skinny_gemm import rms_prologue_available
    x, res, w_norm, w8, act_scale, scale = _inputs(m, n, k, dtype, seed=m + n)
    assert rms_prologue_available(m, n, k, w8)
    one = torch.ones(1).cuda()
    normalized, want_res = residual_rms(x, res.clone(), w_norm, 1e-5, scale_tensor=act_scale)
    want = skinny_gemm_scaled(normalized, w8, scale, one, output=torch.empty(m, n, dtype=dtype).cuda())
    res_before = res.clone()
    got, got_res = skinny_gemm_rms(x, res, w_norm, 1e-5, act_scale, w8, scale)
    assert torch.equal(res, res_before), "the residual is read, not updated in place"
    assert torch.equal(got_res, want_res) and torch.equal(got, want)
    assert got.float().abs().sum() > 0
    # with an addend (the residual stream) and per-channel scales
    sb = (0.5 + torch.rand(n, generator=torch.Generator().manual_seed(1))).cuda()
    base = torch.randn(m, n, generator=torch.Generator().manual_seed(2)).to(dtype).cuda()
    want = skinny_gemm_add(normalized, w8, scale, sb, base)
    got, _ = skinny_gemm_rms(x, res, w_norm, 1e-5, act_scale, w8, scale, scale_b=sb, base=base)
    assert torch.equal(got, want)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("m,n,k", [(1, 28672, 4096), (8, 28672, 4096), (4, 57344, 8192), (6, 8192, 4096)])
def test_gate_up_projection_with_norm_prologue_and_swiglu_epilogue(m, n, k, dtype):
    from hf_rocm_kernels import residual_rms, skinny_gemm_rms, skinny_gemm_swiglu
    x, res, w_norm, w8, act_scale, scale = _inputs(m, n, k, dtype, seed=3 * m + n)
    out_scale = torch.tensor([4.0 / 448]).cuda()
    normalized, want_res = residual_rms(x, res.clone(), w_norm, 1e-5, scale_tensor=act_scale)
    want = skinny_gemm_swiglu(normalized, w8, scale, None, out_scale, intermediate_dtype=dtype)
    got, got_res = skinny_gemm_rms(x, res, w_norm, 1e-5, act_scale, w8, scale, out_scale=out_scale)
    assert got.dtype == torch.float8_e4m3fn and got.shape == (m, n // 2)
    assert torch.equal(got_res, want_res)
    assert torch.equal(got.view(torch.uint8), want.view(torch.uint8))
    assert got.view(torch.uint8).any()


@pytest.mark.parametrize("m,n,k,grid", [(3, 2048, 4096, 4), (7, 1024, 8192, 8), (2, 4096, 4096, 8)])
def test_prologue_under_a_plan_that_rotates_k(m, n, k, grid):
    """Explicit row-split plans whose workgroups start at different points in k (every wave's run is a multiple of 16
    chunks): the staged activations are then read from the rotated position too.  Same bits as the two launches under
    the same plan."""
    from hf_rocm_kernels import _capi, residual_rms
    lib = _capi.load()
    x, res, w_norm, w8, act_scale, scale = _inputs(m, n, k, torch.bfloat16, seed=m + n + grid)
    units = n // 4
    assert (-(-(units // grid) // 4) * (k // 256)) % 128 == 0
    plan = _capi.GemmPlan(1, -2, 1, (m + 3) // 4, grid, units, k // 256, 8 * 2 * 4096)
    one = torch.ones(1).cuda()
    out = torch.full((m, n), float("nan"), dtype=torch.bfloat16).cuda()
    res_out = torch.empty_like(res)
    assert lib.hfrk_skinny_gemm_rms_fused(x.data_ptr(), res.data_ptr(), res_out.data_ptr(), w_norm.data_ptr(), 1e-5, act_scale.data_ptr(),
                                          _capi.BF16, w8.data_ptr(), out.data_ptr(), None, scale.data_ptr(), None, 0, None, m, n, k, k,
                                          _capi.BF16, _capi.EPILOGUE_NONE, ctypes.byref(plan), None) == _capi.SUCCESS
    torch.cuda.synchronize()
    normalized, want_res = residual_rms(x, res.clone(), w_norm, 1e-5, scale_tensor=act_scale)
    want = torch.empty_like(out)
    assert lib.hfrk_skinny_gemm_ex(normalized.data_ptr(), w8.data_ptr(), want.data_ptr(), scale.data_ptr(), 0, one.data_ptr(), 0, m, n, k, k,
                                   _capi.BF16, 0, ctypes.byref(plan), None) == 0
    torch.cuda.synchronize()
    assert torch.equal(res_out, want_res) and torch.equal(out, want)
    assert not out.isnan().any() and out.float().abs().sum() > 0


@pytest.mark.parametrize("add_residual", [False, True])
@pytest.mark.parametrize("m", [1, 4, 8])
def test_mlp_block_in_two_launches_equals_the_three_launch_block(m, add_residual):
    from hf_rocm_kernels.combined_ops.llama_mlp import llama_mlp_combined_ops
    from hf_rocm_kernels.utils.fp8 import amax_scale, fp8_quantize
    hidden, inter = 4096, 14336
    g = torch.Generator().manual_seed(50 + m)
    attn = torch.randn(m, hidden, generator=g).to(torch.bfloat16).cuda()
    resid = torch.randn(m, hidden, generator=g).to(torch.bfloat16).cuda()
    rms_w = (1 + 0.1 * torch.randn(hidden, generator=g)).to(torch.bfloat16).cuda()
    wgu = torch.randn(2 * inter, hidden, generator=g) * 0.02
    wd = torch.randn(hidden, inter, generator=g) * 0.02
    s_gu, s_d = amax_scale(wgu), amax_scale(wd)
    wgu8, wd8 = fp8_quantize(wgu, s_gu)[0].cuda().t(), fp8_quantize(wd, s_d)[0].cuda().t()
    in_gu, in_d = torch.tensor([6.0 / 448]).cuda(), torch.tensor([4.0 / 448]).cuda()
    args = (rms_w, 1e-5, wgu8, in_gu, (in_gu * s_gu.cuda()).reshape(1), wd8, in_d, (in_d * s_d.cuda()).reshape(1))
    want, want_res = llama_mlp_combined_ops(attn, resid.clone(), *args, add_residual=add_residual, fused=True)
    got, got_res = llama_mlp_combined_ops(attn, resid, *args, add_residual=add_residual, fused=True, rms_prologue=True)
    assert torch.equal(got, want) and torch.equal(got_res, want_res)
    assert got_res.data_ptr() != resid.data_ptr()


def test_where_the_prologue_does_not_exist_the_wrapper_runs_two_launches_and_the_library_says_so():
    from hf_rocm_kernels import _capi, residual_rms, skinny_gemm_rms, skinny_gemm_scaled
    from hf_rocm_kernels.operators.skinny_gemm import rms_prologue_available
    from hf_rocm_kernels.utils.weight_format import pack_weight
    lib = _capi.load()
    one = torch.ones(1).cuda()
    for m, n, k in [(9, 4096, 4096), (4, 4096, 2048), (4, 512, 4096)]:   # too many rows; k; too few weight rows to deal out
        x, res, w_norm, w8, act_scale, scale = _inputs(m, n, k, torch.bfloat16, seed=7)
        assert not rms_prologue_available(m, n, k, w8)
        out = torch.empty(m, n, dtype=torch.bfloat16).cuda()
        res_out = torch.empty_like(res)
        st = lib.hfrk_skinny_gemm_rms_fused(x.data_ptr(), res.data_ptr(), res_out.data_ptr(), w_norm.data_ptr(), 1e-5, act_scale.data_ptr(),
                                            _capi.BF16, w8.data_ptr(), out.data_ptr(), None, scale.data_ptr(), None, 0, None, m, n, k, k,
                                            _capi.BF16, _capi.EPILOGUE_NONE, None, None)
        assert st == _capi.BAD_SHAPE, (m, n, k, st)
        normalized, want_res = residual_rms(x, res.clone(), w_norm, 1e-5, scale_tensor=act_scale)
        want = skinny_gemm_scaled(normalized, w8, scale, one, output=torch.empty(m, n, dtype=torch.bfloat16).cuda())
        got, got_res = skinny_gemm_rms(x, res, w_norm, 1e-5, act_scale, w8, scale)
        assert torch.equal(got, want) and torch.equal(got_res, want_res)
    # packed weights run the two launches too; aliasing and misuse come back as status codes
    x, res, w_norm, w8, act_scale, scale = _inputs(4, 4096, 4096, torch.bfloat16, seed=8)
    assert not rms_prologue_available(4, 4096, 4096, pack_weight(w8.t()))
    out = torch.empty(4, 4096, dtype=torch.bfloat16).cuda()
    call = lambda res_out, plan=None: lib.hfrk_skinny_gemm_rms_fused(
        x.data_ptr(), res.data_ptr(), res_out, w_norm.data_ptr(), 1e-5, act_scale.data_ptr(), _capi.BF16, w8.data_ptr(), out.data_ptr(), None,
        scale.data_ptr(), None, 0, None, 4, 4096, 4096, 4096, _capi.BF16, _capi.EPILOGUE_NONE, plan, None)
    assert call(res.data_ptr()) == _capi.BAD_SHAPE and call(x.data_ptr()) == _capi.BAD_SHAPE and call(None) == _capi.BAD_SHAPE
    res_out = torch.empty_like(res)
    assert call(res_out.data_ptr() + 2) == _capi.BAD_ALIGNMENT
    stream_plan = _capi.GemmPlan(1, 0, 1, 1, 256, 256, 16, 8 * 2 * 4096)
    assert call(res_out.data_ptr(), ctypes.byref(stream_plan)) == _capi.INVALID_CONFIG    # the prologue lives in the row-split kernel
    two_tiles = _capi.GemmPlan(1, -2, 2, 1, 256, 1024, 16, 8 * 3 * 4096)
    assert call(res_out.data_ptr(), ctypes.byref(two_tiles)) == _capi.INVALID_CONFIG      # one tile per chunk with the plain epilogue
    rows_plan = _capi.GemmPlan(1, -2, 1, 1, 200, 1024, 16, 8 * 2 * 4096)
    assert call(res_out.data_ptr(), ctypes.byref(rows_plan)) == _capi.SUCCESS
    torch.cuda.synchronize()
    normalized, want_res = residual_rms(x, res.clone(), w_norm, 1e-5, scale_tensor=act_scale)
    assert torch.equal(res_out, want_res)
    want = torch.empty_like(out)
    assert lib.hfrk_skinny_gemm_ex(normalized.data_ptr(), w8.data_ptr(), want.data_ptr(), scale.data_ptr(), 0, one.data_ptr(), 0, 4, 4096, 4096, 4096,
                                   _capi.BF16, 0, ctypes.byref(rows_plan), None) == 0
    torch.cuda.synchronize()
    assert torch.equal(out, want)


def test_the_predicate_and_the_entry_point_agree_on_random_shapes():
    """`rms_prologue_available` (hfrk_skinny_gemm_rms_plan) says yes exactly where `hfrk_skinny_gemm_rms_fused` launches, and
    where it launches the result is the two-launch chain's, bit for bit."""
    import numpy as np
    from hf_rocm_kernels import _capi, residual_rms
    from hf_rocm_kernels.operators.skinny_gemm import rms_prologue_available
    lib = _capi.load()
    rng = np.random.default_rng(5)
    one = torch.ones(1).cuda()
    seen = {True: 0, False: 0}
    for case in range(40):
        m = int(rng.integers(1, 11))
        n = int(rng.choice([256, 512, 1000, 2048, 3584, 4096, 4098, 6144])) + 4 * int(rng.integers(0, 3))
        k = int(rng.choice([2048, 4096, 8192]))
        x, res, w_norm, w8, act_scale, scale = _inputs(m, n, k, torch.bfloat16, seed=100 + case)
        out = torch.empty(m, n, dtype=torch.bfloat16).cuda()
        res_out = torch.empty_like(res)
        st = lib.hfrk_skinny_gemm_rms_fused(x.data_ptr(), res.data_ptr(), res_out.data_ptr(), w_norm.data_ptr(), 1e-5, act_scale.data_ptr(),
                                            _capi.BF16, w8.data_ptr(), out.data_ptr(), None, scale.data_ptr(), None, 0, None, m, n, k, k,
                                            _capi.BF16, _capi.EPILOGUE_NONE, None, None)
        torch.cuda.synchronize()
        available = rms_prologue_available(m, n, k, w8)
        seen[available] += 1
        assert st == (_capi.SUCCESS if available else _capi.BAD_SHAPE), (m, n, k, st, available)
        if available:
            normalized, want_res = residual_rms(x, res.clone(), w_norm, 1e-5, scale_tensor=act_scale)
            want = torch.empty_like(out)
            plan = _capi.rms_plan(m, n, k)
            assert lib.hfrk_skinny_gemm_ex(normalized.data_ptr(), w8.data_ptr(), want.data_ptr(), scale.data_ptr(), 0, one.data_ptr(), 0, m, n, k, k,
                                           _capi.BF16, 0, ctypes.byref(plan), None) == 0
            torch.cuda.synchronize()
            assert torch.equal(res_out, want_res) and torch.equal(out, want), (m, n, k)
    assert seen[True] >= 8 and seen[False] >= 8, seen
