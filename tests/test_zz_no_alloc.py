"""The allocation-free GEMM entry point (hfrk_skinny_gemm_noalloc) against hfrk_skinny_gemm_ex, through the C ABI.

Both run the same kernels under the same plan; the only difference is where partial sums and arrival counters live (an
array inside the library's code object instead of a workspace from the pool), so results must be bit-identical.  The
array keeps the previous call's contents: the second call of each pair is smaller than the first, and its plan reads
other addresses of the same array.
"""
import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu


def _run(entry, a, b, sa, sb, out, plan=None, accumulate=False):
    from hf_rocm_kernels import _capi
    m, k = a.shape
    status = entry(a.data_ptr(), b.data_ptr(), out.data_ptr(), sa.data_ptr(), 0 if sa.numel() == 1 else 1,
                   sb.data_ptr(), 0 if sb.numel() == 1 else 1, m, b.shape[1], k, b.stride(1),
                   _capi.BF16 if out.dtype == torch.bfloat16 else _capi.F16, int(accumulate),
                   None if plan is None else ctypes.byref(plan), torch.cuda.current_stream().cuda_stream)
    return status


def _pair(m, n, k, seed, plan=None, dtype=torch.bfloat16, accumulate=False, per_channel=False):
    """one call through each entry point on the same inputs; returns (allocation-free result, pooled-workspace result)"""
    from hf_rocm_kernels import _capi
    from hf_rocm_kernels.operators.skinny_gemm import generate_llama_gemm_data
    lib = _capi.load()
    a, b, sa, sw = generate_llama_gemm_data(m, n, k, seed=seed, per_token=per_channel, per_channel=per_channel)
    base = torch.randn(m, n, generator=torch.Generator().manual_seed(seed)).to(dtype).cuda()
    got, want = base.clone(), base.clone()
    assert _run(lib.hfrk_skinny_gemm_noalloc, a, b, sa, sw, got, plan, accumulate) == 0
    assert _run(lib.hfrk_skinny_gemm_ex, a, b, sa, sw, want, plan, accumulate) == 0
    torch.cuda.synchronize()
    return got, want, (a, b, sa, sw, base if accumulate else None)


def test_noalloc_gemm_matches_the_pooled_entry_point_on_two_calls_in_a_row():
    from hf_rocm_kernels import _capi
    from tests.test_gemm_gpu import check_against_oracle
    # wave-stream kernel on 120 workgroups: row tiles cut between workgroups, so workspace and counters are used
    big = _capi.GemmPlan(1, 0, 1, 2, 120, 256, 16, 8 * 2 * 4096)
    got, want, (a, b, sa, sw, base) = _pair(8, 4096, 4096, seed=1, plan=big)
    assert torch.equal(got, want)
    check_against_oracle(got, a, b, sa, sw)
    # smaller input right after: 7 workgroups over 65 row tiles x 4 chunks
    small = _capi.GemmPlan(1, 0, 1, 1, 7, 65, 4, 8 * 2 * 4096)
    got, want, (a, b, sa, sw, base) = _pair(3, 1040, 1024, seed=2, plan=small)
    assert torch.equal(got, want)
    check_against_oracle(got, a, b, sa, sw)


@pytest.mark.parametrize("first,second", [((64, 4096, 14336), (32, 1040, 8192)),     # workgroup kernel, exchange between workgroups
                                          ((48, 2304, 16384), (17, 130, 1024)),
                                          ((16, 6144, 4096), (1, 50, 256)),          # planner's own choice at m <= 16
                                          ((8, 8192, 8192), (5, 4096, 14336))])
def test_noalloc_gemm_under_the_library_s_own_plans(first, second):
    from tests.test_gemm_gpu import check_against_oracle
    for i, (m, n, k) in enumerate((first, second)):
        got, want, (a, b, sa, sw, base) = _pair(m, n, k, seed=10 + i, accumulate=(i == 1), per_channel=(i == 0),
                                                dtype=torch.float16 if i else torch.bfloat16)
        assert torch.equal(got, want), (m, n, k)
        check_against_oracle(got, a, b, sa, sw, base=base)


def test_noalloc_gemm_k_split_with_several_windows_then_a_smaller_one():
    from hf_rocm_kernels import _capi
    for (m, n, k, grid) in ((40, 1024, 8192, 200), (20, 528, 4096, 33)):
        mt, tiles, windows = (m + 15) // 16, (n + 15) // 16, k // 2048
        plan = _capi.GemmPlan(mt, -1, 1, 0, grid, tiles, windows, 8 * 4096 + 16 * mt * 1024)
        got, want, _ = _pair(m, n, k, seed=m, plan=plan)
        assert torch.equal(got, want), (m, n, k)


def test_noalloc_gemm_takes_no_workspace_from_the_pool():
    from hf_rocm_kernels import _capi
    from hf_rocm_kernels.operators.skinny_gemm import generate_llama_gemm_data
    lib = _capi.load()
    a, b, sa, sw = generate_llama_gemm_data(8, 1040, 2048, seed=4)
    plan = _capi.GemmPlan(1, 0, 1, 2, 50, 65, 8, 8 * 2 * 4096)
    want = torch.empty((8, 1040), dtype=torch.bfloat16, device="cuda")
    assert _run(lib.hfrk_skinny_gemm_ex, a, b, sa, sw, want, plan) == 0
    side = torch.cuda.Stream()
    torch.cuda.synchronize()
    assert lib.hfrk_release_stream(side.cuda_stream) == 0      # torch hands out pooled streams: an earlier test may have used it
    got = torch.empty_like(want)
    with torch.cuda.stream(side):
        assert _run(lib.hfrk_skinny_gemm_noalloc, a, b, sa, sw, got, plan) == 0
    torch.cuda.synchronize()
    assert lib.hfrk_workspace_id(side.cuda_stream) == -1       # the stream was given no workspace
    assert torch.equal(got, want)


def test_noalloc_gemm_rejects_what_does_not_fit_its_array():
    from hf_rocm_kernels import _capi
    from hf_rocm_kernels.operators.skinny_gemm import generate_llama_gemm_data
    lib = _capi.load()
    m, n, k = 64, 4096, 4096
    a, b, sa, sw = generate_llama_gemm_data(m, n, k, seed=3)
    out = torch.zeros((m, n), dtype=torch.bfloat16, device="cuda")
    # 16 row tiles per panel x 4 activation tiles: 128 KB of partial sums per workgroup, 32 MB on 256 workgroups (the array: 16 MB)
    plan = _capi.GemmPlan(4, 16, 1, 1, 256, 16, 16, 8 * 2 * 4096 + 2 * 64 * 256)
    assert _run(lib.hfrk_skinny_gemm_ex, a, b, sa, sw, out, plan) == 0
    torch.cuda.synchronize()
    keep = out.clone()
    status = _run(lib.hfrk_skinny_gemm_noalloc, a, b, sa, sw, out, plan)
    assert status == _capi.EXCEEDS_SCRATCH and "scratch" in _capi.status_string(status)
    torch.cuda.synchronize()
    assert torch.equal(out, keep)          # nothing was launched
    # the same shape under the library's own plan fits
    assert _run(lib.hfrk_skinny_gemm_noalloc, a, b, sa, sw, out, None) == 0
    torch.cuda.synchronize()
    assert _run(lib.hfrk_skinny_gemm_ex, a, b, sa, sw, keep, None) == 0
    torch.cuda.synchronize()
    assert torch.equal(out, keep)
