"""GPU tests of the single-launch MLP block (hfrk_llama_mlp_block): its three outputs must have the same bits as the
three launches it replaces (hfrk_residual_rms, hfrk_skinny_gemm_fused with the SwiGLU epilogue, hfrk_skinny_gemm_fused
with the residual as addend) run through the C ABI with the same decompositions, and it must agree with the chained
CPU oracle like the separate kernels do."""
import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu

FP8 = torch.float8_e4m3fn


def _stream_plan(capi, m, n_out, k, row_tiles):
    """The wave-stream plan on 256 workgroups (n_out: output columns; with the SwiGLU epilogue a chunk holds a gate
    and an up tile of the same 16 columns)."""
    ma = (m + 3) // 4
    return capi.GemmPlan((ma + 3) // 4, 0, row_tiles, ma, 256, n_out // 16, k // 256, 8 * (row_tiles + (ma + 3) // 4) * 4096)


def _make(m, hidden, inter, dtype, seed, packed):
    from hf_rocm_kernels.utils.fp8 import amax_scale, fp8_quantize
    from hf_rocm_kernels.utils.weight_format import pack_weight
    g = torch.Generator().manual_seed(seed)
    wn = (1 + 0.1 * torch.randn(hidden, generator=g)).to(dtype).cuda()
    wgu = (0.02 * torch.randn(2 * inter, hidden, generator=g)).cuda()
    wd = (0.02 * torch.randn(hidden, inter, generator=g)).cuda()
    qgu, sgu = fp8_quantize(wgu, amax_scale(wgu))
    qd, sd = fp8_quantize(wd, amax_scale(wd))
    s_in, s_mid = torch.full((1,), 0.02, device="cuda"), torch.full((1,), 0.01, device="cuda")
    x = torch.randn(m, hidden, generator=g).to(dtype).cuda()
    res = torch.randn(m, hidden, generator=g).to(dtype).cuda()
    w_gu = pack_weight(qgu) if packed else qgu.t()
    w_d = pack_weight(qd) if packed else qd.t()
    return dict(x=x, res=res, wn=wn, qgu=qgu, qd=qd, w_gu=w_gu, w_d=w_d, s_in=s_in, s_mid=s_mid,
                s_gu=(s_in * sgu).view(1), s_d=(s_mid * sd).view(1))


def _three_launches(d, m, hidden, inter, dtype, packed, add_residual):
    """The same work as three C-ABI calls with the block's decompositions."""
    from hf_rocm_kernels import _capi
    lib = _capi.load()
    io = _capi.BF16 if dtype == torch.bfloat16 else _capi.F16
    stream = torch.cuda.current_stream().cuda_stream
    res = d["res"].clone()
    normalized = torch.empty(m, hidden, dtype=FP8, device="cuda")
    activated = torch.empty(m, inter, dtype=FP8, device="cuda")
    out = torch.empty(m, hidden, dtype=dtype, device="cuda")
    _capi.check(lib.hfrk_residual_rms(d["x"].data_ptr(), res.data_ptr(), d["wn"].data_ptr(), d["s_in"].data_ptr(), 1e-5,
                                      normalized.data_ptr(), None, m, hidden, 0, io, _capi.FP8_E4M3FN, 0, 0, stream), "rms")
    p1 = _stream_plan(_capi, m, inter, hidden, 2)
    p2 = _stream_plan(_capi, m, hidden, inter, 1)
    if packed:
        _capi.check(lib.hfrk_skinny_gemm_packed(normalized.data_ptr(), d["w_gu"].data.data_ptr(), activated.data_ptr(), None,
                                                d["s_gu"].data_ptr(), 0, None, 0, d["s_mid"].data_ptr(), m, 2 * inter, hidden, io,
                                                _capi.EPILOGUE_SWIGLU, ctypes.byref(p1), stream), "gate_up")
        _capi.check(lib.hfrk_skinny_gemm_packed(activated.data_ptr(), d["w_d"].data.data_ptr(), out.data_ptr(),
                                                res.data_ptr() if add_residual else None, d["s_d"].data_ptr(), 0, None, 0, None,
                                                m, hidden, inter, io, _capi.EPILOGUE_NONE, ctypes.byref(p2), stream), "down")
    else:
        _capi.check(lib.hfrk_skinny_gemm_fused(normalized.data_ptr(), d["qgu"].data_ptr(), activated.data_ptr(), None,
                                               d["s_gu"].data_ptr(), 0, None, 0, d["s_mid"].data_ptr(), m, 2 * inter, hidden, hidden, io,
                                               _capi.EPILOGUE_SWIGLU, ctypes.byref(p1), stream), "gate_up")
        _capi.check(lib.hfrk_skinny_gemm_fused(activated.data_ptr(), d["qd"].data_ptr(), out.data_ptr(),
                                               res.data_ptr() if add_residual else None, d["s_d"].data_ptr(), 0, None, 0, None,
                                               m, hidden, inter, inter, io, _capi.EPILOGUE_NONE, ctypes.byref(p2), stream), "down")
    torch.cuda.synchronize()
    return out, res, normalized, activated


def _timeouts():
    from hf_rocm_kernels import _capi
    count = ctypes.c_uint(0)
    _capi.check(_capi.load().hfrk_llama_mlp_block_timeouts(ctypes.byref(count)), "timeouts")
    return count.value


@pytest.mark.parametrize("packed", [False, True])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("m,hidden,inter", [(1, 1024, 2816), (8, 1024, 2816), (16, 2048, 4096), (5, 4096, 14336), (13, 8192, 4096)])
def test_block_has_the_bits_of_the_three_launches(m, hidden, inter, dtype, packed):
    from hf_rocm_kernels.combined_ops.llama_mlp import llama_mlp_block
    print(f"mlp block m={m} hidden={hidden} inter={inter} {dtype} packed={packed}", flush=True)
    d = _make(m, hidden, inter, dtype, seed=m + hidden, packed=packed)
    before = _timeouts()
    for add_residual in (True, False):
        want_out, want_res, want_norm, want_act = _three_launches(d, m, hidden, inter, dtype, packed, add_residual)
        scratch = (torch.empty(m, hidden, dtype=FP8, device="cuda"), torch.empty(m, inter, dtype=FP8, device="cuda"))
        res = d["res"].clone()
        out, res_out = llama_mlp_block(d["x"], res, d["wn"], 1e-5, d["w_gu"], d["s_in"], d["s_gu"], d["w_d"], d["s_mid"], d["s_d"],
                                       add_residual=add_residual, scratch=scratch)
        torch.cuda.synchronize()
        assert res_out is res and torch.equal(res, want_res)
        assert torch.equal(scratch[0].view(torch.uint8), want_norm.view(torch.uint8))
        assert torch.equal(scratch[1].view(torch.uint8), want_act.view(torch.uint8))
        assert torch.equal(out, want_out)
        assert out.float().abs().sum() > 0
    assert _timeouts() == before
