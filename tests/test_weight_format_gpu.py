"""GPU tests of the weight load format: hfrk_pack_weight / hfrk_unpack_weight / hfrk_reencode_fnuz against the CPU
oracle (bit-exact: this is byte shuffling and a 256-entry code map), and the GEMM on a packed weight against the GEMM
on the row-major weight (bit-exact: same operands, same order of sums) and against the exact product.
Through the C ABI and through the Python surface (PackedWeight in place of `b`)."""
import contextlib
import ctypes

import numpy as np
import pytest
import torch

from test_gemm_gpu import all_plans, check_against_oracle

pytestmark = pytest.mark.gpu


def _lib():
    from hf_rocm_kernels import _capi
    lib = _capi.load()
    _capi.check(lib.hfrk_init(), "hfrk_init")
    return lib, _capi


def _pack(w_bytes, fmt=0):
    """[n, k] uint8 device tensor (rows may be strided) -> packed uint8 device tensor, through the C ABI"""
    lib, _capi = _lib()
    n, k = w_bytes.shape
    size = lib.hfrk_packed_weight_bytes(n, k)
    out = torch.full((size,), 0xAB, dtype=torch.uint8, device="cuda")
    _capi.check(lib.hfrk_pack_weight(w_bytes.data_ptr(), w_bytes.stride(0), fmt, out.data_ptr(), n, k, None), "hfrk_pack_weight")
    torch.cuda.synchronize()
    return out


@pytest.mark.parametrize("n,k", [(16, 256), (1, 256), (37, 512), (130, 1024), (1000, 2048), (4096, 4096)])
def test_pack_and_unpack_match_the_oracle(n, k):
    from oracle import weight_format as wf
    lib, _capi = _lib()
    g = torch.Generator().manual_seed(n + k)
    w = torch.randint(0, 256, (n, k), dtype=torch.uint8, generator=g)
    packed = _pack(w.cuda())
    assert np.array_equal(packed.cpu().numpy(), wf.pack_weight(w.numpy()))
    back = torch.full((n, k), 0xCD, dtype=torch.uint8, device="cuda")
    _capi.check(lib.hfrk_unpack_weight(packed.data_ptr(), back.data_ptr(), k, n, k, None), "hfrk_unpack_weight")
    torch.cuda.synchronize()
    assert torch.equal(back.cpu(), w)


def test_pack_reads_strided_rows_and_unpack_writes_them_without_touching_the_gaps():
    from oracle import weight_format as wf
    lib, _capi = _lib()
    n, k, stride = 50, 512, 768
    g = torch.Generator().manual_seed(1)
    buf = torch.randint(0, 256, (n, stride), dtype=torch.uint8, generator=g)
    dev = buf.cuda()
    packed = _pack(dev[:, :k])
    assert np.array_equal(packed.cpu().numpy(), wf.pack_weight(buf[:, :k].numpy()))
    out = torch.full((n, stride), 0x5A, dtype=torch.uint8, device="cuda")
    _capi.check(lib.hfrk_unpack_weight(packed.data_ptr(), out.data_ptr(), stride, n, k, None), "hfrk_unpack_weight")
    torch.cuda.synchronize()
    assert torch.equal(out[:, :k].cpu(), buf[:, :k])
    assert (out[:, k:] == 0x5A).all()


def test_round_trip_at_full_size():
    """Size-independent property at a Llama gate_up weight: unpack(pack(w)) == w, and packing is a permutation
    (same multiset of bytes; 28672 is a multiple of 16, so there is no padding)."""
    lib, _capi = _lib()
    n, k = 28672, 4096
    w = torch.randint(0, 256, (n, k), dtype=torch.uint8, device="cuda")
    packed = _pack(w)
    assert torch.equal(torch.bincount(packed.int(), minlength=256), torch.bincount(w.view(-1).int(), minlength=256))
    back = torch.empty_like(w)
    _capi.check(lib.hfrk_unpack_weight(packed.data_ptr(), back.data_ptr(), k, n, k, None), "hfrk_unpack_weight")
    torch.cuda.synchronize()
    assert torch.equal(back, w)


def test_reencode_fnuz_all_codes_tail_and_in_place():
    from oracle import weight_format as wf
    lib, _capi = _lib()
    table = torch.from_numpy(wf.reencode_table())
    codes = torch.arange(256, dtype=torch.uint8)
    for count in (256, 255, 17, 16, 1, 100003):
        src = codes.repeat(-(-count // 256))[:count].contiguous()
        if count > 256:
            src = src[torch.randperm(count, generator=torch.Generator().manual_seed(count))].contiguous()
        dev = src.cuda()
        out = torch.full((count + 16,), 0xEE, dtype=torch.uint8, device="cuda")
        _capi.check(lib.hfrk_reencode_fnuz(dev.data_ptr(), out.data_ptr(), count, None), "hfrk_reencode_fnuz")
        torch.cuda.synchronize()
        assert torch.equal(out[:count].cpu(), table[src.long()]), count
        assert (out[count:] == 0xEE).all()
        _capi.check(lib.hfrk_reencode_fnuz(dev.data_ptr(), dev.data_ptr(), count, None), "hfrk_reencode_fnuz")
        torch.cuda.synchronize()
        assert torch.equal(dev.cpu(), table[src.long()])
    assert lib.hfrk_reencode_fnuz(None, None, 0, None) == 0


def test_pack_with_fnuz_source_is_pack_of_the_reencoded_weight():
    from oracle import weight_format as wf
    n, k = 77, 512
    g = torch.Generator().manual_seed(5)
    w = torch.randint(0, 256, (n, k), dtype=torch.uint8, generator=g)
    packed = _pack(w.cuda(), fmt=1)
    assert np.array_equal(packed.cpu().numpy(), wf.pack_weight(wf.reencode_fnuz(w.numpy())))


def test_argument_errors_come_back_as_status_codes():
    lib, _capi = _lib()
    buf = torch.zeros(1 << 16, dtype=torch.uint8, device="cuda")
    p = buf.data_ptr()
    assert lib.hfrk_packed_weight_bytes(16, 100) == 0 and lib.hfrk_packed_weight_bytes(0, 256) == 0
    assert lib.hfrk_packed_weight_bytes(17, 256) == 32 * 256
    assert lib.hfrk_pack_weight(p, 100, 0, p + 4096, 16, 100, None) == _capi.K_NOT_DIVISIBLE_BY_WARPTILE_K
    assert lib.hfrk_pack_weight(p, 128, 0, p + 8192, 16, 256, None) == _capi.BAD_SHAPE        # stride < k
    assert lib.hfrk_pack_weight(p + 1, 256, 0, p + 8192, 16, 256, None) == _capi.BAD_ALIGNMENT
    assert lib.hfrk_pack_weight(p, 264, 0, p + 8192, 16, 256, None) == _capi.BAD_ALIGNMENT     # stride % 16
    assert lib.hfrk_pack_weight(p, 256, 7, p + 8192, 16, 256, None) == _capi.BAD_DTYPE
    assert lib.hfrk_pack_weight(None, 256, 0, p, 16, 256, None) == _capi.BAD_SHAPE
    assert lib.hfrk_unpack_weight(p, p + 8192, 256, 0, 256, None) == _capi.BAD_SHAPE
    assert lib.hfrk_reencode_fnuz(p + 3, p + 4096, 64, None) == _capi.BAD_ALIGNMENT


# ---- the GEMM on a packed weight -------------------------------------------------------------------------------------

def _run_fused(a, b, out, base, sa, sb, out_scale, epilogue, plan, packed):
    lib, _capi = _lib()
    m, k = a.shape
    n = b.shape[1]
    d_dtype = _capi.F16 if out.dtype == torch.float16 else _capi.BF16
    args = [a.data_ptr(), None, out.data_ptr(), None if base is None else base.data_ptr(), sa.data_ptr(), 0 if sa.numel() == 1 else 1,
            None if sb is None else sb.data_ptr(), 0 if sb is None or sb.numel() == 1 else 1,
            None if out_scale is None else out_scale.data_ptr(), m, n, k]
    ref = None if plan is None else ctypes.byref(plan)
    if packed is None:
        args[1] = b.data_ptr()
        status = lib.hfrk_skinny_gemm_fused(*args, b.stride(1), d_dtype, epilogue, ref, None)
    else:
        args[1] = packed.data_ptr()
        status = lib.hfrk_skinny_gemm_packed(*args, d_dtype, epilogue, ref, None)
    _capi.check(status, "gemm")
    torch.cuda.synchronize()
    return out


@pytest.mark.parametrize("m,n,k", [(1, 4096, 4096), (8, 6144, 4096), (16, 1040, 4096), (13, 50, 256), (4, 1000, 1024),
                                   (25, 6144, 4096), (32, 2000, 2048), (33, 256, 1024), (48, 4096, 4096), (64, 6144, 4096),
                                   (64, 1040, 8192), (40, 4096, 14336), (17, 130, 1024)])
def test_every_plan_on_a_packed_weight_equals_the_row_major_result_bit_for_bit(m, n, k):
    from hf_rocm_kernels.operators.skinny_gemm import generate_llama_gemm_data
    a, b, sa, sw = generate_llama_gemm_data(m, n, k, seed=m + n + k, per_token=True, per_channel=True)
    packed = _pack(b.t().view(torch.uint8))
    base = torch.randn((m, n), device="cuda").to(torch.bfloat16)
    # the same plan gives the same bits on both layouts; left to itself the library may plan the two layouts differently
    # (the row-split decomposition exists for row-major weights only), so the library's own choice for the packed weight
    # is passed to both
    from hf_rocm_kernels import plan_table
    plans = [plan_table.get_plan(m, n, k, packed=True)] + [p for p in all_plans(m, n, k) if p.wn != -2]
    for p in plans:
        want = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device="cuda")
        got = want.clone()
        _run_fused(a, b, want, base, sa, sw, None, 0, p, None)
        _run_fused(a, b, got, base, sa, sw, None, 0, p, packed)
        assert torch.equal(got.view(torch.int16), want.view(torch.int16)), f"plan {None if p is None else p.as_dict()}"
    check_against_oracle(got, a, b, sa, sw, base=base)


@pytest.mark.parametrize("seed", range(16))
def test_default_plan_on_random_packed_weights(seed):
    """Whatever the planner answers for a packed weight of a shape nobody swept: against the oracle, accumulating onto a base."""
    import random
    from hf_rocm_kernels.operators.skinny_gemm import generate_llama_gemm_data
    rng = random.Random(9100 + seed)
    m = rng.choice([1, 4, 5, 8, 13, 16, 17, 24, 32, 33, 48, 64])
    n = rng.choice([64 * rng.randrange(40, 200), 128 * rng.randrange(20, 100), rng.randrange(2400, 12000)])
    k = 256 * rng.choice([rng.randrange(2, 33), rng.choice([8, 12, 16, 20, 32])])
    print(f"m={m} n={n} k={k}", flush=True)
    a, b, sa, sw = generate_llama_gemm_data(m, n, k, seed=seed, per_token=True, per_channel=True)
    packed = _pack(b.t().view(torch.uint8))
    base = torch.randn((m, n), device="cuda").to(torch.bfloat16)
    got = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device="cuda")
    _run_fused(a, b, got, base, sa, sw, None, 0, None, packed)
    check_against_oracle(got, a, b, sa, sw, base=base)


@pytest.mark.parametrize("m,n,k", [(7, 1000, 1024), (40, 2048, 4096), (64, 1040, 2048)])
def test_float16_output_and_accumulation_on_a_packed_weight(m, n, k):
    from hf_rocm_kernels.operators.skinny_gemm import generate_llama_gemm_data
    a, b, sa, sw = generate_llama_gemm_data(m, n, k, seed=k + m, per_channel=True)
    packed = _pack(b.t().view(torch.uint8))
    base = torch.randn((m, n), device="cuda").to(torch.float16)
    want, got = base.clone(), base.clone()
    from hf_rocm_kernels import plan_table
    plan = plan_table.get_plan(m, n, k, packed=True)             # one decomposition for both layouts
    _run_fused(a, b, want, want, sa, sw, None, 0, plan, None)    # base = D itself: accumulate in place
    _run_fused(a, b, got, got, sa, sw, None, 0, plan, packed)
    assert torch.equal(got.view(torch.int16), want.view(torch.int16))
    check_against_oracle(got, a, b, sa, sw, base=base)


@pytest.mark.parametrize("m,n,k", [(1, 1024, 1024), (8, 28672, 4096), (16, 2080, 2048), (5, 96, 256), (40, 2080, 2048),
                                   (64, 1024, 4096)])
def test_swiglu_epilogue_on_a_packed_weight_equals_the_row_major_result(m, n, k):
    from hf_rocm_kernels import _capi
    from hf_rocm_kernels.operators.skinny_gemm import generate_llama_gemm_data
    a, b, sa, sw = generate_llama_gemm_data(m, n, k, seed=n)
    packed = _pack(b.t().view(torch.uint8))
    out_scale = torch.full((1,), 0.01, device="cuda")
    want = torch.zeros((m, n // 2), dtype=torch.uint8, device="cuda")
    got = torch.ones_like(want)
    _run_fused(a, b, want, None, sa, sw, out_scale, _capi.EPILOGUE_SWIGLU, None, None)
    _run_fused(a, b, got, None, sa, sw, out_scale, _capi.EPILOGUE_SWIGLU, None, packed)
    assert torch.equal(got, want)
    assert want.any()


def test_python_surface_takes_a_packed_weight_everywhere():
    from hf_rocm_kernels import skinny_gemm, skinny_gemm_add, skinny_gemm_scaled, skinny_gemm_swiglu
    from hf_rocm_kernels.operators.skinny_gemm import generate_llama_gemm_data
    from hf_rocm_kernels.utils.weight_format import PackedWeight, pack_weight, unpack_weight
    for m, n, k in [(8, 1024, 1024), (40, 1056, 2048)]:
        a, b, sa, sw = generate_llama_gemm_data(m, n, k, seed=3)
        pw = pack_weight(b.t())
        assert isinstance(pw, PackedWeight) and pw.shape == (k, n) and pw.stride(0) == 1
        assert torch.equal(unpack_weight(pw).view(torch.uint8), b.t().view(torch.uint8))
        scale = (sa.view(-1)[:1] * sw.view(-1)[:1]).contiguous()
        bias = torch.randn((m, n), device="cuda").to(torch.bfloat16)
        assert torch.equal(skinny_gemm(a, pw, scale, bias.clone()), skinny_gemm(a, b, scale, bias.clone()))
        one = torch.ones(1, device="cuda")
        assert torch.equal(skinny_gemm_scaled(a, pw, scale, one), skinny_gemm_scaled(a, b, scale, one))
        assert torch.equal(skinny_gemm_add(a, pw, scale, None, bias), skinny_gemm_add(a, b, scale, None, bias))
        out_scale = torch.full((1,), 0.02, device="cuda")
        assert torch.equal(skinny_gemm_swiglu(a, pw, scale, None, out_scale).view(torch.uint8),
                           skinny_gemm_swiglu(a, b, scale, None, out_scale).view(torch.uint8))


@contextlib.contextmanager
def one_plan_for_both_layouts(*shapes):
    """The same plan gives the same bits on a row-major and on a packed weight, but the library may plan the two layouts
    differently (the row-split decomposition exists for row-major weights only).  Inside this context the row-major key of
    each (m, n, k) holds the plan the library uses for the packed weight, so that the operators, which take no plan, can be
    compared bit for bit."""
    from hf_rocm_kernels import plan_table
    try:
        for m, n, k in shapes:
            plan_table.set_plan(m, n, k, plan_table.get_plan(m, n, k, packed=True))
        yield
    finally:
        plan_table.clear()
        plan_table.load_from_environment()


@pytest.mark.parametrize("fused", [False, True])
def test_llama_mlp_block_on_packed_weights(fused):
    from hf_rocm_kernels.combined_ops.llama_mlp import llama_mlp_combined_ops
    from hf_rocm_kernels.utils.fp8 import amax_scale, fp8_quantize
    from hf_rocm_kernels.utils.weight_format import pack_weight
    g = torch.Generator().manual_seed(11)
    m, hidden, inter = 8, 1024, 2816
    x = torch.randn(m, hidden, generator=g).to(torch.bfloat16).cuda()
    res = torch.randn(m, hidden, generator=g).to(torch.bfloat16).cuda()
    wn = (1 + 0.1 * torch.randn(hidden, generator=g)).to(torch.bfloat16).cuda()
    wgu = (0.02 * torch.randn(2 * inter, hidden, generator=g)).cuda()
    wd = (0.02 * torch.randn(hidden, inter, generator=g)).cuda()
    qgu, sgu = fp8_quantize(wgu, amax_scale(wgu))
    qd, sd = fp8_quantize(wd, amax_scale(wd))
    s_in, s_mid = torch.full((1,), 0.02, device="cuda"), torch.full((1,), 0.01, device="cuda")
    args = dict(rms_weight=wn, rms_epsilon=1e-5, gate_up_input_scale=s_in, gate_up_output_scale=(s_in * sgu).view(1),
                down_input_scale=s_mid, down_output_scale=(s_mid * sd).view(1), add_residual=True, fused=fused)
    with one_plan_for_both_layouts((m, 2 * inter, hidden), (m, hidden, inter)):
        want, want_res = llama_mlp_combined_ops(x, res.clone(), gate_up_weight=qgu.t(), down_weight=qd.t(), **args)
        got, got_res = llama_mlp_combined_ops(x, res.clone(), gate_up_weight=pack_weight(qgu), down_weight=pack_weight(qd), **args)
    assert torch.equal(got, want) and torch.equal(got_res, want_res)
    assert got.float().abs().sum() > 0


def test_fnuz_weights_from_the_reference_recipe_give_the_same_product_either_way():
    """A weight quantised the reference's way (utils/fp8.py:6-29: fn bits relabelled fnuz, scale doubled) computes
    the same product through the zero-copy view (scale halved), through reencode_fnuz and through pack_weight."""
    from hf_rocm_kernels import skinny_gemm_scaled
    from hf_rocm_kernels.operators.skinny_gemm import generate_llama_gemm_data
    from hf_rocm_kernels.utils.weight_format import fnuz_bits_as_ocp, pack_weight, reencode_fnuz
    m, n, k = 8, 1024, 1024
    a, b, sa, sw = generate_llama_gemm_data(m, n, k, seed=9)
    bits = b.t().contiguous().view(torch.uint8).clone()
    bits[bits == 0x80] = 0  # the reference clears -0, which is NaN in fnuz
    w_fnuz, scale_fnuz = bits.view(torch.float8_e4m3fnuz), sw * 2
    sa1, one = sa.view(-1)[:1].contiguous(), torch.ones(1, device="cuda")
    want = skinny_gemm_scaled(a, bits.view(torch.float8_e4m3fn).t(), sa1 * sw.view(-1)[:1], one)

    view, scale = fnuz_bits_as_ocp(w_fnuz, scale_fnuz)
    assert torch.equal(skinny_gemm_scaled(a, view.t(), sa1 * scale.view(-1)[:1], one), want)
    # value-preserving re-encode: values are halved on the way in, the scale stays doubled; bytes below 2^-6 round,
    # so the products agree to the GEMM's own tolerance rather than bit for bit
    re = reencode_fnuz(w_fnuz)
    got = skinny_gemm_scaled(a, re.t(), sa1 * scale_fnuz.view(-1)[:1], one)
    assert torch.allclose(got.float(), want.float(), rtol=2e-2, atol=2e-2)
    assert torch.equal(skinny_gemm_scaled(a, pack_weight(w_fnuz), sa1 * scale_fnuz.view(-1)[:1], one), got)
    bad = w_fnuz.clone().view(torch.uint8)
    bad[0, 0] = 0x80
    with pytest.raises(ValueError):
        fnuz_bits_as_ocp(bad.view(torch.float8_e4m3fnuz), scale_fnuz)


def test_packed_gemm_replays_in_a_graph():
    from hf_rocm_kernels import skinny_gemm_scaled
    from hf_rocm_kernels.operators.skinny_gemm import generate_llama_gemm_data
    from hf_rocm_kernels.utils.weight_format import pack_weight
    m, n, k = 8, 4096, 4096
    a, b, sa, sw = generate_llama_gemm_data(m, n, k, seed=2)
    pw = pack_weight(b.t())
    scale, one = (sa.view(-1)[:1] * sw.view(-1)[:1]).contiguous(), torch.ones(1, device="cuda")
    with one_plan_for_both_layouts((m, n, k)):
        want = skinny_gemm_scaled(a, b, scale, one)
    out = torch.empty_like(want)
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        skinny_gemm_scaled(a, pw, scale, one, output=out)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        skinny_gemm_scaled(a, pw, scale, one, output=out)
    for _ in range(3):
        out.zero_()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, want)


# ---- per-channel scales carried in the packed buffer ---------------------------------------------------------------------

@pytest.mark.parametrize("m,n,k", [(8, 4096, 4096), (3, 1000, 1024), (33, 50, 256), (16, 2080, 2048)])
def test_scales_stored_behind_the_packed_bytes(m, n, k):
    """hfrk_pack_weight_scaled: the packed bytes, then the n per-channel scales (zeros up to the padded row count), in one
    buffer.  The GEMM told to use them (sb_stride = HFRK_SCALES_IN_PACKED_BUFFER through the C ABI; `pw.scales`, or no
    scale_b to skinny_gemm_scaled, in Python) gives the bits of the GEMM that is handed the scales separately, on the packed
    and on the row-major weight.  In every wrapper whose scale_b may be None for "1" it means 1 for this buffer too: the
    same call gives the same numbers in both layouts."""
    from hf_rocm_kernels import skinny_gemm, skinny_gemm_add, skinny_gemm_scaled
    from hf_rocm_kernels.operators.skinny_gemm import generate_llama_gemm_data
    from hf_rocm_kernels.utils.weight_format import PackedWeight, pack_weight, packed_weight_bytes, unpack_weight
    lib, _capi = _lib()
    a, b, sa, sw = generate_llama_gemm_data(m, n, k, seed=n + k, per_token=True, per_channel=True)
    w = b.t()
    plain, scaled = packed_weight_bytes(n, k), packed_weight_bytes(n, k, scaled=True)
    n_pad = (n + 15) // 16 * 16
    assert scaled == plain + 4 * n_pad == lib.hfrk_packed_weight_bytes_scaled(n, k)
    # through the C ABI, into a buffer of a known fill
    buf = torch.full((scaled,), 0xAB, dtype=torch.uint8, device="cuda")
    _capi.check(lib.hfrk_pack_weight_scaled(w.data_ptr(), w.stride(0), 0, sw.data_ptr(), buf.data_ptr(), n, k, None), "hfrk_pack_weight_scaled")
    torch.cuda.synchronize()
    assert torch.equal(buf[:plain], _pack(w.contiguous().view(torch.uint8)))
    tail = buf[plain:].view(torch.float32)
    assert torch.equal(tail[:n], sw) and (tail[n:] == 0).all() and tail.numel() == n_pad
    assert lib.hfrk_packed_weight_scales(buf.data_ptr(), n, k) == buf.data_ptr() + plain
    assert lib.hfrk_packed_weight_scales(buf.data_ptr(), n, k + 16) is None and lib.hfrk_packed_weight_bytes_scaled(n, k + 16) == 0
    assert lib.hfrk_pack_weight_scaled(w.data_ptr(), w.stride(0), 0, None, buf.data_ptr(), n, k, None) == _capi.BAD_SHAPE
    want = torch.empty((m, n), dtype=torch.bfloat16, device="cuda")
    _run_fused(a, b, want, None, sa, sw, None, _capi.EPILOGUE_NONE, None, None)
    check_against_oracle(want, a, b, sa, sw)
    got = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device="cuda")
    status = lib.hfrk_skinny_gemm_packed(a.data_ptr(), buf.data_ptr(), got.data_ptr(), None, sa.data_ptr(), 1, None,
                                         _capi.SCALES_IN_PACKED_BUFFER, None, m, n, k, _capi.BF16, _capi.EPILOGUE_NONE, None, None)
    _capi.check(status, "hfrk_skinny_gemm_packed")
    torch.cuda.synchronize()
    with one_plan_for_both_layouts((m, n, k)):
        _run_fused(a, b, want, None, sa, sw, None, _capi.EPILOGUE_NONE, None, None)
        status = lib.hfrk_skinny_gemm_packed(a.data_ptr(), buf.data_ptr(), got.data_ptr(), None, sa.data_ptr(), 1, None,
                                             _capi.SCALES_IN_PACKED_BUFFER, None, m, n, k, _capi.BF16, _capi.EPILOGUE_NONE, None, None)
        _capi.check(status, "hfrk_skinny_gemm_packed")
        torch.cuda.synchronize()
        assert torch.equal(got, want)
    # the Python surface
    pw = pack_weight(w, sw)
    assert isinstance(pw, PackedWeight) and pw.data.numel() == scaled and torch.equal(pw.scales, sw)
    assert torch.equal(pw.data.view(torch.uint8), buf)
    assert torch.equal(unpack_weight(pw).view(torch.uint8), w.contiguous().view(torch.uint8))
    check_against_oracle(skinny_gemm_scaled(a, pw, sa, None), a, b, sa, sw)
    assert torch.equal(skinny_gemm_scaled(a, pw, sa, None), skinny_gemm_scaled(a, pack_weight(w), sa, sw))
    base = torch.randn(m, n, generator=torch.Generator().manual_seed(2)).to(torch.bfloat16).cuda()
    assert torch.equal(skinny_gemm_add(a, pw, sa, pw.scales, base), skinny_gemm_add(a, pack_weight(w), sa, sw, base))
    # no scale_b = 1, whatever the weight carries: skinny_gemm / skinny_gemm_add on the scaled buffer equal the row-major call
    with one_plan_for_both_layouts((m, n, k)):
        assert torch.equal(skinny_gemm_add(a, pw, sa, None, base), skinny_gemm_add(a, b, sa, None, base))
        one = sa[:1].contiguous()
        zeros = lambda: torch.zeros((m, n), dtype=torch.bfloat16, device="cuda")
        assert torch.equal(skinny_gemm(a, pw, one, zeros()), skinny_gemm(a, b, one, zeros()))
    # scales handed over explicitly win over the stored ones
    other = (sw * 2).contiguous()
    assert torch.equal(skinny_gemm_scaled(a, pw, sa, other), skinny_gemm_scaled(a, pack_weight(w), sa, other))
    with pytest.raises(AssertionError):
        skinny_gemm_scaled(a, pack_weight(w), sa, None)


def test_fp8_linear_keeps_packed_weight_and_scales_in_one_buffer():
    from hf_rocm_kernels.layers import Fp8Linear
    torch.manual_seed(4)
    lin = torch.nn.Linear(1024, 520, bias=True).to(torch.bfloat16).cuda()
    layer = Fp8Linear.from_float(lin, per_channel=True, packed=True)
    assert layer.weight_scale is None and layer.weight.scales is not None and layer.weight.scales.numel() == 520
    assert set(layer.state_dict()) == {"weight_data", "bias"}
    apart = Fp8Linear.from_float(lin, per_channel=True, packed=False)
    assert torch.equal(layer.weight.scales, apart.weight_scale)
    x = torch.randn(9, 1024, device="cuda").to(torch.bfloat16)
    want = lin(x).float()
    got = layer(x)
    assert (got.float() - want).norm() / want.norm() < 0.06
    twin = Fp8Linear.from_float(torch.nn.Linear(1024, 520, bias=True).to(torch.bfloat16).cuda(), per_channel=True, packed=True)
    twin.load_state_dict(layer.state_dict())
    assert torch.equal(twin(x), got)
    assert torch.equal(layer.half().to("cuda")(x), got)  # the cast reaches the bias only (x stays bfloat16: so does the output)
