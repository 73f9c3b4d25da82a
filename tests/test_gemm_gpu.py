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


def oracle_checker(a, b, sa, sb, out_dtype, base=None, rtol=1e-2, atol=1e-2):
    """The oracle's answers for one set of inputs, computed once: returns check(out) for any number of device results of
    the same product (e.g. one per plan)."""
    og = _oracle()
    a_c, b_c = a.cpu(), b.cpu()
    sa_c, sb_c = sa.cpu(), sb.cpu()
    base_c = None if base is None else base.cpu()
    ref32 = og.reference_skinny_gemm(a_c, b_c, sa_c, sb_c, output=base_c, out_dtype=out_dtype).float()
    exact = og.exact_skinny_gemm(a_c, b_c, sa_c, sb_c, output=base_c)
    tol = atol + rtol * ref32.abs()
    bound = og.error_bound(a_c, b_c, sa_c, sb_c, out_dtype, exact)

    def check(out):
        assert out.dtype == out_dtype
        got = out.cpu()
        assert not got.isnan().any()
        err32 = (got.float() - ref32).abs()
        assert (err32 <= tol).all(), f"max excess over rtol/atol: {(err32 - tol).max().item()}"
        worst = ((got.double() - exact).abs() / bound).max().item()
        assert worst <= 1.0, f"error is {worst} x the bound (1 ulp + 2^-16 sum|a b|) from the exact product"
    return check


def check_against_oracle(out, a, b, sa, sb, base=None, rtol=1e-2, atol=1e-2):
    oracle_checker(a, b, sa, sb, out.dtype, base=base, rtol=rtol, atol=atol)(out)


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
    if m <= 32:  # wave-stream decomposition: grids that split row groups between workgroups in different ways
        ma, kc = (m + 3) // 4, k // 256
        for rt in (1, 2):
            if not ((rt == 1 and ma <= 4) or (rt == 2 and 3 <= ma <= 8)):
                continue
            groups = (n + 16 * rt - 1) // (16 * rt)
            for grid in sorted({min(g, groups * kc) for g in (256, 200, 7, 512, 1)}):
                plans.append(_capi.GemmPlan((ma + 3) // 4, 0, rt, ma, grid, groups, kc, 8 * (rt + (ma + 3) // 4) * 4096))
    if m <= 32 and k >= 512:  # row-split decomposition: bands of rows per workgroup, cut into tiles of different heights
        units = (n + 3) // 4
        ma = (m + 3) // 4 if m <= 16 else (6 if m <= 24 else 8)  # above 16 rows: two activation tiles, two weight tiles per chunk
        for rt in ((1, 2) if m <= 16 else (2,)):
            for grid in sorted({min(g, units) for g in (256, 200, 7, 512, 1, 77)}):
                plans.append(_capi.GemmPlan(1, -2, rt, ma, grid, units, k // 256, 8 * (rt + (ma + 3) // 4) * 4096))
        tiles = (n + 15) // 16  # the same on bands of whole 16-row tiles (the form that also reads the packed load format)
        for rt in ((1, 2) if m <= 16 else (2,)):
            for grid in sorted({min(g, tiles) for g in (256, 200, 7, 384, 1, 77)}):
                plans.append(_capi.GemmPlan(1, -3, rt, ma, grid, tiles, k // 256, 8 * (rt + (ma + 3) // 4) * 4096))
    for wave_k in (256, 512, 1024):  # K-split decomposition
        if k % (8 * wave_k) == 0 and (wave_k < 1024 or mt <= 2):
            tiles, windows = (n + 15) // 16, k // (8 * wave_k)
            for grid in sorted({min(g, tiles * windows) for g in (256, 200, 7, 1)}):
                plans.append(_capi.GemmPlan(mt, -1, wave_k // 256, 0, grid, tiles, windows, 8 * (wave_k // 256) * 4096 + 16 * mt * 1024))
    for wn, rt in [(w, r) for w in (1, 2, 4, 8) for r in (1, 2)]:  # row waves x weight tiles per wave
        wk = 8 // wn
        for ch in ((1, 2) if rt == 1 else (1,)):
            ks = 256 * wk * ch
            if k % ks:
                continue
            lds = 8 * rt * 4096 + 2 * 16 * mt * ks
            if lds > 160 * 1024:
                continue
            panels = (n + 16 * wn * rt - 1) // (16 * wn * rt)
            slabs = k // ks
            units = panels * slabs
            for grid in sorted({min(256, units), min(200, units), min(7, units)}):
                p = _capi.GemmPlan(mt, wn * rt, wk, ch, grid, panels, slabs, lds)
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


@pytest.mark.parametrize("m,n,k", [(1, 16384, 8192), (8, 8192, 16384), (5, 14336, 8192), (24, 8192, 8192), (32, 6144, 4096), (19, 16384, 2048),
                                   (33, 28672, 4096), (64, 57344, 8192), (40, 16384, 4096), (36, 14336, 4096), (48, 32768, 2048),
                                   (20, 5120, 5120), (32, 3072, 3072), (28, 4096, 5120), (64, 10240, 3072), (48, 12288, 8192),
                                   (33, 13312, 14336), (48, 24576, 16384), (64, 20480, 3072), (40, 16384, 16384),
                                   (48, 13312, 16384), (32, 6144, 16384), (64, 8192, 16384), (17, 6144, 14336),
                                   (20, 14336, 5120), (24, 16384, 14336), (18, 13312, 8192),
                                   (8, 5120, 8192), (4, 5120, 8192), (16, 5120, 5120), (7, 7168, 14336), (5, 11264, 5120),
                                   (48, 8192, 3072), (33, 7168, 5120), (40, 5120, 5120)])
def test_default_plan_on_shapes_with_rules_of_their_own(m, n, k):
    """Weights whose bands come to 512 KB (two weight tiles per chunk, or 256 workgroups instead of 224), ragged bands of
    20..44 rows (two weight tiles per chunk from 5 rows on), the 17..32 row
    variants of the row-split kernel, and from 17 rows on the workgroup kernel on whole row panels per workgroup (256,
    128 or 64 rows tall, on 160 to 256 workgroups, or 128-row panels whose k is cut between 2 or 4 workgroups), as the planner
    chooses them: against the oracle, plain and accumulating."""
    from hf_rocm_kernels import _capi
    from hf_rocm_kernels.operators.skinny_gemm import generate_llama_gemm_data
    p = _capi.plan(m, n, k)
    if m <= 16 or (m <= 32 and (n <= 8192 or k == 2048) and (k <= 8192 or m <= 24)):
        assert p.wn == -2
    else:
        panels = n // (16 * p.wn)
        assert p.wn in (2, 4, 8, 16) and (panels % p.grid == 0 or p.grid % panels == 0), p.as_dict()   # whole panels, or whole fractions
    a, b, sa, sw = generate_llama_gemm_data(m, n, k, seed=m + n + k, per_token=True, per_channel=True)
    out = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device="cuda")
    run_ex(a, b, sa, sw, out, accumulate=False)
    check_against_oracle(out, a, b, sa, sw)
    base = torch.randn(m, n, generator=torch.Generator().manual_seed(5)).to(torch.bfloat16).cuda()
    out = base.clone()
    run_ex(a, b, sa, sw, out, accumulate=True)
    check_against_oracle(out, a, b, sa, sw, base=base)


@pytest.mark.parametrize("seed", range(24))
def test_default_plan_on_random_shapes(seed):
    """The planner's rules were read off sweeps of particular shapes; whatever they answer for a shape nobody swept must still
    be the right product: seeded random row counts, weight heights (ragged ones too) and k, per-token and per-channel scales,
    plain and accumulating, against the oracle."""
    import random
    from hf_rocm_kernels.operators.skinny_gemm import generate_llama_gemm_data
    rng = random.Random(7000 + seed)
    m = rng.choice([1, 3, 4, 5, 8, 9, 13, 16, 17, 20, 24, 25, 31, 32, 33, 47, 48, 50, 64])
    n = rng.choice([4 * rng.randrange(600, 3100), 64 * rng.randrange(40, 200), 128 * rng.randrange(20, 100), rng.randrange(2400, 12000)])
    k = 256 * rng.choice([rng.randrange(2, 33), rng.choice([8, 12, 16, 20, 32])])
    a, b, sa, sw = generate_llama_gemm_data(m, n, k, seed=seed, per_token=True, per_channel=True)
    print(f"m={m} n={n} k={k}", flush=True)
    out = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device="cuda")
    run_ex(a, b, sa, sw, out, accumulate=False)
    check_against_oracle(out, a, b, sa, sw)
    base = torch.randn(m, n, generator=torch.Generator().manual_seed(seed)).to(torch.bfloat16).cuda()
    out = base.clone()
    run_ex(a, b, sa, sw, out, accumulate=True)
    check_against_oracle(out, a, b, sa, sw, base=base)


@pytest.mark.parametrize("m,n,k", [(8, 512, 2048), (16, 1040, 4096), (33, 256, 1024), (64, 6144, 4096), (5, 4096, 14336),
                                   (1, 50, 256), (13, 6144, 4096), (4, 1000, 1024),
                                   (32, 2000, 2048), (20, 1040, 1024), (25, 6144, 4096), (12, 28672, 4096),
                                   (32, 1040, 8192), (48, 4096, 4096), (9, 528, 16384), (17, 4096, 14336), (24, 1000, 2048), (29, 4100, 1024),
                                   (5, 1027, 768), (16, 4099, 512), (2, 2050, 1024), (11, 1533, 2048)])   # n % 4 != 0: element-wise stores
def test_every_plan_gives_the_same_answer(m, n, k):
    from hf_rocm_kernels.operators.skinny_gemm import generate_llama_gemm_data
    a, b, sa, sw = generate_llama_gemm_data(m, n, k, seed=7)
    plans = all_plans(m, n, k)
    assert plans
    check = oracle_checker(a, b, sa, sw, torch.bfloat16)
    for p in plans:
        out = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device="cuda")
        run_ex(a, b, sa, sw, out, accumulate=False, plan=p)
        try:
            check(out)
        except AssertionError as e:
            raise AssertionError(f"plan {p.as_dict()}: {e}")


@pytest.mark.parametrize("m,n,k,grid,rt", [(3, 2048, 4096, 4, 1), (8, 2048, 4096, 2, 2), (5, 1024, 8192, 2, 1), (1, 4096, 4096, 8, 1),
                                          (16, 2048, 4096, 4, 2), (12, 1024, 8192, 3, 1), (9, 6144, 4096, 256, 2)])
def test_row_split_plans_that_rotate_k(m, n, k, grid, rt):
    """Row-split plans under which every workgroup starts at its own point in k and wraps round (rows a multiple of 4 KB
    apart and either every wave's run a multiple of 16 chunks long, or 9+ activation rows on bands of 4+ units): against
    the oracle, on a contiguous weight and on one whose rows are 8 KB / 12 KB apart with NaN codes behind k (a rotation that
    left the row's k bytes could not pass), plain and accumulating."""
    from hf_rocm_kernels import _capi
    from hf_rocm_kernels.operators.skinny_gemm import generate_llama_gemm_data
    units = (n + 3) // 4
    per_band = units // grid
    tiles = -(-per_band // (4 * rt))
    assert (tiles * (k // 256)) % 128 == 0 or (m >= 9 and units >= 4 * grid), "the case is meant to switch the rotation on"
    a, b, sa, sw = generate_llama_gemm_data(m, n, k, seed=m + n + k + grid, per_token=True, per_channel=True)
    wide = torch.full((n, k + 4096), 0x7F, dtype=torch.uint8, device="cuda")
    wide[:, :k] = b.t().contiguous().view(torch.uint8)
    b_view = wide.view(torch.float8_e4m3fn)[:, :k].t()
    plan = _capi.GemmPlan(1, -2, rt, (m + 3) // 4, grid, units, k // 256, 8 * (rt + 1) * 4096)
    for weight in (b, b_view):
        out = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device="cuda")
        run_ex(a, weight, sa, sw, out, accumulate=False, plan=plan)
        check_against_oracle(out, a, b, sa, sw)
    base = torch.randn(m, n, generator=torch.Generator().manual_seed(3)).to(torch.float16).cuda()
    out = base.clone()
    run_ex(a, b_view, sa, sw, out, accumulate=True, plan=plan)
    check_against_oracle(out, a, b, sa, sw, base=base)


@pytest.mark.parametrize("m,n,k", [(1, 4096, 4096 + 128), (8, 1000, 640), (16, 6144, 4096 + 64), (32, 2048, 1152),
                                   (33, 1024, 640), (64, 4096, 4096 + 128), (5, 256, 144), (3, 128, 16), (12, 4096, 1008)])
def test_k_that_ends_inside_a_chunk(m, n, k):
    """k % 16 == 0 but k % 256 != 0 (the reference takes such k with its narrow tiles, skinny_gemm_caller.cu:33-48): the
    last chunk of every row is cut short.  The weight is a view of wider rows whose bytes beyond k are NaN codes, so a
    kernel that reads past k, in either operand, cannot pass; above 32 rows the call runs as two launches."""
    from hf_rocm_kernels import _capi
    from hf_rocm_kernels.operators.skinny_gemm import generate_llama_gemm_data
    lib = _capi.load()
    a, b, sa, sw = generate_llama_gemm_data(m, n, k, seed=m + n + k, per_token=True, per_channel=True)
    wide = torch.full((n, k + 112), 0x7F, dtype=torch.uint8, device="cuda")
    wide[:, :k] = b.t().contiguous().view(torch.uint8)
    b_view = wide.view(torch.float8_e4m3fn)[:, :k].t()
    assert b_view.stride() == (1, k + 112)
    for weight in (b, b_view):
        out = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device="cuda")
        run_ex(a, weight, sa, sw, out, accumulate=False)
        check_against_oracle(out, a, b, sa, sw)
    base = torch.randn(m, n, generator=torch.Generator().manual_seed(1)).to(torch.float16).cuda()
    out = base.clone()
    run_ex(a, b_view, sa, sw, out, accumulate=True)
    check_against_oracle(out, a, b, sa, sw, base=base)
    # every explicit plan of the kernel that cuts a chunk short; the others and the packed format refuse
    kc = (k + 255) // 256
    plans = [p for p in all_plans(m, n, (k // 256) * 256 or 256) if p.wn == 0] if m <= 32 else []
    for p in plans:
        p.slabs = kc
        p.grid = min(p.grid, p.panels * kc)
        out = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device="cuda")
        try:
            run_ex(a, b_view, sa, sw, out, accumulate=False, plan=p)
            check_against_oracle(out, a, b, sa, sw)
        except (AssertionError, RuntimeError) as e:
            raise AssertionError(f"plan {p.as_dict()}: {e}")
    refused = _capi.GemmPlan((m + 15) // 16, 8, 1, 1, 1, (n + 127) // 128, max(1, k // 256), 8 * 4096 + 2 * 16 * ((m + 15) // 16) * 256)
    out = torch.zeros((m, n), dtype=torch.bfloat16, device="cuda")
    assert lib.hfrk_skinny_gemm_ex(a.data_ptr(), b.data_ptr(), out.data_ptr(), sa.data_ptr(), 1, sw.data_ptr(), 1, m, n, k, k,
                                   _capi.BF16, 0, ctypes.byref(refused), None) == _capi.K_NOT_DIVISIBLE_BY_WARPTILE_K
    assert lib.hfrk_packed_weight_bytes(n, k) == 0
    if k % 64 == 0:  # the reference's operator: one combined scale, accumulating into float16
        from hf_rocm_kernels import skinny_gemm
        scale = (sa[:1] * sw[:1]).contiguous()
        check_against_oracle(skinny_gemm(a, b_view, scale), a, b, scale, torch.ones(1).cuda())


# ---- the operator surface: torch.ops._HFRK_C / hf_rocm_kernels.skinny_gemm ----------------------------------------

_reference_matrix_oracle = {}


@pytest.mark.parametrize("repeat_id", "abcde")
@pytest.mark.parametrize("k", [256, 1024, 16384])
@pytest.mark.parametrize("n", [128, 1024, 6656, 13312])
@pytest.mark.parametrize("m", [1, 2, 3, 4, 5, 6, 7, 8, 10, 11, 12, 16, 17, 32])
def test_skinny_gemm_reference_matrix(m, n, k, repeat_id):
    """The reference's own test matrix and data recipe (tests/test_skinny_gemm.py:21-34: the same seed five times, its only
    probe for run-to-run differences), with its pass criterion (max abs error <= 0.125) and the tighter ones of this build.
    The five repeats see the same operands, so the oracle's three results are computed once per shape."""
    from hf_rocm_kernels import skinny_gemm
    from hf_rocm_kernels.operators.skinny_gemm import generate_skinny_gemm_data
    from hf_rocm_kernels.utils.testing import compare_x_with_ref
    a, b, scale, out = generate_skinny_gemm_data(m, n, k, seed=0, out_dtype=torch.float16)
    got = skinny_gemm(a, b, scale, out.clone())
    assert got.dtype == torch.float16
    og = _oracle()
    one = torch.ones(1)
    if (m, n, k) not in _reference_matrix_oracle:
        _reference_matrix_oracle.clear()   # (parametrisation keeps a shape's repeats next to each other)
        a_c, b_c, s_c = a.cpu(), b.cpu(), scale.cpu()
        exact = og.exact_skinny_gemm(a_c, b_c, s_c, one)
        _reference_matrix_oracle[(m, n, k)] = (a_c.view(torch.uint8).clone(), og.reference_skinny_gemm(a_c, b_c, s_c, one, out_dtype=torch.float16),
                                               exact, og.error_bound(a_c, b_c, s_c, one, torch.float16, exact))
    a_codes, ref, exact, bound = _reference_matrix_oracle[(m, n, k)]
    assert torch.equal(a.cpu().view(torch.uint8), a_codes)   # same seed, same operands
    g = got.cpu()
    assert not g.isnan().any()
    max_err, _, _ = compare_x_with_ref(g.float(), ref.float())
    # 0.125 is the reference's threshold; where |result| >= 256 one float16 step is already 0.25, so a single
    # rounding-boundary flip against the fp32 path is allowed there (the exact-product check below is the tight one)
    assert max_err <= max(0.125, float(og.ulp16(ref.float().abs().max(), torch.float16)))
    err32 = (g.float() - ref.float()).abs()
    assert (err32 <= 1e-2 + 1e-2 * ref.float().abs()).all()                       # rtol / atol 1e-2 against the fp32 path
    worst = ((g.double() - exact).abs() / bound).max().item()
    assert worst <= 1.0, f"error is {worst} x the bound (1 ulp + 2^-16 sum|a b|) from the exact product"
    again = skinny_gemm(a, b, scale, out.clone())
    assert torch.equal(got, again), "results differ between two runs on the same input"


def test_accumulates_into_output_like_the_reference():
    from hf_rocm_kernels import skinny_gemm
    from hf_rocm_kernels.operators.skinny_gemm import generate_llama_gemm_data
    m, n, k = 8, 4096, 4096
    a, b, sa, sw = generate_llama_gemm_data(m, n, k, seed=5)
    scale = (sa * sw).contiguous()
    g = torch.Generator().manual_seed(6)
    bias = torch.randn(m, n, generator=g).to(torch.bfloat16).cuda()
    out = skinny_gemm(a, b, scale, bias.clone())
    check_against_oracle(out, a, b, scale, torch.ones(1).cuda(), base=bias)
    # output=None allocates float16 zeros, as the reference does (operators/skinny_gemm/wrapped.py:119)
    out0 = skinny_gemm(a, b, scale)
    assert out0.dtype == torch.float16
    check_against_oracle(out0, a, b, scale, torch.ones(1).cuda())


@pytest.mark.parametrize("m,n,k", [(m, n, k) for n, k in [(4096, 4096), (28672, 4096), (4096, 14336)] for m in (16, 32, 64)] + [(17, 1000, 512)])
def test_per_token_and_per_channel_scales(m, n, k):
    """Per-token activation scales with two outlier rows scaled x20, per-output-channel weight scales: every (shape, row count)
    cell of the benchmark configuration that exercises them, at full size against the oracle, plus a ragged shape."""
    from hf_rocm_kernels import skinny_gemm_scaled
    from hf_rocm_kernels.operators.skinny_gemm import generate_llama_gemm_data
    a, b, sa, sw = generate_llama_gemm_data(m, n, k, seed=9, per_token=True, per_channel=True, outlier_rows=(1, m - 1))
    out = skinny_gemm_scaled(a, b, sa, sw)
    check_against_oracle(out, a, b, sa, sw)
    g = torch.Generator().manual_seed(10)
    base = torch.randn(m, n, generator=g).to(torch.float16).cuda()
    out = skinny_gemm_scaled(a, b, sa, sw, output=base.clone(), accumulate=True)
    check_against_oracle(out, a, b, sa, sw, base=base)


def test_full_size_properties_llama70b_down():
    """The largest K of the Llama-3-70B shapes (8192 x 28672), checked through size-independent properties instead of the oracle:
    zero activations give the bias back bit for bit, a one-hot activation row returns a scaled weight column
    exactly, and the product is linear in the output scale."""
    from hf_rocm_kernels import skinny_gemm
    n, k, m = 8192, 28672, 4
    g = torch.Generator().manual_seed(12)
    w = (torch.randn(n, k, generator=g) * 0.02 / 0.0003).clamp(-448, 448).to(torch.float8_e4m3fn).cuda()
    bias = torch.randn(m, n, generator=g).to(torch.bfloat16).cuda()
    zero = torch.zeros(m, k).to(torch.float8_e4m3fn).cuda()
    one = torch.ones(1).cuda()
    assert torch.equal(skinny_gemm(zero, w.t(), one, bias.clone()), bias)
    hot = torch.zeros(m, k)
    cols = [0, 255, 14336, 28671]
    for i, c in enumerate(cols):
        hot[i, c] = 2.0
    out = skinny_gemm(hot.to(torch.float8_e4m3fn).cuda(), w.t(), torch.tensor([0.5]).cuda())
    for i, c in enumerate(cols):
        assert torch.equal(out[i].float(), w[:, c].float())   # every e4m3 value is a float16 value
    a = torch.randn(m, k, generator=g).clamp(-4, 4).to(torch.float8_e4m3fn).cuda()
    o1 = skinny_gemm(a, w.t(), torch.tensor([2.0 ** -12]).cuda(), torch.zeros_like(bias))
    o4 = skinny_gemm(a, w.t(), torch.tensor([2.0 ** -10]).cuda(), torch.zeros_like(bias))
    assert torch.equal(o4.float(), o1.float() * 4)       # power-of-two scales commute with the rounding


def test_status_codes_and_misuse():
    from hf_rocm_kernels import _capi, skinny_gemm
    from hf_rocm_kernels.operators.skinny_gemm.binding import _skinny_gemm
    a = torch.zeros(8, 384).to(torch.float8_e4m3fn).cuda()
    b = torch.zeros(128, 384).to(torch.float8_e4m3fn).cuda().t()
    d = torch.zeros(8, 128, dtype=torch.bfloat16).cuda()
    one = torch.ones(1).cuda()
    knobs = dict(split_k=1, A_producers=3, B_producers=4, consumers=3, a_lanes=1, b_lanes=4, qsize=3, op_m=8, ops=4)
    assert _skinny_gemm(a, b, one, d, **knobs) == _capi.K_NOT_DIVISIBLE_BY_WARPTILE_K      # k = 384
    assert torch.equal(skinny_gemm(a, b, one, d), torch.zeros_like(d))   # the wrapper names a tile that divides 384: (512/16)*4
    a = torch.zeros(8, 392).to(torch.float8_e4m3fn).cuda()
    b = torch.zeros(128, 392).to(torch.float8_e4m3fn).cuda().t()
    with pytest.raises(RuntimeError, match="status 3"):
        skinny_gemm(a, b, one, d)                                                          # k % 16 != 0: the wrapper raises
    a = torch.zeros(8, 256).to(torch.float8_e4m3fn).cuda()
    b = torch.zeros(127, 256).to(torch.float8_e4m3fn).cuda().t()
    d = torch.zeros(8, 127, dtype=torch.bfloat16).cuda()
    assert _skinny_gemm(a, b, one, d, **knobs) == _capi.N_NOT_EVEN
    b = torch.zeros(128, 256).to(torch.float8_e4m3fn).cuda().t()
    d = torch.zeros(8, 128, dtype=torch.bfloat16).cuda()
    assert _skinny_gemm(a, b, one, d, **dict(knobs, consumers=12)) == _capi.TOO_MANY_WARPS
    assert _skinny_gemm(a, b, one, d, **dict(knobs, qsize=1)) == _capi.QSIZE_TOO_SMALL
    assert _skinny_gemm(a, b, one, d, **dict(knobs, op_m=7)) == _capi.INVALID_CONFIG
    assert _skinny_gemm(a, b, one, d, **knobs) == _capi.SUCCESS
    fnuz = a.view(torch.uint8).view(torch.float8_e4m3fnuz)
    with pytest.raises(RuntimeError, match="e4m3fnuz"):
        torch.ops._HFRK_C.skinny_gemm_tb(fnuz, b, d, one, 1, 3, 4, 3, 1, 4, 3, 8, 4)
    with pytest.raises(RuntimeError, match="float16 or bfloat16"):
        torch.ops._HFRK_C.skinny_gemm_tb(a, b, d.float(), one, 1, 3, 4, 3, 1, 4, 3, 8, 4)


def test_weight_view_with_row_stride():
    """B may be a column slice of a wider weight: row stride larger than k (reference: b_stride = B.stride(1))."""
    from hf_rocm_kernels import skinny_gemm
    from hf_rocm_kernels.operators.skinny_gemm import generate_llama_gemm_data
    m, n, k = 8, 512, 1024
    a, b_full, sa, sw = generate_llama_gemm_data(m, n, 2 * k, seed=13)
    a = a[:, :k].contiguous()
    b = b_full[k:, :]                      # [k, n] view, stride (1, 2k)
    assert b.stride() == (1, 2 * k)
    scale = (sa * sw).contiguous()
    out = skinny_gemm(a, b, scale)
    check_against_oracle(out, a, b.contiguous() if False else b, scale, torch.ones(1).cuda())


def test_capturable_in_a_hip_graph():
    from hf_rocm_kernels import skinny_gemm
    from hf_rocm_kernels.operators.skinny_gemm import generate_llama_gemm_data
    m, n, k = 8, 6144, 4096
    a, b, sa, sw = generate_llama_gemm_data(m, n, k, seed=14)
    scale = (sa * sw).contiguous()
    eager = skinny_gemm(a, b, scale)
    out = torch.zeros_like(eager)
    stream = torch.cuda.Stream()
    with torch.cuda.stream(stream):
        skinny_gemm(a, b, scale, out)      # warm-up outside capture
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    out.zero_()
    with torch.cuda.graph(graph, stream=stream):
        skinny_gemm(a, b, scale, out)
    for _ in range(3):
        out.zero_()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, eager)


# ---- fused forms: residual addend and SwiGLU epilogue -----------------------------------------------------------------

@pytest.mark.parametrize("m,n,k", [(1, 4096, 14336), (8, 4096, 4096), (16, 1040, 1024), (13, 130, 512), (32, 4096, 4096),
                                   (64, 1000, 2048)])
def test_base_addend_is_read_not_written(m, n, k):
    """D = base + scale * A.B with base a separate tensor: one fp32 sum, one rounding; base stays untouched."""
    from hf_rocm_kernels import skinny_gemm_add
    from hf_rocm_kernels.operators.skinny_gemm import generate_llama_gemm_data
    a, b, sa, sw = generate_llama_gemm_data(m, n, k, seed=31)
    base = torch.randn(m, n, generator=torch.Generator().manual_seed(5)).to(torch.bfloat16).cuda()
    keep = base.clone()
    out = skinny_gemm_add(a, b, sa, sw, base)
    assert torch.equal(base, keep)
    check_against_oracle(out, a, b, sa, sw, base=keep)
    # in place (base is the output) gives the same bits
    again = skinny_gemm_add(a, b, sa, sw, base, output=base)
    assert again.data_ptr() == base.data_ptr() and torch.equal(again, out)


def _swiglu_oracle(a, w, sa, sb, out_scale, dtype):
    """(fp8 result of the oracle chain, tolerance in fp8 units).  Two correct GEMMs may round a 16-bit projection
    differently: each lies within `error_bound` (1 ulp + 2^-16 sum|a b|) of the exact product, so gate and up can
    differ by twice that, which moves silu(gate) * up by at most 1.1 |up| dgate + |silu(gate)| dup (|silu'| <= 1.1);
    on top of that the fp8 rounding may flip by one step."""
    og = _oracle()
    from oracle import swiglu as osw
    a_c, w_c, sa_c, sb_c = a.cpu(), w.cpu(), sa.cpu(), sb.cpu()
    gate_up = og.reference_skinny_gemm(a_c, w_c, sa_c, sb_c, out_dtype=dtype)
    ref = osw.reference_swiglu(gate_up, out_scale.cpu())
    exact = og.exact_skinny_gemm(a_c, w_c, sa_c, sb_c)
    bound = og.error_bound(a_c, w_c, sa_c, sb_c, dtype, exact)
    half = exact.shape[1] // 2
    g, u = exact[:, :half], exact[:, half:]
    dg, du = 2 * bound[:, :half], 2 * bound[:, half:]
    silu = g / (1 + torch.exp(-g))
    moved = (1.1 * u.abs() * dg + silu.abs() * du + 1.1 * dg * du) / float(out_scale)
    step = torch.maximum(ref.float().abs() * 2.0 ** -3, torch.tensor(2.0 ** -9))
    return ref, (step + moved).float()


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("per_channel", [False, True])
@pytest.mark.parametrize("m,n,k", [(1, 512, 1024), (5, 2080, 512), (8, 28672, 4096), (13, 1024, 2048), (16, 28672, 4096),
                                   (16, 64, 256), (17, 1024, 4096), (32, 28672, 4096), (40, 4160, 2048), (64, 2048, 2048),
                                   (64, 28672, 4096), (8, 1024, 640), (3, 4160, 4096 + 128),
                                   (32, 16384, 8192), (20, 4160, 3072), (24, 8192, 1024), (17, 2080, 8192)])
def test_swiglu_epilogue_matches_the_two_kernel_chain(m, n, k, per_channel, dtype):
    """One launch (GEMM with SwiGLU epilogue) against GEMM -> 16-bit -> swiglu, on the device and in the oracle.
    The two device paths may sum K in a different order, so a 16-bit projection can differ by one rounding and an
    fp8 output by one step; such flips must be rare and never larger."""
    from hf_rocm_kernels import skinny_gemm_scaled, skinny_gemm_swiglu, swiglu
    from hf_rocm_kernels.operators.skinny_gemm import generate_llama_gemm_data
    a, w, sa, sw = generate_llama_gemm_data(m, n, k, seed=40 + m, per_token=(m > 4), per_channel=per_channel, weight_std=0.05)
    out_scale = torch.tensor([8.0 / 448], dtype=torch.float32).cuda()
    fused = skinny_gemm_swiglu(a, w, sa, sw, out_scale, intermediate_dtype=dtype)
    assert fused.dtype == torch.float8_e4m3fn and fused.shape == (m, n // 2)
    gate_up = skinny_gemm_scaled(a, w, sa, sw, output=torch.empty(m, n, dtype=dtype).cuda())
    chain = swiglu(gate_up, out_scale)
    ref, tol = _swiglu_oracle(a, w, sa, sw, out_scale, dtype)
    f = fused.cpu().float()
    assert not f.isnan().any()
    for name, other in (("device chain", chain.cpu().float()), ("oracle", ref.float())):
        d = (f - other).abs()
        assert (d <= tol).all(), (name, float((d / tol).max()))
        assert (d > 0).float().mean() < 0.02, (name, float((d > 0).float().mean()))


@pytest.mark.parametrize("seed", range(12))
def test_swiglu_epilogue_on_random_shapes(seed):
    """The fused projection + SwiGLU under whatever plan the library picks for a shape nobody swept (row-split bands of output
    columns, wave-stream, K-split above 16 rows, or the two-kernel fallback where no epilogue exists): against the oracle."""
    import random
    from hf_rocm_kernels import skinny_gemm_swiglu
    from hf_rocm_kernels.operators.skinny_gemm import generate_llama_gemm_data
    rng = random.Random(5300 + seed)
    m = rng.choice([1, 2, 4, 5, 8, 12, 16, 17, 32, 40, 64])
    n = 32 * rng.choice([rng.randrange(16, 400), rng.randrange(100, 900)])
    k = 256 * rng.choice([rng.randrange(2, 33), 8, 16, 16, 32])
    print(f"m={m} n={n} k={k}", flush=True)
    a, w, sa, sw = generate_llama_gemm_data(m, n, k, seed=seed, per_token=(m > 4), per_channel=bool(seed & 1), weight_std=0.05)
    out_scale = torch.tensor([8.0 / 448], dtype=torch.float32).cuda()
    fused = skinny_gemm_swiglu(a, w, sa, sw, out_scale)
    assert fused.dtype == torch.float8_e4m3fn and fused.shape == (m, n // 2)
    ref, tol = _swiglu_oracle(a, w, sa, sw, out_scale, torch.bfloat16)
    f = fused.cpu().float()
    assert not f.isnan().any()
    d = (f - ref.float()).abs()
    assert (d <= tol).all(), float((d / tol).max())
    assert (d > 0).float().mean() < 0.02, float((d > 0).float().mean())


def test_swiglu_epilogue_limits_and_fallback():
    from hf_rocm_kernels import _capi, skinny_gemm_swiglu
    from hf_rocm_kernels.operators.skinny_gemm import generate_llama_gemm_data
    lib = _capi.load()
    a, w, sa, sw = generate_llama_gemm_data(17, 512, 512, seed=3)
    out_scale = torch.ones(1).cuda()
    out = torch.empty(17, 256, dtype=torch.float8_e4m3fn).cuda()
    args = lambda m, n: (a.data_ptr(), w.data_ptr(), out.data_ptr(), None, sa.data_ptr(), 0, sw.data_ptr(), 0,
                         out_scale.data_ptr(), m, n, 512, 512, _capi.BF16, _capi.EPILOGUE_SWIGLU, None, None)
    assert lib.hfrk_skinny_gemm_fused(*args(17, 512)) == _capi.BAD_SHAPE      # m > 16 on a weight too small to deal out: callers run the two kernels
    assert lib.hfrk_skinny_gemm_fused(*args(8, 496)) == _capi.BAD_SHAPE       # n % 32 != 0
    bad = list(args(8, 512)); bad[3] = out.data_ptr()
    assert lib.hfrk_skinny_gemm_fused(*bad) == _capi.BAD_SHAPE                # base with the SwiGLU epilogue
    bad = list(args(8, 512)); bad[14] = 7
    assert lib.hfrk_skinny_gemm_fused(*bad) == _capi.INVALID_CONFIG
    # above 16 rows the epilogue exists where one K-split window covers k (2048, 4096): k = 512 is not among them, and the
    # K-split kernel takes no plan that cuts k into several windows with it
    a4, w4, sa4, sw4 = generate_llama_gemm_data(32, 512, 4096, seed=4)
    out4 = torch.empty(32, 256, dtype=torch.float8_e4m3fn).cuda()
    args4 = (a4.data_ptr(), w4.data_ptr(), out4.data_ptr(), None, sa4.data_ptr(), 0, sw4.data_ptr(), 0, out_scale.data_ptr(),
             32, 512, 4096, 4096, _capi.BF16, _capi.EPILOGUE_SWIGLU)
    assert lib.hfrk_skinny_gemm_fused(*args4, None, None) == _capi.SUCCESS
    windows = _capi.GemmPlan(2, -1, 1, 0, 32, 16, 2, 8 * 4096 + 16 * 2 * 1024)   # 256 bytes per wave: two windows
    assert lib.hfrk_skinny_gemm_fused(*args4, ctypes.byref(windows), None) == _capi.INVALID_CONFIG
    workgroup = _capi.GemmPlan(2, 4, 2, 1, 32, 4, 8, 8 * 4096 + 2 * 16 * 2 * 512)
    assert lib.hfrk_skinny_gemm_fused(*args4, ctypes.byref(workgroup), None) == _capi.INVALID_CONFIG
    torch.cuda.synchronize()
    # the Python wrapper falls back to GEMM + swiglu where the epilogue does not exist
    got = skinny_gemm_swiglu(a, w, sa, sw, out_scale)
    ref, tol = _swiglu_oracle(a, w, sa, sw, out_scale, torch.bfloat16)
    assert ((got.cpu().float() - ref.float()).abs() <= tol).all()


@pytest.mark.parametrize("m,n,k", [(8, 1024, 2048), (16, 6144, 1024), (3, 2080 * 2, 512), (40, 2080 * 2, 4096), (64, 1024, 2048),
                                   (20, 2080 * 2, 1536), (32, 6144, 8192)])
def test_swiglu_epilogue_under_every_split(m, n, k):
    """Forced plans: grids that cut (gate, up) tile pairs between waves and between workgroups in different places."""
    from hf_rocm_kernels import _capi
    from hf_rocm_kernels.operators.skinny_gemm import generate_llama_gemm_data
    lib = _capi.load()
    a, w, sa, sw = generate_llama_gemm_data(m, n, k, seed=77, weight_std=0.05)
    out_scale = torch.tensor([8.0 / 448], dtype=torch.float32).cuda()
    ref, tol = _swiglu_oracle(a, w, sa, sw, out_scale, torch.bfloat16)
    ma, kc, groups = (m + 3) // 4, k // 256, (n // 2) // 16
    if k in (2048, 4096):  # K-split plans: one window covers k, the workgroup's 8 waves split it
        mt, wave_k = (m + 15) // 16, k // 8
        for grid in sorted({min(g, groups) for g in (256, 200, 7, 1)}):
            plan = _capi.GemmPlan(mt, -1, wave_k // 256, 0, grid, groups, 1, 8 * (wave_k // 256) * 4096 + 16 * mt * 1024)
            out = torch.full((m, n // 2), float("nan"), dtype=torch.float32).cuda().to(torch.float8_e4m3fn)
            st = lib.hfrk_skinny_gemm_fused(a.data_ptr(), w.data_ptr(), out.data_ptr(), None, sa.data_ptr(), 0, sw.data_ptr(), 0,
                                            out_scale.data_ptr(), m, n, k, k, _capi.BF16, _capi.EPILOGUE_SWIGLU,
                                            ctypes.byref(plan), torch.cuda.current_stream().cuda_stream)
            assert st == 0, ("k-split", grid, st)
            torch.cuda.synchronize()
            f = out.cpu().float()
            assert not f.isnan().any(), ("k-split", grid)
            assert ((f - ref.float()).abs() <= tol).all(), ("k-split", grid)
    if m > 32:
        return
    for grid in (sorted({min(g, groups * kc) for g in (256, 200, 64, 7, 1)}) if m <= 16 else []):   # wave-stream plans: up to 16 rows
        plan = _capi.GemmPlan((ma + 3) // 4, 0, 2, ma, grid, groups, kc, 8 * (2 + (ma + 3) // 4) * 4096)
        out = torch.full((m, n // 2), float("nan"), dtype=torch.float32).cuda().to(torch.float8_e4m3fn)
        st = lib.hfrk_skinny_gemm_fused(a.data_ptr(), w.data_ptr(), out.data_ptr(), None, sa.data_ptr(), 0, sw.data_ptr(), 0,
                                        out_scale.data_ptr(), m, n, k, k, _capi.BF16, _capi.EPILOGUE_SWIGLU,
                                        ctypes.byref(plan), torch.cuda.current_stream().cuda_stream)
        assert st == 0, (grid, st)
        torch.cuda.synchronize()
        f = out.cpu().float()
        assert not f.isnan().any(), grid
        assert ((f - ref.float()).abs() <= tol).all(), grid
    if k < 512:
        return
    # row-split plans: bands of output columns, cut between waves inside a workgroup only (17..32 rows: two activation tiles)
    units = (n // 2 + 3) // 4
    if m > 16:
        ma = 6 if m <= 24 else 8
    rows_lds = 8 * (2 + (ma + 3) // 4) * 4096
    for grid in sorted({min(g, units) for g in (512, 256, 224, 200, 64, 7, 1)}):
        plan = _capi.GemmPlan(1, -2, 2, ma, grid, units, kc, rows_lds)
        out = torch.full((m, n // 2), float("nan"), dtype=torch.float32).cuda().to(torch.float8_e4m3fn)
        st = lib.hfrk_skinny_gemm_fused(a.data_ptr(), w.data_ptr(), out.data_ptr(), None, sa.data_ptr(), 0, sw.data_ptr(), 0,
                                        out_scale.data_ptr(), m, n, k, k, _capi.BF16, _capi.EPILOGUE_SWIGLU,
                                        ctypes.byref(plan), torch.cuda.current_stream().cuda_stream)
        assert st == 0, ("rows", grid, st)
        torch.cuda.synchronize()
        f = out.cpu().float()
        assert not f.isnan().any(), ("rows", grid)
        assert ((f - ref.float()).abs() <= tol).all(), ("rows", grid)
    # the same on bands of whole tiles of 16 output columns, from the row-major and from the packed weight
    from hf_rocm_kernels.utils.weight_format import pack_weight
    packed = pack_weight(w.t())
    tiles = (n // 2 + 15) // 16
    for grid in sorted({min(g, tiles) for g in (384, 256, 200, 64, 7, 1)}):
        plan = _capi.GemmPlan(1, -3, 2, ma, grid, tiles, kc, rows_lds)
        outs = []
        for layout in ("row-major", "packed"):
            out = torch.full((m, n // 2), float("nan"), dtype=torch.float32).cuda().to(torch.float8_e4m3fn)
            if layout == "packed":
                st = lib.hfrk_skinny_gemm_packed(a.data_ptr(), packed.data.data_ptr(), out.data_ptr(), None, sa.data_ptr(), 0, sw.data_ptr(), 0,
                                                 out_scale.data_ptr(), m, n, k, _capi.BF16, _capi.EPILOGUE_SWIGLU, ctypes.byref(plan),
                                                 torch.cuda.current_stream().cuda_stream)
            else:
                st = lib.hfrk_skinny_gemm_fused(a.data_ptr(), w.data_ptr(), out.data_ptr(), None, sa.data_ptr(), 0, sw.data_ptr(), 0,
                                                out_scale.data_ptr(), m, n, k, k, _capi.BF16, _capi.EPILOGUE_SWIGLU,
                                                ctypes.byref(plan), torch.cuda.current_stream().cuda_stream)
            assert st == 0, ("rows on tiles", layout, grid, st)
            torch.cuda.synchronize()
            f = out.cpu().float()
            assert not f.isnan().any(), ("rows on tiles", layout, grid)
            assert ((f - ref.float()).abs() <= tol).all(), ("rows on tiles", layout, grid)
            outs.append(out.view(torch.uint8))
        assert torch.equal(outs[0], outs[1]), ("rows on tiles: the two layouts differ", grid)
    one_tile = _capi.GemmPlan(1, -2, 1, min(ma, 4), 64, units, kc, 8 * 2 * 4096)  # a chunk must hold a gate and an up tile
    assert lib.hfrk_skinny_gemm_fused(a.data_ptr(), w.data_ptr(), out.data_ptr(), None, sa.data_ptr(), 0, sw.data_ptr(), 0,
                                      out_scale.data_ptr(), m, n, k, k, _capi.BF16, _capi.EPILOGUE_SWIGLU,
                                      ctypes.byref(one_tile), torch.cuda.current_stream().cuda_stream) == _capi.INVALID_CONFIG


def test_benchmarking_helpers_and_the_library_gemm_agree_with_scaled_mm():
    """The reference times its kernel against torch._scaled_mm (hipBLASLt) and uses it as its oracle
    (operators/skinny_gemm/reference.py:18-25): same cross-check here, plus the timing helpers on a tiny budget."""
    from hf_rocm_kernels import skinny_gemm
    from hf_rocm_kernels.operators.skinny_gemm import generate_llama_gemm_data
    from hf_rocm_kernels.operators.skinny_gemm.benchmarking_fn import benchmark_skinny_gemm
    from hf_rocm_kernels.utils.benchmarking import Bench, benchmark_cuda_graph_no_cache
    a, b, sa, sw = generate_llama_gemm_data(8, 1024, 2048, seed=12)
    ours = skinny_gemm(a, b, (sa * sw).contiguous())
    try:
        theirs = torch._scaled_mm(a, b, scale_a=sa.reshape(1), scale_b=sw.reshape(1), out_dtype=ours.dtype)
    except Exception as e:  # not every torch build has the fp8 hipBLASLt path
        theirs = None
        print("torch._scaled_mm unavailable:", e)
    if theirs is not None:
        assert torch.allclose(ours.float(), theirs.float(), rtol=1e-2, atol=1e-2)
    mean, std = benchmark_skinny_gemm(8, 1024, 2048, {}, graph_size=2, warmups=1, iterations=4)
    assert 0 < mean < 1e4 and std >= 0
    med, _ = benchmark_skinny_gemm(8, 1024, 2048, dict(split_k=4, A_producers=2, B_producers=6, consumers=2, a_lanes=2,
                                                        b_lanes=3, qsize=4, op_m=16, ops=8),
                                   graph_size=2, warmups=1, iterations=4, mode="median")
    assert 0 < med < 1e4
    t = benchmark_cuda_graph_no_cache(lambda x: x.add_(1), (torch.zeros(1024, device="cuda"),), {}, graph_size=2, warmups=1, iterations=4)
    assert 0 < t < 1e4
    bench = Bench()
    bench.add_measure("add", 1024, lambda: torch.zeros(1024, device="cuda").add_(1), rep=4)
    assert bench.table("n")["add"][0] > 0


def test_a_plan_table_entry_is_what_a_call_without_a_plan_runs():
    """An entry that moves m = 8 to the workgroup kernel with an odd grid: the default call then gives, bit for bit,
    what the explicit plan gives, on the row-major and on the packed key, and the oracle's answer."""
    from hf_rocm_kernels import plan_table, skinny_gemm_scaled
    from hf_rocm_kernels import _capi
    from hf_rocm_kernels.operators.skinny_gemm import generate_llama_gemm_data
    from hf_rocm_kernels.utils.weight_format import pack_weight
    m, n, k = 8, 2048, 4096
    a, b, sa, sw = generate_llama_gemm_data(m, n, k, seed=21)
    entry = _capi.GemmPlan(1, 2, 4, 1, 23, n // 32, k // 1024, 8 * 4096 + 2 * 16 * 1024)
    explicit = torch.empty((m, n), dtype=torch.bfloat16, device="cuda")
    run_ex(a, b, sa, sw, explicit, accumulate=False, plan=entry)
    plan_table.clear()
    try:
        before = skinny_gemm_scaled(a, b, sa, sw)
        plan_table.set_plan(m, n, k, entry)
        plan_table.set_plan(m, n, k, entry, packed=True)
        assert plan_table.get_plan(m, n, k).as_dict() == entry.as_dict()
        after = skinny_gemm_scaled(a, b, sa, sw)
        after_packed = skinny_gemm_scaled(a, pack_weight(b.t()), sa, sw)
        # the entry also serves m = 5..7 (same activation loads): same plan, first rows of the same product
        assert plan_table.get_plan(6, n, k).as_dict() == entry.as_dict()
        six = skinny_gemm_scaled(a[:6].contiguous(), b, sa, sw)
    finally:
        plan_table.clear()
        plan_table.load_from_environment()
    assert torch.equal(after, explicit) and torch.equal(after_packed, explicit)
    assert torch.equal(six, explicit[:6])
    check_against_oracle(after, a, b, sa, sw)
    check_against_oracle(before, a, b, sa, sw)


def _shipped_entries():
    import json
    from hf_rocm_kernels import plan_table
    entries = []
    for path in plan_table.shipped_tables():
        for e in json.load(open(path))["entries"]:
            entries.append(pytest.param(e, id=f"{e['m']}x{e['n']}x{e['k']}{'p' if e['packed'] else ''}"))
    return entries


@pytest.mark.parametrize("entry", _shipped_entries())
def test_every_shipped_plan_table_entry_computes_what_the_planner_s_plan_computes(entry):
    """Each tuned entry is another decomposition of the same product, run here on the entry's own full-size shape and weight
    layout through a call that picks it up from the table.  Against the oracle (exact product and fp32 path, the bounds of
    check_against_oracle) on all columns of weights up to 8192 rows and on eight 1024-column slices spread over the larger
    ones (first and last included, the others at seeded offsets); and on every column against the same call run on the
    planner's plan, to within the reassociation of fp32 sums."""
    from hf_rocm_kernels import _capi, plan_table, skinny_gemm_scaled
    from hf_rocm_kernels.utils.weight_format import pack_weight
    m, n, k, packed = entry["m"], entry["n"], entry["k"], entry["packed"]
    assert plan_table.get_plan(m, n, k, packed).as_dict() == entry["plan"], "the shipped table is not installed"
    # the benchmark's data recipe (activations ~ N(0,1), weights ~ N(0,0.02), per-tensor scales amax / 448), drawn on the device
    g = torch.Generator(device="cuda").manual_seed(m + n + k)
    def quantised(rows, cols, std):
        x = torch.randn((rows, cols), generator=g, device="cuda") * std
        scale = (x.abs().amax() / 448.0).reshape(1)
        return (x / scale).clamp(-448, 448).to(torch.float8_e4m3fn), scale
    (a, sa), (w, sw) = quantised(m, k, 1.0), quantised(n, k, 0.02)
    want = torch.empty((m, n), dtype=torch.bfloat16, device="cuda")
    run_ex(a, w.t(), sa, sw, want, accumulate=False, plan=_capi.plan(m, n, k))
    got = skinny_gemm_scaled(a, pack_weight(w) if packed else w.t(), sa, sw)
    torch.cuda.synchronize()
    err = (got.float() - want.float()).abs()
    bound = want.float().abs() * 2.0 ** -7 + 2.0 ** -6   # one bf16 step of the result, plus the cancellation floor
    assert bool((err <= bound).all()), float((err - bound).max())
    assert float(want.float().abs().mean()) > 0.01
    if n <= 8192:
        slices = None
    else:
        import random
        rng = random.Random(m * 1000003 + n * 101 + k)
        starts = {0, n - 1024} | {1024 * rng.randrange(1, (n - 1024) // 1024) for _ in range(6)}
        slices = [(c, c + 1024) for c in sorted(starts)]
    _check_columns_against_oracle([(f"table entry {m}x{n}x{k}", got, a.cpu(), sa.cpu()), (f"planner {m}x{n}x{k}", want, a.cpu(), sa.cpu())],
                                  w.cpu(), sw.cpu(), slices=slices)


# ---- the Llama-3-70B projections (unsharded) at full size against the oracle ------------------------------------------

def _check_columns_against_oracle(cases, b_codes_nk, sw, cols=4096, slices=None):
    """cases: [(label, out [m,n] on the device, a [m,k] fp8 on the host, sa [1 or m] on the host)].  The oracle's two
    checks of `check_against_oracle` (rtol/atol 1e-2 against the fp32 path; 1 ulp + 2^-16 sum|a b| against the exact
    product), evaluated one slice of output columns at a time so that the float64 copy of a 470 MB weight is never
    held whole, and with each slice decoded once for all the cases that share the weight.  slices: the (c0, c1) column ranges
    to check instead of all of them."""
    og = _oracle()
    from oracle import fp8 as ofp8
    n = b_codes_nk.shape[0]
    outs = [(label, out.cpu(), a, sa) for label, out, a, sa in cases]
    for c0, c1 in (slices if slices is not None else [(c, min(n, c + cols)) for c in range(0, n, cols)]):
        w64 = torch.from_numpy(ofp8.decode(b_codes_nk[c0:c1].view(torch.uint8)))   # [cols, k] float64
        w64_abs = w64.abs()
        w32 = w64.float()
        swc = sw if sw.numel() == 1 else sw[c0:c1]
        for label, got, a, sa in outs:
            a64 = torch.from_numpy(ofp8.decode(a.view(torch.uint8)))
            scale = sa.double().reshape(-1, 1) * swc.double().reshape(1, -1)
            exact = (a64 @ w64.t()) * scale
            bound = og.ulp16(exact, got.dtype) + (a64.abs() @ w64_abs.t()) * scale.abs() * 2.0 ** -16
            g = got[:, c0:c1]
            assert not g.isnan().any(), label
            worst = ((g.double() - exact).abs() / bound).max().item()
            assert worst <= 1.0, f"{label}, columns {c0}..{c1}: error is {worst} x the bound from the exact product"
            ref32 = ((a64.float() * sa.float().reshape(-1, 1)) @ (w32 * swc.float().reshape(-1, 1)).t()).to(got.dtype).float()
            err = (g.float() - ref32).abs()
            tol = 1e-2 + 1e-2 * ref32.abs()
            assert (err <= tol).all(), f"{label}, columns {c0}..{c1}: excess over rtol/atol 1e-2: {(err - tol).max().item()}"


@pytest.mark.parametrize("name,n,k", [("qkv", 10240, 8192), ("o_proj", 8192, 8192), ("gate_up", 57344, 8192),
                                      ("down", 8192, 28672)])
def test_llama3_70b_shapes_match_the_oracle(name, n, k):
    """Every (N, K) of the Llama-3-70B projections, row-major at M = 1, 4, 8, 16, 32 (each takes its own plan, from the
    installed table or the planner) and from the packed weight at M = 8, through the operator (so with the plan the installed table or the planner gives the shape), against the
    exact oracle at full size."""
    from hf_rocm_kernels import plan_table, skinny_gemm, skinny_gemm_scaled
    from hf_rocm_kernels.operators.skinny_gemm import generate_llama_gemm_data
    from hf_rocm_kernels.utils.weight_format import pack_weight
    _, b, _, sw = generate_llama_gemm_data(1, n, k, seed=70 + n % 7, device="cpu")
    b_dev = b.t().contiguous().cuda().t()      # [k, n] view of the [n, k] weight
    sw_dev = sw.cuda()
    cases = []
    for m in (1, 4, 8, 16, 32):
        a, _, sa, _ = generate_llama_gemm_data(m, 16, k, seed=700 + m, device="cpu")
        print(f"{name} m={m}: plan {plan_table.get_plan(m, n, k).as_dict()}", flush=True)
        out = skinny_gemm(a.cuda(), b_dev, (sa * sw).cuda())              # the 13-argument operator, one combined scale
        cases.append((f"{name} m={m} row-major", out, a, sa))
        if m == 8:
            print(f"{name} m={m} packed: plan {plan_table.get_plan(m, n, k, True).as_dict()}", flush=True)
            out_p = skinny_gemm_scaled(a.cuda(), pack_weight(b_dev.t()), sa.cuda(), sw_dev)
            cases.append((f"{name} m={m} packed", out_p, a, sa))
    torch.cuda.synchronize()
    _check_columns_against_oracle(cases, b.t(), sw)


def test_committed_gemm_fixtures_on_the_device():
    """tests/golden/gemm_*.npz hold operand codes, the oracle's bf16 result and the exact integer dot products: the
    device result, through the C ABI, must be the correctly rounded exact product up to rare one-ulp boundary cases."""
    import glob
    import os

    import numpy as np
    og = _oracle()
    files = sorted(glob.glob(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "gemm_*.npz")))
    assert len(files) >= 3
    for f in files:
        z = np.load(f)
        a = torch.from_numpy(z["a_codes"]).view(torch.float8_e4m3fn).cuda()
        w = torch.from_numpy(z["w_codes"]).view(torch.float8_e4m3fn).cuda()
        sa, sw = torch.from_numpy(z["scale_a"]).cuda(), torch.from_numpy(z["scale_w"]).cuda()
        m, n = a.shape[0], w.shape[0]
        out = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device="cuda")
        run_ex(a, w.t(), sa, sw, out, accumulate=False)
        got = out.cpu()
        exact = torch.from_numpy(z["int_dots"].astype(np.float64) * 2.0 ** -18) * sa.cpu().double().reshape(-1, 1) * sw.cpu().double().reshape(1, -1)
        err = (got.double() - exact).abs()
        bound = og.error_bound(a.cpu(), w.cpu().t(), sa.cpu(), sw.cpu(), torch.bfloat16, exact)
        assert (err <= bound).all(), (f, float((err / bound).max()))
        # the exact product rounded once: the device's fp32 sums of 256..1024 cancelling terms carry an error of about
        # 2^-17 of the result, so about one result in a hundred lands on the other side of a bf16 rounding boundary
        differs = got.view(torch.int16) != exact.to(torch.bfloat16).view(torch.int16)
        assert differs.float().mean() <= 0.03, (f, float(differs.float().mean()))
        # the fixture's own result comes from the fp32 path, which scales the operands before multiplying: more boundary
        # flips, none beyond one step
        want = torch.from_numpy(z["out_bf16_bits"]).view(torch.bfloat16)
        differs = got.view(torch.int16) != want.view(torch.int16)
        assert differs.float().mean() <= 0.03, (f, float(differs.float().mean()))
        assert ((got.double() - want.double()).abs() <= 2 * bound).all(), f   # each within `bound` of the exact product


# ---- workspaces: one per stream, arrival counters shared by every launch on a stream -----------------------------------

def _launch_ex(lib, a, b, sa, sb, out, plan, stream):
    from hf_rocm_kernels import _capi
    m, k = a.shape
    st = lib.hfrk_skinny_gemm_ex(a.data_ptr(), b.data_ptr(), out.data_ptr(), sa.data_ptr(), 0 if sa.numel() == 1 else 1,
                                 sb.data_ptr(), 0 if sb.numel() == 1 else 1, m, b.shape[1], k, b.stride(1), _capi.BF16, 0,
                                 None if plan is None else ctypes.byref(plan), stream.cuda_stream)
    assert st == 0, st


def test_two_streams_run_independent_gemms():
    """Two streams, two shapes whose row tiles are shared between workgroups (so both use workspace and counters),
    launched interleaved without synchronisation 50 times: every result equals the one the same launch gives alone.
    The reference's calls are independent of each other because it accumulates into the caller's output
    (csrc/op_src/skinny_gemm/consumers/mfma_16x16x32_consumer.cu:155-163); here each stream owns a workspace."""
    from hf_rocm_kernels import _capi
    from hf_rocm_kernels.operators.skinny_gemm import generate_llama_gemm_data
    lib = _capi.load()
    a1, b1, sa1, sw1 = generate_llama_gemm_data(8, 4096, 4096, seed=91)
    a2, b2, sa2, sw2 = generate_llama_gemm_data(32, 4096, 14336, seed=92)
    p1 = _capi.GemmPlan(1, 0, 1, 2, 120, 256, 16, 8 * 2 * 4096)       # wave-stream on 120 workgroups: tiles cut between them
    p2 = _capi.GemmPlan(2, 4, 2, 1, 120, 64, 28, 8 * 4096 + 2 * 32 * 512)  # workgroup kernel, 4 x 2 waves, 120 workgroups
    s1, s2 = torch.cuda.Stream(), torch.cuda.Stream()
    alone1 = torch.empty((8, 4096), dtype=torch.bfloat16, device="cuda")
    alone2 = torch.empty((32, 4096), dtype=torch.bfloat16, device="cuda")
    torch.cuda.synchronize()
    _launch_ex(lib, a1, b1, sa1, sw1, alone1, p1, s1)
    torch.cuda.synchronize()
    _launch_ex(lib, a2, b2, sa2, sw2, alone2, p2, s2)
    torch.cuda.synchronize()
    check_against_oracle(alone1, a1, b1, sa1, sw1)
    check_against_oracle(alone2, a2, b2, sa2, sw2)
    id1, id2 = lib.hfrk_workspace_id(s1.cuda_stream), lib.hfrk_workspace_id(s2.cuda_stream)
    assert id1 >= 0 and id2 >= 0 and id1 != id2, (id1, id2)
    per_iter = 4
    outs1 = [torch.full((8, 4096), float("nan"), dtype=torch.bfloat16, device="cuda") for _ in range(per_iter)]
    outs2 = [torch.full((32, 4096), float("nan"), dtype=torch.bfloat16, device="cuda") for _ in range(per_iter)]
    torch.cuda.synchronize()
    for it in range(50):
        for j in range(per_iter):
            _launch_ex(lib, a1, b1, sa1, sw1, outs1[j], p1, s1)
            _launch_ex(lib, a2, b2, sa2, sw2, outs2[j], p2, s2)
        torch.cuda.synchronize()
        for j in range(per_iter):
            assert torch.equal(outs1[j], alone1), f"iteration {it}, launch {j}: stream 1 differs from its run alone"
            assert torch.equal(outs2[j], alone2), f"iteration {it}, launch {j}: stream 2 differs from its run alone"
            outs1[j].fill_(float("nan"))
            outs2[j].fill_(float("nan"))
        torch.cuda.synchronize()
    # a stream keeps its workspace; releasing it hands the workspace to the next stream that asks
    assert lib.hfrk_workspace_id(s1.cuda_stream) == id1
    assert lib.hfrk_release_stream(s1.cuda_stream) == 0 and lib.hfrk_workspace_id(s1.cuda_stream) == -1
    assert lib.hfrk_release_stream(s1.cuda_stream) == 0
    assert lib.hfrk_reset_workspace(torch.cuda.current_stream().cuda_stream) == 0
    torch.cuda.synchronize()
    _launch_ex(lib, a1, b1, sa1, sw1, outs1[0], p1, s1)
    torch.cuda.synchronize()
    assert lib.hfrk_workspace_id(s1.cuda_stream) == id1 and torch.equal(outs1[0], alone1)


def test_back_to_back_launches_of_different_plans_share_counters_safely():
    """Every plan of one shape uses the same arrival counters and workspace addresses with a different meaning.  300
    launches cycling through them on one stream with no synchronisation in between: each must give the bits its plan
    gave when it ran alone (the partial sums are exchanged past the caches and the counters reset themselves, with
    no fence between launches)."""
    from hf_rocm_kernels import _capi
    from hf_rocm_kernels.operators.skinny_gemm import generate_llama_gemm_data
    lib = _capi.load()
    m, n, k = 24, 1040, 4096
    a, b, sa, sw = generate_llama_gemm_data(m, n, k, seed=93)
    plans = all_plans(m, n, k)
    stream = torch.cuda.current_stream()
    alone = []
    for p in plans:
        out = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device="cuda")
        _launch_ex(lib, a, b, sa, sw, out, p, stream)
        torch.cuda.synchronize()
        alone.append(out)
    check_against_oracle(alone[0], a, b, sa, sw)
    launches = 300
    outs = [torch.full((m, n), float("nan"), dtype=torch.bfloat16, device="cuda") for _ in range(launches)]
    torch.cuda.synchronize()
    for i in range(launches):
        _launch_ex(lib, a, b, sa, sw, outs[i], plans[(i * 7) % len(plans)], stream)
    torch.cuda.synchronize()
    for i in range(launches):   # stops at the first mismatch
        j = (i * 7) % len(plans)
        assert torch.equal(outs[i], alone[j]), f"launch {i} (plan {plans[j].as_dict()}) differs from the same plan run alone"
