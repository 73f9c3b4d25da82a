"""Pins the GEMM part of the oracle without a GPU: exact integer dot products (plain C) == float64 matmul ==
pure-Python integers; closed forms; the fp32 reference path against the exact one; the committed fixtures."""
import os

import numpy as np
import pytest
import torch

from oracle import c_oracle, fp8
from oracle import skinny_gemm as og

GOLDEN = os.path.join(os.path.dirname(__file__), "golden")


def _codes(t):
    return t.contiguous().view(torch.uint8).numpy()


def test_exact_paths_agree_tiny_pure_python():
    a, b, s, _ = og.generate_skinny_gemm_data(3, 5, 128, seed=0)
    table = fp8.decode_table()
    ac, wc = _codes(a), _codes(b.t())
    ints = [[sum(int(round(table[ac[i, t]] * 512)) * int(round(table[wc[j, t]] * 512)) for t in range(128))
             for j in range(5)] for i in range(3)]
    assert np.array_equal(np.array(ints, dtype=np.int64), c_oracle.gemm_int(ac, wc))
    assert np.array_equal(np.array(ints, dtype=np.int64), og.int_dot_products(a, b))
    one = torch.ones(1)
    exact = og.exact_skinny_gemm(a, b, one, one).numpy()
    assert np.array_equal(exact, np.array(ints, dtype=np.float64) / 2.0 ** 18)


@pytest.mark.parametrize("m,n,k", [(8, 96, 1024), (33, 64, 4096), (2, 16, 28672)])
def test_c_integer_gemm_equals_float64_matmul(m, n, k):
    a, b, s, _ = og.generate_skinny_gemm_data(m, n, k, seed=k + m)
    one = torch.ones(1)
    exact = og.exact_skinny_gemm(a, b, one, one).numpy()
    ints = c_oracle.gemm_int(_codes(a), _codes(b.t()))
    assert np.array_equal(exact * 2.0 ** 18, ints.astype(np.float64))


def test_closed_forms():
    k, n, m = 256, 256, 4
    one = torch.ones(1)
    g = torch.Generator().manual_seed(3)
    a = fp8.fp8_quantize(torch.randn(m, k, generator=g), torch.tensor([0.01]))[0]
    # zero weights / zero activations
    z = torch.zeros(n, k).to(torch.float8_e4m3fn)
    assert (og.reference_skinny_gemm(a, z.t(), one, one).float() == 0).all()
    assert (og.exact_skinny_gemm(torch.zeros(m, k).to(torch.float8_e4m3fn), z.t(), one, one) == 0).all()
    # identity weights scaled by a power of two return the activations times that scale, exactly
    eye = (torch.eye(n, k) * 2.0).to(torch.float8_e4m3fn)
    out = og.reference_skinny_gemm(a, eye.t(), torch.tensor([0.5]), one, out_dtype=torch.float16)
    assert torch.equal(out.float(), a.float())
    # a one-hot activation row picks one weight column (row of the [n,k] weight transposed)
    w = fp8.fp8_quantize(torch.randn(n, k, generator=g), torch.tensor([0.02]))[0]
    hot = torch.zeros(1, k)
    hot[0, 37] = 4.0
    out = og.exact_skinny_gemm(hot.to(torch.float8_e4m3fn), w.t(), one, one)
    assert torch.equal(out[0], 4.0 * w.float().double()[:, 37])
    # linearity in the output scale and row-permutation equivariance
    base = og.exact_skinny_gemm(a, w.t(), one, one)
    assert torch.equal(og.exact_skinny_gemm(a, w.t(), torch.tensor([4.0]), one), 4 * base)
    perm = torch.tensor([2, 0, 3, 1])
    assert torch.equal(og.exact_skinny_gemm(a[perm], w.t(), one, one), base[perm])
    # K split invariance: summing two half-K products equals the full product exactly
    h = k // 2
    parts = og.exact_skinny_gemm(a[:, :h].contiguous(), w[:, :h].contiguous().t(), one, one) + \
        og.exact_skinny_gemm(a[:, h:].contiguous(), w[:, h:].contiguous().t(), one, one)
    assert torch.equal(parts, base)
    # the accumulator argument is added before the single rounding
    bias = torch.randn(m, n, generator=g).to(torch.bfloat16)
    with_bias = og.reference_skinny_gemm(a, w.t(), one, one, output=bias)
    assert torch.equal(with_bias, (og.reference_skinny_gemm(a, w.t(), one, one, out_dtype=torch.float32) + bias.float()).to(torch.bfloat16))


@pytest.mark.parametrize("per_token,per_channel", [(False, False), (True, True)])
def test_fp32_reference_within_one_ulp_of_exact(per_token, per_channel):
    m, n, k = 16, 512, 4096
    g = torch.Generator().manual_seed(11)
    act = torch.randn(m, k, generator=g).to(torch.bfloat16).float()
    w = torch.randn(n, k, generator=g) * 0.02
    sa = fp8.amax_scale(act, dim=1 if per_token else None)
    sw = fp8.amax_scale(w, dim=1 if per_channel else None)
    a8, w8 = fp8.fp8_quantize(act, sa)[0], fp8.fp8_quantize(w, sw)[0]
    ref = og.reference_skinny_gemm(a8, w8.t(), sa.reshape(-1), sw.reshape(-1))
    exact = og.exact_skinny_gemm(a8, w8.t(), sa.reshape(-1), sw.reshape(-1))
    assert ref.dtype == torch.bfloat16
    bound = og.error_bound(a8, w8.t(), sa.reshape(-1), sw.reshape(-1), torch.bfloat16, exact)
    assert ((ref.double() - exact).abs() <= bound).all()
    # and the scalar C restatement of the fp32 path (sequential sum) lands on the same bf16 values almost everywhere
    c32 = c_oracle.gemm_f32(_codes(a8), _codes(w8), sa.numpy(), sw.numpy())
    c16 = torch.from_numpy(c32).to(torch.bfloat16)
    assert ((c16.double() - exact).abs() <= bound).all()
    assert (c16 != ref).float().mean() < 0.02


def test_config1_shape_matches_torch_scaled_mm_on_cpu():
    """The reference test shape (M=8, N=K=4096, per-tensor amax/448 scales): torch's own CPU _scaled_mm on e4m3fn -- the
    library routine behind the reference's oracle -- agrees with the restated path to one bf16 ulp."""
    m, n, k = 8, 4096, 4096
    g = torch.Generator().manual_seed(0)
    act = torch.randn(m, k, generator=g).to(torch.bfloat16).float()
    w = torch.randn(n, k, generator=g) * 0.02
    sa, sw = fp8.amax_scale(act), fp8.amax_scale(w)
    a8, w8 = fp8.fp8_quantize(act, sa)[0], fp8.fp8_quantize(w, sw)[0]
    ref = og.reference_skinny_gemm(a8, w8.t(), sa.reshape(1), sw.reshape(1))
    try:
        lib = torch._scaled_mm(a8, w8.t(), scale_a=sa.reshape(()), scale_b=sw.reshape(()), out_dtype=torch.bfloat16)
    except (RuntimeError, NotImplementedError) as e:  # not every torch build has the CPU kernel
        pytest.skip(f"torch._scaled_mm unavailable on CPU: {e}")
    exact = og.exact_skinny_gemm(a8, w8.t(), sa.reshape(1), sw.reshape(1))
    bound = og.error_bound(a8, w8.t(), sa.reshape(1), sw.reshape(1), torch.bfloat16, exact)
    assert ((lib.double() - exact).abs() <= bound).all()
    assert ((ref.double() - exact).abs() <= bound).all()
    assert (lib != ref).float().mean() < 0.02


def test_golden_fixtures_reproduce():
    import glob
    files = sorted(glob.glob(os.path.join(GOLDEN, "gemm_*.npz")))
    assert files, "run tests/golden/make_fixtures.py"
    for f in files:
        z = np.load(f)
        a = torch.from_numpy(z["a_codes"]).view(torch.float8_e4m3fn)
        w = torch.from_numpy(z["w_codes"]).view(torch.float8_e4m3fn)
        sa, sw = torch.from_numpy(z["scale_a"]), torch.from_numpy(z["scale_w"])
        out = og.reference_skinny_gemm(a, w.t(), sa, sw)
        assert np.array_equal(out.view(torch.int16).numpy(), z["out_bf16_bits"]), f
        ints = c_oracle.gemm_int(z["a_codes"], z["w_codes"])
        assert np.array_equal(ints, z["int_dots"]), f
