"""Pins the residual-RMSNorm, SwiGLU and MLP-chain parts of the oracle without a GPU."""
import glob
import os

import numpy as np
import pytest
import torch

from oracle import c_oracle, fp8
from oracle import llama_mlp as omlp
from oracle import residual_rms as orr
from oracle import skinny_gemm as og
from oracle import swiglu as osw

GOLDEN = os.path.join(os.path.dirname(__file__), "golden")


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_residual_is_one_ieee_16bit_add(dtype):
    g = torch.Generator().manual_seed(0)
    x = (torch.randn(7, 300, generator=g) * 3).to(dtype)
    r = (torch.randn(7, 300, generator=g) * 3).to(dtype)
    w = torch.ones(300, dtype=dtype)
    _, res, _ = orr.reference_residual_rms(x, r, w, 1e-5, None)
    if dtype == torch.float16:
        # numpy adds float16 with a single IEEE rounding: an independent implementation of the same operation
        expect = torch.from_numpy(x.numpy() + r.numpy())
    else:
        # bfloat16: the exact sum of two 8-bit-mantissa numbers rounded to nearest even by integer arithmetic
        s = (x.double() + r.double()).float()            # exact in fp32 for these magnitudes
        bits = s.view(torch.int32)
        rounded = ((bits + 0x7FFF + ((bits >> 16) & 1)) >> 16).to(torch.int16)
        expect = rounded.view(torch.bfloat16)
    assert torch.equal(res.view(torch.int16), expect.view(torch.int16))
    # and the inputs are left untouched
    assert res.data_ptr() != x.data_ptr()


def test_rms_against_textbook_and_c():
    g = torch.Generator().manual_seed(1)
    z = torch.randn(5, 1024, generator=g, dtype=torch.float64)
    w = 1 + 0.1 * torch.randn(1024, generator=g, dtype=torch.float64)
    eps = 1e-5
    ours = orr.reference_rms(z.float(), eps).double() * w
    for i in range(5):
        c = c_oracle.rms_row(z[i].numpy(), w.numpy(), eps)
        assert np.allclose(ours[i].numpy(), c, rtol=2e-6, atol=1e-7)
    # closed forms: a constant row normalises to +-1 (eps aside), scaling the row by 4 leaves the result unchanged
    const = torch.full((1, 64), 3.0)
    assert torch.allclose(orr.reference_rms(const, 0.0), torch.ones(1, 64))
    assert torch.allclose(orr.reference_rms(z.float() * 4, 0.0), orr.reference_rms(z.float(), 0.0), rtol=1e-6, atol=1e-7)
    # mean of squares of the normalised row is 1
    assert torch.allclose(orr.reference_rms(z.float(), 0.0).pow(2).mean(-1), torch.ones(5), rtol=1e-5)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_reference_no_worse_than_quantisation_vs_precise(dtype):
    g = torch.Generator().manual_seed(2)
    x = torch.randn(16, 4096, generator=g).to(dtype)
    r = torch.randn(16, 4096, generator=g).to(dtype)
    w = (1 + 0.1 * torch.randn(4096, generator=g)).to(dtype)
    scale = torch.tensor([0.02])
    q, res, s = orr.reference_residual_rms(x, r, w, 1e-5, scale)
    p, _ = orr.precise_residual_rms(x, r, w, 1e-5, scale)
    assert q.dtype == torch.float8_e4m3fn and s is scale
    # both are fp8 roundings of nearly the same real number: they differ by at most one fp8 step, rarely
    d = (q.float() - p.float()).abs()
    step = torch.maximum(p.float().abs() * 2.0 ** -3, torch.tensor(2.0 ** -9))
    assert (d <= step).all() and (d > 0).float().mean() < 0.1
    # 16-bit output: cast to weight dtype, then a 16-bit multiply
    h, _, _ = orr.reference_residual_rms(x, r, w, 1e-5, None)
    manual = (orr.reference_rms(x + r, 1e-5).to(dtype) * w)
    assert h.dtype == dtype and torch.equal(h, manual)
    # next buffer is zeroed only on the fp8 path, as in the reference
    nb = torch.full((16, 8), 7.0, dtype=dtype)
    orr.reference_residual_rms(x, r, w, 1e-5, scale, nb)
    assert nb.abs().sum() == 0


def test_swiglu_closed_forms_and_c():
    g = torch.Generator().manual_seed(3)
    gu = (torch.randn(6, 2 * 160, generator=g) * 2).to(torch.float16)
    ours = osw.swiglu_fp32(gu).double().numpy()
    c = c_oracle.swiglu(gu.double().numpy())
    assert np.allclose(ours, c, rtol=1e-6, atol=1e-7)
    # x*sigmoid(x) identities: silu(0)=0, silu(x)-silu(-x)=x, silu(x)->x for large x; gate is the first half
    x = torch.linspace(-20, 20, 401)
    silu = torch.nn.functional.silu
    assert silu(torch.zeros(1)) == 0
    assert torch.allclose(silu(x) - silu(-x), x, atol=1e-5)
    assert abs(silu(torch.tensor(30.0)) - 30.0) < 1e-5
    probe = torch.zeros(1, 8, dtype=torch.float16)
    probe[0, :4] = 10.0      # gate
    probe[0, 4:] = 2.0       # up
    assert torch.allclose(osw.swiglu_fp32(probe), torch.full((1, 4), 2.0 * float(silu(torch.tensor(10.0)))))
    # quantised output = fp8_quantize of the fp32 value
    scale = torch.tensor([0.05])
    q = osw.reference_swiglu(gu, scale)
    assert torch.equal(q.view(torch.uint8), fp8.fp8_quantize(osw.swiglu_fp32(gu), scale)[0].view(torch.uint8))
    nb = torch.full((6, 4), 3.0, dtype=torch.float16)
    osw.reference_swiglu(gu, scale, nb)
    assert nb.abs().sum() == 0


def test_golden_fixtures_reproduce():
    for f in sorted(glob.glob(os.path.join(GOLDEN, "rms_*.npz"))):
        z = np.load(f)
        dtype = torch.bfloat16 if "bf16" in f else torch.float16
        x = torch.from_numpy(z["input_bits"]).view(dtype)
        r = torch.from_numpy(z["residual_bits"]).view(dtype)
        w = torch.from_numpy(z["weight_bits"]).view(dtype)
        q, res, _ = orr.reference_residual_rms(x, r, w, float(z["eps"]), torch.from_numpy(z["scale"]))
        h, _, _ = orr.reference_residual_rms(x, r, w, float(z["eps"]), None)
        assert np.array_equal(q.view(torch.uint8).numpy(), z["out_fp8"]), f
        assert np.array_equal(h.view(torch.int16).numpy(), z["out16_bits"]), f
        assert np.array_equal(res.view(torch.int16).numpy(), z["new_residual_bits"]), f
    for f in sorted(glob.glob(os.path.join(GOLDEN, "swiglu_*.npz"))):
        z = np.load(f)
        dtype = torch.bfloat16 if "bf16" in f else torch.float16
        gu = torch.from_numpy(z["gate_up_bits"]).view(dtype)
        q = osw.reference_swiglu(gu, torch.from_numpy(z["scale"]))
        assert np.array_equal(q.view(torch.uint8).numpy(), z["out_fp8"]), f


def test_mlp_chain_is_the_composition_of_its_parts():
    g = torch.Generator().manual_seed(4)
    m, hidden, inter = 3, 256, 512
    dtype = torch.bfloat16
    x = torch.randn(m, hidden, generator=g).to(dtype)
    r = torch.randn(m, hidden, generator=g).to(dtype)
    w = (1 + 0.1 * torch.randn(hidden, generator=g)).to(dtype)
    wgu = torch.randn(2 * inter, hidden, generator=g) * 0.02
    wd = torch.randn(hidden, inter, generator=g) * 0.02
    s_gu, s_d = fp8.amax_scale(wgu), fp8.amax_scale(wd)
    wgu8, wd8 = fp8.fp8_quantize(wgu, s_gu)[0].t(), fp8.fp8_quantize(wd, s_d)[0].t()
    in_gu, in_d = torch.tensor([0.02]), torch.tensor([0.01])
    out, res = omlp.reference_llama_mlp(x, r, w, 1e-5, wgu8, in_gu, in_gu * s_gu, wd8, in_d, in_d * s_d)
    one = torch.ones(())
    n8, res2, _ = orr.reference_residual_rms(x, r, w, 1e-5, in_gu)
    gu = og.reference_skinny_gemm(n8, wgu8, in_gu * s_gu, one, out_dtype=dtype)
    a8 = osw.reference_swiglu(gu, in_d)
    expect = og.reference_skinny_gemm(a8, wd8, in_d * s_d, one, out_dtype=dtype)
    assert torch.equal(out, expect) and torch.equal(res, res2) and out.shape == (m, hidden)
    out_res, _ = omlp.reference_llama_mlp(x, r, w, 1e-5, wgu8, in_gu, in_gu * s_gu, wd8, in_d, in_d * s_d, add_residual=True)
    manual = (og.reference_skinny_gemm(a8, wd8, in_d * s_d, one, out_dtype=torch.float32) + res2.float()).to(dtype)
    assert torch.equal(out_res, manual)


# ---- per-row dynamic quantisation (oracle of the *_dynamic operators) ----------------------------------------------------

@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_dynamic_quantisation_oracles_are_fixed_by_their_scaling(dtype):
    """What the definition forces: the row maximum lands on +-448 exactly, the scale is amax/448, and dequantising
    reproduces y to within half an fp8 step (relative 2^-4 for normals, 2^-10 absolute in code units below)."""
    from oracle import residual_rms as orms
    from oracle import swiglu as osw
    g = torch.Generator().manual_seed(3)
    x = torch.randn(6, 512, generator=g).to(dtype)
    r = torch.randn(6, 512, generator=g).to(dtype)
    w = (1 + 0.1 * torch.randn(512, generator=g)).to(dtype)
    q, z, scales, y = orms.precise_residual_rms_dynamic(x, r, w, 1e-5)
    assert torch.equal(z, (x.float() + r.float()).to(dtype))
    gu = torch.randn(5, 2 * 384, generator=g).mul(3)
    gu[1] *= 8.0  # an outlier row gets its own scale
    gu = gu.to(dtype)
    q2, scales2, y2 = osw.precise_swiglu_dynamic(gu)
    for qq, ss, yy in ((q, scales, y), (q2, scales2, y2)):
        assert ss.dtype == torch.float32 and ss.shape == (yy.shape[0],)
        assert torch.allclose(ss.double(), yy.abs().amax(dim=1) / 448.0, rtol=1e-6)
        assert (qq.float().abs().amax(dim=1) == 448.0).all()
        deq = qq.double() * ss.double()[:, None]
        half_step = torch.maximum(yy.abs() * 2.0 ** -4, ss.double()[:, None] * 2.0 ** -10)
        assert ((deq - yy).abs() <= half_step * 1.0001).all()
    # rows scale independently: the outlier row does not cost the others their resolution
    assert scales2[1] > 10 * scales2[0]
    # textbook check of y against plain float64 arithmetic written out
    zz = z.double()
    manual = w.double() * zz / torch.sqrt((zz * zz).mean(dim=1, keepdim=True) + 1e-5)
    assert torch.allclose(y, manual, rtol=1e-12, atol=0)
    gate, up = gu[:, :384].double(), gu[:, 384:].double()
    assert torch.allclose(y2, gate / (1 + torch.exp(-gate)) * up, rtol=1e-12, atol=1e-300)
