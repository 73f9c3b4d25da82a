"""GPU tests of the stand-alone FP8 quantisation kernel (bit-exact against the oracle: a division, a clamp and one
rounding per element) and of the linear-layer front end built on it (same bar as the GEMM tests)."""
import pytest
import torch

from test_gemm_gpu import check_against_oracle

pytestmark = pytest.mark.gpu


def _data(rows, cols, dtype, seed, outliers=True):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(rows, cols, generator=g)
    if outliers and rows > 1:
        x[rows - 1] *= 30.0
        x[0, ::7] *= 1e-3
    return x.to(dtype)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("rows,cols", [(1, 8), (7, 4096), (64, 14336), (3, 32768), (5, 1000), (16, 8192)])
def test_dynamic_quantisation_is_bit_exact(rows, cols, dtype):
    from hf_rocm_kernels import quantize_fp8
    from oracle import fp8 as ofp8
    x = _data(rows, cols, dtype, seed=rows + cols)
    q, scales = quantize_fp8(x.cuda())
    want_scale = ofp8.amax_scale(x, dim=1)
    assert torch.equal(scales.cpu(), want_scale.reshape(-1))
    want_q, _ = ofp8.fp8_quantize(x, want_scale)
    assert torch.equal(q.cpu().view(torch.uint8), want_q.view(torch.uint8))
    # the row maximum lands on +-448
    assert (q.cpu().float().abs().amax(dim=1) == 448).all()


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("scale", [1.0, 0.0123, 3.0])
def test_static_quantisation_is_bit_exact_and_saturates(scale, dtype):
    from hf_rocm_kernels import quantize_fp8
    from oracle import fp8 as ofp8
    x = _data(9, 2048, dtype, seed=3)
    s = torch.tensor([scale])
    q, s_out = quantize_fp8(x.cuda(), s.cuda())
    want_q, _ = ofp8.fp8_quantize(x, s)
    assert torch.equal(q.cpu().view(torch.uint8), want_q.view(torch.uint8))
    assert s_out.item() == pytest.approx(scale)
    if scale < 0.1:
        assert (q.cpu().float().abs() == 448).any()


def test_zero_rows_and_empty_input():
    from hf_rocm_kernels import quantize_fp8
    x = torch.zeros(4, 256, dtype=torch.bfloat16, device="cuda")
    x[2, 5] = 1.5
    q, scales = quantize_fp8(x)
    assert (q.view(torch.uint8)[[0, 1, 3]] == 0).all()
    assert scales[0].item() == torch.finfo(torch.float32).tiny and scales[2].item() == pytest.approx(1.5 / 448)
    q, scales = quantize_fp8(torch.empty(0, 256, dtype=torch.bfloat16, device="cuda"))
    assert q.shape == (0, 256) and scales.shape == (0,)
    with pytest.raises(AssertionError):
        quantize_fp8(torch.zeros(2, 12, dtype=torch.bfloat16, device="cuda"))


def test_c_abi_argument_errors():
    from hf_rocm_kernels import _capi
    lib = _capi.load()
    buf = torch.zeros(4096, dtype=torch.uint8, device="cuda")
    p = buf.data_ptr()
    assert lib.hfrk_quantize_fp8(p, None, p + 2048, None, 1, 64, _capi.BF16, None) == _capi.BAD_SHAPE      # no scales
    assert lib.hfrk_quantize_fp8(p, None, p + 2048, p + 1024, 1, 60, _capi.BF16, None) == _capi.BAD_SHAPE  # cols % 8
    assert lib.hfrk_quantize_fp8(p + 2, None, p + 2048, p + 1024, 1, 64, _capi.BF16, None) == _capi.BAD_ALIGNMENT
    assert lib.hfrk_quantize_fp8(p, None, p + 2048, p + 1024, 1, 64, _capi.FP8_E4M3FN, None) == _capi.BAD_DTYPE
    assert lib.hfrk_quantize_fp8(p, None, p + 2048, p + 1024, 0, 64, _capi.BF16, None) == _capi.SUCCESS


def _linear_case(m, n, k, seed, dtype=torch.bfloat16):
    from hf_rocm_kernels.utils.fp8 import amax_scale, fp8_quantize
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(m, k, generator=g).to(dtype)
    w = torch.randn(n, k, generator=g) * 0.02
    sw = amax_scale(w, dim=1)
    wq, _ = fp8_quantize(w, sw)
    bias = torch.randn(n, generator=g).to(dtype)
    return x, w, wq, sw.reshape(-1), bias


@pytest.mark.parametrize("packed", [False, True])
@pytest.mark.parametrize("m,n,k", [(1, 1024, 1024), (8, 4096, 4096), (33, 1000, 2048), (130, 512, 1024)])
def test_apply_fp8_linear_matches_the_oracle(m, n, k, packed):
    from hf_rocm_kernels.layers import apply_fp8_linear
    from hf_rocm_kernels.utils.weight_format import pack_weight
    from oracle import fp8 as ofp8
    x, _, wq, sw, bias = _linear_case(m, n, k, seed=m + n)
    weight = pack_weight(wq.cuda()) if packed else wq.cuda()
    got = apply_fp8_linear(x.cuda(), weight, sw.cuda(), bias=bias.cuda())
    assert got.shape == (m, n) and got.dtype == x.dtype
    sa = ofp8.amax_scale(x, dim=1)
    xq, _ = ofp8.fp8_quantize(x, sa)
    base = bias.expand(m, n).contiguous()
    check_against_oracle(got, xq, wq.t(), sa.reshape(-1), sw, base=base)
    # static activation scale, residual and bias, leading batch dimensions
    s_in = torch.tensor([4.0 / 448])
    res = torch.randn(2, m, n).to(x.dtype)
    x3 = torch.stack([x, x.flip(0)])
    got3 = apply_fp8_linear(x3.cuda(), weight, sw.cuda(), input_scale=s_in.cuda(), bias=bias.cuda(), residual=res.cuda())
    assert got3.shape == (2, m, n)
    xq3, _ = ofp8.fp8_quantize(x3.reshape(-1, k), s_in)
    check_against_oracle(got3.reshape(-1, n), xq3, wq.t(), s_in, sw, base=(res.reshape(-1, n) + bias).contiguous())


def test_fp8_linear_module_tracks_the_float_layer_and_accepts_quantised_activations():
    from hf_rocm_kernels import residual_rms_dynamic
    from hf_rocm_kernels.layers import Fp8Linear, apply_fp8_linear
    torch.manual_seed(0)
    lin = torch.nn.Linear(2048, 1536, bias=True).to(torch.bfloat16).cuda()
    x = torch.randn(4, 6, 2048, device="cuda").to(torch.bfloat16)
    want = lin(x).float()
    for packed in (False, True):
        for per_channel in (False, True):
            layer = Fp8Linear.from_float(lin, per_channel=per_channel, packed=packed)
            got = layer(x).float()
            rel = (got - want).norm() / want.norm()
            assert rel < 0.06, (packed, per_channel, float(rel))  # two fp8 roundings: a few per cent of the norm
    # activations that arrive quantised (from the fused RMSNorm) skip the quantisation kernel and give the same result
    layer = Fp8Linear.from_float(lin)
    h = torch.randn(8, 2048, device="cuda").to(torch.bfloat16)
    res = torch.randn(8, 2048, device="cuda").to(torch.bfloat16)
    wn = torch.ones(2048, device="cuda", dtype=torch.bfloat16)
    q, res_out, scales = residual_rms_dynamic(h, res.clone(), wn, 1e-5)
    got = layer(q, input_scale=scales)
    want = apply_fp8_linear(q, layer.weight, layer.weight_scale, scales, layer.bias)
    assert torch.equal(got, want) and got.dtype == torch.bfloat16
    assert "in_features=2048" in repr(layer)


@pytest.mark.parametrize("packed", [False, True])
def test_traced_fp8_linear_equals_the_eager_layer(packed):
    """The layer traces as one graph (quantisation kernel and GEMM have shape-only implementations, and the GEMM
    goes through the operator that raises instead of returning a status); traced and eager outputs are identical."""
    from hf_rocm_kernels.layers import Fp8Linear
    torch.manual_seed(1)
    lin = torch.nn.Linear(1024, 768, bias=True).to(torch.bfloat16).cuda()
    layer = Fp8Linear.from_float(lin, per_channel=True, packed=packed)
    traced = torch.compile(layer, backend="aot_eager", fullgraph=True)
    for rows in (1, 8, 8, 70):  # 70 rows: two GEMM launches of at most 64 rows
        x = torch.randn(rows, 1024, device="cuda").to(torch.bfloat16)
        assert torch.equal(traced(x), layer(x)), rows


def test_checked_gemm_operator_raises_where_the_status_operator_returns_a_code():
    import hf_rocm_kernels  # noqa: F401
    a = torch.zeros(4, 512, device="cuda").to(torch.float8_e4m3fn)
    w = torch.zeros(64, 512, device="cuda").to(torch.float8_e4m3fn)
    one = torch.ones(1, device="cuda")
    d = torch.zeros(4, 64, device="cuda", dtype=torch.bfloat16)
    torch.ops._HFRK_C.skinny_gemm_checked(a, w.t(), False, 64, d, None, one, None, None, 0, 0)
    bad_a = torch.zeros(4, 392, device="cuda").to(torch.float8_e4m3fn)  # k not a multiple of 16
    bad_w = torch.zeros(64, 392, device="cuda").to(torch.float8_e4m3fn)
    assert torch.ops._HFRK_C.skinny_gemm_fused(bad_a, bad_w.t(), d, None, one, None, None, 0, 0) == 3
    with pytest.raises(RuntimeError, match="status 3"):
        torch.ops._HFRK_C.skinny_gemm_checked(bad_a, bad_w.t(), False, 64, d, None, one, None, None, 0, 0)


def test_converted_model_tracks_the_float_model_and_reloads_its_state():
    """convert_linear_layers on a small MLP: outputs track the float model, the state dict (fp8 weights, scales)
    reloads into a freshly converted model bit for bit, for row-major and packed weights, and a model converted on the
    CPU works after .to("cuda")."""
    from hf_rocm_kernels.layers import Fp8Linear, convert_linear_layers

    class Mlp(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.up = torch.nn.Linear(1024, 2048, bias=False)
            self.down = torch.nn.Linear(2048, 1024, bias=True)

        def forward(self, x):
            return self.down(torch.nn.functional.silu(self.up(x)))

    torch.manual_seed(2)
    float_model = Mlp().to(torch.bfloat16).cuda()
    x = torch.randn(6, 1024, device="cuda").to(torch.bfloat16)
    want = float_model(x).float()
    for packed in (False, True):
        model = Mlp().to(torch.bfloat16).cuda()
        model.load_state_dict(float_model.state_dict())
        assert convert_linear_layers(model, packed=packed) == 2
        got = model(x)
        rel = (got.float() - want).norm() / want.norm()
        assert rel < 0.08, (packed, float(rel))
        state = {k: v.clone() for k, v in model.state_dict().items()}
        assert state["up.weight_data"].dim() == (1 if packed else 2)
        other = Mlp().to(torch.bfloat16).cuda()
        convert_linear_layers(other, packed=packed)
        other.load_state_dict(state)
        assert torch.equal(other(x), got), packed
    # converted on the host, moved afterwards: the operand follows the buffer
    host = Mlp().to(torch.bfloat16)
    host.load_state_dict({k: v.cpu() for k, v in float_model.state_dict().items()})
    convert_linear_layers(host)
    moved = host.to("cuda")
    assert moved.up.weight.device.type == "cuda" and isinstance(moved.up, Fp8Linear)
    rel = (moved(x).float() - want).norm() / want.norm()
    assert rel < 0.08, float(rel)
