"""The operators trace with fake tensors: every wrapper runs under FakeTensorMode without a GPU and returns outputs of
the right shape and dtype (no kernel runs, no device is touched)."""
import pytest
import torch
from torch._subclasses import FakeTensorMode

import hf_rocm_kernels
from hf_rocm_kernels.combined_ops.llama_mlp import llama_mlp_combined_ops
from hf_rocm_kernels.layers import apply_fp8_linear

FP8 = torch.float8_e4m3fn


def _fp8(*shape):
    return torch.empty(*shape, device="cuda", dtype=FP8)


def test_every_operator_has_a_fake_implementation():
    from hf_rocm_kernels import _fake_kernels
    names = set(_fake_kernels._RETURNS_NOTHING) | set(_fake_kernels._RETURNS_STATUS)
    defined = {n.split("::")[1].split(".")[0] for n in torch._C._dispatch_get_all_op_names() if n.startswith("_HFRK_C::")}
    assert defined == names


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_wrappers_under_fake_tensors(dtype):
    with FakeTensorMode():
        m, hidden, inter = 8, 4096, 14336
        one = torch.empty(1, device="cuda")
        x = torch.empty(m, hidden, device="cuda", dtype=dtype)
        res = torch.empty_like(x)
        w = torch.empty(hidden, device="cuda", dtype=dtype)

        q, res2 = hf_rocm_kernels.residual_rms(input=x, residual=res, weight=w, epsilon=1e-5, scale_tensor=one)
        assert q.shape == (m, hidden) and q.dtype == FP8 and res2.shape == res.shape
        q, _, scales = hf_rocm_kernels.residual_rms_dynamic(input=x, residual=res, weight=w, epsilon=1e-5)
        assert q.dtype == FP8 and scales.shape == (m,)

        gate_up_w = _fp8(2 * inter, hidden)
        proj = hf_rocm_kernels.skinny_gemm(q, gate_up_w.t(), one, output=torch.empty(m, 2 * inter, device="cuda", dtype=dtype))
        assert proj.shape == (m, 2 * inter) and proj.dtype == dtype
        act = hf_rocm_kernels.swiglu(gate_up_proj=proj, scale_tensor=one)
        assert act.shape == (m, inter) and act.dtype == FP8
        act, act_scales = hf_rocm_kernels.swiglu_dynamic(proj)[:2]
        assert act.shape == (m, inter) and act_scales.shape == (m,)

        down_w = _fp8(hidden, inter)
        out = hf_rocm_kernels.skinny_gemm_scaled(act, down_w.t(), act_scales, torch.empty(hidden, device="cuda"))
        assert out.shape == (m, hidden) and out.dtype == torch.bfloat16
        out = hf_rocm_kernels.skinny_gemm_add(act, down_w.t(), one, None, base=res)
        assert out.shape == (m, hidden)
        fused = hf_rocm_kernels.skinny_gemm_swiglu(q, gate_up_w.t(), one, None, one, intermediate_dtype=dtype)
        assert fused.shape == (m, inter) and fused.dtype == FP8

        q, s = hf_rocm_kernels.quantize_fp8(x)
        assert q.shape == x.shape and q.dtype == FP8 and s.shape == (m,)
        y = apply_fp8_linear(x, down_w[:, :hidden].contiguous(), torch.empty(hidden, device="cuda"))
        assert y.shape == (m, hidden) and y.dtype == dtype


@pytest.mark.parametrize("fused", [False, True])
def test_mlp_chain_under_fake_tensors(fused):
    with FakeTensorMode():
        m, hidden, inter = 4, 4096, 14336
        one = torch.empty(1, device="cuda")
        x = torch.empty(m, hidden, device="cuda", dtype=torch.bfloat16)
        out, res = llama_mlp_combined_ops(x, torch.empty_like(x), torch.empty(hidden, device="cuda", dtype=torch.bfloat16), 1e-5,
                                          _fp8(2 * inter, hidden).t(), one, one, _fp8(hidden, inter).t(), one, one,
                                          add_residual=True, fused=fused)
        assert out.shape == (m, hidden) and out.dtype == torch.bfloat16 and res.shape == (m, hidden)


class _Block(torch.nn.Module):
    def __init__(self):
        super().__init__()
        self.gate_up = torch.nn.Linear(512, 1024, bias=False)
        self.down = torch.nn.Linear(512, 512, bias=True)
        self.odd = torch.nn.Linear(100, 8)        # in_features not a multiple of 256: stays
        self.lm_head = torch.nn.Linear(512, 64)   # skipped by name
        self.inner = torch.nn.Sequential(torch.nn.Linear(256, 256), torch.nn.ReLU())


def test_convert_linear_layers_and_state_dict_round_trip_on_the_cpu():
    """Conversion and (de)serialisation are host work: which layers are replaced, what the state dict holds, and that
    a freshly converted model takes another one's state."""
    from hf_rocm_kernels.layers import Fp8Linear, convert_linear_layers
    from oracle import fp8 as ofp8
    torch.manual_seed(0)
    model = _Block().to(torch.bfloat16)
    float_weight = model.down.weight.detach().clone()
    assert convert_linear_layers(model, skip=("lm_head",)) == 3
    assert isinstance(model.gate_up, Fp8Linear) and isinstance(model.down, Fp8Linear) and isinstance(model.inner[0], Fp8Linear)
    assert type(model.odd) is torch.nn.Linear and type(model.lm_head) is torch.nn.Linear
    assert convert_linear_layers(model) == 1          # a second pass finds only lm_head left
    # the quantised weight is the oracle's quantisation with per-channel amax/448 scales
    scale = ofp8.amax_scale(float_weight, dim=1)
    want, _ = ofp8.fp8_quantize(float_weight, scale)
    assert torch.equal(model.down.weight_data.view(torch.uint8), want.view(torch.uint8))
    assert torch.equal(model.down.weight_scale, scale.reshape(-1))
    state = model.state_dict()
    assert state["down.weight_data"].dtype == FP8 and state["down.weight_scale"].shape == (512,) and "gate_up.bias" not in state
    other = _Block().to(torch.bfloat16)
    convert_linear_layers(other)
    result = other.load_state_dict(state)
    assert not result.missing_keys and not result.unexpected_keys
    for name in ("gate_up", "down", "lm_head"):
        a, b = getattr(model, name), getattr(other, name)
        assert torch.equal(a.weight_data.view(torch.uint8), b.weight_data.view(torch.uint8)) and torch.equal(a.weight_scale, b.weight_scale)
        assert b.weight is b.weight_data and not b.packed
    assert "weight=row-major" in repr(other.down)
