"""Pins the FP8 part of the oracle (oracle/fp8.py, oracle/c/hfrk_oracle.c) without a GPU.

The decode table is checked against the format's closed form and torch's own bit reinterpretation; the
round-to-nearest-even encoder (written against the value grid) against torch's cast on every midpoint and on a
dense sweep; the quantiser through invariants a wrong clamp, a wrong rounding mode or a lost sign would break.
"""
import numpy as np
import torch

from oracle import c_oracle, fp8


def test_decode_table_matches_torch_bit_view():
    codes = torch.arange(256, dtype=torch.uint8)
    ref = codes.view(torch.float8_e4m3fn).float().double().numpy()
    mine = fp8.decode_table()
    assert np.array_equal(np.isnan(ref), np.isnan(mine))
    ok = ~np.isnan(ref)
    assert np.array_equal(ref[ok], mine[ok])


def test_decode_known_values():
    t = fp8.decode_table()
    assert t[0x00] == 0.0 and t[0x80] == 0.0 and np.signbit(t[0x80])
    assert t[0x01] == 2.0 ** -9          # smallest subnormal
    assert t[0x07] == 7 * 2.0 ** -9      # largest subnormal
    assert t[0x08] == 2.0 ** -6          # smallest normal
    assert t[0x38] == 1.0
    assert t[0x7E] == 448.0 and t[0xFE] == -448.0
    assert np.isnan(t[0x7F]) and np.isnan(t[0xFF])
    assert np.count_nonzero(np.isnan(t)) == 2     # no infinities, two NaNs
    # every finite value is an integer multiple of 2^-9 below 2^18 * 2^-9: what makes exact dot products possible
    fin = t[~np.isnan(t)] * 512
    assert np.array_equal(fin, np.rint(fin)) and np.abs(fin).max() == 448 * 512


def test_c_decode_matches_python_table():
    lib = c_oracle.load()
    t = fp8.decode_table()
    for code in range(256):
        v = lib.hfrk_oracle_decode_e4m3fn(code)
        assert (np.isnan(v) and np.isnan(t[code])) or v == t[code]


def _torch_cast(x):
    return torch.from_numpy(np.asarray(x, dtype=np.float32)).to(torch.float8_e4m3fn).view(torch.uint8).numpy()


def test_encoder_matches_torch_on_every_midpoint_and_neighbours():
    t = fp8.decode_table()[:0x7F]
    mids = (t[:-1] + t[1:]) / 2           # exactly representable in fp32
    pts = np.concatenate([t, mids, np.nextafter(mids.astype(np.float32), np.float32(0)),
                          np.nextafter(mids.astype(np.float32), np.float32(1e9))]).astype(np.float32)
    pts = np.concatenate([pts, -pts])
    assert np.array_equal(fp8.encode_rne(pts), _torch_cast(pts))


def test_encoder_matches_torch_on_dense_sweep_and_c_encoder():
    rng = np.random.default_rng(0)
    x = np.concatenate([rng.normal(0, 1, 20000), rng.normal(0, 100, 20000), rng.uniform(-448, 448, 20000),
                        rng.normal(0, 1e-3, 5000)]).astype(np.float32)
    # torch's cast maps values beyond the last rounding boundary (464) to NaN; the quantiser clamps to +-448 first,
    # which is the case the encoder restates (it saturates), so compare on clamped inputs
    x = np.clip(x, -448, 448)
    mine = fp8.encode_rne(x)
    assert np.array_equal(mine, _torch_cast(x))
    lib = c_oracle.load()
    sample = x[::97]
    c_codes = np.array([lib.hfrk_oracle_encode_e4m3fn(float(v)) for v in sample], dtype=np.uint8)
    assert np.array_equal(c_codes, fp8.encode_rne(sample))


def test_quantize_invariants():
    g = torch.Generator().manual_seed(1)
    x = torch.randn(64, 257, generator=g) * 50
    scale = torch.tensor([2.5])
    q, s = fp8.fp8_quantize(x, scale)
    assert s is scale and q.dtype == torch.float8_e4m3fn
    qf = q.float()
    # saturation instead of NaN/inf, and nothing beyond +-448
    assert not qf.isnan().any() and qf.abs().max() <= 448
    big = fp8.fp8_quantize(torch.tensor([1e6, -1e6, 448 * 2.5, 449 * 2.5]), scale)[0].float()
    assert big.tolist() == [448.0, -448.0, 448.0, 448.0]
    # idempotent on representable values
    q2, _ = fp8.fp8_quantize(qf * scale, scale)
    assert torch.equal(q2.view(torch.uint8), q.view(torch.uint8))
    # odd symmetry (sign is kept, including -0) and monotonicity
    qn, _ = fp8.fp8_quantize(-x, scale)
    assert torch.equal(qn.float(), -qf)
    xs, _ = torch.sort(x.flatten())
    assert (fp8.fp8_quantize(xs, scale)[0].float().diff() >= 0).all()
    # error at most half a unit in the last place of the result (relative 2^-4) or half a subnormal step
    err = (qf - x / scale).abs()
    assert (err <= torch.maximum((x / scale).abs() * 2.0 ** -4, torch.tensor(2.0 ** -10))).all()
    # own encoder agrees with the torch path used by the quantiser
    assert np.array_equal(fp8.encode_rne((x / scale).numpy().clip(-448, 448)), q.view(torch.uint8).numpy())


def test_amax_scale_maps_extreme_to_448():
    g = torch.Generator().manual_seed(2)
    x = torch.randn(8, 512, generator=g)
    s = fp8.amax_scale(x)
    assert fp8.fp8_quantize(x, s)[0].float().abs().max() == 448
    srow = fp8.amax_scale(x, dim=1)
    assert srow.shape == (8, 1)
    assert (fp8.fp8_quantize(x, srow)[0].float().abs().amax(dim=1) == 448).all()
