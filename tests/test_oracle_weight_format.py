"""Pins the CPU oracle of the weight load format (oracle/weight_format.py): the e4m3fnuz table and the fnuz -> fn
re-encoder against torch's own float8 casts (library routines) and against the "same bits, half the value" rule
the reference relies on (hf_rocm_kernels/utils/fp8.py:27-29); the packed layout against an element loop written
from the MFMA operand definition, plus its inverse.  No GPU."""
import numpy as np
import pytest
import torch

from oracle import fp8, weight_format as wf


def test_fnuz_table_matches_torch_for_all_codes():
    codes = torch.arange(256, dtype=torch.uint8)
    want = codes.view(torch.float8_e4m3fnuz).float().numpy().astype(np.float64)
    got = wf.decode_table_fnuz()
    assert np.isnan(got[0x80]) and np.isnan(want[0x80])
    keep = np.arange(256) != 0x80
    assert np.array_equal(got[keep], want[keep])


def test_fnuz_is_half_the_fn_value_on_the_same_bits():
    fnuz, fn = wf.decode_table_fnuz(), fp8.decode_table()
    for code in range(256):
        if code in (0x80, 0x7F, 0xFF):  # fnuz NaN; fn NaN (fnuz +-240)
            continue
        assert fnuz[code] == fn[code] / 2
    assert fnuz[0x7F] == 240.0 and fnuz[0xFF] == -240.0


def test_reencode_table_matches_torch_casts_for_all_codes():
    codes = torch.arange(256, dtype=torch.uint8)
    want = codes.view(torch.float8_e4m3fnuz).float().to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    got = wf.reencode_table()
    keep = np.arange(256) != 0x80
    assert np.array_equal(got[keep], want[keep])
    assert got[0x80] == 0x7F  # NaN stays NaN (torch gives a NaN code too)
    assert np.isnan(fp8.decode_table()[want[0x80]])


def test_reencode_is_exact_from_two_to_the_minus_six_up_and_rounds_to_even_below():
    fnuz, fn = wf.decode_table_fnuz(), fp8.decode_table()
    table = wf.reencode_table()
    for code in range(256):
        if code == 0x80:
            continue
        v, r = fnuz[code], fn[table[code]]
        if abs(v) >= 2.0 ** -6:
            assert r == v
        else:
            assert abs(r - v) <= 2.0 ** -10  # half a step of fn's subnormal grid
            if abs(r - v) == 2.0 ** -10:  # a tie: the even multiple of 2^-9 wins
                assert (abs(r) / 2.0 ** -9) % 2 == 0
    assert table[0x00] == 0x00 and fn[table[0x7F]] == 240.0 and fn[table[0xFF]] == -240.0
    # codes at and around the boundary, by hand: fnuz 0x0f = 15 * 2^-10 -> 7.5 units -> 8 = fn 0x08 (2^-6)
    assert table[0x0F] == 0x08 and table[0x10] == 0x08 and table[0x01] == 0x00 and table[0x03] == 0x02


@pytest.mark.parametrize("n,k", [(16, 256), (37, 512), (1, 256), (130, 1024)])
def test_pack_matches_the_operand_definition_element_by_element(n, k):
    rng = np.random.default_rng(n * 1000 + k)
    w = rng.integers(0, 256, (n, k), dtype=np.uint8)
    packed = wf.pack_weight(w)
    assert packed.size == wf.packed_bytes(n, k) == -(-n // 16) * 16 * k
    seen = np.zeros(packed.size, dtype=bool)
    for r in range(n):
        for c in range(k):
            off = wf.packed_offset(r, c, k)
            assert packed[off] == w[r, c]
            seen[off] = True
    assert not packed[~seen].any()  # padding rows are zero
    assert seen.sum() == n * k      # the offsets are a bijection onto the non-padding bytes
    assert np.array_equal(wf.unpack_weight(packed, n, k), w)


def test_a_lane_operand_is_thirty_two_contiguous_k_bytes_of_one_row():
    """The property the GEMM relies on: pieces 2h and 2h+1 of lane l, concatenated, are bytes h*128 + (l/16)*32 .. +32
    of row l%16 of the chunk."""
    k = 512
    w = np.arange(16 * k, dtype=np.uint32).reshape(16, k)
    w8 = (w % 251).astype(np.uint8)
    packed = wf.pack_weight(w8)
    for kc in range(k // 256):
        chunk = packed[kc * 4096:(kc + 1) * 4096]
        for lane in range(64):
            for h in range(2):
                operand = np.concatenate([chunk[(2 * h) * 1024 + lane * 16:][:16], chunk[(2 * h + 1) * 1024 + lane * 16:][:16]])
                c0 = kc * 256 + h * 128 + (lane // 16) * 32
                assert np.array_equal(operand, w8[lane % 16, c0:c0 + 32])


def test_pack_unpack_round_trip_on_random_shapes():
    """Property check over many (n, k): unpack(pack(w)) == w, the packed size is the padded size, padding is zero."""
    from hypothesis import given, settings, strategies as st

    @settings(max_examples=60, deadline=None)
    @given(n=st.integers(1, 70), kc=st.integers(1, 3), seed=st.integers(0, 2 ** 31 - 1))
    def check(n, kc, seed):
        k = 256 * kc
        w = np.random.default_rng(seed).integers(0, 256, (n, k), dtype=np.uint8)
        packed = wf.pack_weight(w)
        assert packed.size == wf.packed_bytes(n, k)
        assert np.array_equal(wf.unpack_weight(packed, n, k), w)
        assert int(packed.astype(np.int64).sum()) == int(w.astype(np.int64).sum())  # padding adds nothing
        r, c = (seed % n), (seed // 7) % k
        assert packed[wf.packed_offset(r, c, k)] == w[r, c]

    check()


def test_reencode_preserves_order_and_sign_symmetry():
    """The code map is monotone in value (no two fnuz values swap order) and odd: map(-x) = -map(x)."""
    fnuz, fn = wf.decode_table_fnuz(), fp8.decode_table()
    table = wf.reencode_table()
    codes = [c for c in range(256) if c != 0x80]
    by_value = sorted(codes, key=lambda c: fnuz[c])
    mapped = [fn[table[c]] for c in by_value]
    assert all(a <= b for a, b in zip(mapped, mapped[1:]))
    for c in range(1, 0x80):
        assert fn[table[c | 0x80]] == -fn[table[c]]
