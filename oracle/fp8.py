"""OCP float8 e4m3fn on the CPU: decode table, encoder, quantiser.  Test infrastructure only (see __init__.py).

e4m3fn: 1 sign, 4 exponent (bias 7), 3 mantissa bits; no infinities; S.1111.111 is NaN; largest finite value
S.1111.110 = 448; subnormals are multiples of 2^-9.  (The reference's e4m3fnuz has bias 8, max 240, 0x80 = NaN
and reads the same bits as half the value: hf_rocm_kernels/utils/fp8.py:17-29.)
"""
import numpy as np
import torch

FP8_MAX = 448.0


def decode_table() -> np.ndarray:
    """float64 value of each of the 256 codes, from the format's definition (no library call)."""
    out = np.empty(256, dtype=np.float64)
    for code in range(256):
        sign = -1.0 if code & 0x80 else 1.0
        exp = (code >> 3) & 0xF
        man = code & 0x7
        if exp == 0xF and man == 0x7:
            out[code] = np.nan
        elif exp == 0:
            out[code] = sign * man * 2.0 ** -9
        else:
            out[code] = sign * (1.0 + man / 8.0) * 2.0 ** (exp - 7)
    return out


_TABLE = decode_table()


def decode(codes) -> np.ndarray:
    """uint8 codes (numpy array or torch tensor of dtype uint8 / float8_e4m3fn) -> float64 values."""
    if isinstance(codes, torch.Tensor):
        if codes.dtype == torch.float8_e4m3fn:
            codes = codes.view(torch.uint8)
        codes = codes.cpu().numpy()
    return _TABLE[np.asarray(codes, dtype=np.uint8)]


def encode_rne(x: np.ndarray) -> np.ndarray:
    """float -> nearest e4m3fn code, ties to even mantissa, |x| > 448 saturating to +-448, NaN -> 0x7F (the device
    kernels clamp with a median-of-three that turns NaN into -448, code 0xFE, before converting: NaN inputs are the one
    place where the two differ, pinned by a GPU test).

    Written against the value grid (search in the sorted table of the 127 non-negative finite values), not by
    bit manipulation, so that it is independent of torch's cast."""
    x = np.asarray(x, dtype=np.float64)
    pos = _TABLE[:0x7F]  # 0 .. 448, increasing with the code
    mag = np.minimum(np.abs(x), FP8_MAX)
    hi = np.searchsorted(pos, mag, side="left")  # first code with value >= mag
    hi = np.clip(hi, 0, 0x7E)
    lo = np.clip(hi - 1, 0, 0x7E)
    d_hi = pos[hi] - mag
    d_lo = mag - pos[lo]
    pick_lo = (d_lo < d_hi) | ((d_lo == d_hi) & ((lo & 1) == 0))
    code = np.where(pick_lo, lo, hi).astype(np.uint8)
    code = np.where(np.signbit(x), code | 0x80, code).astype(np.uint8)
    return np.where(np.isnan(x), np.uint8(0x7F), code).astype(np.uint8)


def fp8_quantize(x_full_precision: torch.Tensor, scale: torch.Tensor):
    """(x / scale) clamped to +-448 and cast to float8_e4m3fn; returns (quantised, scale).

    Follows hf_rocm_kernels/utils/fp8.py:6-29 up to the cast: multiply by scale.reciprocal() in fp32, clamp to
    the e4m3fn range, cast (round to nearest even).  The reference's last two steps -- zeroing 0x80 and
    relabelling the bits as fnuz with the scale doubled -- exist only because gfx942 is fnuz and are dropped."""
    q = (x_full_precision.float() * scale.reciprocal()).clamp(min=-FP8_MAX, max=FP8_MAX)
    return q.to(torch.float8_e4m3fn), scale


def amax_scale(x: torch.Tensor, dim=None) -> torch.Tensor:
    """amax/448, over the tensor or per slice along `dim` (kept as a size-1 dimension)."""
    x = x.float().abs()
    amax = x.amax() if dim is None else x.amax(dim=dim, keepdim=True)
    return (amax / FP8_MAX).clamp_min(torch.finfo(torch.float32).tiny).to(torch.float32)
