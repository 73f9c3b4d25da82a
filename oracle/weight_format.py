"""Weight load format on the CPU: packed tile layout and e4m3fnuz -> e4m3fn re-encoding.  Test infrastructure only
(see __init__.py).

The reference has no packed format and no re-encoder: its kernel reads the row-major [n, k] weight
(csrc/op_src/skinny_gemm/producers/n_full_tiles.cu:4-127) and its fp8 tensors are fn bits viewed as fnuz with a
doubled scale (hf_rocm_kernels/utils/fp8.py:17-29).  What is restated here is the format's own definition:

  packed layout   16-row x 256-byte chunks, rows zero-padded to a multiple of 16, chunk (tile, kc) at
                  (tile * k/256 + kc) * 4096; inside a chunk, 16-byte piece j (0..3) of lane l (0..63) at
                  j*1024 + l*16 holds row l%16, bytes (j/2)*128 + (l/16)*32 + (j%2)*16 .. +16 -- i.e. lane l's
                  operand of v_mfma_f32_16x16x128_f8f6f4 step h = j/2 is the 32 contiguous K bytes
                  h*128 + (l/16)*32 .. +32 of row l%16.
  e4m3fnuz        1 sign, 4 exponent (bias 8), 3 mantissa bits; 0x80 is NaN, no negative zero, no infinities;
                  largest value 240; subnormals are multiples of 2^-10.

Pinned by tests/test_oracle_weight_format.py: the fnuz table against torch's float8_e4m3fnuz decode for all 256
codes and against "fn value / 2 on the same bits"; the re-encoder against torch's fnuz -> float -> fn casts for all
256 codes; the layout by an element-by-element loop written from the MFMA operand definition, and by the
pack/unpack round trip.
"""
import numpy as np

from . import fp8

CHUNK_ROWS = 16
CHUNK_COLS = 256
CHUNK_BYTES = CHUNK_ROWS * CHUNK_COLS


def decode_table_fnuz() -> np.ndarray:
    """float64 value of each of the 256 e4m3fnuz codes, from the format's definition (no library call)."""
    out = np.empty(256, dtype=np.float64)
    for code in range(256):
        sign = -1.0 if code & 0x80 else 1.0
        exp = (code >> 3) & 0xF
        man = code & 0x7
        if code == 0x80:
            out[code] = np.nan
        elif exp == 0:
            out[code] = sign * man * 2.0 ** -10
        else:
            out[code] = sign * (1.0 + man / 8.0) * 2.0 ** (exp - 8)
    return out


def reencode_table() -> np.ndarray:
    """fn code with the value of each fnuz code (nearest, ties to even; NaN -> 0x7f), built on the value grids."""
    values = decode_table_fnuz()
    table = fp8.encode_rne(values)
    table[0x80] = 0x7F
    return table.astype(np.uint8)


_REENCODE = None


def reencode_fnuz(codes: np.ndarray) -> np.ndarray:
    """uint8 e4m3fnuz codes -> uint8 e4m3fn codes of the same values."""
    global _REENCODE
    if _REENCODE is None:
        _REENCODE = reencode_table()
    return _REENCODE[np.asarray(codes, dtype=np.uint8)]


def packed_bytes(n: int, k: int) -> int:
    return -(-n // CHUNK_ROWS) * CHUNK_ROWS * k


def pack_weight(w: np.ndarray) -> np.ndarray:
    """[n, k] uint8 (k % 256 == 0) -> packed uint8 vector, by array reshapes."""
    w = np.asarray(w, dtype=np.uint8)
    n, k = w.shape
    assert k % CHUNK_COLS == 0
    tiles = -(-n // CHUNK_ROWS)
    padded = np.zeros((tiles * CHUNK_ROWS, k), dtype=np.uint8)
    padded[:n] = w
    # [tile, row li, kc, step h, k-group lg, half p, 16 bytes]  ->  [tile, kc, h, p, lg, li, 16]; piece j = 2h + p
    x = padded.reshape(tiles, 16, k // 256, 2, 4, 2, 16)
    return np.ascontiguousarray(x.transpose(0, 2, 3, 5, 4, 1, 6)).reshape(-1)


def unpack_weight(packed: np.ndarray, n: int, k: int) -> np.ndarray:
    """Inverse of pack_weight (padding rows dropped)."""
    tiles = -(-n // CHUNK_ROWS)
    x = np.asarray(packed, dtype=np.uint8).reshape(tiles, k // 256, 2, 2, 4, 16, 16)
    rows = np.ascontiguousarray(x.transpose(0, 5, 1, 2, 4, 3, 6)).reshape(tiles * CHUNK_ROWS, k)
    return rows[:n].copy()


def packed_offset(row: int, col: int, k: int) -> int:
    """Byte offset of weight element (row, col) in the packed buffer, straight from the layout's definition."""
    tile, li = divmod(row, 16)
    kc, c = divmod(col, 256)
    h, c = divmod(c, 128)   # MFMA step
    lg, c = divmod(c, 32)   # k-group of the lane
    p, byte = divmod(c, 16) # first or second 16-byte piece of the lane's 32-byte operand
    lane = lg * 16 + li
    return (tile * (k // 256) + kc) * CHUNK_BYTES + (2 * h + p) * 1024 + lane * 16 + byte
