"""OCP FP8 e4m3fn / E8M0 / bf16 codecs in numpy (test infrastructure, see oracle/__init__.py).

The reference leans on ``tensor.to(torch.float8_e4m3fn)``
(test/test_es_grouped_gemm.py:43,57) and on ``__nv_fp8x2_e4m3(float2)``
(expert_specialization/csrc/cuda/es_sm100_mxfp8_blockscaled_group_quant.cuh:108-115)
for the fp32 -> e4m3 step; both are round-to-nearest-even onto the e4m3fn grid.
This module builds that grid from the format definition (1 sign, 4 exponent bits
with bias 7, 3 mantissa bits, no infinities, 0x7f/0xff = NaN) and rounds by a
nearest-value search, so it shares no code with torch's bit-twiddling cast.
"""
import numpy as np

E4M3_MAX = 448.0


def _build_decode_table():
    t = np.zeros(256, dtype=np.float64)
    for b in range(256):
        s = -1.0 if b & 0x80 else 1.0
        e = (b >> 3) & 0xF
        m = b & 0x7
        if e == 0xF and m == 0x7:
            t[b] = np.nan
        elif e == 0:
            t[b] = s * (m / 8.0) * 2.0 ** (-6)
        else:
            t[b] = s * (1.0 + m / 8.0) * 2.0 ** (e - 7)
    return t


_DECODE64 = _build_decode_table()
_DECODE32 = _DECODE64.astype(np.float32)
# non-negative finite grid: codes 0x00..0x7e, strictly increasing
_POS = _DECODE64[:0x7F].copy()
_MID = (_POS[:-1] + _POS[1:]) / 2.0  # midpoint between code i and i+1


def e4m3fn_decode(codes):
    """uint8 codes -> float32 values (exact; NaN for 0x7f / 0xff)."""
    return _DECODE32[np.asarray(codes, dtype=np.uint8)]


def e4m3fn_encode_rne(x, saturate=False):
    """float array -> uint8 e4m3fn codes, round to nearest, ties to even code.

    ``saturate=False`` follows torch's cast (magnitudes that round above 448
    become NaN 0x7f); ``saturate=True`` follows the CUDA ``satfinite`` converts
    (clamped to +-448).  NaN input gives 0x7f | sign.
    """
    x = np.asarray(x)
    xf = x.astype(np.float64)
    sign = (np.signbit(xf)).astype(np.uint8) << 7
    mag = np.abs(xf)
    # index of the first midpoint that is >= mag  -> candidate code
    idx = np.searchsorted(_MID, mag, side="left")
    idx = np.minimum(idx, 0x7E)
    # ties: mag == MID[idx] -> choose the even code of (idx, idx+1)
    tie = (idx < len(_MID)) & (mag == _MID[np.minimum(idx, len(_MID) - 1)])
    up = tie & ((idx & 1) == 1)
    idx = np.where(up, idx + 1, idx)
    # overflow: strictly beyond the midpoint between 448 and the would-be next
    # value 480 (464 itself is a tie and goes to the even code 0x7e = 448)
    over = mag > 464.0
    if saturate:
        idx = np.where(over, 0x7E, idx)
    else:
        idx = np.where(over, 0x7F, idx)
    idx = np.where(np.isnan(xf), 0x7F, idx)
    return (idx.astype(np.uint8) | sign).astype(np.uint8)


def bf16_round(x):
    """float32 array -> float32 array holding the nearest bf16 value (RNE)."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    u = x.view(np.uint32).astype(np.uint64)
    rounded = ((u + 0x7FFF + ((u >> 16) & 1)) >> 16) << 16
    out = rounded.astype(np.uint32).view(np.float32)
    return np.where(np.isnan(x), x, out).astype(np.float32)


def bf16_bits(x):
    """float32 array of bf16-representable values -> uint16 bit patterns."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    return (x.view(np.uint32) >> 16).astype(np.uint16)


def bf16_from_bits(b):
    b = np.ascontiguousarray(b, dtype=np.uint16)
    return (b.astype(np.uint32) << 16).view(np.float32)


def fp16_round(x):
    return np.asarray(x, dtype=np.float32).astype(np.float16).astype(np.float32)


def e8m0_decode(codes):
    """uint8 E8M0 codes -> float64 2^(code-127) (0xff = NaN)."""
    c = np.asarray(codes, dtype=np.uint8).astype(np.int32)
    out = np.ldexp(1.0, c - 127)
    return np.where(c == 255, np.nan, out)
