"""FP8-blockwise grouped GEMM oracle (test infrastructure, see oracle/__init__.py).

Restates, in numpy, the torch helpers the reference defines next to its op:

* ``quant_act_1x128``      <- per_token_cast_to_fp8   test/test_es_grouped_gemm.py:36-44
* ``quant_weight_128x128`` <- per_block_cast_to_fp8   test/test_es_grouped_gemm.py:47-59
* ``grouped_mm``           <- baseline_scaled_mm      test/test_es_grouped_gemm.py:62-86
  applied per expert with the pointer arithmetic of
  expert_specialization/csrc/cuda/es_fp8_blockwise_functor.cuh:57-74
* ``calc_diff``            <- test/test_es_grouped_gemm.py:25-29

Tensors are numpy arrays: fp8 data as uint8 codes, bf16 data as float32 arrays
holding bf16-representable values.
"""
import numpy as np

from . import fp8

BLOCK = 128


def quant_act_1x128(x, scale_via_reciprocal=False):
    """[M, K] float32 (K % 128 == 0) -> (codes uint8 [M, K], scales float32 [M, K/128]).

    amax over each 1x128 block, clamped below at 1e-4; data = e4m3(x * (448 / amax))
    with the product formed in fp32; scale = amax / 448.  The reference writes the multiplier as
    ``448.0 / x_amax`` with a Python scalar on the left, which torch evaluates as
    ``reciprocal(x_amax) * 448.0`` (two fp32 roundings, not one division); the same is done here.
    The scale ``x_amax / 448.0`` is a true division when torch runs the helper on the CPU; on a GPU
    torch divides a tensor by a Python scalar as ``x_amax * fl(1 / 448)`` (one ulp apart for some
    values), which is what the reference's callers get: ``scale_via_reciprocal=True`` selects that.
    """
    x = np.asarray(x, dtype=np.float32)
    m, k = x.shape
    assert k % BLOCK == 0
    xv = x.reshape(m, k // BLOCK, BLOCK)
    amax = np.maximum(np.abs(xv).max(axis=2), np.float32(1e-4)).astype(np.float32)
    mult = ((np.float32(1.0) / amax).astype(np.float32) * np.float32(448.0)).astype(np.float32)
    scaled = (xv * mult[:, :, None]).astype(np.float32)
    codes = fp8.e4m3fn_encode_rne(scaled).reshape(m, k)
    if scale_via_reciprocal:
        return codes, (amax * (np.float32(1.0) / np.float32(448.0))).astype(np.float32)
    return codes, (amax / np.float32(448.0)).astype(np.float32)


def swiglu(x, out_dtype="bf16"):
    """[M, 2*I] float32 (values representable in out_dtype) -> [M, I] float32: silu(gate) * up with gate the
    first half of a row and up the second, the product formed in fp32 and rounded once to out_dtype.
    Defines the fused SwiGLU + quantisation operator of this build (no counterpart in the reference);
    silu(x) = x / (1 + exp(-x)) with exp evaluated in float64 and rounded, i.e. the correctly rounded
    fp32 exp that a device routine approximates to within an ulp or two."""
    x = np.asarray(x, dtype=np.float32)
    inter = x.shape[1] // 2
    g, u = x[:, :inter], x[:, inter:]
    e = np.exp(-g.astype(np.float64)).astype(np.float32)
    h = ((g / (np.float32(1.0) + e)).astype(np.float32) * u).astype(np.float32)
    return fp8.bf16_round(h) if out_dtype == "bf16" else fp8.fp16_round(h)


def quant_weight_128x128(w, scale_via_reciprocal=False):
    """[N, K] float32 (both % 128 == 0) -> (codes uint8 [N, K], scales float32 [N/128, K/128]).

    The reference quantises the (K, N) view and transposes data and scales back
    (test/test_es_grouped_gemm.py:127,132-134,160,166-168), which equals
    quantising the physical [N, K] matrix directly.
    """
    w = np.asarray(w, dtype=np.float32)
    n, k = w.shape
    assert n % BLOCK == 0 and k % BLOCK == 0
    wv = w.reshape(n // BLOCK, BLOCK, k // BLOCK, BLOCK)
    amax = np.maximum(np.abs(wv).max(axis=(1, 3)), np.float32(1e-4)).astype(np.float32)
    mult = ((np.float32(1.0) / amax).astype(np.float32) * np.float32(448.0)).astype(np.float32)
    scaled = (wv * mult[:, None, :, None]).astype(np.float32)
    codes = fp8.e4m3fn_encode_rne(scaled).reshape(n, k)
    if scale_via_reciprocal:   # torch's GPU evaluation of amax / 448.0, see quant_act_1x128
        return codes, (amax * (np.float32(1.0) / np.float32(448.0))).astype(np.float32)
    return codes, (amax / np.float32(448.0)).astype(np.float32)


def dequant_act(a_codes, sa, dtype=np.float32):
    """scale * value, formed in `dtype` (fp32 as the reference does; fp64 is exact)."""
    return fp8.e4m3fn_decode(a_codes).astype(dtype) * np.repeat(sa, BLOCK, axis=1).astype(dtype)


def dequant_weight(b_codes, sb, dtype=np.float32):
    return fp8.e4m3fn_decode(b_codes).astype(dtype) * np.repeat(np.repeat(sb, BLOCK, axis=0), BLOCK, axis=1).astype(dtype)


def _round_out(y, out_dtype):
    if out_dtype == "bf16":
        return fp8.bf16_round(y.astype(np.float32))
    if out_dtype == "fp16":
        return fp8.fp16_round(y.astype(np.float32))
    if out_dtype in ("fp32", "fp64"):
        return y
    raise ValueError(out_dtype)


def grouped_mm(a_codes, b_codes, sa, sb, problem_sizes, expert_offsets, out_dtype="bf16", acc="fp32", out=None):
    """Dequantise-then-matmul per expert.

    a_codes [sumM, K] uint8, b_codes [E, N, K] uint8 (physical layout),
    sa [sumM, K/128] f32, sb [E, N/128, K/128] f32, problem_sizes int [E, 3] rows
    (M_e, N, K), expert_offsets int [E] (exclusive prefix sum of M_e).
    Rows of experts with M_e == 0 and rows not covered by any expert are left
    as they are in ``out`` (NaN when ``out`` is None).
    """
    a_codes = np.asarray(a_codes, dtype=np.uint8)
    b_codes = np.asarray(b_codes, dtype=np.uint8)
    e_cnt, n, k = b_codes.shape
    dt = np.float64 if acc == "fp64" else np.float32
    if out is None:
        out = np.full((a_codes.shape[0], n), np.nan, dtype=dt if out_dtype in ("fp32", "fp64") else np.float32)
    for e in range(e_cnt):
        m_e, n_e, k_e = (int(v) for v in problem_sizes[e])
        if m_e == 0:
            continue
        assert n_e == n and k_e == k
        off = int(expert_offsets[e])
        a32 = dequant_act(a_codes[off:off + m_e], sa[off:off + m_e], dt)
        b32 = dequant_weight(b_codes[e], sb[e], dt)
        y = _matmul_nt(a32, b32)
        out[off:off + m_e] = _round_out(y, out_dtype)
    return out


def _matmul_nt(a, b):
    """a [M, K] @ b[N, K]^T in the dtype of the inputs (torch CPU for speed when available)."""
    try:
        import torch

        ta = torch.from_numpy(np.ascontiguousarray(a))
        tb = torch.from_numpy(np.ascontiguousarray(b))
        return torch.mm(ta, tb.t()).numpy()
    except ImportError:  # pragma: no cover
        return a @ b.T


def calc_diff(x, y):
    x = np.asarray(x, dtype=np.float64)
    y = np.asarray(y, dtype=np.float64)
    den = (x * x + y * y).sum()
    return 1.0 - 2.0 * (x * y).sum() / den
