"""MXFP8 (e4m3 data, E8M0 1x32 scales) oracle (test infrastructure, see oracle/__init__.py).

* ``scale_code_from_amax`` / ``quant_rows`` <- cvt_warp_fp16_to_mxfp8
  expert_specialization/csrc/cuda/es_sm100_mxfp8_blockscaled_group_quant.cuh:36-134
* ``sf_offset`` <- ScaleFactorTileLayout and its tiling, same file :25,294-310
* ``grouped_quant`` <- mxfp8_group_quant kernel loop, same file :261-355
* ``grouped_mm`` <- the arithmetic of the SM100 block-scaled GEMM as the
  reference configures it (es_sm100_mxfp8_blockscaled_traits.cuh:44-72) with
  the per-expert bases of es_sm100_mxfp8_blockscaled_functor.cuh:61-75.

Scale rule.  The reference computes ``sf = amax * rcp.approx.ftz(448)`` and
converts it to E8M0 rounding towards +inf (group_quant.cuh:81-88), i.e. the
smallest power of two >= amax/448.  On the fp32 bit pattern of
``amax = (1+f) * 2^e`` that is ``E = e - 8 + 127 + (f > 0.75)`` because
448 = 1.75 * 2^8.  At f == 0.75 exactly the reference's result hinges on the
last bit of NVIDIA's approximate reciprocal; this oracle takes the correctly
rounded reciprocal, for which fl(1.75*2^e * fl(1/448)) == 2^(e-8) and no
round-up happens.  PARITY UNPINNED for that single tie (see oracle/__init__.py).

Domain.  Block amax must be 0 or lie in [2^-110, 2^118]; outside it the
reference's flush-to-zero reciprocal produces infinities/saturation that this
oracle does not model.  NaN/Inf inputs are out of domain too.
"""
import numpy as np

from . import fp8

MX_BLOCK = 32


def scale_code_from_amax(amax):
    """float32 amax array (>= 0, finite) -> uint8 E8M0 code (integer rule above)."""
    amax = np.ascontiguousarray(amax, dtype=np.float32)
    bits = amax.view(np.uint32).astype(np.int64)
    exp_field = (bits >> 23) & 0xFF
    mant = bits & 0x7FFFFF
    code = exp_field - 8 + (mant > 0x600000).astype(np.int64)
    code = np.clip(code, 0, 254)
    code = np.where(amax == 0, 0, code)
    return code.astype(np.uint8)


def scale_code_float_eval(amax):
    """Same quantity through the float route the reference takes, with a
    correctly rounded fp32 reciprocal: ceil-to-power-of-two of fl(amax*fl(1/448))."""
    amax = np.ascontiguousarray(amax, dtype=np.float32)
    rcp = np.float32(1.0) / np.float32(448.0)
    sf = (amax * rcp).astype(np.float32)
    bits = sf.view(np.uint32).astype(np.int64)
    exp_field = (bits >> 23) & 0xFF
    mant = bits & 0x7FFFFF
    code = exp_field + (mant != 0).astype(np.int64)
    code = np.clip(code, 0, 254)
    code = np.where(amax == 0, 0, code)
    return code.astype(np.uint8)


def quant_rows(x):
    """[M, K] float32 holding bf16/fp16-representable values, K % 32 == 0
    -> (codes uint8 [M, K], scale codes uint8 [M, K/32])."""
    x = np.asarray(x, dtype=np.float32)
    m, k = x.shape
    assert k % MX_BLOCK == 0
    xv = x.reshape(m, k // MX_BLOCK, MX_BLOCK)
    amax = np.abs(xv).max(axis=2).astype(np.float32)
    sc = scale_code_from_amax(amax)
    # multiplier 2^(127 - E), exact in fp32; 0 when the block is all zero (keeps the sign of zero)
    inv = np.ldexp(np.float32(1.0), 127 - sc.astype(np.int32)).astype(np.float32)
    inv = np.where(amax == 0, np.float32(0.0), inv)
    scaled = (xv * inv[:, :, None]).astype(np.float32)
    codes = fp8.e4m3fn_encode_rne(scaled, saturate=True).reshape(m, k)
    return codes, sc


def sf_offset(r, c, k):
    """Byte offset of scale (row r, scale column c) inside one expert's scale block.

    The block is tiled 128 rows x 4 scale columns = 512 bytes, K-tile fastest.
    """
    r = np.asarray(r, dtype=np.int64)
    c = np.asarray(c, dtype=np.int64)
    return ((r // 128) * (k // 128) + c // 4) * 512 + (r % 32) * 16 + ((r % 128) // 32) * 4 + c % 4


def sf_block_bytes(rows, k):
    """Size in bytes of a swizzled scale block that holds ``rows`` rows."""
    return ((rows + 127) // 128) * 128 * (k // MX_BLOCK)


def swizzle_scales(sc, k, out=None, base=0):
    """[M, K/32] scale codes -> written into flat uint8 ``out`` at ``base`` in tile layout."""
    m, kc = sc.shape
    assert kc == k // MX_BLOCK
    if out is None:
        out = np.zeros(sf_block_bytes(m, k), dtype=np.uint8)
    rr, cc = np.meshgrid(np.arange(m), np.arange(kc), indexing="ij")
    out[base + sf_offset(rr, cc, k)] = sc
    return out


def unswizzle_scales(flat, rows, k, base=0):
    kc = k // MX_BLOCK
    rr, cc = np.meshgrid(np.arange(rows), np.arange(kc), indexing="ij")
    return np.asarray(flat, dtype=np.uint8)[base + sf_offset(rr, cc, k)]


def grouped_quant(x, problem_sizes, expert_offsets, blockscale_offsets, sf_total_rows=None, fill=0):
    """Grouped quantisation with the reference op's argument meaning.

    x [sumM, K] float32 (bf16/fp16-representable).  Returns (codes uint8 [sumM, K],
    sf uint8 flat of ``sf_total_rows * K/32`` bytes, valid mask of the same size).
    Only bytes whose mask is True are defined by the reference (padding rows of
    each 128-row tile hold unspecified bytes there); they are ``fill`` here.
    """
    x = np.asarray(x, dtype=np.float32)
    total, k = x.shape
    e_cnt = len(problem_sizes)
    if sf_total_rows is None:
        sf_total_rows = max(int(blockscale_offsets[e]) + (int(problem_sizes[e][0]) + 127) // 128 * 128 for e in range(e_cnt))
    codes = np.zeros((total, k), dtype=np.uint8)
    sf = np.full(sf_total_rows * (k // MX_BLOCK), fill, dtype=np.uint8)
    mask = np.zeros(sf.shape, dtype=bool)
    for e in range(e_cnt):
        m_e = int(problem_sizes[e][0])
        k_e = int(problem_sizes[e][2])
        assert k_e == k
        if m_e == 0:
            continue
        off = int(expert_offsets[e])
        base = int(blockscale_offsets[e]) * (k // MX_BLOCK)
        q, sc = quant_rows(x[off:off + m_e])
        codes[off:off + m_e] = q
        swizzle_scales(sc, k, out=sf, base=base)
        rr, cc = np.meshgrid(np.arange(m_e), np.arange(k // MX_BLOCK), indexing="ij")
        mask[base + sf_offset(rr, cc, k)] = True
    return codes, sf, mask


def dequant_rows(codes, sc):
    """codes [M, K] uint8, sc [M, K/32] uint8 -> float64 [M, K] (exact)."""
    return fp8.e4m3fn_decode(codes).astype(np.float64) * np.repeat(fp8.e8m0_decode(sc), MX_BLOCK, axis=1)


def grouped_mm(a_codes, b_codes, sfa, sfb, problem_sizes, expert_offsets, blockscale_offsets,
               out_dtype="bf16", acc="fp32", out=None):
    """d[off_e + m, n] = sum_k a[m,k] 2^(sfa[m,k/32]-127) * b[e,n,k] 2^(sfb[e,n,k/32]-127).

    a_codes [sumM, K], b_codes [E, N, K] (physical), sfa/sfb flat swizzled uint8;
    expert e's A scales start at blockscale_offsets[e]*(K/32), its B scales at
    e*N*(K/32) with N rows.
    """
    from .fp8_blockwise import _matmul_nt, _round_out

    a_codes = np.asarray(a_codes, dtype=np.uint8)
    b_codes = np.asarray(b_codes, dtype=np.uint8)
    sfa = np.asarray(sfa, dtype=np.uint8).reshape(-1)
    sfb = np.asarray(sfb, dtype=np.uint8).reshape(-1)
    e_cnt, n, k = b_codes.shape
    dt = np.float64 if acc == "fp64" else np.float32
    if out is None:
        out = np.full((a_codes.shape[0], n), np.nan, dtype=dt if out_dtype in ("fp32", "fp64") else np.float32)
    for e in range(e_cnt):
        m_e = int(problem_sizes[e][0])
        if m_e == 0:
            continue
        off = int(expert_offsets[e])
        sa = unswizzle_scales(sfa, m_e, k, base=int(blockscale_offsets[e]) * (k // MX_BLOCK))
        sb = unswizzle_scales(sfb, n, k, base=e * n * (k // MX_BLOCK))
        a = dequant_rows(a_codes[off:off + m_e], sa).astype(dt)
        b = dequant_rows(b_codes[e], sb).astype(dt)
        out[off:off + m_e] = _round_out(_matmul_nt(a, b), out_dtype)
    return out
