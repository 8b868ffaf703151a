"""Pins oracle/mxfp8.py: scale rule, quantised bytes, swizzled scale layout and the block-scaled GEMM."""
import numpy as np
import pytest

from oracle import brute, fp8
from oracle import mxfp8 as o


def _positive_patterns(fmt):
    if fmt == "bf16":
        bits = np.arange(1, 0x7F80, dtype=np.uint32) << 16
        return bits.view(np.float32)
    h = np.arange(1, 0x7C00, dtype=np.uint16).view(np.float16)
    return h.astype(np.float32)


@pytest.mark.parametrize("fmt", ["bf16", "fp16"])
def test_scale_code_integer_rule_equals_float_route_exhaustively(fmt):
    """The bit-pattern rule equals ceil-to-power-of-two of fl(amax * fl(1/448)) for every positive
    bf16 / fp16 amax inside the stated domain (the tie amax = 448*2^j included)."""
    amax = _positive_patterns(fmt)
    amax = amax[(amax >= 2.0 ** -110) & (amax <= 2.0 ** 118)]
    assert np.array_equal(o.scale_code_from_amax(amax), o.scale_code_float_eval(amax))


def test_scale_code_known_values_and_minimality():
    a = np.array([448.0, 449.0, 447.0, 224.0, 1.75, 1.7578125, 3.5, 1.0, 0.0, 2.0 ** -20], dtype=np.float32)
    code = o.scale_code_from_amax(a).astype(int)
    assert code.tolist() == [127, 128, 127, 126, 119, 120, 120, 119, 0, 127 - 28]
    # minimality: 2^(code-127) >= amax/448 > 2^(code-128)
    rng = np.random.default_rng(0)
    x = fp8.bf16_round(np.exp(rng.uniform(-30, 30, 20000)).astype(np.float32))
    c = o.scale_code_from_amax(x).astype(np.int64)
    s = np.ldexp(1.0, c - 127)
    assert (s >= x.astype(np.float64) / 448.0).all() and (s / 2 < x.astype(np.float64) / 448.0).all()


def test_quant_rows_properties():
    rng = np.random.default_rng(1)
    x = fp8.bf16_round((rng.standard_normal((33, 256)) * np.exp(rng.uniform(-8, 8, (33, 1)))).astype(np.float32))
    x[4, 32:64] = 0.0
    x[5, 64:96] = -0.0
    q, sc = o.quant_rows(x)
    v = fp8.e4m3fn_decode(q).astype(np.float64)
    assert np.abs(v).max() <= 448.0 and not np.isnan(v).any()
    assert sc[4, 1] == 0 and not q[4, 32:64].any()
    assert sc[5, 2] == 0 and (q[5, 64:96] == 0x80).all()     # sign of zero survives x * 0.0f
    deq = o.dequant_rows(q, sc)
    scale = np.repeat(fp8.e8m0_decode(sc), 32, axis=1)
    # e4m3 RNE: half an ulp is 2^-4 relative for normals, 2^-10 * scale absolute for subnormals
    assert (np.abs(deq - x) <= 2.0 ** -4 * np.abs(x) + scale * 2.0 ** -10 + 1e-300).all()
    # the block maximum lands in the top binade of e4m3: 224 < |q| <= 448
    xb = np.abs(x.reshape(33, 8, 32)); vb = np.abs(v.reshape(33, 8, 32))
    top = np.take_along_axis(vb, xb.argmax(axis=2)[..., None], axis=2)[..., 0]
    nz = xb.max(axis=2) > 0
    assert (top[nz] > 224.0 - 1e-9).all() and (top[nz] <= 448.0).all()


def _cute_index(coord, shape, stride):
    """Index of a natural coordinate in a (possibly nested) CuTe layout; integers against nested
    modes are split colexicographically (first sub-mode fastest)."""
    if isinstance(shape, tuple):
        if isinstance(coord, tuple):
            return sum(_cute_index(c, s, d) for c, s, d in zip(coord, shape, stride))
        idx = 0
        for s, d in zip(shape, stride):
            size = int(np.prod(s))
            idx += _cute_index(coord % size, s, d)
            coord //= size
        return idx
    return coord * stride


@pytest.mark.parametrize("rows,k", [(1, 128), (127, 128), (128, 384), (129, 384), (300, 384)])
def test_sf_offset_equals_cute_layout_enumeration(rows, k):
    """ScaleFactorTileLayout ((32,4),4):((16,4),1), tiles laid out K-tile fastest, 512 bytes apart."""
    tile_shape, tile_stride = ((32, 4), 4), ((16, 4), 1)
    kc = k // 32
    seen = set()
    for r in range(rows):
        for c in range(kc):
            tile = (r // 128) * (k // 128) + c // 4
            lit = tile * 512 + _cute_index((r % 128, c % 4), tile_shape, tile_stride)
            assert int(o.sf_offset(r, c, k)) == lit == brute.sf_offset(r, c, k)
            seen.add(lit)
    assert len(seen) == rows * kc and max(seen) < o.sf_block_bytes(rows, k)
    sc = np.arange(rows * kc, dtype=np.int64).reshape(rows, kc).astype(np.uint8)
    flat = o.swizzle_scales(sc, k)
    assert np.array_equal(o.unswizzle_scales(flat, rows, k), sc)


def test_grouped_quant_layout_and_mask():
    rng = np.random.default_rng(2)
    rows = [5, 0, 130]
    k = 256
    x = fp8.bf16_round(rng.standard_normal((sum(rows), k)).astype(np.float32))
    ps = [[m, 9, k] for m in rows]
    eo = [0, 5, 5]
    bso = [0, 128, 128]
    q, sf, mask = o.grouped_quant(x, ps, eo, bso, fill=0xEE)
    assert sf.size == (128 + 256) * (k // 32) and mask.sum() == sum(rows) * (k // 32)
    q0, s0 = o.quant_rows(x[:5])
    assert np.array_equal(q[:5], q0)
    assert np.array_equal(o.unswizzle_scales(sf, 5, k, base=0), s0)
    q2, s2 = o.quant_rows(x[5:])
    assert np.array_equal(o.unswizzle_scales(sf, 130, k, base=128 * (k // 32)), s2)
    assert (sf[~mask] == 0xEE).all()


def _mx_problem(rng, rows, n, k):
    e = len(rows)
    total = sum(rows)
    a = fp8.bf16_round(rng.standard_normal((total, k)).astype(np.float32))
    ps = np.array([[m, n, k] for m in rows], dtype=np.int32)
    eo = np.concatenate([[0], np.cumsum(rows)[:-1]]).astype(np.int32)
    aligned = [(m + 127) // 128 * 128 for m in rows]
    bso = np.concatenate([[0], np.cumsum(aligned)[:-1]]).astype(np.int32)
    a_q, sfa, _ = o.grouped_quant(a, ps, eo, bso, sf_total_rows=sum(aligned))
    b_q = np.zeros((e, n, k), dtype=np.uint8)
    sfb = np.zeros(e * n * (k // 32), dtype=np.uint8)
    for i in range(e):
        w = fp8.bf16_round((rng.standard_normal((n, k)) * 0.05).astype(np.float32))
        b_q[i], sc = o.quant_rows(w)
        o.swizzle_scales(sc, k, out=sfb, base=i * n * (k // 32))
    return a_q, b_q, sfa, sfb, ps, eo, bso


def test_grouped_mm_against_c_brute_force():
    rng = np.random.default_rng(3)
    a_q, b_q, sfa, sfb, ps, eo, bso = _mx_problem(rng, [3, 0, 2], 128, 256)
    ref = brute.mxfp8(a_q, b_q, sfa, sfb, ps, eo, bso)
    y64 = o.grouped_mm(a_q, b_q, sfa, sfb, ps, eo, bso, out_dtype="fp64", acc="fp64")
    assert np.allclose(y64, ref, rtol=1e-12, atol=0, equal_nan=True)
    y32 = o.grouped_mm(a_q, b_q, sfa, sfb, ps, eo, bso, out_dtype="fp32")
    assert np.allclose(y32, ref, rtol=2e-5, atol=1e-6)


def test_grouped_mm_unit_scales_is_plain_fp8_gemm_and_scale_bump_doubles_a_slice():
    rng = np.random.default_rng(4)
    rows, n, k = [4], 128, 128
    ai = rng.integers(-4, 5, size=(4, k)); bi = rng.integers(-4, 5, size=(1, n, k))
    a_q = fp8.e4m3fn_encode_rne(ai.astype(np.float32)); b_q = fp8.e4m3fn_encode_rne(bi.astype(np.float32))
    sfa = np.full(o.sf_block_bytes(4, k), 127, dtype=np.uint8)
    sfb = np.full(n * (k // 32), 127, dtype=np.uint8)
    ps = np.array([[4, n, k]], dtype=np.int32)
    y = o.grouped_mm(a_q, b_q, sfa, sfb, ps, [0], [0], out_dtype="fp32")
    assert np.array_equal(y, ai @ bi[0].T)
    sfa2 = sfa.copy()
    sfa2[o.sf_offset(2, 1, k)] = 128          # row 2, K columns 32..63 count twice
    y2 = o.grouped_mm(a_q, b_q, sfa2, sfb, ps, [0], [0], out_dtype="fp32")
    extra = ai[2, 32:64] @ bi[0][:, 32:64].T
    assert np.array_equal(y2[2], y[2] + extra) and np.array_equal(y2[[0, 1, 3]], y[[0, 1, 3]])
