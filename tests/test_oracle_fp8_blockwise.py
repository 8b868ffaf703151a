"""Pins oracle/fp8_blockwise.py: quantiser closed forms and the dequantise+matmul against
independent evaluations (torch restatement, C brute force, fp64, exact special cases)."""
import numpy as np
import pytest
import torch

from oracle import brute, fp8
from oracle import fp8_blockwise as o


def _bf16_randn(rng, shape, scale=1.0):
    return fp8.bf16_round((rng.standard_normal(shape) * scale).astype(np.float32))


def test_quant_act_closed_form_invariants():
    rng = np.random.default_rng(0)
    x = _bf16_randn(rng, (37, 384))
    x[3, 128:256] = 0.0              # all-zero block
    x[5, :128] *= 1e-6               # tiny block, still above the 1e-4 clamp after amax? (no: below)
    q, s = o.quant_act_1x128(x)
    v = fp8.e4m3fn_decode(q)
    assert np.abs(v).max() <= 448.0
    xb = x.reshape(37, 3, 128)
    amax = np.abs(xb).max(axis=2)
    # scale is amax/448 with the 1e-4 clamp
    assert np.array_equal(s, (np.maximum(amax, np.float32(1e-4)) / np.float32(448.0)).astype(np.float32))
    assert s[3, 1] == np.float32(1e-4) / np.float32(448.0) and not q[3, 128:256].any()
    # the block's largest element maps to +-448 (unless clamped)
    vb = v.reshape(37, 3, 128)
    for i, j in [(0, 0), (10, 2), (36, 1)]:
        k = np.abs(xb[i, j]).argmax()
        assert abs(vb[i, j, k]) == 448.0 and np.sign(vb[i, j, k]) == np.sign(xb[i, j, k])
    # dequantised value within half an e4m3 ulp (2^-4 relative) plus the subnormal floor
    deq = o.dequant_act(q, s)
    bound = 2.0 ** -4 * np.abs(x) + np.repeat(s, 128, axis=1) * 2.0 ** -10
    assert (np.abs(deq - x) <= bound + 1e-12).all()


def test_quant_matches_independent_torch_restatement():
    """Same arithmetic written with stock torch ops (amax, fp32 divide, fp32 multiply, cast)."""
    rng = np.random.default_rng(1)
    x = _bf16_randn(rng, (64, 512))
    t = torch.from_numpy(x).to(torch.bfloat16)
    tv = t.view(64, 4, 128)
    amax = tv.abs().float().amax(dim=2).clamp(1e-4)
    tq = (tv * (448.0 / amax.unsqueeze(2))).to(torch.float8_e4m3fn).view(64, 512)
    q, s = o.quant_act_1x128(x)
    assert np.array_equal(q, tq.view(torch.uint8).numpy())
    assert np.array_equal(s, (amax / 448.0).numpy())
    w = (rng.standard_normal((256, 384)) * 0.02).astype(np.float32)
    tw = torch.from_numpy(w).view(2, 128, 3, 128)
    wmax = tw.abs().float().amax(dim=(1, 3), keepdim=True).clamp(1e-4)
    twq = (tw * (448.0 / wmax)).to(torch.float8_e4m3fn).view(256, 384)
    qw, sw = o.quant_weight_128x128(w)
    assert np.array_equal(qw, twq.view(torch.uint8).numpy())
    assert np.array_equal(sw, (wmax / 448.0).view(2, 3).numpy())


def test_weight_quant_transpose_equivalence():
    """Quantising the (K, N) view and transposing back (what the reference's test does) equals
    quantising the physical [N, K] matrix."""
    rng = np.random.default_rng(2)
    w = (rng.standard_normal((256, 384)) * 0.02).astype(np.float32)
    q1, s1 = o.quant_weight_128x128(w)
    q2, s2 = o.quant_weight_128x128(np.ascontiguousarray(w.T))
    assert np.array_equal(q1, q2.T) and np.array_equal(s1, s2.T)


def _small_problem(rng, rows, n, k):
    e = len(rows)
    total = sum(rows)
    a_q, sa = o.quant_act_1x128(_bf16_randn(rng, (total, k)))
    b_q = np.zeros((e, n, k), dtype=np.uint8)
    sb = np.zeros((e, n // 128, k // 128), dtype=np.float32)
    for i in range(e):
        b_q[i], sb[i] = o.quant_weight_128x128((rng.standard_normal((n, k)) * 0.02).astype(np.float32))
    ps = np.array([[m, n, k] for m in rows], dtype=np.int32)
    eo = np.concatenate([[0], np.cumsum(rows)[:-1]]).astype(np.int32)
    return a_q, b_q, sa, sb, ps, eo


def test_grouped_mm_against_c_brute_force_and_fp64():
    rng = np.random.default_rng(3)
    a_q, b_q, sa, sb, ps, eo = _small_problem(rng, [3, 0, 2], 128, 256)
    ref = brute.fp8_blockwise(a_q, b_q, sa, sb, ps, eo)
    y64 = o.grouped_mm(a_q, b_q, sa, sb, ps, eo, out_dtype="fp64", acc="fp64")
    y32 = o.grouped_mm(a_q, b_q, sa, sb, ps, eo, out_dtype="fp32", acc="fp32")
    assert np.allclose(y64, ref, rtol=1e-12, atol=1e-14, equal_nan=True)
    assert np.isnan(ref[3:3]).all() and np.isfinite(ref).all()  # (the empty expert owns no rows)
    assert np.allclose(y32, ref, rtol=2e-5, atol=1e-6)
    ybf = o.grouped_mm(a_q, b_q, sa, sb, ps, eo, out_dtype="bf16")
    assert np.array_equal(ybf, fp8.bf16_round(y32.astype(np.float32)))


def test_grouped_mm_exact_integer_case():
    """Unit scales and small-integer fp8 values: the result is the integer matmul, exactly."""
    rng = np.random.default_rng(4)
    rows, n, k = [5, 7], 128, 256
    ai = rng.integers(-4, 5, size=(sum(rows), k))
    bi = rng.integers(-4, 5, size=(2, n, k))
    a_q = fp8.e4m3fn_encode_rne(ai.astype(np.float32))
    b_q = fp8.e4m3fn_encode_rne(bi.astype(np.float32))
    assert np.array_equal(fp8.e4m3fn_decode(a_q), ai)
    sa = np.ones((sum(rows), k // 128), dtype=np.float32)
    sb = np.ones((2, n // 128, k // 128), dtype=np.float32)
    ps = np.array([[m, n, k] for m in rows], dtype=np.int32)
    y = o.grouped_mm(a_q, b_q, sa, sb, ps, [0, 5], out_dtype="fp32")
    assert np.array_equal(y[:5], ai[:5] @ bi[0].T)
    assert np.array_equal(y[5:], ai[5:] @ bi[1].T)


def test_grouped_mm_one_hot_rows_and_scale_shift():
    rng = np.random.default_rng(5)
    a_q, b_q, sa, sb, ps, eo = _small_problem(rng, [4], 128, 256)
    a_q[:] = 0
    a_q[2, 130] = 0x38  # 1.0 at k = 130 (second K block)
    y = o.grouped_mm(a_q, b_q, sa, sb, ps, eo, out_dtype="fp32")
    expect = sa[2, 1] * (sb[0, 0, 1] * fp8.e4m3fn_decode(b_q[0, :, 130]))
    assert np.allclose(y[2], expect, rtol=1e-6)
    assert not y[[0, 1, 3]].any()
    # scaling sa by 2^j scales the output by exactly 2^j
    a_q2, b_q2, sa2, sb2, ps2, eo2 = _small_problem(rng, [6], 128, 256)
    y1 = o.grouped_mm(a_q2, b_q2, sa2, sb2, ps2, eo2, out_dtype="fp32")
    y2 = o.grouped_mm(a_q2, b_q2, sa2 * np.float32(8.0), sb2, ps2, eo2, out_dtype="fp32")
    assert np.array_equal(y2, y1 * np.float32(8.0))


def test_grouped_mm_empty_experts_untouched_and_permutation():
    rng = np.random.default_rng(6)
    rows = [3, 0, 5, 2]
    a_q, b_q, sa, sb, ps, eo = _small_problem(rng, rows, 128, 128)
    out = np.full((sum(rows) + 2, 128), 123.0, dtype=np.float32)
    o.grouped_mm(np.vstack([a_q, a_q[:2]]), b_q, np.vstack([sa, sa[:2]]), sb, ps, eo, out=out)
    assert (out[-2:] == 123.0).all()  # rows beyond every expert are not written
    y = o.grouped_mm(a_q, b_q, sa, sb, ps, eo)
    # expert order permuted: output blocks permute with it
    perm = [2, 0, 3, 1]
    rows_p = [rows[i] for i in perm]
    starts = np.concatenate([[0], np.cumsum(rows)[:-1]])
    a_p = np.vstack([a_q[starts[i]:starts[i] + rows[i]] for i in perm])
    sa_p = np.vstack([sa[starts[i]:starts[i] + rows[i]] for i in perm])
    ps_p = np.array([[m, 128, 128] for m in rows_p], dtype=np.int32)
    eo_p = np.concatenate([[0], np.cumsum(rows_p)[:-1]]).astype(np.int32)
    y_p = o.grouped_mm(a_p, b_q[perm], sa_p, sb[perm], ps_p, eo_p)
    y_expect = np.vstack([y[starts[i]:starts[i] + rows[i]] for i in perm])
    assert np.array_equal(y_p, y_expect)


def test_calc_diff_properties():
    x = np.arange(12.0).reshape(3, 4)
    assert o.calc_diff(x, x) == pytest.approx(0.0, abs=1e-15)
    assert o.calc_diff(x, -x) == pytest.approx(2.0)


def test_quant_act_scale_variants_agree_within_one_ulp():
    """The GPU flavour of the scale (amax * fl(1/448)) is the CPU flavour (amax / 448) up to one ulp, and
    the quantised bytes do not depend on the flavour."""
    import numpy as np
    from oracle import fp8_blockwise as ofp8

    rng = np.random.default_rng(11)
    x = (rng.standard_normal((64, 512)) * np.exp(rng.standard_normal((64, 1)) * 3)).astype(np.float32)
    q0, s0 = ofp8.quant_act_1x128(x)
    q1, s1 = ofp8.quant_act_1x128(x, scale_via_reciprocal=True)
    assert np.array_equal(q0, q1)
    d = np.abs(s0.view(np.int32).astype(np.int64) - s1.view(np.int32).astype(np.int64))
    assert d.max() <= 1 and (d == 1).any()
    assert np.array_equal(s1, s0 if False else (np.maximum(np.abs(x.reshape(64, 4, 128)).max(axis=2), np.float32(1e-4)) * (np.float32(1) / np.float32(448))).astype(np.float32))


def test_swiglu_oracle_closed_forms():
    """swiglu(): gate 0 -> 0; large positive gate -> gate * up; large negative gate -> (-)0; and agreement with a
    float64 evaluation to one rounding of the output type."""
    import numpy as np
    from oracle import fp8
    from oracle import fp8_blockwise as ofp8

    x = np.array([[0.0, 30.0, -100.0, 1.5, 2.0, 0.5, 3.0, -2.0]], dtype=np.float32)   # gates | ups
    with np.errstate(over="ignore"):
        h = ofp8.swiglu(x)
    assert h[0, 0] == 0.0 and h[0, 1] == 15.0 and h[0, 2] == 0.0
    exact = 1.5 / (1.0 + np.exp(-1.5)) * -2.0
    assert h[0, 3] == fp8.bf16_round(np.float32(exact))
    rng = np.random.default_rng(3)
    g = fp8.bf16_round(rng.standard_normal((16, 256)).astype(np.float32) * 3)
    u = fp8.bf16_round(rng.standard_normal((16, 256)).astype(np.float32))
    h = ofp8.swiglu(np.concatenate([g, u], axis=1))
    ref = (g.astype(np.float64) / (1.0 + np.exp(-g.astype(np.float64)))) * u.astype(np.float64)
    assert np.abs(h - ref).max() <= np.abs(ref).max() * 2.0 ** -8
    assert (h == fp8.bf16_round(ref.astype(np.float32))).mean() > 0.999
