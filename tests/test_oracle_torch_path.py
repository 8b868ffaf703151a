"""The torch-only restatement of the reference's CPU path (oracle/torch_path.py, the benchmark's CPU baseline) against
the numpy oracles that the parity tests use, and against exact integer cases."""
import numpy as np
import torch

from oracle import fp8, fp8_blockwise as ofp8, mxfp8 as omx, torch_path as otp


def _as_fp8(codes):
    return torch.from_numpy(np.ascontiguousarray(codes)).view(torch.float8_e4m3fn)


def test_scaled_mm_matches_the_numpy_oracle():
    rng = np.random.default_rng(3)
    rows, n, k = [5, 0, 130, 17], 256, 384
    total = sum(rows)
    a_codes, sa = ofp8.quant_act_1x128(rng.standard_normal((total, k)).astype(np.float32))
    b_codes = np.empty((len(rows), n, k), dtype=np.uint8)
    sb = np.empty((len(rows), n // 128, k // 128), dtype=np.float32)
    for e in range(len(rows)):
        b_codes[e], sb[e] = ofp8.quant_weight_128x128((rng.standard_normal((n, k)) * 0.05).astype(np.float32))
    offs = np.concatenate([[0], np.cumsum(rows)[:-1]])
    ref = ofp8.grouped_mm(a_codes, b_codes, sa, sb, [[m, n, k] for m in rows], offs)
    got = otp.grouped_scaled_mm(_as_fp8(a_codes), _as_fp8(b_codes), torch.from_numpy(sa), torch.from_numpy(sb), rows)
    # same arithmetic (scale times value in fp32, fp32 matmul, one rounding to bf16): a blocked matmul may sum in
    # another order, which moves a result by a bf16 step at most
    g = got.float().numpy()
    assert np.abs(g - ref).max() <= 2.0 ** -7 * np.abs(ref).max()
    assert (g == ref).mean() > 0.99


def test_scaled_mm_is_exact_on_small_integers():
    rng = np.random.default_rng(4)
    m, n, k = 9, 128, 256
    a = rng.integers(-3, 4, size=(m, k)).astype(np.float32)
    b = rng.integers(-2, 3, size=(n, k)).astype(np.float32)
    sa = np.exp2(rng.integers(-2, 3, size=(m, k // 128))).astype(np.float32)
    sb = np.exp2(rng.integers(-2, 3, size=(n // 128, k // 128))).astype(np.float32)
    want = (a * np.repeat(sa, 128, 1)).astype(np.float64) @ (b * np.repeat(np.repeat(sb, 128, 0), 128, 1)).astype(np.float64).T
    got = otp.scaled_mm(_as_fp8(fp8.e4m3fn_encode_rne(a)), _as_fp8(fp8.e4m3fn_encode_rne(b)), torch.from_numpy(sa),
                        torch.from_numpy(sb), torch.float32)
    assert np.array_equal(got.numpy().astype(np.float64), want)


def test_mx_scaled_mm_matches_the_numpy_oracle():
    rng = np.random.default_rng(5)
    rows, n, k = [40, 129], 128, 256
    total = sum(rows)
    x = fp8.bf16_round(rng.standard_normal((total, k)).astype(np.float32))
    w = fp8.bf16_round((rng.standard_normal((len(rows) * n, k)) * 0.05).astype(np.float32))
    a_codes, sca = omx.quant_rows(x)
    b_codes, scb = omx.quant_rows(w)
    ps = [[m, n, k] for m in rows]
    offs = [0, rows[0]]
    bso = [0, (rows[0] + 127) // 128 * 128]
    sf_rows = sum((m + 127) // 128 * 128 for m in rows)
    sfa = np.zeros(sf_rows * (k // 32), dtype=np.uint8)
    for e, m in enumerate(rows):
        omx.swizzle_scales(sca[offs[e]:offs[e] + m], k, out=sfa, base=bso[e] * (k // 32))
    sfb = np.zeros(len(rows) * n * (k // 32), dtype=np.uint8)
    for e in range(len(rows)):
        omx.swizzle_scales(scb[e * n:(e + 1) * n], k, out=sfb, base=e * n * (k // 32))
    ref = omx.grouped_mm(a_codes, b_codes.reshape(len(rows), n, k), sfa, sfb, ps, offs, bso)
    got = otp.grouped_mx_scaled_mm(_as_fp8(a_codes), _as_fp8(b_codes.reshape(len(rows), n, k)), torch.from_numpy(sca),
                                   torch.from_numpy(scb.reshape(len(rows), n, k // 32)), rows)
    g = got.float().numpy()
    assert np.abs(g - ref).max() <= 2.0 ** -7 * np.abs(ref).max()
    assert (g == ref).mean() > 0.99
