"""Pins oracle/fp8.py: the e4m3fn codec against the OCP format definition and torch's cast."""
import numpy as np
import torch

from oracle import fp8


def test_decode_known_values():
    # OCP FP8 E4M3 (fn): bias 7, no infinities, max 448, min normal 2^-6, min subnormal 2^-9
    assert fp8.e4m3fn_decode(np.array([0x7E]))[0] == 448.0
    assert fp8.e4m3fn_decode(np.array([0xFE]))[0] == -448.0
    assert fp8.e4m3fn_decode(np.array([0x38]))[0] == 1.0
    assert fp8.e4m3fn_decode(np.array([0x08]))[0] == 2.0 ** -6
    assert fp8.e4m3fn_decode(np.array([0x01]))[0] == 2.0 ** -9
    assert fp8.e4m3fn_decode(np.array([0x00]))[0] == 0.0
    assert np.isnan(fp8.e4m3fn_decode(np.array([0x7F, 0xFF]))).all()


def test_decode_matches_torch_all_codes():
    codes = np.arange(256, dtype=np.uint8)
    ref = torch.from_numpy(codes.copy()).view(torch.float8_e4m3fn).float().numpy()
    mine = fp8.e4m3fn_decode(codes)
    assert np.array_equal(np.isnan(ref), np.isnan(mine))
    ok = ~np.isnan(ref)
    assert np.array_equal(ref[ok], mine[ok])


def test_encode_matches_torch_all_bf16_patterns():
    bits = (np.arange(1 << 16, dtype=np.uint32) << 16).view(np.float32)
    finite = np.isfinite(bits)
    ref = torch.from_numpy(bits.copy()).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    mine = fp8.e4m3fn_encode_rne(bits, saturate=False)
    # both give a NaN code (0x7f | sign) above the rounding boundary 464
    assert np.array_equal(ref[finite], mine[finite])


def test_encode_matches_torch_random_fp32_and_ties():
    rng = np.random.default_rng(0)
    x = (rng.standard_normal(400000) * np.exp(rng.uniform(-12, 6.5, 400000))).astype(np.float32)
    # exact midpoints between neighbouring codes (ties) and their float32 neighbours
    grid = fp8.e4m3fn_decode(np.arange(0x7F, dtype=np.uint8)).astype(np.float64)
    mids = ((grid[:-1] + grid[1:]) / 2).astype(np.float32)
    ties = np.concatenate([mids, np.nextafter(mids, np.float32(np.inf)), np.nextafter(mids, np.float32(-np.inf)), -mids])
    x = np.concatenate([x, ties, np.array([464.0, 463.99997, 0.0, -0.0], dtype=np.float32)])
    ref = torch.from_numpy(x.copy()).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    mine = fp8.e4m3fn_encode_rne(x, saturate=False)
    assert np.array_equal(ref, mine)


def test_encode_saturate_and_roundtrip():
    codes = np.arange(256, dtype=np.uint8)
    vals = fp8.e4m3fn_decode(codes)
    ok = ~np.isnan(vals)
    back = fp8.e4m3fn_encode_rne(vals[ok], saturate=True)
    assert np.array_equal(back, codes[ok])  # includes -0.0 -> 0x80
    big = np.array([465.0, 1e9, -1e9, np.inf, -np.inf], dtype=np.float32)
    assert np.array_equal(fp8.e4m3fn_encode_rne(big, saturate=True), np.array([0x7E, 0x7E, 0xFE, 0x7E, 0xFE], dtype=np.uint8))


def test_bf16_round_matches_torch():
    rng = np.random.default_rng(1)
    x = (rng.standard_normal(200000) * np.exp(rng.uniform(-20, 20, 200000))).astype(np.float32)
    ref = torch.from_numpy(x.copy()).to(torch.bfloat16).float().numpy()
    assert np.array_equal(fp8.bf16_round(x), ref)
    assert np.array_equal(fp8.bf16_from_bits(fp8.bf16_bits(ref)), ref)


def test_e8m0_decode_matches_torch():
    codes = np.arange(255, dtype=np.uint8)
    ref = torch.from_numpy(codes.copy()).view(torch.float8_e8m0fnu).to(torch.float64).numpy()
    assert np.array_equal(fp8.e8m0_decode(codes), ref)
