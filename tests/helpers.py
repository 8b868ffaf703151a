"""Shared test helpers: tensor <-> numpy conversions, C-ABI callers, tolerance checks."""
import ctypes

import numpy as np
import torch

# Tolerance of the GEMM parity tests (bf16/fp16 output, fp32 accumulation), per expert:
#   max |y - ref| / max |ref| <= 1e-2,  |y - ref| <= 1e-2 |ref| + 1e-2 rms(ref),  cosine >= 0.9999
REL_MAX = 1e-2
COS_MIN = 0.9999


def codes(t: torch.Tensor) -> np.ndarray:
    """fp8 / uint8 tensor -> numpy uint8 codes (on the host)."""
    return t.contiguous().view(torch.uint8).cpu().numpy()


def f32(t: torch.Tensor) -> np.ndarray:
    return t.detach().float().cpu().numpy()


def check_close(y, ref, what=""):
    y = np.asarray(y, dtype=np.float64)
    ref = np.asarray(ref, dtype=np.float64)
    assert y.shape == ref.shape, (y.shape, ref.shape)
    assert np.isfinite(y).all(), f"{what}: non-finite values in result"
    scale = np.abs(ref).max()
    if scale == 0:
        assert np.abs(y).max() == 0, what
        return
    err = np.abs(y - ref)
    rms = np.sqrt((ref * ref).mean())
    assert err.max() / scale <= REL_MAX, f"{what}: max rel err {err.max() / scale:.3e}"
    bad = err > REL_MAX * np.abs(ref) + REL_MAX * rms
    assert not bad.any(), f"{what}: {bad.sum()} elements outside elementwise tolerance, worst {err.max():.3e}"
    cos = (y * ref).sum() / np.sqrt((y * y).sum() * (ref * ref).sum())
    assert cos >= COS_MIN, f"{what}: cosine {cos}"


def check_ulps(y, ref, out_dtype, what="", ulps=2.0, abs_rms=2e-3):
    """Tight form of the tolerance: every element within `ulps` units in the last place of the output type (bf16:
    2^-8 relative, fp16: 2^-11) plus abs_rms of the result's rms.  The oracle dequantises and then multiplies in
    fp32, the kernels scale per K block (fp8-blockwise) or inside the MFMA (mxfp8) and sum in another order: both
    are fp32 evaluations of the same real number, and the rms term is what absorbs their difference where K blocks
    cancel."""
    y = np.asarray(y, dtype=np.float64)
    ref = np.asarray(ref, dtype=np.float64)
    ok = np.isfinite(ref)
    eps = 2.0 ** -8 if out_dtype == torch.bfloat16 else 2.0 ** -11
    rms = np.sqrt((ref[ok] ** 2).mean()) if ok.any() else 0.0
    err = np.abs(y - ref)[ok]
    bound = (ulps * eps * np.abs(ref) + abs_rms * rms)[ok]
    bad = err > bound
    assert not bad.any(), f"{what}: {bad.sum()} of {bad.size} elements beyond {ulps} ulps, worst ratio {(err / np.maximum(bound, 1e-300)).max():.2f}"


def check_grouped(y, ref, rows, offsets, what=""):
    for e, (m, off) in enumerate(zip(rows, offsets)):
        if m:
            check_close(y[off:off + m], ref[off:off + m], f"{what} expert {e} (M={m})")


def ptr(t):
    return ctypes.c_void_p(t.data_ptr()) if t is not None else None


def stream_ptr():
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def capi_fp8_mm(native, ops, force_bm=0, out=None):
    """Call esmoe_fp8_blockwise_grouped_mm through ctypes on the operand dict of
    workloads.make_fp8_blockwise_operands."""
    lib = native.lib
    out = ops["output"] if out is None else out
    e = ops["problem_sizes"].size(0)
    total, k = ops["a"].shape
    n = ops["b_phys"].size(1)
    need = lib.esmoe_gemm_workspace_bytes(e)
    ws = torch.empty((need,), dtype=torch.uint8, device=out.device)
    rc = lib.esmoe_fp8_blockwise_grouped_mm(
        ptr(out), 0 if out.dtype == torch.bfloat16 else 1, ptr(ops["a"]), ptr(ops["b_phys"]), ptr(ops["scales_a"]),
        ptr(ops["scales_b_phys"]), ptr(ops["problem_sizes"]), ptr(ops["expert_offsets"]), e, total, n, k, force_bm,
        ptr(ws), need, stream_ptr())
    assert rc == 0, (rc, native.last_error())
    torch.cuda.synchronize()
    return out


def capi_mx_mm(native, ops, force_bm=0, out=None):
    lib = native.lib
    out = ops["output"] if out is None else out
    e = ops["problem_sizes"].size(0)
    total, k = ops["a"].shape
    n = ops["b_phys"].size(1)
    need = lib.esmoe_gemm_workspace_bytes(e)
    ws = torch.empty((need,), dtype=torch.uint8, device=out.device)
    rc = lib.esmoe_mxfp8_grouped_mm(
        ptr(out), 0 if out.dtype == torch.bfloat16 else 1, ptr(ops["a"]), ptr(ops["b_phys"]), ptr(ops["sfa"]),
        ptr(ops["sfb_phys"]), ptr(ops["problem_sizes"]), ptr(ops["expert_offsets"]), ptr(ops["blockscale_offsets"]),
        e, total, n, k, force_bm, ptr(ws), need, stream_ptr())
    assert rc == 0, (rc, native.last_error())
    torch.cuda.synchronize()
    return out


def hp_to_f32(t: torch.Tensor) -> np.ndarray:
    """bf16/fp16 tensor -> float32 numpy (exact)."""
    return t.detach().float().cpu().numpy()
