"""The reference's torch CPU path, stock torch ops only (test infrastructure, see oracle/__init__.py).

* ``scaled_mm`` <- ``baseline_scaled_mm``, test/test_es_grouped_gemm.py:62-86: broadcast the
  per-1x128 activation scales and the per-128x128 weight scales over their blocks, multiply into
  the fp32 casts of the fp8 operands, ``torch.mm`` in fp32, cast to the output type.
* ``grouped_scaled_mm`` applies it per expert over the packed rows, as the reference's test loop
  does (test/test_es_grouped_gemm.py:143-199).
* ``mx_scaled_mm`` / ``grouped_mx_scaled_mm`` are the same path for the MXFP8 operands: E8M0
  scale bytes decoded as 2^(b - 127) (es_sm100_mxfp8_blockscaled_traits.cuh:44-72), one per 1x32
  block of either operand; the scale tensors come in row-major [rows, K/32] form.

These exist for the benchmark's CPU baseline: nothing but torch runs inside them, so timing them
measures torch's CPU path and not numpy.  Pinned against ``fp8_blockwise.grouped_mm`` and
``mxfp8.grouped_mm`` (tests/test_oracle_torch_path.py), which are pinned by closed forms.
"""
import torch


def scaled_mm(a, b, scale_a, scale_b, out_dtype=torch.bfloat16):
    """a [M, K] float8_e4m3fn, b [N, K] float8_e4m3fn (the physical weight layout),
    scale_a [M, K/128] f32, scale_b [N/128, K/128] f32 -> [M, N] in out_dtype."""
    sa = scale_a.repeat_interleave(128, dim=1)
    sb = scale_b.repeat_interleave(128, dim=0).repeat_interleave(128, dim=1)
    return torch.mm(sa * a.to(torch.float32), (sb * b.to(torch.float32)).t()).to(out_dtype)


def grouped_scaled_mm(a, b, scale_a, scale_b, rows, out_dtype=torch.bfloat16, out=None):
    """Packed rows of all experts: a [sumM, K], b [E, N, K], scale_a [sumM, K/128], scale_b [E, N/128, K/128]."""
    if out is None:
        out = torch.empty((a.shape[0], b.shape[1]), dtype=out_dtype)
    off = 0
    for e, m in enumerate(rows):
        if m:
            out[off:off + m] = scaled_mm(a[off:off + m], b[e], scale_a[off:off + m], scale_b[e], out_dtype)
        off += m
    return out


def mx_scaled_mm(a, b, sfa, sfb, out_dtype=torch.bfloat16):
    """a [M, K], b [N, K] float8_e4m3fn; sfa [M, K/32], sfb [N, K/32] uint8 E8M0 codes (row-major)."""
    da = torch.exp2(sfa.to(torch.float32) - 127.0).repeat_interleave(32, dim=1)
    db = torch.exp2(sfb.to(torch.float32) - 127.0).repeat_interleave(32, dim=1)
    return torch.mm(da * a.to(torch.float32), (db * b.to(torch.float32)).t()).to(out_dtype)


def grouped_mx_scaled_mm(a, b, sfa_rows, sfb_rows, rows, out_dtype=torch.bfloat16, out=None):
    """a [sumM, K], b [E, N, K]; sfa_rows [sumM, K/32] and sfb_rows [E, N, K/32] row-major E8M0 codes."""
    if out is None:
        out = torch.empty((a.shape[0], b.shape[1]), dtype=out_dtype)
    off = 0
    for e, m in enumerate(rows):
        if m:
            out[off:off + m] = mx_scaled_mm(a[off:off + m], b[e], sfa_rows[off:off + m], sfb_rows[e], out_dtype)
        off += m
    return out
