"""Torch-side quantisers that prepare operands for the grouped GEMMs (run on any device).

They produce the tensors the reference's callers build with its test helpers
(test/test_es_grouped_gemm.py:36-59): e4m3fn data with fp32 scales per 1x128
block of an activation row and per 128x128 block of a weight matrix.  They are
input preparation, not part of the measured path.
"""
import torch

FP8_MAX = 448.0


def quant_act_1x128(x: torch.Tensor):
    """[M, K] (K % 128 == 0) -> (e4m3fn [M, K], fp32 scales [M, K/128])."""
    assert x.dim() == 2 and x.size(1) % 128 == 0
    m, k = x.shape
    xv = x.view(m, k // 128, 128)
    amax = xv.abs().float().amax(dim=2).clamp(1e-4)
    q = (xv * (FP8_MAX / amax.unsqueeze(2))).to(torch.float8_e4m3fn)
    return q.view(m, k), amax / FP8_MAX


def quant_weight_128x128(w: torch.Tensor):
    """[..., N, K] (both % 128 == 0) -> (e4m3fn [..., N, K], fp32 scales [..., N/128, K/128])."""
    assert w.size(-1) % 128 == 0 and w.size(-2) % 128 == 0
    lead = w.shape[:-2]
    n, k = w.shape[-2:]
    wv = w.reshape(*lead, n // 128, 128, k // 128, 128)
    amax = wv.abs().float().amax(dim=(-3, -1), keepdim=True).clamp(1e-4)
    q = (wv * (FP8_MAX / amax)).to(torch.float8_e4m3fn)
    return q.reshape(*lead, n, k), (amax / FP8_MAX).reshape(*lead, n // 128, k // 128)
