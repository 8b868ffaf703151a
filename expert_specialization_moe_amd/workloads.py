"""Synthetic workloads: routing generators, operand builders and the roofline model.

Routing follows the benchmark configurations of this project:
  * uniform top-k routing as benchmark/benchmark_es_fp8_blockwise_moe.py:44-56 of the reference;
  * Zipf(s) expert popularity (rank permuted by the seed), either sampled per token
    with distinct top-k experts (Gumbel top-k) or as a multinomial over local experts.
"""
import math
from dataclasses import dataclass, field
from typing import List

import numpy as np
import torch

from .quant import quant_act_1x128, quant_weight_128x128

HBM_BYTES_PER_S = 8.0e12     # MI355X HBM3E peak
FP8_FLOPS_PER_S = 5.0e15     # MI355X dense FP8 MFMA peak


def zipf_popularity(rng, num_experts, s):
    rank = rng.permutation(num_experts)
    p = (rank + 1.0) ** (-s)
    return p / p.sum()


def zipf_topk_rows(seed, tokens, topk, total_experts, s, local_experts):
    """Rows per local expert (ids 0..local_experts-1) when `tokens` tokens each pick `topk`
    distinct experts out of `total_experts` with Zipf(s) popularity."""
    rng = np.random.default_rng(seed)
    p = zipf_popularity(rng, total_experts, s)
    gumbel = rng.gumbel(size=(tokens, total_experts))
    picks = np.argsort(-(np.log(p)[None, :] + gumbel), axis=1)[:, :topk]
    counts = np.bincount(picks.reshape(-1), minlength=total_experts)
    return [int(c) for c in counts[:local_experts]]


def zipf_multinomial_rows(seed, rows, num_experts, s):
    rng = np.random.default_rng(seed)
    p = zipf_popularity(rng, num_experts, s)
    return [int(c) for c in rng.multinomial(rows, p)]


def uniform_topk_rows(seed, tokens, topk, num_experts):
    rng = np.random.default_rng(seed)
    ids = rng.integers(0, num_experts, size=tokens * topk)
    return [int(c) for c in np.bincount(ids, minlength=num_experts)]


@dataclass
class Problem:
    name: str
    n: int
    k: int
    rows: List[int]
    kind: str = "fp8_blockwise"   # or "mxfp8"
    meta: dict = field(default_factory=dict)

    @property
    def num_experts(self):
        return len(self.rows)

    @property
    def total_rows(self):
        return int(sum(self.rows))


def config_problem(name, seed=0, tokens=None, routing="zipf"):
    """The benchmark configurations by name: c0 .. c4, and a single large expert (dense, dense_mx)."""
    if name == "c0":
        rng = np.random.default_rng(seed)
        return Problem("c0", 256, 512, [int(v) for v in rng.integers(1, 65, size=8)])
    if name == "c1":
        return Problem("c1", 4096, 7168, zipf_topk_rows(seed, 4096, 8, 256, 1.2, 32),
                       meta={"tokens": 4096, "topk": 8, "experts_total": 256, "zipf_s": 1.2})
    if name == "c2":
        return Problem("c2", 7168, 2048, zipf_multinomial_rows(seed, 256, 32, 1.2), meta={"rows": 256, "zipf_s": 1.2})
    if name == "c3":
        t = tokens or 2048
        rows = zipf_topk_rows(seed, t, 8, 128, 1.2, 128) if routing == "zipf" else uniform_topk_rows(seed, t, 8, 128)
        return Problem(f"c3_T{t}_{routing}", 3072, 4096, rows, meta={"tokens": t, "routing": routing})
    if name == "c4":
        return Problem("c4", 4096, 7168, zipf_multinomial_rows(seed, 8192, 32, 1.0), kind="mxfp8",
                       meta={"rows": 8192, "zipf_s": 1.0})
    if name in ("dense", "dense_mx"):
        # one large expert: what the tall tiles do when nothing else runs beside them (no counterpart among the
        # reference's benchmark shapes; it isolates the matrix-bound part of c1/c3/c4)
        return Problem(name, 4096, 7168, [12288], kind="mxfp8" if name == "dense_mx" else "fp8_blockwise", meta={"rows": 12288})
    raise ValueError(name)


# ---------------------------------------------------------------------------- roofline
def gemm_flops(rows, n, k):
    return 2.0 * n * k * float(sum(rows))


def gemm_bytes(rows, n, k, kind="fp8_blockwise"):
    """Algorithmic HBM bytes of one grouped GEMM call: every operand byte once, output once."""
    total = float(sum(rows))
    active = sum(1 for m in rows if m > 0)
    if kind == "fp8_blockwise":
        return total * (k + 4.0 * k / 128) + active * (n * k + 4.0 * (n // 128) * (k // 128)) + 2.0 * n * total
    return total * (k + k / 32.0) + active * (n * k + n * k / 32.0) + 2.0 * n * total


def quant_bytes(rows, k):
    return float(sum(rows)) * k * (2 + 1 + 1 / 32.0)


def gemm_roofline_seconds(rows, n, k, kind="fp8_blockwise"):
    return max(gemm_flops(rows, n, k) / FP8_FLOPS_PER_S, gemm_bytes(rows, n, k, kind) / HBM_BYTES_PER_S)


def gemm_roofline_per_expert_seconds(rows, n, k, kind="fp8_blockwise"):
    """Looser secondary figure: every expert priced on its own bound, sum over experts of max(F_e / P, B_e / BW)."""
    return sum(gemm_roofline_seconds([m], n, k, kind) for m in rows if m > 0)


# ---------------------------------------------------------------------------- operands
def offsets_of(rows):
    off = np.zeros(len(rows), dtype=np.int64)
    off[1:] = np.cumsum(rows)[:-1]
    return off


def blockscale_offsets_of(rows):
    aligned = [(m + 127) // 128 * 128 for m in rows]
    return offsets_of(aligned), int(sum(aligned))


def make_fp8_blockwise_operands(prob: Problem, device, seed=0, out_dtype=torch.bfloat16, weight_std=0.02):
    """Operands of es_fp8_blockwise_scaled_grouped_mm in the layouts the reference's callers build
    (test/test_es_grouped_gemm.py:143-179).  Returns a dict of tensors on `device`."""
    e, n, k = prob.num_experts, prob.n, prob.k
    gdev = device if torch.device(device).type == "cuda" else "cpu"   # values are seeded per device type
    gen = torch.Generator(device=gdev).manual_seed(seed)
    total = prob.total_rows
    a = torch.randn((total, k), generator=gen, dtype=torch.float32, device=gdev).to(torch.bfloat16).to(device)
    a_q, sa = quant_act_1x128(a)
    b_q = torch.empty((e, n, k), dtype=torch.float8_e4m3fn, device=device)
    sb = torch.empty((e, n // 128, k // 128), dtype=torch.float32, device=device)
    for i in range(e):
        w = (torch.randn((n, k), generator=gen, dtype=torch.float32, device=gdev) * weight_std).to(device)
        b_q[i], sb[i] = quant_weight_128x128(w)
    ps = torch.tensor([[m, n, k] for m in prob.rows], dtype=torch.int32, device=device)
    eo = torch.tensor(offsets_of(prob.rows), dtype=torch.int32, device=device)
    return {
        "a": a_q.contiguous(), "b": b_q.transpose(1, 2), "b_phys": b_q,
        "scales_a": sa.contiguous(), "scales_b": sb.transpose(1, 2), "scales_b_phys": sb,
        "stride_a": torch.full((e,), k, dtype=torch.int64, device=device),
        "stride_b": torch.full((e,), k, dtype=torch.int64, device=device),
        "stride_d": torch.full((e,), n, dtype=torch.int64, device=device),
        "problem_sizes": ps, "expert_offsets": eo,
        "workspace": torch.empty((1 << 16,), dtype=torch.uint8, device=device),
        "output": torch.empty((total, n), dtype=out_dtype, device=device),
        "a_hp": a,
    }


def make_mxfp8_operands(prob: Problem, device, seed=0, out_dtype=torch.bfloat16, weight_std=0.02, in_dtype=torch.bfloat16):
    """Operands of the MXFP8 quant + GEMM pair, built the way the reference's end-to-end test does
    (test/test_es_sm100_mxfp8_blockscaled_grouped_quant.py:42-101): activations and weights are both
    quantised by the grouped quant op, the weights through the auxiliary problem list [N, M, K] with
    offsets e*N.  Needs a GPU (it calls the op)."""
    from . import ops

    e, n, k = prob.num_experts, prob.n, prob.k
    total = prob.total_rows
    gdev = device if torch.device(device).type == "cuda" else "cpu"
    gen = torch.Generator(device=gdev).manual_seed(seed)
    a = torch.randn((total, k), generator=gen, dtype=torch.float32, device=gdev).to(in_dtype).to(device)
    w = torch.empty((e * n, k), dtype=in_dtype, device=device)
    for i in range(e):
        w[i * n:(i + 1) * n] = (torch.randn((n, k), generator=gen, dtype=torch.float32, device=gdev) * weight_std).to(in_dtype)
    ps = torch.tensor([[m, n, k] for m in prob.rows], dtype=torch.int32, device=device)
    eo = torch.tensor(offsets_of(prob.rows), dtype=torch.int32, device=device)
    bso_np, sf_rows = blockscale_offsets_of(prob.rows)
    bso = torch.tensor(bso_np, dtype=torch.int32, device=device)
    aux_ps = torch.tensor([[n, m, k] for m in prob.rows], dtype=torch.int32, device=device)
    aux_eo = torch.arange(e, dtype=torch.int32, device=device) * n
    a_q = torch.zeros((total, k), dtype=torch.float8_e4m3fn, device=device)
    sfa = torch.zeros((max(sf_rows, 128), k // 32), dtype=torch.uint8, device=device)
    b_q = torch.zeros((e * n, k), dtype=torch.float8_e4m3fn, device=device)
    sfb = torch.zeros((e, n, k // 32), dtype=torch.uint8, device=device)
    ops.es_sm100_mxfp8_blockscaled_grouped_quant(a, ps, eo, bso, a_q, sfa)
    ops.es_sm100_mxfp8_blockscaled_grouped_quant(w, aux_ps, aux_eo, aux_eo, b_q, sfb)
    return {
        "a_hp": a, "w_hp": w, "a": a_q, "b": b_q.view(e, n, k).transpose(1, 2), "b_phys": b_q.view(e, n, k),
        "sfa": sfa, "sfb": sfb.view(e, n, k // 32).transpose(1, 2), "sfb_phys": sfb,
        "problem_sizes": ps, "expert_offsets": eo, "blockscale_offsets": bso,
        "aux_problem_sizes": aux_ps, "aux_expert_offsets": aux_eo,
        "output": torch.empty((total, n), dtype=out_dtype, device=device),
    }
