#!/usr/bin/env python3
"""Writes the golden fixtures in this directory from the CPU oracle (closed forms pinned in
tests/test_oracle_*.py).  The reference holds no golden vectors for this path, so these are the
project's own known-answer vectors:

  c0_fp8_blockwise.npz   config 0 (E=8, K=512, N=256, rows ~ U{1..64}, seed 0): quantised operands,
                         scales, metadata and the oracle's bf16 output
  mx_quant_small.npz     a ragged MXFP8 grouped-quant case: bf16 input bits, expected e4m3 bytes,
                         swizzled E8M0 scale bytes and the mask of defined scale bytes
  sf_swizzle_table.npz   byte offsets of the swizzled scale layout for M in {1,127,128,129,300}, K in {128,384}
  caller_side_small.npz  the caller-side steps on a 40-token, top-2, 6-expert case (ids 0..7, so two experts are
                         remote): routing metadata and packing order, packed bf16 rows, their 1x128 quantisation
                         (scale = amax * fl(1/448), the GPU flavour) and a 128x128 weight quantisation

Run from the repository root:  python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import fp8, mxfp8  # noqa: E402
from oracle import fp8_blockwise as ofp8  # noqa: E402
from oracle import routing as oroute  # noqa: E402

HERE = os.path.dirname(os.path.abspath(__file__))


def c0():
    rng = np.random.default_rng(0)
    rows = [int(v) for v in rng.integers(1, 65, size=8)]
    n, k = 256, 512
    total = sum(rows)
    a = fp8.bf16_round(rng.standard_normal((total, k)).astype(np.float32))
    a_q, sa = ofp8.quant_act_1x128(a)
    b_q = np.zeros((8, n, k), dtype=np.uint8)
    sb = np.zeros((8, n // 128, k // 128), dtype=np.float32)
    for e in range(8):
        w = (rng.standard_normal((n, k)) * 0.02).astype(np.float32)
        b_q[e], sb[e] = ofp8.quant_weight_128x128(w)
    ps = np.array([[m, n, k] for m in rows], dtype=np.int32)
    eo = np.concatenate([[0], np.cumsum(rows)[:-1]]).astype(np.int32)
    out = ofp8.grouped_mm(a_q, b_q, sa, sb, ps, eo, out_dtype="bf16")
    np.savez_compressed(os.path.join(HERE, "c0_fp8_blockwise.npz"), a=a_q, b=b_q, scales_a=sa, scales_b=sb,
                        problem_sizes=ps, expert_offsets=eo, out_bf16_bits=fp8.bf16_bits(out))


def mx_quant():
    rng = np.random.default_rng(1)
    rows = [1, 127, 0, 130]
    k = 256
    total = sum(rows)
    x = fp8.bf16_round((rng.standard_normal((total, k)) * np.exp(rng.uniform(-6, 6, (total, 1)))).astype(np.float32))
    x[3, :32] = 0.0
    x[7, 32:64] = 1.75      # amax exactly on the documented tie 448 * 2^-8
    ps = np.array([[m, 5, k] for m in rows], dtype=np.int32)
    eo = np.concatenate([[0], np.cumsum(rows)[:-1]]).astype(np.int32)
    aligned = [(m + 127) // 128 * 128 for m in rows]
    bso = np.concatenate([[0], np.cumsum(aligned)[:-1]]).astype(np.int32)
    q, sf, mask = mxfp8.grouped_quant(x, ps, eo, bso, sf_total_rows=sum(aligned))
    np.savez_compressed(os.path.join(HERE, "mx_quant_small.npz"), x_bf16_bits=fp8.bf16_bits(x), problem_sizes=ps,
                        expert_offsets=eo, blockscale_offsets=bso, q=q, sf=sf, sf_mask=mask)


def sf_table():
    out = {}
    for m in (1, 127, 128, 129, 300):
        for k in (128, 384):
            rr, cc = np.meshgrid(np.arange(m), np.arange(k // 32), indexing="ij")
            out[f"m{m}_k{k}"] = mxfp8.sf_offset(rr, cc, k).astype(np.int32)
    np.savez_compressed(os.path.join(HERE, "sf_swizzle_table.npz"), **out)


def caller_side():
    rng = np.random.default_rng(2)
    tokens, topk, experts, k = 40, 2, 6, 256
    ids = np.stack([rng.permutation(8)[:topk] for _ in range(tokens)]).astype(np.int32)
    x = fp8.bf16_round((rng.standard_normal((tokens, k)) * np.exp(rng.uniform(-3, 3, (tokens, 1)))).astype(np.float32))
    x[5, :128] = 0.0
    ps, eo, bso, dst = oroute.route_metadata(ids, 0, experts, 128, k)
    packed = oroute.permute_rows(x, dst, topk, int(eo[-1]))
    q, sc = ofp8.quant_act_1x128(packed, scale_via_reciprocal=True)
    w = fp8.bf16_round((rng.standard_normal((128, k)) * 0.03).astype(np.float32))
    wq, wsc = ofp8.quant_weight_128x128(w, scale_via_reciprocal=True)
    np.savez_compressed(os.path.join(HERE, "caller_side_small.npz"), topk_ids=ids, x_bf16_bits=fp8.bf16_bits(x),
                        problem_sizes=ps, expert_offsets=eo, blockscale_offsets=bso, dst_row=dst,
                        packed_bf16_bits=fp8.bf16_bits(packed), q=q, scales=sc, w_bf16_bits=fp8.bf16_bits(w), wq=wq,
                        wscales=wsc)


if __name__ == "__main__":
    caller_side()
    c0()
    mx_quant()
    sf_table()
    print("golden fixtures written to", HERE)
