"""Routing metadata oracle (test infrastructure, see oracle/__init__.py).

Restates what the reference's callers compute on the host before they call the grouped operators:
per-expert row counts and their exclusive prefix sum
(benchmark/benchmark_es_fp8_blockwise_moe.py:44-56 counts, :72-88 expert_offsets / problem_sizes) and
blockscale_offsets as the prefix sum of the counts rounded up to 128
(test/test_es_sm100_mxfp8_blockscaled_grouped_quant.py:42-60), plus the stable packing order of the
(token, choice) pairs that those layouts imply.  Plain Python loops: pinned by construction, and by
a numpy argsort cross-check in the tests.
"""
import numpy as np


def route_metadata(topk_ids, first_expert, num_experts, n, k):
    """topk_ids: int array [num_pairs] -> (problem_sizes [E,3], expert_offsets [E+1], blockscale_offsets [E+1],
    dst_row [num_pairs]) as int32 arrays."""
    ids = [int(v) - first_expert for v in np.asarray(topk_ids).reshape(-1)]
    counts = [0] * num_experts
    for i in ids:
        if 0 <= i < num_experts:
            counts[i] += 1
    eo, bso = [0], [0]
    for c in counts:
        eo.append(eo[-1] + c)
        bso.append(bso[-1] + (c + 127) // 128 * 128)
    nxt = list(eo[:-1])
    dst = []
    for i in ids:
        if 0 <= i < num_experts:
            dst.append(nxt[i])
            nxt[i] += 1
        else:
            dst.append(-1)
    ps = [[c, n, k] for c in counts]
    return (np.array(ps, dtype=np.int32).reshape(num_experts, 3), np.array(eo, dtype=np.int32),
            np.array(bso, dtype=np.int32), np.array(dst, dtype=np.int32))


def permute_rows(x, dst_row, topk, total_rows):
    """out[dst_row[p]] = x[p // topk]; rows nobody writes stay NaN (float input) or 0."""
    x = np.asarray(x)
    out = np.full((total_rows, x.shape[1]), np.nan if x.dtype.kind == "f" else 0, dtype=x.dtype)
    for p, d in enumerate(np.asarray(dst_row)):
        if d >= 0:
            out[d] = x[p // topk]
    return out
