"""GPU parity of the FP8-blockwise grouped GEMM against the CPU oracle (through the torch op and the C ABI)."""
import numpy as np
import pytest
import torch

from oracle import fp8_blockwise as ofp8
from tests import helpers as H

pytestmark = pytest.mark.gpu


def _oracle(ops, prob, out_dtype="bf16"):
    return ofp8.grouped_mm(H.codes(ops["a"]), H.codes(ops["b_phys"]), H.f32(ops["scales_a"]),
                           H.f32(ops["scales_b_phys"]), [[m, prob.n, prob.k] for m in prob.rows],
                           ops["expert_offsets"].cpu().numpy(), out_dtype=out_dtype)


def _call_op(esmoe, ops):
    esmoe.es_fp8_blockwise_scaled_grouped_mm(
        ops["output"], ops["a"], ops["b"], ops["scales_a"], ops["scales_b"], ops["stride_a"], ops["stride_b"],
        ops["stride_d"], ops["problem_sizes"], ops["expert_offsets"], ops["workspace"])
    torch.cuda.synchronize()
    return ops["output"]


def test_c0_through_torch_op(esmoe):
    from expert_specialization_moe_amd import workloads as W

    prob = W.config_problem("c0", seed=0)
    ops = W.make_fp8_blockwise_operands(prob, "cuda", seed=0)
    ops["output"].fill_(float("nan"))
    y = H.f32(_call_op(esmoe, ops))
    ref = _oracle(ops, prob)
    H.check_grouped(y, ref, prob.rows, W.offsets_of(prob.rows), "c0")


@pytest.mark.parametrize("force_bm", [0, 16, 32, 64, 128, 192])
@pytest.mark.parametrize("out_dtype", [torch.bfloat16, torch.float16])
def test_forced_tile_shapes(esmoe, force_bm, out_dtype):
    """Every tile height of the menu and the device schedule (0), both output types, against the oracle; also the
    tight form of the tolerance (helpers.check_ulps)."""
    from expert_specialization_moe_amd import _native
    from expert_specialization_moe_amd import workloads as W

    # ragged rows incl. empty experts, N not a multiple of 256, odd number of K blocks
    prob = W.Problem("ragged", 384, 640, [0, 1, 17, 130, 0, 64, 300, 15, 33, 200])
    ops = W.make_fp8_blockwise_operands(prob, "cuda", seed=3, out_dtype=out_dtype)
    ops["output"].fill_(float("nan"))
    y = H.f32(H.capi_fp8_mm(_native, ops, force_bm=force_bm))
    ref = _oracle(ops, prob, "bf16" if out_dtype == torch.bfloat16 else "fp16")
    H.check_grouped(y, ref, prob.rows, W.offsets_of(prob.rows), f"ragged bm={force_bm}")
    H.check_ulps(y, ref, out_dtype, f"ragged bm={force_bm}")


@pytest.mark.parametrize("k", [128, 384, 512, 640, 1024, 1536])
@pytest.mark.parametrize("force_bm", [0, 128, 192])
def test_tall_tiles_with_whole_and_ragged_scale_chunks(esmoe, force_bm, k):
    """The hand-scheduled K block of the 128- and 192-row tiles fetches the activation scales four K blocks at a time:
    K of one, three and five K blocks (a single short chunk; a last chunk that overlaps the one before) and of one to
    three whole chunks, full and ragged tiles, a last column tile that is half empty, against the oracle."""
    from expert_specialization_moe_amd import _native
    from expert_specialization_moe_amd import workloads as W

    prob = W.Problem("tall", 384, k, [0, 1, 17, 130, 192, 300, 193, 500, 96, 97])
    for out_dtype in (torch.bfloat16, torch.float16):
        ops = W.make_fp8_blockwise_operands(prob, "cuda", seed=7, out_dtype=out_dtype)
        ops["output"].fill_(float("nan"))
        y = H.f32(H.capi_fp8_mm(_native, ops, force_bm=force_bm))
        ref = _oracle(ops, prob, "bf16" if out_dtype == torch.bfloat16 else "fp16")
        H.check_grouped(y, ref, prob.rows, W.offsets_of(prob.rows), f"tall k={k} bm={force_bm}")
        H.check_ulps(y, ref, out_dtype, f"tall k={k} bm={force_bm}")


def test_tall_tiles_distinct_scales_per_row_and_k_block(esmoe):
    """Scales that differ for every (row, K block) and every (column block, K block), with integer-valued operands:
    a scale taken from a neighbouring row, K block or chunk shows as a large error, not as rounding."""
    from expert_specialization_moe_amd import _native
    from expert_specialization_moe_amd import workloads as W
    from oracle import fp8

    rows, n, k = [200, 0, 385, 33], 512, 2048
    rng = np.random.default_rng(9)
    e, total = len(rows), sum(rows)
    ai = rng.integers(-2, 3, size=(total, k)).astype(np.float32)
    bi = rng.integers(-2, 3, size=(e, n, k)).astype(np.float32)
    sa = (2.0 ** rng.integers(-2, 3, size=(total, k // 128))).astype(np.float32)
    sb = (2.0 ** rng.integers(-2, 3, size=(e, n // 128, k // 128))).astype(np.float32)
    ops = {
        "a": torch.from_numpy(fp8.e4m3fn_encode_rne(ai)).cuda().view(torch.float8_e4m3fn),
        "b_phys": torch.from_numpy(fp8.e4m3fn_encode_rne(bi)).cuda().view(torch.float8_e4m3fn),
        "scales_a": torch.from_numpy(sa).cuda(), "scales_b_phys": torch.from_numpy(sb).cuda(),
        "problem_sizes": torch.tensor([[m, n, k] for m in rows], dtype=torch.int32, device="cuda"),
        "expert_offsets": torch.tensor(W.offsets_of(rows), dtype=torch.int32, device="cuda"),
        "output": torch.full((total, n), float("nan"), dtype=torch.bfloat16, device="cuda"),
    }
    y = H.f32(H.capi_fp8_mm(_native, ops))
    for g, (m, off) in enumerate(zip(rows, W.offsets_of(rows))):
        if not m:
            continue
        exact = np.zeros((m, n), dtype=np.float64)
        for kb in range(k // 128):
            part = ai[off:off + m, kb * 128:(kb + 1) * 128].astype(np.float64) @ bi[g][:, kb * 128:(kb + 1) * 128].T
            exact += part * sa[off:off + m, kb:kb + 1] * np.repeat(sb[g][:, kb], 128)[None, :]
        # integers times powers of two: every partial sum is exact in fp32, only the final rounding remains
        assert np.array_equal(y[off:off + m], fp8.bf16_round(exact.astype(np.float32))), f"expert {g}"


def test_two_streams_with_their_own_workspaces(esmoe):
    """Two calls in flight at once on two streams, each with its own workspace (the hand-out counters live there),
    against the oracle."""
    from expert_specialization_moe_amd import workloads as W

    probs = [W.Problem("s0", 512, 1024, [300, 0, 17, 700, 64, 5]), W.Problem("s1", 384, 768, [40, 129, 0, 260, 33])]
    opss = [W.make_fp8_blockwise_operands(p, "cuda", seed=40 + i) for i, p in enumerate(probs)]
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    torch.cuda.synchronize()
    for rep in range(3):
        for ops, st in zip(opss, streams):
            ops["output"].fill_(float("nan"))
        torch.cuda.synchronize()
        for ops, st in zip(opss, streams):
            with torch.cuda.stream(st):
                esmoe.es_fp8_blockwise_scaled_grouped_mm(
                    ops["output"], ops["a"], ops["b"], ops["scales_a"], ops["scales_b"], ops["stride_a"], ops["stride_b"],
                    ops["stride_d"], ops["problem_sizes"], ops["expert_offsets"], ops["workspace"])
        torch.cuda.synchronize()
    for prob, ops in zip(probs, opss):
        H.check_grouped(H.f32(ops["output"]), _oracle(ops, prob), prob.rows, W.offsets_of(prob.rows), prob.name)
