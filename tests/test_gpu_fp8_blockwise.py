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


@pytest.mark.parametrize("force_bm", [0, 16, 32, 64, 128, 192, 256])
@pytest.mark.parametrize("out_dtype", [torch.bfloat16, torch.float16])
def test_forced_tile_shapes(esmoe, force_bm, out_dtype):
    """Every tile height of the menu and the device schedule (0), both output types, against the oracle; also the
    tight form of the tolerance (the oracle accumulates per K block in the kernel's order)."""
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
