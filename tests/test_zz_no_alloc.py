"""The entry point that allocates nothing (static schedule workspace inside the library) against the entry point
that takes a caller workspace: identical output bits, two calls in a row, the second on a smaller problem; a call
leaves the device's free memory as it found it, and can be captured in a graph and replayed."""
import ctypes

import pytest
import torch

from tests import helpers as H

pytestmark = pytest.mark.gpu


def _static_mm(native, ops, out):
    e = ops["problem_sizes"].size(0)
    total, k = ops["a"].shape
    n = ops["b_phys"].size(1)
    rc = native.lib.esmoe_fp8_blockwise_grouped_mm_static(
        H.ptr(out), 0 if out.dtype == torch.bfloat16 else 1, H.ptr(ops["a"]), H.ptr(ops["b_phys"]), H.ptr(ops["scales_a"]),
        H.ptr(ops["scales_b_phys"]), H.ptr(ops["problem_sizes"]), H.ptr(ops["expert_offsets"]), e, total, n, k, 0,
        H.stream_ptr())
    assert rc == 0, (rc, native.last_error())
    torch.cuda.synchronize()
    return out


def test_static_workspace_entry_point_matches_workspace_entry_point(esmoe):
    from expert_specialization_moe_amd import _native
    from expert_specialization_moe_amd import workloads as W

    big = W.Problem("first", 512, 640, [300, 0, 17, 64, 700, 5, 129, 33, 1, 200, 0, 90])
    small = W.Problem("second", 256, 384, [3, 130, 0, 40])
    for prob, seed in ((big, 31), (small, 32)):
        ops = W.make_fp8_blockwise_operands(prob, "cuda", seed=seed)
        want = H.capi_fp8_mm(_native, ops, out=torch.full_like(ops["output"], float("nan"))).clone()
        got = _static_mm(_native, ops, torch.full_like(ops["output"], float("nan")))
        assert torch.equal(got.view(torch.int16), want.view(torch.int16)), prob.name
        assert not torch.isnan(got).any()
        # the property the entry point exists for: after its first call on the device (which looks the array's
        # address up), a call takes no device memory and returns none
        out = torch.full_like(ops["output"], float("nan"))
        torch.cuda.synchronize()
        free_before = torch.cuda.mem_get_info()[0]
        _static_mm(_native, ops, out)
        assert torch.cuda.mem_get_info()[0] == free_before
        assert torch.equal(out.view(torch.int16), want.view(torch.int16))


def test_static_workspace_entry_point_rejects_too_many_experts(esmoe):
    from expert_specialization_moe_amd import _native

    buf = torch.zeros(4096, dtype=torch.uint8, device="cuda")
    p = H.ptr(buf)
    rc = _native.lib.esmoe_fp8_blockwise_grouped_mm_static(p, 0, p, p, p, p, p, p, 1025, 10, 128, 128, 0, None)
    assert rc == -1 and "at most 1024" in _native.last_error()


def test_static_workspace_entry_point_replays_in_a_graph(esmoe):
    """Captured after one eager call on the device (the address look-up is not capturable): every replay, with eager
    work between the replays, gives the eager result."""
    from expert_specialization_moe_amd import _native
    from expert_specialization_moe_amd import workloads as W

    prob = W.Problem("graph", 384, 512, [33, 0, 200, 7, 129])
    ops = W.make_fp8_blockwise_operands(prob, "cuda", seed=33)
    eager = _static_mm(_native, ops, torch.full_like(ops["output"], float("nan"))).clone()
    out = torch.zeros_like(ops["output"])
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        e = ops["problem_sizes"].size(0)
        total, k = ops["a"].shape
        n = ops["b_phys"].size(1)
        rc = _native.lib.esmoe_fp8_blockwise_grouped_mm_static(
            H.ptr(out), 0, H.ptr(ops["a"]), H.ptr(ops["b_phys"]), H.ptr(ops["scales_a"]), H.ptr(ops["scales_b_phys"]),
            H.ptr(ops["problem_sizes"]), H.ptr(ops["expert_offsets"]), e, total, n, k, 0, H.stream_ptr())
        assert rc == 0, _native.last_error()
    for rep in range(3):
        out.fill_(float("nan"))
        torch.cuda.synchronize()
        graph.replay()
        assert torch.isfinite(torch.randn(1024, device="cuda").sum()).item()   # eager work between replays
        torch.cuda.synchronize()
        assert torch.equal(out, eager), f"replay {rep}"
