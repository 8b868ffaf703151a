"""GPU parity of the gate_up grouped GEMM with the fused SwiGLU + 1x128 quantisation epilogue."""
import numpy as np
import pytest
import torch

from oracle import fp8
from oracle import fp8_blockwise as ofp8
from tests import helpers as H

pytestmark = pytest.mark.gpu


def _fused(native, ops, inter, mid_dtype, force_bm=0, q=None, sc=None):
    lib = native.lib
    e = ops["problem_sizes"].size(0)
    total, k = ops["a"].shape
    q = torch.full((total, inter), 0x55, dtype=torch.uint8, device="cuda") if q is None else q
    sc = torch.full((total, inter // 128), -1.0, dtype=torch.float32, device="cuda") if sc is None else sc
    need = lib.esmoe_gemm_workspace_bytes(e)
    ws = torch.empty((need,), dtype=torch.uint8, device="cuda")
    rc = lib.esmoe_fp8_blockwise_grouped_mm_swiglu_quant(
        H.ptr(q), H.ptr(sc), 0 if mid_dtype == torch.bfloat16 else 1, H.ptr(ops["a"]), H.ptr(ops["b_phys"]),
        H.ptr(ops["scales_a"]), H.ptr(ops["scales_b_phys"]), H.ptr(ops["problem_sizes"]), H.ptr(ops["expert_offsets"]), e,
        total, 2 * inter, k, force_bm, H.ptr(ws), need, H.stream_ptr())
    assert rc == 0, (rc, native.last_error())
    torch.cuda.synchronize()
    return q, sc


@pytest.mark.parametrize("force_bm", [0, 16, 32, 64, 128, 192])
@pytest.mark.parametrize("mid_dtype", [torch.bfloat16, torch.float16])
def test_fused_equals_projection_then_swiglu_quant(esmoe, force_bm, mid_dtype):
    """Bit-exact against this library's own separate route: grouped GEMM into `mid_dtype`, then the fused
    SwiGLU + 1x128 quantiser (itself checked against the oracle in test_gpu_fp8_quant_act.py)."""
    from expert_specialization_moe_amd import _native
    from expert_specialization_moe_amd import workloads as W

    inter = 384
    rows = [0, 5, 70, 200, 130, 1, 333, 64]
    prob = W.Problem("gate_up", 2 * inter, 512, rows)
    ops = W.make_fp8_blockwise_operands(prob, "cuda", seed=3, out_dtype=mid_dtype, weight_std=0.05)
    total = prob.total_rows
    q, sc = _fused(_native, ops, inter, mid_dtype, force_bm)
    y = H.capi_fp8_mm(_native, ops, force_bm)
    q_ref, sc_ref = esmoe.es_swiglu_quant_1x128(y)
    torch.cuda.synchronize()
    assert torch.equal(q, q_ref.view(torch.uint8)), f"{(q != q_ref.view(torch.uint8)).sum().item()} bytes differ"
    assert torch.equal(sc, sc_ref)
    assert total == q.shape[0]


def test_fused_against_oracle_chain(esmoe):
    """Against the CPU oracle chain grouped_mm -> swiglu -> quant_act_1x128 on the same quantised operands.

    Floating point: the projection differs from the oracle's by fp32 summation order (a few bf16 roundings flip),
    and the device exp is within an ulp or two; a flipped rounding moves one byte or, at a block maximum, one scale.
    Tolerance: dequantised values within 2 % of the block's largest value plus one e4m3 step of the oracle's."""
    from expert_specialization_moe_amd import _native
    from expert_specialization_moe_amd import workloads as W

    inter = 256
    rows = [3, 140, 0, 65]
    prob = W.Problem("gate_up", 2 * inter, 384, rows)
    ops = W.make_fp8_blockwise_operands(prob, "cuda", seed=9, weight_std=0.05)
    q, sc = _fused(_native, ops, inter, torch.bfloat16)
    ps = [[m, 2 * inter, 384] for m in rows]
    y = ofp8.grouped_mm(H.codes(ops["a"]), H.codes(ops["b_phys"]), ops["scales_a"].cpu().numpy(),
                        ops["scales_b_phys"].cpu().numpy(), ps, W.offsets_of(rows), out_dtype="bf16")
    with np.errstate(over="ignore"):
        h = ofp8.swiglu(y, "bf16")
    q_ref, sc_ref = ofp8.quant_act_1x128(h, scale_via_reciprocal=True)
    deq_g = fp8.e4m3fn_decode(q.cpu().numpy()) * np.repeat(sc.cpu().numpy(), 128, axis=1)
    deq_r = fp8.e4m3fn_decode(q_ref) * np.repeat(sc_ref, 128, axis=1)
    blockmax = np.repeat(sc_ref, 128, axis=1) * 448.0
    assert (np.abs(deq_g - deq_r) <= 0.02 * blockmax + 0.13 * np.abs(deq_r)).all()
    assert np.allclose(sc.cpu().numpy(), sc_ref, rtol=2e-2)
    assert (q.cpu().numpy() != q_ref).mean() <= 0.05


def test_fused_through_operator_and_untouched_rows(esmoe):
    """Operator form equals the C ABI call; rows of no expert are left alone."""
    from expert_specialization_moe_amd import _native
    from expert_specialization_moe_amd import workloads as W

    inter = 128
    rows = [17, 0, 40]
    prob = W.Problem("gate_up", 2 * inter, 256, rows)
    ops = W.make_fp8_blockwise_operands(prob, "cuda", seed=4, weight_std=0.05)
    q, sc = _fused(_native, ops, inter, torch.bfloat16)
    q2 = torch.zeros_like(q)
    sc2 = torch.zeros_like(sc)
    esmoe.es_fp8_blockwise_scaled_grouped_mm_swiglu_quant(q2, sc2, ops["a"], ops["b"], ops["scales_a"], ops["scales_b"],
                                                          ops["problem_sizes"], ops["expert_offsets"], ops["workspace"])
    torch.cuda.synchronize()
    assert torch.equal(q, q2) and torch.equal(sc, sc2)
    # n not a multiple of 256 is refused
    rc = _native.lib.esmoe_fp8_blockwise_grouped_mm_swiglu_quant(
        H.ptr(q), H.ptr(sc), 0, H.ptr(ops["a"]), H.ptr(ops["b_phys"]), H.ptr(ops["scales_a"]), H.ptr(ops["scales_b_phys"]),
        H.ptr(ops["problem_sizes"]), H.ptr(ops["expert_offsets"]), 3, prob.total_rows, 384, 256, 0, H.ptr(ops["workspace"]),
        ops["workspace"].numel(), H.stream_ptr())
    assert rc != 0


def test_fused_equals_separate_route_at_c1_size(esmoe):
    """Full DeepSeek-V3 gate_up share (E=32, K=7168, N=4096, Zipf rows): the fused operator and the two separate
    operators give identical bytes and scales; nothing outside the experts' rows is written."""
    from expert_specialization_moe_amd import workloads as W

    prob = W.config_problem("c1")
    ops = W.make_fp8_blockwise_operands(prob, "cuda", seed=0)
    total, inter = prob.total_rows, prob.n // 2
    q = torch.full((total, inter), 0x55, dtype=torch.uint8, device="cuda")
    sc = torch.full((total, inter // 128), -1.0, dtype=torch.float32, device="cuda")
    esmoe.es_fp8_blockwise_scaled_grouped_mm_swiglu_quant(q, sc, ops["a"], ops["b"], ops["scales_a"], ops["scales_b"],
                                                          ops["problem_sizes"], ops["expert_offsets"], ops["workspace"])
    esmoe.es_fp8_blockwise_scaled_grouped_mm(ops["output"], ops["a"], ops["b"], ops["scales_a"], ops["scales_b"],
                                             ops["stride_a"], ops["stride_b"], ops["stride_d"], ops["problem_sizes"],
                                             ops["expert_offsets"], ops["workspace"])
    q_ref, sc_ref = esmoe.es_swiglu_quant_1x128(ops["output"])
    torch.cuda.synchronize()
    assert torch.equal(q, q_ref.view(torch.uint8))
    assert torch.equal(sc, sc_ref)
    assert (sc > 0).all()


def test_fused_replays_in_a_graph(esmoe):
    """The fused operator captured in a HIP graph gives the eager result on every replay (no allocation, no memset
    node: the workspace is passed in and the schedule kernel clears its own counters)."""
    from expert_specialization_moe_amd import workloads as W

    prob = W.Problem("gate_up", 512, 384, [40, 0, 300, 7])
    ops = W.make_fp8_blockwise_operands(prob, "cuda", seed=8, weight_std=0.05)
    total, inter = prob.total_rows, 256
    q_e = torch.zeros((total, inter), dtype=torch.uint8, device="cuda")
    sc_e = torch.zeros((total, inter // 128), dtype=torch.float32, device="cuda")
    args = (ops["a"], ops["b"], ops["scales_a"], ops["scales_b"], ops["problem_sizes"], ops["expert_offsets"], ops["workspace"])
    esmoe.es_fp8_blockwise_scaled_grouped_mm_swiglu_quant(q_e, sc_e, *args)
    torch.cuda.synchronize()
    q_g = torch.zeros_like(q_e)
    sc_g = torch.zeros_like(sc_e)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        esmoe.es_fp8_blockwise_scaled_grouped_mm_swiglu_quant(q_g, sc_g, *args)   # warm-up on the capture stream
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        esmoe.es_fp8_blockwise_scaled_grouped_mm_swiglu_quant(q_g, sc_g, *args)
    for _ in range(3):
        q_g.zero_()
        sc_g.zero_()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(q_g, q_e) and torch.equal(sc_g, sc_e)
