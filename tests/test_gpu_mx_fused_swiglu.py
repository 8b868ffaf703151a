"""GPU parity of the mxfp8 gate_up grouped GEMM with the fused SwiGLU + 1x32 E8M0 quantisation epilogue."""
import numpy as np
import pytest
import torch

from oracle import fp8
from oracle import fp8_blockwise as ofp8
from oracle import mxfp8 as omx
from tests import helpers as H

pytestmark = pytest.mark.gpu


def _sf_rows(ops, rows):
    from expert_specialization_moe_amd import workloads as W

    return max(W.blockscale_offsets_of(rows)[1], 128)


def _fused(native, ops, rows, inter, mid_dtype, force_bm=0, fill=0x55):
    lib = native.lib
    e = ops["problem_sizes"].size(0)
    total, k = ops["a"].shape
    sf_rows = _sf_rows(ops, rows)
    q = torch.full((total, inter), fill, dtype=torch.uint8, device="cuda")
    sf = torch.full((sf_rows, inter // 32), fill, dtype=torch.uint8, device="cuda")
    need = lib.esmoe_gemm_workspace_bytes(e)
    ws = torch.empty((need,), dtype=torch.uint8, device="cuda")
    rc = lib.esmoe_mxfp8_grouped_mm_swiglu_quant(
        H.ptr(q), H.ptr(sf), 0 if mid_dtype == torch.bfloat16 else 1, H.ptr(ops["a"]), H.ptr(ops["b_phys"]),
        H.ptr(ops["sfa"]), H.ptr(ops["sfb_phys"]), H.ptr(ops["problem_sizes"]), H.ptr(ops["expert_offsets"]),
        H.ptr(ops["blockscale_offsets"]), e, total, sf_rows, 2 * inter, k, force_bm, H.ptr(ws), need, H.stream_ptr())
    assert rc == 0, (rc, native.last_error())
    torch.cuda.synchronize()
    return q, sf


def _separate(esmoe, native, ops, rows, inter, mid_dtype, force_bm=0, fill=0x55):
    """This library's own separate route: grouped GEMM into `mid_dtype`, then SwiGLU + grouped quantisation."""
    total = ops["a"].shape[0]
    y = H.capi_mx_mm(native, ops, force_bm, out=torch.empty((total, 2 * inter), dtype=mid_dtype, device="cuda"))
    q = torch.full((total, inter), fill, dtype=torch.uint8, device="cuda")
    sf = torch.full((_sf_rows(ops, rows), inter // 32), fill, dtype=torch.uint8, device="cuda")
    esmoe.es_swiglu_mxfp8_grouped_quant(y, ops["problem_sizes"], ops["expert_offsets"], ops["blockscale_offsets"], q, sf)
    torch.cuda.synchronize()
    return q, sf


@pytest.mark.parametrize("force_bm", [0, 16, 32, 64, 128, 192])
@pytest.mark.parametrize("mid_dtype", [torch.bfloat16, torch.float16])
def test_fused_equals_projection_then_swiglu_quant(esmoe, force_bm, mid_dtype):
    """Bit-exact against the separate route (each step of which is checked against the oracle in test_gpu_mxfp8.py):
    every byte of q and of the scale tiles, padding rows and untouched bytes included, at every tile height."""
    from expert_specialization_moe_amd import _native
    from expert_specialization_moe_amd import workloads as W

    inter = 384
    rows = [0, 5, 70, 200, 130, 1, 333, 64, 530]
    prob = W.Problem("gate_up", 2 * inter, 512, rows)
    ops = W.make_mxfp8_operands(prob, "cuda", seed=3, out_dtype=mid_dtype, weight_std=0.05)
    q, sf = _fused(_native, ops, rows, inter, mid_dtype, force_bm)
    q_ref, sf_ref = _separate(esmoe, _native, ops, rows, inter, mid_dtype, force_bm)
    assert torch.equal(q, q_ref), f"{(q != q_ref).sum().item()} bytes differ"
    assert torch.equal(sf, sf_ref), f"{(sf != sf_ref).sum().item()} scale bytes differ"


def test_fused_against_oracle_chain(esmoe):
    """Against the CPU oracle chain grouped_mm -> swiglu -> grouped_quant on the same quantised operands.

    Floating point: the projection differs from the oracle's by fp32 summation order (a few bf16 roundings flip) and
    the device exp is within an ulp or two; a flipped rounding moves one byte or, at a block maximum on a power-of-two
    boundary, one scale code.  Tolerance: dequantised values within 2 % of the block's range plus one e4m3 step."""
    from expert_specialization_moe_amd import _native
    from expert_specialization_moe_amd import workloads as W

    inter = 256
    rows = [3, 140, 0, 65]
    k = 384
    prob = W.Problem("gate_up", 2 * inter, k, rows)
    ops = W.make_mxfp8_operands(prob, "cuda", seed=9, weight_std=0.05)
    q, sf = _fused(_native, ops, rows, inter, torch.bfloat16, fill=0)
    ps = [[m, 2 * inter, k] for m in rows]
    eo = W.offsets_of(rows)
    bso, sf_rows = W.blockscale_offsets_of(rows)
    y = omx.grouped_mm(H.codes(ops["a"]), H.codes(ops["b_phys"]), ops["sfa"].cpu().numpy().reshape(-1),
                       ops["sfb_phys"].cpu().numpy().reshape(-1), ps, eo, bso, out_dtype="bf16")
    with np.errstate(over="ignore"):
        h = ofp8.swiglu(y, "bf16")
    ps_q = [[m, inter, inter] for m in rows]
    q_ref, sf_ref, _ = omx.grouped_quant(h, ps_q, eo, bso, sf_total_rows=max(sf_rows, 128))
    qg, sfg = q.cpu().numpy(), sf.cpu().numpy().reshape(-1)
    for e, m in enumerate(rows):
        if m == 0:
            continue
        base = int(bso[e]) * (inter // 32)
        sg = omx.unswizzle_scales(sfg, m, inter, base=base)
        sr = omx.unswizzle_scales(sf_ref, m, inter, base=base)
        assert (np.abs(sg.astype(int) - sr.astype(int)) <= 1).all()
        assert (sg != sr).mean() <= 0.02
        dg = omx.dequant_rows(qg[eo[e]:eo[e] + m], sg)
        dr = omx.dequant_rows(q_ref[eo[e]:eo[e] + m], sr)
        blockmax = np.repeat(fp8.e8m0_decode(sr), 32, axis=1) * 448.0
        assert (np.abs(dg - dr) <= 0.02 * blockmax + 0.13 * np.abs(dr)).all()


def test_fused_through_operator_and_untouched_bytes(esmoe):
    """Operator form equals the C ABI call; scale tiles of no expert and rows of no expert are left alone; sizes the
    layouts cannot express are refused."""
    from expert_specialization_moe_amd import _native
    from expert_specialization_moe_amd import workloads as W

    inter = 128
    rows = [17, 0, 40]
    prob = W.Problem("gate_up", 2 * inter, 256, rows)
    ops = W.make_mxfp8_operands(prob, "cuda", seed=4, weight_std=0.05)
    q, sf = _fused(_native, ops, rows, inter, torch.bfloat16)
    q2 = torch.full_like(q, 0x55)
    sf2 = torch.full_like(sf, 0x55)
    esmoe.es_mxfp8_blockscaled_grouped_mm_swiglu_quant(q2, sf2, ops["a"], ops["b"], ops["sfa"], ops["sfb"],
                                                       ops["problem_sizes"], ops["expert_offsets"],
                                                       ops["blockscale_offsets"])
    torch.cuda.synchronize()
    assert torch.equal(q, q2) and torch.equal(sf, sf2)
    # padding rows of the two written scale tiles are 0
    sfn = sf.cpu().numpy().reshape(-1)
    bso, _ = W.blockscale_offsets_of(rows)
    for e, m in enumerate(rows):
        if m == 0:
            continue
        tile = sfn[bso[e] * (inter // 32):(bso[e] + 128) * (inter // 32)].reshape(-1, 32, 4, 4)   # [k tile][row % 32][row / 32][col]
        pad = np.array([[tile[0, r % 32, r // 32, c] for c in range(4)] for r in range(m, 128)])
        assert (pad == 0).all()
    lib = _native.lib
    ws = torch.empty((lib.esmoe_gemm_workspace_bytes(3),), dtype=torch.uint8, device="cuda")
    args = lambda n, sf_rows: (H.ptr(q), H.ptr(sf), 0, H.ptr(ops["a"]), H.ptr(ops["b_phys"]), H.ptr(ops["sfa"]),
                               H.ptr(ops["sfb_phys"]), H.ptr(ops["problem_sizes"]), H.ptr(ops["expert_offsets"]),
                               H.ptr(ops["blockscale_offsets"]), 3, prob.total_rows, sf_rows, n, 256, 0,
                               H.ptr(ws), ws.numel(), H.stream_ptr())
    assert lib.esmoe_mxfp8_grouped_mm_swiglu_quant(*args(384, 256)) != 0      # n not a multiple of 256
    assert lib.esmoe_mxfp8_grouped_mm_swiglu_quant(*args(256, 0)) != 0        # scale rows smaller than the rows
    assert lib.esmoe_mxfp8_grouped_mm_swiglu_quant(*args(256, 100)) != 0      # not a multiple of 128


def test_fused_equals_separate_route_at_c4_size(esmoe):
    """Full C4 share (E=32, K=7168, N=4096, 8192 rows): the fused operator and the two separate operators give identical
    bytes and scale tiles."""
    from expert_specialization_moe_amd import _native
    from expert_specialization_moe_amd import workloads as W

    prob = W.config_problem("c4")
    ops = W.make_mxfp8_operands(prob, "cuda", seed=0)
    inter = prob.n // 2
    q, sf = _fused(_native, ops, prob.rows, inter, torch.bfloat16)
    q_ref, sf_ref = _separate(esmoe, _native, ops, prob.rows, inter, torch.bfloat16)
    assert torch.equal(q, q_ref)
    assert torch.equal(sf, sf_ref)


def test_fused_output_feeds_the_down_projection(esmoe):
    """gate_up (fused) -> down projection, against gate_up -> SwiGLU + quantisation -> down projection: the same
    result, bit for bit, through the operators."""
    from expert_specialization_moe_amd import workloads as W

    inter, hidden = 256, 512
    rows = [130, 7, 0, 260]
    prob = W.Problem("gate_up", 2 * inter, hidden, rows)
    ops = W.make_mxfp8_operands(prob, "cuda", seed=12, weight_std=0.05)
    down = W.make_mxfp8_operands(W.Problem("down", hidden, inter, rows), "cuda", seed=13, weight_std=0.05)
    total = prob.total_rows
    q = torch.zeros((total, inter), dtype=torch.uint8, device="cuda")
    sf = torch.zeros_like(down["sfa"])
    esmoe.es_mxfp8_blockscaled_grouped_mm_swiglu_quant(q, sf, ops["a"], ops["b"], ops["sfa"], ops["sfb"],
                                                       ops["problem_sizes"], ops["expert_offsets"],
                                                       ops["blockscale_offsets"])
    d1 = torch.zeros((total, hidden), dtype=torch.bfloat16, device="cuda")
    esmoe.es_sm100_mxfp8_blockscaled_grouped_mm(d1, q.view(torch.float8_e4m3fn), down["b"], sf, down["sfb"],
                                                down["problem_sizes"], down["expert_offsets"], down["blockscale_offsets"])
    esmoe.es_sm100_mxfp8_blockscaled_grouped_mm(ops["output"], ops["a"], ops["b"], ops["sfa"], ops["sfb"],
                                                ops["problem_sizes"], ops["expert_offsets"], ops["blockscale_offsets"])
    q2 = torch.zeros_like(q)
    sf2 = torch.zeros_like(sf)
    esmoe.es_swiglu_mxfp8_grouped_quant(ops["output"], ops["problem_sizes"], ops["expert_offsets"],
                                        ops["blockscale_offsets"], q2, sf2)
    d2 = torch.zeros_like(d1)
    esmoe.es_sm100_mxfp8_blockscaled_grouped_mm(d2, q2.view(torch.float8_e4m3fn), down["b"], sf2, down["sfb"],
                                                down["problem_sizes"], down["expert_offsets"], down["blockscale_offsets"])
    torch.cuda.synchronize()
    assert torch.equal(d1, d2)
    assert d1.float().abs().max().item() > 0
