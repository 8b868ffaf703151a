"""GPU parity of the FP8 1x128 activation quantiser: bytes and scales bit-exact against the CPU oracle
(the restatement of per_token_cast_to_fp8, test/test_es_grouped_gemm.py:36-44), through the C ABI."""
import ctypes

import numpy as np
import pytest
import torch

from oracle import fp8_blockwise as ofp8
from tests import helpers as H

pytestmark = pytest.mark.gpu


def _run_capi(x):
    from expert_specialization_moe_amd import _native

    m, k = x.shape
    xd = x.cuda()
    q = torch.full((m, k), 0x55, dtype=torch.uint8, device="cuda")
    sc = torch.full((m, k // 128), -1.0, dtype=torch.float32, device="cuda")
    rc = _native.lib.esmoe_fp8_quant_act_1x128(
        ctypes.c_void_p(xd.data_ptr()), 0 if x.dtype == torch.bfloat16 else 1, ctypes.c_void_p(q.data_ptr()),
        ctypes.c_void_p(sc.data_ptr()), m, k, ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
    assert rc == 0, _native.last_error()
    torch.cuda.synchronize()
    return q.cpu().numpy(), sc.cpu().numpy()


def _inputs(m, k, dtype, seed):
    gen = torch.Generator().manual_seed(seed)
    x = (torch.randn((m, k), generator=gen) * torch.exp(2.0 * torch.randn((m, 1), generator=gen))).to(dtype)
    if m:
        x[0, :128] = 0                                   # all-zero block: amax clamps to 1e-4
        x[m // 2, 128:256] = torch.tensor(3e-5).to(dtype)   # below the clamp
        x[m - 1, :128] = torch.tensor(448.0).to(dtype)
        x[m - 1, 5] = torch.tensor(-1.75).to(dtype)
    return x


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("shape", [(1, 128), (7, 384), (333, 512), (1030, 7168)])
def test_quant_act_bit_exact(esmoe, dtype, shape):
    x = _inputs(*shape, dtype, seed=shape[0])
    q, sc = _run_capi(x)
    q_ref, sc_ref = ofp8.quant_act_1x128(H.hp_to_f32(x), scale_via_reciprocal=True)
    assert np.array_equal(q, q_ref), f"{(q != q_ref).sum()} bytes differ"
    assert np.array_equal(sc.view(np.uint32), sc_ref.view(np.uint32)), "scales differ"


def test_quant_act_matches_torch_helper_and_feeds_the_gemm(esmoe):
    """Operator path: same bytes as the torch quantiser, and its outputs drive the grouped GEMM."""
    from expert_specialization_moe_amd import quant as Q
    from expert_specialization_moe_amd import workloads as W

    prob = W.Problem("ragged", 256, 512, [3, 40, 0, 130])
    ops = W.make_fp8_blockwise_operands(prob, "cuda", seed=3)
    gen = torch.Generator().manual_seed(9)
    x = torch.randn((prob.total_rows, prob.k), generator=gen).to(torch.bfloat16).cuda()
    q, sc = esmoe.es_fp8_quant_act_1x128(x)
    q_t, sc_t = Q.quant_act_1x128(x)
    assert torch.equal(q.view(torch.uint8), q_t.view(torch.uint8)) and torch.equal(sc, sc_t)
    out = torch.empty_like(ops["output"])
    esmoe.es_fp8_blockwise_scaled_grouped_mm(out, q, ops["b"], sc, ops["scales_b"], ops["stride_a"], ops["stride_b"],
                                             ops["stride_d"], ops["problem_sizes"], ops["expert_offsets"], ops["workspace"])
    torch.cuda.synchronize()
    ref = ofp8.grouped_mm(q.view(torch.uint8).cpu().numpy(), ops["b_phys"].view(torch.uint8).cpu().numpy(),
                          sc.cpu().numpy(), ops["scales_b_phys"].cpu().numpy(), [[m, prob.n, prob.k] for m in prob.rows],
                          W.offsets_of(prob.rows))
    H.check_grouped(H.f32(out), ref, prob.rows, W.offsets_of(prob.rows), "gemm on device-quantised rows")


def test_quant_act_empty_and_rejects(esmoe):
    from expert_specialization_moe_amd import _native

    x = torch.empty((0, 256), dtype=torch.bfloat16)
    q, sc = _run_capi(x)
    assert q.shape == (0, 256) and sc.shape == (0, 2)
    p = ctypes.c_void_p(16)
    assert _native.lib.esmoe_fp8_quant_act_1x128(p, 0, p, p, 4, 100, None) == -1
    assert _native.lib.esmoe_fp8_quant_act_1x128(p, 5, p, p, 4, 128, None) == -1
    with pytest.raises(RuntimeError, match="align to 128"):
        esmoe.es_fp8_quant_act_1x128(torch.zeros((2, 100), dtype=torch.bfloat16, device="cuda"))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("shape", [(1, 128, 128), (3, 256, 384), (2, 512, 7168)])
def test_quant_weight_bit_exact(esmoe, dtype, shape):
    """128x128 weight quantiser through the C ABI: bytes and scales bit-exact against the oracle's restatement
    of per_block_cast_to_fp8 (test/test_es_grouped_gemm.py:47-59) and against the torch helper on the GPU."""
    from expert_specialization_moe_amd import _native
    from expert_specialization_moe_amd import quant as Q

    e, n, k = shape
    gen = torch.Generator().manual_seed(e * 7 + n)
    w = (torch.randn((e, n, k), generator=gen) * 0.02 * torch.exp(torch.randn((e, 1, 1), generator=gen))).to(dtype)
    w[0, :128, :128] = 0                         # all-zero block: amax clamps to 1e-4
    wd = w.cuda()
    q = torch.full((e, n, k), 0x55, dtype=torch.uint8, device="cuda")
    sc = torch.full((e, n // 128, k // 128), -1.0, dtype=torch.float32, device="cuda")
    rc = _native.lib.esmoe_fp8_quant_weight_128x128(
        ctypes.c_void_p(wd.data_ptr()), 0 if dtype == torch.bfloat16 else 1, ctypes.c_void_p(q.data_ptr()),
        ctypes.c_void_p(sc.data_ptr()), e * n, k, ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
    assert rc == 0, _native.last_error()
    torch.cuda.synchronize()
    for i in range(e):
        q_ref, sc_ref = ofp8.quant_weight_128x128(H.hp_to_f32(w[i]), scale_via_reciprocal=True)
        assert np.array_equal(q[i].cpu().numpy(), q_ref), f"expert {i}: bytes differ"
        assert np.array_equal(sc[i].cpu().numpy().view(np.uint32), sc_ref.view(np.uint32)), f"expert {i}: scales differ"
    q_t, sc_t = Q.quant_weight_128x128(wd)
    q_o, sc_o = esmoe.es_fp8_quant_weight_128x128(wd)
    assert torch.equal(q_o.view(torch.uint8), q_t.view(torch.uint8)) and torch.equal(sc_o, sc_t)
    assert torch.equal(q_o.view(torch.uint8), q)
    assert _native.lib.esmoe_fp8_quant_weight_128x128(ctypes.c_void_p(16), 0, ctypes.c_void_p(16), ctypes.c_void_p(16), 100, 128, None) == -1


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("shape", [(1, 128), (37, 384), (1030, 2048)])
def test_swiglu_quant_against_oracle(esmoe, dtype, shape):
    """Fused SwiGLU + 1x128 quantisation through the C ABI against oracle swiglu() -> quant_act_1x128().

    Floating point with a transcendental: the device forms silu with the hardware's base-2 exponential and
    reciprocal, each about an ulp from the oracle's correctly rounded float64 route, so a product that lands within
    that distance of a bf16/fp16 rounding boundary may round the other way and move one byte (or, if it is the
    block maximum, the block's scale) by one step (seen on 4096 x 2048 outputs: 1e-6 of the bytes, 1e-4 of the scales).
    Tolerance: at most 1e-3 of the bytes and of the scales differ, and every dequantised value is within one
    e4m3 step (12.5 % relative, plus the subnormal step) of the oracle's.  Zero products may carry either sign."""
    from expert_specialization_moe_amd import _native
    from oracle import fp8

    m, inter = shape
    gen = torch.Generator().manual_seed(m + inter)
    x = (torch.randn((m, 2 * inter), generator=gen) * 2.0).to(dtype)
    x[0, :8] = torch.tensor([-100.0, -20.0, 0.0, 20.0, 100.0, -0.0, 1e-3, -1e-3]).to(dtype)   # saturated and tiny gates
    xd = x.cuda()
    q = torch.full((m, inter), 0x55, dtype=torch.uint8, device="cuda")
    sc = torch.full((m, inter // 128), -1.0, dtype=torch.float32, device="cuda")
    rc = _native.lib.esmoe_swiglu_quant_1x128(H.ptr(xd), 0 if dtype == torch.bfloat16 else 1, H.ptr(q), H.ptr(sc), m, inter,
                                              H.stream_ptr())
    assert rc == 0, _native.last_error()
    torch.cuda.synchronize()
    with np.errstate(over="ignore"):
        h = ofp8.swiglu(H.hp_to_f32(x), "bf16" if dtype == torch.bfloat16 else "fp16")
    q_ref, sc_ref = ofp8.quant_act_1x128(h, scale_via_reciprocal=True)
    qg, sg = q.cpu().numpy(), sc.cpu().numpy()
    # the sign of a zero product (gate -0.0) is not pinned: 0x80 and 0x00 both decode to zero
    canon = lambda c: np.where(c == 0x80, 0, c)
    assert (canon(qg) != canon(q_ref)).mean() <= 1e-3, f"{(canon(qg) != canon(q_ref)).sum()} of {qg.size} bytes differ"
    assert (sg != sc_ref).mean() <= 1e-3 + 1.0 / sg.size, f"{(sg != sc_ref).sum()} of {sg.size} scales differ"
    deq_g = fp8.e4m3fn_decode(qg) * np.repeat(sg, 128, axis=1)
    deq_r = fp8.e4m3fn_decode(q_ref) * np.repeat(sc_ref, 128, axis=1)
    tol = 0.13 * np.abs(deq_r) + 1.1 * np.repeat(sc_ref, 128, axis=1) * 2.0 ** -9
    assert (np.abs(deq_g - deq_r) <= tol).all()
    # operator path gives the same bytes as the C ABI call
    q_o, sc_o = esmoe.es_swiglu_quant_1x128(xd)
    assert torch.equal(q_o.view(torch.uint8), q) and torch.equal(sc_o, sc)
    # and stays close to the unfused torch sequence (two roundings instead of one)
    hd = (torch.nn.functional.silu(xd[:, :inter].float()) * xd[:, inter:].float()).to(dtype)
    q_t, sc_t = esmoe.es_fp8_quant_act_1x128(hd)
    assert (q_t.view(torch.uint8) != q).float().mean().item() <= 2e-2
