"""GPU parity of the MXFP8 grouped quant (bit-exact) and block-scaled grouped GEMM against the CPU oracle."""
import numpy as np
import pytest
import torch

from oracle import mxfp8 as omx
from tests import helpers as H

pytestmark = pytest.mark.gpu


def _quant_case(esmoe, rows, k, in_dtype, seed):
    from expert_specialization_moe_amd import workloads as W

    e = len(rows)
    total = sum(rows)
    gen = torch.Generator().manual_seed(seed)
    x = (torch.randn((total, k), generator=gen) * torch.exp(2.0 * torch.randn((total, 1), generator=gen))).to(in_dtype)
    # sprinkle exact zeros blocks, tie values (amax = 448 * 2^j is the documented unpinned tie) and tiny values
    if total:
        x[0, :32] = 0
        x[total // 2, 32:64] = 0
        x[total - 1, :32] = torch.tensor(1e-30).to(in_dtype)
    xd = x.cuda()
    ps = torch.tensor([[m, 7, k] for m in rows], dtype=torch.int32, device="cuda")
    eo = torch.tensor(W.offsets_of(rows), dtype=torch.int32, device="cuda")
    bso_np, sf_rows = W.blockscale_offsets_of(rows)
    bso = torch.tensor(bso_np, dtype=torch.int32, device="cuda")
    q = torch.full((total, k), 0x55, dtype=torch.uint8, device="cuda")
    sf = torch.full((sf_rows * (k // 32),), 0xEE, dtype=torch.uint8, device="cuda")
    esmoe.es_sm100_mxfp8_blockscaled_grouped_quant(xd, ps, eo, bso, q, sf)
    torch.cuda.synchronize()
    q_ref, sf_ref, mask = omx.grouped_quant(H.hp_to_f32(x), [[m, 7, k] for m in rows], W.offsets_of(rows), bso_np,
                                            sf_total_rows=sf_rows)
    q_gpu = q.cpu().numpy()
    sf_gpu = sf.cpu().numpy()
    assert np.array_equal(q_gpu, q_ref), f"{(q_gpu != q_ref).sum()} quantised bytes differ"
    assert np.array_equal(sf_gpu[mask], sf_ref[mask]), f"{(sf_gpu[mask] != sf_ref[mask]).sum()} scale bytes differ"
    # padding rows of touched 128-row tiles are zero, untouched tiles keep the poison
    return sf_gpu, mask


@pytest.mark.parametrize("in_dtype", [torch.bfloat16, torch.float16])
def test_quant_bit_exact_ragged(esmoe, in_dtype):
    sf, mask = _quant_case(esmoe, [1, 127, 128, 129, 0, 300, 5], 384, in_dtype, seed=1)
    assert set(np.unique(sf[~mask]).tolist()) <= {0}, "padding rows of a written scale tile must be 0"


def test_quant_bit_exact_wide(esmoe):
    _quant_case(esmoe, [513, 64, 0, 0, 1000], 7168, torch.bfloat16, seed=2)


@pytest.mark.parametrize("force_bm", [0, 16, 64, 128, 256])
@pytest.mark.parametrize("out_dtype", [torch.bfloat16, torch.float16])
def test_mx_gemm_parity(esmoe, force_bm, out_dtype):
    from expert_specialization_moe_amd import _native
    from expert_specialization_moe_amd import workloads as W

    prob = W.Problem("ragged", 384, 640, [0, 1, 17, 130, 0, 64, 300, 15, 33], kind="mxfp8")
    ops = W.make_mxfp8_operands(prob, "cuda", seed=5, out_dtype=out_dtype, weight_std=1.0)
    ops["output"].fill_(float("nan"))
    y = H.f32(H.capi_mx_mm(_native, ops, force_bm=force_bm))
    ref = omx.grouped_mm(H.codes(ops["a"]), H.codes(ops["b_phys"]), ops["sfa"].cpu().numpy().reshape(-1),
                         ops["sfb_phys"].cpu().numpy().reshape(-1), [[m, prob.n, prob.k] for m in prob.rows],
                         W.offsets_of(prob.rows), ops["blockscale_offsets"].cpu().numpy(),
                         out_dtype="bf16" if out_dtype == torch.bfloat16 else "fp16")
    H.check_grouped(y, ref, prob.rows, W.offsets_of(prob.rows), f"mx bm={force_bm}")
    # rows of empty experts / nothing else: every row belongs to an expert here, so no NaN may remain
    assert np.isfinite(y).all()


def test_mx_end_to_end_through_ops(esmoe):
    """quant -> GEMM through the Python entry points, compared like the reference's own test
    (calc_diff < 1e-3 against the unquantised product)."""
    from expert_specialization_moe_amd import workloads as W
    from oracle.fp8_blockwise import calc_diff

    prob = W.Problem("e2e", 256, 512, [77, 200, 3, 129], kind="mxfp8")
    ops = W.make_mxfp8_operands(prob, "cuda", seed=9, weight_std=1.0)
    esmoe.es_sm100_mxfp8_blockscaled_grouped_mm(ops["output"], ops["a"], ops["b"], ops["sfa"], ops["sfb"],
                                                ops["problem_sizes"], ops["expert_offsets"], ops["blockscale_offsets"])
    torch.cuda.synchronize()
    y = H.f32(ops["output"])
    a = H.hp_to_f32(ops["a_hp"]).astype(np.float64)
    w = H.hp_to_f32(ops["w_hp"]).astype(np.float64).reshape(prob.num_experts, prob.n, prob.k)
    for e, (m, off) in enumerate(zip(prob.rows, W.offsets_of(prob.rows))):
        ref = a[off:off + m] @ w[e].T
        assert calc_diff(y[off:off + m], ref) < 1e-3
