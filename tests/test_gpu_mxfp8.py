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


@pytest.mark.parametrize("force_bm", [0, 16, 32, 64, 128, 192])
@pytest.mark.parametrize("out_dtype", [torch.bfloat16, torch.float16])
def test_mx_gemm_parity(esmoe, force_bm, out_dtype):
    from expert_specialization_moe_amd import _native
    from expert_specialization_moe_amd import workloads as W

    prob = W.Problem("ragged", 384, 640, [0, 1, 17, 130, 0, 64, 300, 15, 33, 530], kind="mxfp8")
    ops = W.make_mxfp8_operands(prob, "cuda", seed=5, out_dtype=out_dtype, weight_std=1.0)
    ops["output"].fill_(float("nan"))
    y = H.f32(H.capi_mx_mm(_native, ops, force_bm=force_bm))
    ref = omx.grouped_mm(H.codes(ops["a"]), H.codes(ops["b_phys"]), ops["sfa"].cpu().numpy().reshape(-1),
                         ops["sfb_phys"].cpu().numpy().reshape(-1), [[m, prob.n, prob.k] for m in prob.rows],
                         W.offsets_of(prob.rows), ops["blockscale_offsets"].cpu().numpy(),
                         out_dtype="bf16" if out_dtype == torch.bfloat16 else "fp16")
    H.check_grouped(y, ref, prob.rows, W.offsets_of(prob.rows), f"mx bm={force_bm}")
    H.check_ulps(y, ref, out_dtype, f"mx bm={force_bm}")
    # rows of empty experts / nothing else: every row belongs to an expert here, so no NaN may remain
    assert np.isfinite(y).all()


@pytest.mark.parametrize("force_bm", [0, 16, 32, 64, 128, 192])
def test_mx_tiles_exact_with_distinct_scale_bytes(esmoe, force_bm):
    """Small-integer e4m3 operands and E8M0 scale bytes that differ for every (token row, 32-wide K sub-block) and every
    (weight row, K sub-block): every partial sum is exact in fp32, so the result must EQUAL the fp64 evaluation rounded
    once, and a scale byte taken from a neighbouring row, sub-block, K block or scale tile shows as a wrong value, not as
    rounding.  Experts of 200 / 385 / 530 rows make 192-row tiles start in the middle of a 128-row scale tile.  Every
    tile height, and the fused SwiGLU + quantisation epilogue against the stand-alone quantiser fed the exact result."""
    from expert_specialization_moe_amd import _native
    from expert_specialization_moe_amd import workloads as W
    from oracle import fp8

    rows, n, k = [200, 0, 385, 33, 530], 512, 2048
    kc = k // 32
    rng = np.random.default_rng(12)
    e, total = len(rows), sum(rows)
    ai = rng.integers(-2, 3, size=(total, k)).astype(np.float32)
    bi = rng.integers(-2, 3, size=(e, n, k)).astype(np.float32)
    ca = rng.integers(125, 130, size=(total, kc)).astype(np.uint8)      # 2^-2 .. 2^2 per (row, sub-block)
    cb = rng.integers(125, 130, size=(e, n, kc)).astype(np.uint8)
    offs = W.offsets_of(rows)
    bso_np, sf_rows = W.blockscale_offsets_of(rows)
    sfa = np.zeros(sf_rows * kc, dtype=np.uint8)
    for g, (m, off) in enumerate(zip(rows, offs)):
        if m:
            omx.swizzle_scales(ca[off:off + m], k, out=sfa, base=int(bso_np[g]) * kc)
    sfb = np.zeros(e * n * kc, dtype=np.uint8)
    for g in range(e):
        omx.swizzle_scales(cb[g], k, out=sfb, base=g * n * kc)
    ops = {
        "a": torch.from_numpy(fp8.e4m3fn_encode_rne(ai)).cuda().view(torch.float8_e4m3fn),
        "b_phys": torch.from_numpy(fp8.e4m3fn_encode_rne(bi)).cuda().view(torch.float8_e4m3fn),
        "sfa": torch.from_numpy(sfa).cuda().view(sf_rows, kc), "sfb_phys": torch.from_numpy(sfb).cuda().view(e, n, kc),
        "problem_sizes": torch.tensor([[m, n, k] for m in rows], dtype=torch.int32, device="cuda"),
        "expert_offsets": torch.tensor(offs, dtype=torch.int32, device="cuda"),
        "blockscale_offsets": torch.tensor(bso_np, dtype=torch.int32, device="cuda"),
        "output": torch.full((total, n), float("nan"), dtype=torch.bfloat16, device="cuda"),
    }
    y = H.f32(H.capi_mx_mm(_native, ops, force_bm=force_bm))
    want = np.empty((total, n), dtype=np.float32)
    for g, (m, off) in enumerate(zip(rows, offs)):
        if m:
            da = ai[off:off + m].astype(np.float64) * np.repeat(np.exp2(ca[off:off + m].astype(np.float64) - 127), 32, 1)
            db = bi[g].astype(np.float64) * np.repeat(np.exp2(cb[g].astype(np.float64) - 127), 32, 1)
            want[off:off + m] = fp8.bf16_round((da @ db.T).astype(np.float32))
            assert np.array_equal(y[off:off + m], want[off:off + m]), f"expert {g} ({m} rows), tile height {force_bm}"
    # fused epilogue: the bytes and scale bytes of the stand-alone quantiser applied to the (exact) projection
    inter = n // 2
    lib = _native.lib
    ws_bytes = lib.esmoe_gemm_workspace_bytes(e)
    ws = torch.empty((ws_bytes,), dtype=torch.uint8, device="cuda")
    q = torch.full((total, inter), 0x55, dtype=torch.uint8, device="cuda")
    sf = torch.zeros((sf_rows, inter // 32), dtype=torch.uint8, device="cuda")
    rc = lib.esmoe_mxfp8_grouped_mm_swiglu_quant(
        H.ptr(q), H.ptr(sf), 0, H.ptr(ops["a"]), H.ptr(ops["b_phys"]), H.ptr(ops["sfa"]), H.ptr(ops["sfb_phys"]),
        H.ptr(ops["problem_sizes"]), H.ptr(ops["expert_offsets"]), H.ptr(ops["blockscale_offsets"]), e, total, sf_rows, n, k,
        force_bm, H.ptr(ws), ws_bytes, H.stream_ptr())
    assert rc == 0, _native.last_error()
    q2, sf2 = torch.zeros_like(q), torch.zeros_like(sf)
    esmoe.es_swiglu_mxfp8_grouped_quant(torch.from_numpy(want).cuda().to(torch.bfloat16), ops["problem_sizes"], ops["expert_offsets"],
                                        ops["blockscale_offsets"], q2, sf2)
    torch.cuda.synchronize()
    assert torch.equal(q, q2) and torch.equal(sf, sf2), f"fused epilogue, tile height {force_bm}"


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


@pytest.mark.parametrize("in_dtype", [torch.bfloat16, torch.float16])
def test_weight_quant_equals_transposed_problem_list(esmoe, in_dtype):
    """esmoe_mxfp8_quant_weight through the C ABI: bit-exact against the oracle applied the way the reference
    quantises weights (activation operator, problem list [N, M, K], offsets e*N), and equal to this library's
    grouped operator called that way."""
    from expert_specialization_moe_amd import _native

    e, n, k = 3, 256, 384
    gen = torch.Generator().manual_seed(11)
    w = (torch.randn((e, n, k), generator=gen) * 0.05).to(in_dtype)
    w[1, 5, 32:64] = 0
    wd = w.cuda()
    q = torch.full((e, n, k), 0x55, dtype=torch.uint8, device="cuda")
    sf = torch.full((e, n, k // 32), 0xEE, dtype=torch.uint8, device="cuda")
    rc = _native.lib.esmoe_mxfp8_quant_weight(H.ptr(wd), 0 if in_dtype == torch.bfloat16 else 1, H.ptr(q), H.ptr(sf), e * n, k,
                                              H.stream_ptr())
    assert rc == 0, _native.last_error()
    torch.cuda.synchronize()
    aux_ps = [[n, 5, k]] * e
    aux_off = [i * n for i in range(e)]
    q_ref, sf_ref, mask = omx.grouped_quant(H.hp_to_f32(w.reshape(e * n, k)), aux_ps, aux_off, aux_off, sf_total_rows=e * n)
    assert mask.all()
    assert np.array_equal(q.cpu().numpy().reshape(e * n, k), q_ref)
    assert np.array_equal(sf.cpu().numpy().reshape(-1), sf_ref)
    # the grouped operator with the transposed problem list gives the same bytes
    q2 = torch.zeros((e * n, k), dtype=torch.uint8, device="cuda")
    sf2 = torch.zeros((e * n * (k // 32),), dtype=torch.uint8, device="cuda")
    ps_d = torch.tensor(aux_ps, dtype=torch.int32, device="cuda")
    off_d = torch.tensor(aux_off, dtype=torch.int32, device="cuda")
    esmoe.es_sm100_mxfp8_blockscaled_grouped_quant(wd.reshape(e * n, k), ps_d, off_d, off_d, q2, sf2)
    assert torch.equal(q2, q.reshape(e * n, k)) and torch.equal(sf2, sf.reshape(-1))
    # operator form
    q3, sf3 = esmoe.es_mxfp8_quant_weight(wd)
    assert torch.equal(q3.view(torch.uint8), q) and torch.equal(sf3, sf)
    # rows that are not a multiple of 128 are refused
    assert _native.lib.esmoe_mxfp8_quant_weight(H.ptr(wd), 0, H.ptr(q), H.ptr(sf), 100, k, H.stream_ptr()) != 0


@pytest.mark.parametrize("in_dtype", [torch.bfloat16, torch.float16])
def test_swiglu_mxfp8_grouped_quant_against_oracle(esmoe, in_dtype):
    """Fused SwiGLU + MXFP8 grouped quantisation through the C ABI against oracle swiglu() -> grouped_quant().

    Floating point with a transcendental (the device's fp32 exp is within an ulp or two of the oracle's correctly
    rounded one): a product within that distance of a rounding boundary of the input type may round the other way
    and move one quantised byte, or a block's scale when it is the block maximum at a power-of-two boundary.
    Tolerance: at most 1e-3 of the bytes and of the scale bytes differ; zero products may carry either sign."""
    from expert_specialization_moe_amd import _native
    from expert_specialization_moe_amd import workloads as W
    from oracle import fp8_blockwise as ofp8

    rows, inter = [3, 130, 0, 257, 64], 384
    total = sum(rows)
    gen = torch.Generator().manual_seed(21)
    x = (torch.randn((total, 2 * inter), generator=gen) * 2.0).to(in_dtype)
    x[0, :8] = torch.tensor([-100.0, -20.0, 0.0, 20.0, 100.0, -0.0, 1e-3, -1e-3]).to(in_dtype)
    xd = x.cuda()
    ps = [[m, 9, inter] for m in rows]
    eo = W.offsets_of(rows)
    bso_np, sf_rows = W.blockscale_offsets_of(rows)
    ps_d = torch.tensor(ps, dtype=torch.int32, device="cuda")
    eo_d = torch.tensor(eo, dtype=torch.int32, device="cuda")
    bso_d = torch.tensor(bso_np, dtype=torch.int32, device="cuda")
    q = torch.full((total, inter), 0x55, dtype=torch.uint8, device="cuda")
    sf = torch.full((sf_rows * (inter // 32),), 0xEE, dtype=torch.uint8, device="cuda")
    rc = _native.lib.esmoe_swiglu_mxfp8_grouped_quant(H.ptr(xd), 0 if in_dtype == torch.bfloat16 else 1, H.ptr(ps_d), H.ptr(eo_d),
                                                      H.ptr(bso_d), H.ptr(q), H.ptr(sf), len(rows), total, sf_rows, inter,
                                                      H.stream_ptr())
    assert rc == 0, _native.last_error()
    torch.cuda.synchronize()
    with np.errstate(over="ignore"):
        h = ofp8.swiglu(H.hp_to_f32(x), "bf16" if in_dtype == torch.bfloat16 else "fp16")
    q_ref, sf_ref, mask = omx.grouped_quant(h, ps, eo, bso_np, sf_total_rows=sf_rows)
    canon = lambda c: np.where(c == 0x80, 0, c)
    qg, sg = q.cpu().numpy(), sf.cpu().numpy()
    assert (canon(qg) != canon(q_ref)).mean() <= 1e-3, f"{(canon(qg) != canon(q_ref)).sum()} of {qg.size} bytes differ"
    assert (sg[mask] != sf_ref[mask]).mean() <= 1e-3, f"{(sg[mask] != sf_ref[mask]).sum()} of {mask.sum()} scale bytes differ"
    # the unfused sequence of this library (torch SwiGLU rounded to the input type, then the grouped quant) agrees
    hd = (torch.nn.functional.silu(xd[:, :inter].float()) * xd[:, inter:].float()).to(in_dtype)
    q_u = torch.zeros((total, inter), dtype=torch.uint8, device="cuda")
    sf_u = torch.zeros_like(sf)
    esmoe.es_sm100_mxfp8_blockscaled_grouped_quant(hd, ps_d, eo_d, bso_d, q_u, sf_u)
    assert (canon(q_u.cpu().numpy()) != canon(qg)).mean() <= 2e-2
    # operator form gives the bytes of the C ABI call
    q_o = torch.zeros_like(q)
    sf_o = torch.zeros_like(sf)
    esmoe.es_swiglu_mxfp8_grouped_quant(xd, ps_d, eo_d, bso_d, q_o, sf_o)
    assert torch.equal(q_o, q)
    assert np.array_equal(sf_o.cpu().numpy()[mask], sg[mask])


def test_reference_callers_two_byte_buffers_give_the_same_bytes(esmoe):
    """The reference's end-to-end test hands the quant operator zeros_like(bf16 input) buffers, lets it write e4m3 bytes
    into them and passes those 2-byte tensors on to the GEMM as `a` and `b`
    (test/test_es_sm100_mxfp8_blockscaled_grouped_quant.py:72-101).  Same calls, same dtypes: the bytes written and the
    GEMM result must equal those of the uint8 / float8 route."""
    from expert_specialization_moe_amd import workloads as W

    prob = W.Problem("two_byte", 256, 384, [77, 0, 200, 3, 129], kind="mxfp8")
    ops = W.make_mxfp8_operands(prob, "cuda", seed=17, weight_std=1.0)
    e, n, k, total = prob.num_experts, prob.n, prob.k, prob.total_rows
    a, w = ops["a_hp"], ops["w_hp"]
    a_quant = torch.zeros_like(a)                      # bf16 [rows, k]: twice the bytes needed
    b_quant = torch.zeros_like(w)                      # bf16 [e * n, k]
    sfa = torch.zeros_like(ops["sfa"])
    sfb = torch.zeros((e, n, k // 32), dtype=torch.uint8, device="cuda")
    esmoe.es_sm100_mxfp8_blockscaled_grouped_quant(a, ops["problem_sizes"], ops["expert_offsets"], ops["blockscale_offsets"],
                                                   a_quant, sfa)
    esmoe.es_sm100_mxfp8_blockscaled_grouped_quant(w, ops["aux_problem_sizes"], ops["aux_expert_offsets"],
                                                   ops["aux_expert_offsets"], b_quant, sfb)
    torch.cuda.synchronize()
    a_bytes = a_quant.view(torch.uint8).reshape(-1)[: total * k].reshape(total, k)
    b_bytes = b_quant.view(torch.uint8).reshape(-1)[: e * n * k].reshape(e, n, k)
    assert torch.equal(a_bytes, ops["a"].view(torch.uint8)) and torch.equal(b_bytes, ops["b_phys"].view(torch.uint8))
    assert torch.equal(sfa, ops["sfa"]) and torch.equal(sfb, ops["sfb_phys"])
    # the untouched second half of the 2-byte buffers stays zero
    assert not a_quant.view(torch.uint8).reshape(-1)[total * k:].any()
    want = torch.empty_like(ops["output"])
    esmoe.es_sm100_mxfp8_blockscaled_grouped_mm(want, ops["a"], ops["b"], ops["sfa"], ops["sfb"], ops["problem_sizes"],
                                                ops["expert_offsets"], ops["blockscale_offsets"])
    got = torch.full_like(want, float("nan"))
    # the reference reshapes the 2-byte weight buffer to (e, n, k) and hands over its (e, k, n) view
    esmoe.es_sm100_mxfp8_blockscaled_grouped_mm(got, a_quant, b_quant.view(e, n, k).transpose(1, 2), sfa,
                                                sfb.view(e, n, k // 32).transpose(1, 2), ops["problem_sizes"],
                                                ops["expert_offsets"], ops["blockscale_offsets"])
    torch.cuda.synchronize()
    assert torch.equal(got, want)


def test_grouped_quant_through_the_c_abi(esmoe):
    """esmoe_mxfp8_grouped_quant called through ctypes (the other quant tests go through the torch operator)."""
    from expert_specialization_moe_amd import _native
    from expert_specialization_moe_amd import workloads as W

    rows, k = [5, 0, 200, 128, 1], 256
    total = sum(rows)
    x = torch.randn((total, k), generator=torch.Generator().manual_seed(4)).to(torch.float16)
    xd = x.cuda()
    ps = [[m, 11, k] for m in rows]
    bso_np, sf_rows = W.blockscale_offsets_of(rows)
    ps_d = torch.tensor(ps, dtype=torch.int32, device="cuda")
    eo_d = torch.tensor(W.offsets_of(rows), dtype=torch.int32, device="cuda")
    bso_d = torch.tensor(bso_np, dtype=torch.int32, device="cuda")
    q = torch.full((total, k), 0x55, dtype=torch.uint8, device="cuda")
    sf = torch.full((sf_rows * (k // 32),), 0xEE, dtype=torch.uint8, device="cuda")
    rc = _native.lib.esmoe_mxfp8_grouped_quant(H.ptr(xd), 1, H.ptr(ps_d), H.ptr(eo_d), H.ptr(bso_d), H.ptr(q), H.ptr(sf), len(rows),
                                               total, sf_rows, k, H.stream_ptr())
    assert rc == 0, _native.last_error()
    torch.cuda.synchronize()
    q_ref, sf_ref, mask = omx.grouped_quant(H.hp_to_f32(x), ps, W.offsets_of(rows), bso_np, sf_total_rows=sf_rows)
    assert np.array_equal(q.cpu().numpy(), q_ref)
    assert np.array_equal(sf.cpu().numpy()[mask], sf_ref[mask])
