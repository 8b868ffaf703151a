"""The torch operators exist under the reference's names and reject bad arguments before any launch
(checked with CPU tensors; the reference's checks: es_fp8_blockwise.cu:47-56,
es_sm100_mxfp8_blockscaled.cu:15-25, es_sm100_mxfp8_blockscaled_group_quant.cu:13-24)."""
import pytest
import torch


def _fp8_args(e=2, rows=(3, 5), n=128, k=256):
    total = sum(rows)
    return dict(
        output=torch.empty((total, n), dtype=torch.bfloat16),
        a=torch.zeros((total, k), dtype=torch.float8_e4m3fn),
        b=torch.zeros((e, n, k), dtype=torch.float8_e4m3fn).transpose(1, 2),
        scales_a=torch.ones((total, k // 128)),
        scales_b=torch.ones((e, n // 128, k // 128)).transpose(1, 2),
        stride_a=torch.full((e,), k, dtype=torch.int64), stride_b=torch.full((e,), k, dtype=torch.int64),
        stride_d=torch.full((e,), n, dtype=torch.int64),
        problem_sizes=torch.tensor([[m, n, k] for m in rows], dtype=torch.int32),
        expert_offsets=torch.tensor([0, rows[0]], dtype=torch.int32),
        workspace=torch.empty((1024,), dtype=torch.uint8))


def test_operators_registered_with_reference_schemas(esmoe):
    ns = torch.ops.expert_specialization
    s = str(ns.es_fp8_blockwise_scaled_grouped_mm.default._schema)
    assert "Tensor output, Tensor a, Tensor b, Tensor scales_a, Tensor scales_b, Tensor stride_a" in s and "-> ()" in s
    s = str(ns.es_sm100_mxfp8_blockscaled_grouped_mm.default._schema)
    assert "Tensor a, Tensor b, Tensor sfa, Tensor sfb, Tensor d, Tensor problem_sizes" in s
    s = str(ns.es_sm100_mxfp8_blockscaled_grouped_quant.default._schema)
    assert "Tensor input, Tensor problem_sizes, Tensor expert_offsets, Tensor blockscale_offsets, Tensor quant_output" in s


def test_fp8_op_rejects_bad_arguments(esmoe):
    good = _fp8_args()
    with pytest.raises(RuntimeError, match="no CPU implementation"):
        esmoe.es_fp8_blockwise_scaled_grouped_mm(*good.values())
    bad = dict(good, problem_sizes=good["problem_sizes"].to(torch.int64))
    with pytest.raises(RuntimeError, match="problem_sizes must be int32"):
        esmoe.es_fp8_blockwise_scaled_grouped_mm(*bad.values())
    bad = dict(good, problem_sizes=good["problem_sizes"][:1])
    with pytest.raises(RuntimeError, match="must match expert_offsets"):
        esmoe.es_fp8_blockwise_scaled_grouped_mm(*bad.values())
    bad = dict(good, a=good["a"].view(torch.uint8))
    with pytest.raises(RuntimeError, match="a must be kFloat8_e4m3fn"):
        esmoe.es_fp8_blockwise_scaled_grouped_mm(*bad.values())
    bad = dict(good, output=good["output"].float())
    with pytest.raises(RuntimeError, match="output must be bfloat16 or half"):
        esmoe.es_fp8_blockwise_scaled_grouped_mm(*bad.values())
    bad = dict(good, b=good["b"].transpose(1, 2))  # row-major (E, N, K) handed over as is
    with pytest.raises(RuntimeError, match="column-major"):
        esmoe.es_fp8_blockwise_scaled_grouped_mm(*bad.values())
    bad = dict(good, problem_sizes=good["problem_sizes"].reshape(-1))
    with pytest.raises(RuntimeError, match="problem_sizes must be 2D"):
        esmoe.es_fp8_blockwise_scaled_grouped_mm(*bad.values())


def test_mx_ops_reject_bad_arguments(esmoe):
    e, n, k, rows = 2, 128, 256, (3, 5)
    total = sum(rows)
    a = torch.zeros((total, k), dtype=torch.float8_e4m3fn)
    b = torch.zeros((e, n, k), dtype=torch.float8_e4m3fn).transpose(1, 2)
    sfa = torch.zeros((256, k // 32), dtype=torch.uint8)
    sfb = torch.zeros((e, n, k // 32), dtype=torch.uint8).transpose(1, 2)
    d = torch.empty((total, n), dtype=torch.bfloat16)
    ps = torch.tensor([[m, n, k] for m in rows], dtype=torch.int32)
    eo = torch.tensor([0, 3], dtype=torch.int32)
    bso = torch.tensor([0, 128], dtype=torch.int32)
    with pytest.raises(RuntimeError, match="no CPU implementation"):
        esmoe.es_sm100_mxfp8_blockscaled_grouped_mm(d, a, b, sfa, sfb, ps, eo, bso)
    with pytest.raises(RuntimeError, match="b must be a 3D tensor"):
        esmoe.es_sm100_mxfp8_blockscaled_grouped_mm(d, a, b[0], sfa, sfb, ps, eo, bso)
    with pytest.raises(RuntimeError, match="k should align 128"):
        esmoe.es_sm100_mxfp8_blockscaled_grouped_mm(d, a[:, :192], b, sfa, sfb, ps, eo, bso)
    with pytest.raises(RuntimeError, match="dtype must be kFloat16 or kBFloat16"):
        esmoe.es_sm100_mxfp8_blockscaled_grouped_mm(d.float(), a, b, sfa, sfb, ps, eo, bso)
    x = torch.zeros((total, k), dtype=torch.bfloat16)
    q = torch.zeros((total, k), dtype=torch.uint8)
    with pytest.raises(RuntimeError, match="no CPU implementation"):
        esmoe.es_sm100_mxfp8_blockscaled_grouped_quant(x, ps, eo, bso, q, sfa)
    with pytest.raises(RuntimeError, match="k must align to 128"):
        esmoe.es_sm100_mxfp8_blockscaled_grouped_quant(x[:, :200].contiguous(), ps, eo, bso, q, sfa)
    with pytest.raises(RuntimeError, match="dtype must be kFloat16 or kBFloat16"):
        esmoe.es_sm100_mxfp8_blockscaled_grouped_quant(x.float(), ps, eo, bso, q, sfa)
    with pytest.raises(RuntimeError, match="blockscale_offsets must be 1D"):
        esmoe.es_sm100_mxfp8_blockscaled_grouped_quant(x, ps, eo, bso[:1], q, sfa)
