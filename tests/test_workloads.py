"""Routing generators and the roofline model of the benchmark configurations (host logic)."""
import numpy as np


def test_routing_is_seeded_and_shaped(esmoe):
    from expert_specialization_moe_amd import workloads as W

    c1 = W.config_problem("c1", seed=0)
    assert c1.num_experts == 32 and c1.n == 4096 and c1.k == 7168
    assert c1.rows == W.config_problem("c1", seed=0).rows
    assert c1.total_rows == 6579 and max(c1.rows) == 3841  # the seed-0 draw documented with the configs
    c2 = W.config_problem("c2", seed=0)
    assert c2.total_rows == 256 and sorted(c2.rows, reverse=True)[:3] == [70, 39, 24]
    c4 = W.config_problem("c4", seed=0)
    assert c4.total_rows == 8192 and c4.kind == "mxfp8"
    c3 = W.config_problem("c3", seed=0, tokens=512, routing="uniform")
    assert c3.total_rows == 512 * 8 and c3.num_experts == 128


def test_roofline_model(esmoe):
    from expert_specialization_moe_amd import workloads as W

    rows, n, k = [16, 0, 100], 256, 512
    total, active = 116, 2
    assert W.gemm_flops(rows, n, k) == 2.0 * n * k * total
    expect = total * (k + 4 * k / 128) + active * (n * k + 4 * (n // 128) * (k // 128)) + 2 * n * total
    assert W.gemm_bytes(rows, n, k) == expect
    expect_mx = total * (k + k / 32) + active * (n * k + n * k / 32) + 2 * n * total
    assert W.gemm_bytes(rows, n, k, "mxfp8") == expect_mx
    c1 = W.config_problem("c1", seed=0)
    t = W.gemm_roofline_seconds(c1.rows, c1.n, c1.k)
    assert 120e-6 < t < 135e-6  # HBM bound: ~1.04 GB at 8 TB/s
    assert W.gemm_bytes(c1.rows, c1.n, c1.k) / W.HBM_BYTES_PER_S > W.gemm_flops(c1.rows, c1.n, c1.k) / W.FP8_FLOPS_PER_S


def test_operand_builder_layouts_on_cpu(esmoe):
    import torch
    from expert_specialization_moe_amd import workloads as W

    prob = W.Problem("t", 256, 384, [3, 0, 130])
    ops = W.make_fp8_blockwise_operands(prob, "cpu", seed=1)
    assert ops["b"].shape == (3, 384, 256) and ops["b"].stride() == (256 * 384, 1, 384)
    assert ops["scales_b"].shape == (3, 3, 2) and ops["scales_b"].stride(1) == 1
    assert ops["expert_offsets"].tolist() == [0, 3, 3]
    bso, total = W.blockscale_offsets_of(prob.rows)
    assert bso.tolist() == [0, 128, 128] and total == 384
