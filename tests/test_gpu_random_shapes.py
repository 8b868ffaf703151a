"""Randomised self-consistency of the grouped GEMMs on the GPU.

Every output element is accumulated K block by K block in the same order whatever the tile height, so forcing the
tile height (16 ... 192 rows) must give the bytes of the device schedule; FP8-blockwise results are also checked
against a torch fp32 product of the dequantised operands (tolerance of the path: 1e-2 of the expert's largest output),
and where the shape allows it the fused SwiGLU + quantisation entry points against projection -> stand-alone
quantiser, byte for byte.  Shapes are drawn from lists that mix empty, one-row, ragged and many-row experts, column
counts that are no multiple of 256 and K from one block to 7168.
"""
import random

import pytest
import torch

from tests import helpers as H

pytestmark = pytest.mark.gpu

ROW_POOLS = [[0, 1, 3, 7, 16, 17, 31], [0, 5, 33, 64, 65, 100, 128, 129], [0, 1, 190, 192, 193, 250, 384, 385, 500],
             [2, 40, 70, 130, 200, 333, 577, 800], [0, 0, 0, 1, 2000, 1500, 191, 383], [96, 97, 95, 48, 49, 47, 0]]


def _cases(seed, count):
    rng = random.Random(seed)
    for case in range(count):
        kind = rng.choice(["fp8", "mx"])
        e = rng.choice([1, 2, 3, 5, 8, 9, 17, 33, 40, 64])
        n = rng.choice([128, 256, 384, 512, 768, 1024, 1152, 2048])
        k = rng.choice([128, 256, 384, 512, 640, 896, 1024, 1536, 2048, 7168])
        pool = rng.choice(ROW_POOLS)
        rows = [rng.choice(pool) for _ in range(e)]
        if sum(rows) == 0:
            rows[0] = 9
        if sum(rows) * (n + k) > 40_000_000 or e * n * k > 400_000_000:
            continue   # keep the suite's memory and time small
        yield case, kind, n, k, rows, rng.choice([torch.bfloat16, torch.float16])


@pytest.mark.parametrize("seed", [5, 6])
def test_forced_heights_fused_forms_and_torch_agree(seed):
    import expert_specialization_moe_amd as es
    from expert_specialization_moe_amd import _native, workloads as W

    ran = 0
    for case, kind, n, k, rows, dt in _cases(seed, 60):
        prob = W.Problem("rand", n, k, rows, kind="mxfp8" if kind == "mx" else "fp8_blockwise")
        tag = f"seed {seed} case {case}: {kind} n={n} k={k} {dt} rows={rows}"
        print(tag, flush=True)
        if kind == "mx":
            ops = W.make_mxfp8_operands(prob, "cuda", seed=case, out_dtype=dt, weight_std=0.05)
            mm = H.capi_mx_mm
        else:
            ops = W.make_fp8_blockwise_operands(prob, "cuda", seed=case, out_dtype=dt, weight_std=0.05)
            mm = H.capi_fp8_mm
        base = mm(_native, ops, 0, out=torch.full_like(ops["output"], 3.0)).clone()
        for bm in (16, 64, 128, 192):
            forced = mm(_native, ops, bm, out=torch.full_like(ops["output"], 3.0))
            assert torch.equal(base.view(torch.int16), forced.view(torch.int16)), f"{tag}: tile height {bm}"
        if kind == "fp8":
            a = ops["a"].float() * ops["scales_a"].repeat_interleave(128, dim=1)
            sb = ops["scales_b_phys"].repeat_interleave(128, dim=1).repeat_interleave(128, dim=2)
            off = 0
            for i, m in enumerate(rows):
                if m:
                    ref = a[off:off + m] @ (ops["b_phys"][i].float() * sb[i]).t()
                    err = (base[off:off + m].float() - ref).abs().max().item() / max(ref.abs().max().item(), 1e-6)
                    assert err <= 1e-2, f"{tag}: expert {i}: {err}"
                off += m
        if n % 256 == 0:
            inter, total = n // 2, prob.total_rows
            q = torch.zeros((total, inter), dtype=torch.uint8, device="cuda")
            if kind == "fp8":
                sc = torch.zeros((total, inter // 128), dtype=torch.float32, device="cuda")
                es.es_fp8_blockwise_scaled_grouped_mm_swiglu_quant(q, sc, ops["a"], ops["b"], ops["scales_a"], ops["scales_b"],
                                                                   ops["problem_sizes"], ops["expert_offsets"], ops["workspace"], dt)
                q2, sc2 = es.es_swiglu_quant_1x128(base)
                torch.cuda.synchronize()
                assert torch.equal(q, q2.view(torch.uint8)) and torch.equal(sc, sc2), f"{tag}: fused fp8"
            else:
                sf = torch.zeros((ops["sfa"].shape[0], inter // 32), dtype=torch.uint8, device="cuda")
                es.es_mxfp8_blockscaled_grouped_mm_swiglu_quant(q, sf, ops["a"], ops["b"], ops["sfa"], ops["sfb"], ops["problem_sizes"],
                                                                ops["expert_offsets"], ops["blockscale_offsets"], dt)
                q2, sf2 = torch.zeros_like(q), torch.zeros_like(sf)
                es.es_swiglu_mxfp8_grouped_quant(base, ops["problem_sizes"], ops["expert_offsets"], ops["blockscale_offsets"], q2, sf2)
                torch.cuda.synchronize()
                assert torch.equal(q, q2) and torch.equal(sf, sf2), f"{tag}: fused mxfp8"
        ran += 1
    assert ran >= 30
