"""Golden fixtures: the oracle reproduces them (CPU) and the HIP path matches them (GPU)."""
import os

import numpy as np
import pytest
import torch

from oracle import fp8, mxfp8
from oracle import fp8_blockwise as ofp8
from tests import helpers as H

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def test_oracle_reproduces_c0_fixture():
    g = np.load(os.path.join(GOLD, "c0_fp8_blockwise.npz"))
    out = ofp8.grouped_mm(g["a"], g["b"], g["scales_a"], g["scales_b"], g["problem_sizes"], g["expert_offsets"])
    assert np.array_equal(fp8.bf16_bits(out), g["out_bf16_bits"])


def test_oracle_reproduces_quant_and_layout_fixtures():
    g = np.load(os.path.join(GOLD, "mx_quant_small.npz"))
    x = fp8.bf16_from_bits(g["x_bf16_bits"])
    q, sf, mask = mxfp8.grouped_quant(x, g["problem_sizes"], g["expert_offsets"], g["blockscale_offsets"],
                                      sf_total_rows=g["sf"].size // (x.shape[1] // 32))
    assert np.array_equal(q, g["q"]) and np.array_equal(sf, g["sf"]) and np.array_equal(mask, g["sf_mask"])
    t = np.load(os.path.join(GOLD, "sf_swizzle_table.npz"))
    for name in t.files:
        m, k = (int(v[1:]) for v in name.split("_"))
        rr, cc = np.meshgrid(np.arange(m), np.arange(k // 32), indexing="ij")
        assert np.array_equal(mxfp8.sf_offset(rr, cc, k), t[name])


@pytest.mark.gpu
def test_gpu_matches_c0_fixture(esmoe):
    g = np.load(os.path.join(GOLD, "c0_fp8_blockwise.npz"))
    dev = "cuda"
    e, n, k = g["b"].shape
    a = torch.from_numpy(g["a"]).to(dev).view(torch.float8_e4m3fn)
    b = torch.from_numpy(g["b"]).to(dev).view(torch.float8_e4m3fn)
    sa = torch.from_numpy(g["scales_a"]).to(dev)
    sb = torch.from_numpy(g["scales_b"]).to(dev)
    ps = torch.from_numpy(g["problem_sizes"]).to(dev)
    eo = torch.from_numpy(g["expert_offsets"]).to(dev)
    out = torch.full((a.size(0), n), float("nan"), dtype=torch.bfloat16, device=dev)
    stride = torch.full((e,), k, dtype=torch.int64, device=dev)
    esmoe.es_fp8_blockwise_scaled_grouped_mm(out, a, b.transpose(1, 2), sa, sb.transpose(1, 2), stride, stride,
                                             torch.full((e,), n, dtype=torch.int64, device=dev), ps, eo,
                                             torch.empty((4096,), dtype=torch.uint8, device=dev))
    torch.cuda.synchronize()
    ref = fp8.bf16_from_bits(g["out_bf16_bits"])
    rows = g["problem_sizes"][:, 0].tolist()
    H.check_grouped(H.f32(out), ref, rows, g["expert_offsets"].tolist(), "c0 golden")


@pytest.mark.gpu
def test_gpu_matches_quant_fixture_bit_exact(esmoe):
    g = np.load(os.path.join(GOLD, "mx_quant_small.npz"))
    dev = "cuda"
    x = torch.from_numpy(g["x_bf16_bits"].astype(np.int16)).view(torch.bfloat16).to(dev)
    ps = torch.from_numpy(g["problem_sizes"]).to(dev)
    eo = torch.from_numpy(g["expert_offsets"]).to(dev)
    bso = torch.from_numpy(g["blockscale_offsets"]).to(dev)
    q = torch.zeros(g["q"].shape, dtype=torch.uint8, device=dev)
    sf = torch.zeros(g["sf"].shape, dtype=torch.uint8, device=dev)
    esmoe.es_sm100_mxfp8_blockscaled_grouped_quant(x, ps, eo, bso, q, sf)
    torch.cuda.synchronize()
    assert np.array_equal(q.cpu().numpy(), g["q"])
    assert np.array_equal(sf.cpu().numpy()[g["sf_mask"]], g["sf"][g["sf_mask"]])


def test_oracle_reproduces_caller_side_fixture():
    from oracle import routing as oroute

    g = np.load(os.path.join(GOLD, "caller_side_small.npz"))
    ids, x = g["topk_ids"], fp8.bf16_from_bits(g["x_bf16_bits"])
    ps, eo, bso, dst = oroute.route_metadata(ids, 0, 6, 128, x.shape[1])
    assert np.array_equal(ps, g["problem_sizes"]) and np.array_equal(eo, g["expert_offsets"])
    assert np.array_equal(bso, g["blockscale_offsets"]) and np.array_equal(dst, g["dst_row"])
    packed = oroute.permute_rows(x, dst, ids.shape[1], int(eo[-1]))
    assert np.array_equal(fp8.bf16_bits(packed), g["packed_bf16_bits"])
    q, sc = ofp8.quant_act_1x128(packed, scale_via_reciprocal=True)
    assert np.array_equal(q, g["q"]) and np.array_equal(sc, g["scales"])
    wq, wsc = ofp8.quant_weight_128x128(fp8.bf16_from_bits(g["w_bf16_bits"]), scale_via_reciprocal=True)
    assert np.array_equal(wq, g["wq"]) and np.array_equal(wsc, g["wscales"])


@pytest.mark.gpu
def test_gpu_matches_caller_side_fixture_bit_exact(esmoe):
    g = np.load(os.path.join(GOLD, "caller_side_small.npz"))
    ids = torch.from_numpy(g["topk_ids"]).cuda()
    x = torch.from_numpy(g["x_bf16_bits"].astype(np.int16)).view(torch.bfloat16).cuda()
    ps, eo, bso, dst = esmoe.es_route_metadata(ids, 0, 6, 128, x.shape[1])
    assert np.array_equal(ps.cpu().numpy(), g["problem_sizes"]) and np.array_equal(eo.cpu().numpy(), g["expert_offsets"])
    assert np.array_equal(bso.cpu().numpy(), g["blockscale_offsets"]) and np.array_equal(dst.cpu().numpy(), g["dst_row"])
    packed = torch.zeros((int(g["expert_offsets"][-1]), x.shape[1]), dtype=torch.bfloat16, device="cuda")
    esmoe.es_permute_rows(x, dst, ids.shape[1], packed)
    assert np.array_equal(packed.view(torch.int16).cpu().numpy().view(np.uint16), g["packed_bf16_bits"])
    q, sc = esmoe.es_fp8_quant_act_1x128(packed)
    assert np.array_equal(q.view(torch.uint8).cpu().numpy(), g["q"]) and np.array_equal(sc.cpu().numpy(), g["scales"])
    w = torch.from_numpy(g["w_bf16_bits"].astype(np.int16)).view(torch.bfloat16).cuda()
    wq, wsc = esmoe.es_fp8_quant_weight_128x128(w)
    assert np.array_equal(wq.view(torch.uint8).cpu().numpy(), g["wq"]) and np.array_equal(wsc.cpu().numpy(), g["wscales"])
