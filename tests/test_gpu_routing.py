"""GPU parity of the routing metadata builder and the row packer: integers bit-exact against the oracle,
through the C ABI; then the whole caller-side chain on the device feeding the FP8 grouped GEMM."""
import ctypes

import numpy as np
import pytest
import torch

from oracle import fp8_blockwise as ofp8
from oracle import routing as oroute
from tests import helpers as H

pytestmark = pytest.mark.gpu


def _capi_route(native, ids, first, experts, n, k):
    lib = native.lib
    pairs = ids.size
    d_ids = torch.from_numpy(ids.reshape(-1)).cuda()
    ps = torch.full((experts, 3), -7, dtype=torch.int32, device="cuda")
    eo = torch.full((experts + 1,), -7, dtype=torch.int32, device="cuda")
    bso = torch.full((experts + 1,), -7, dtype=torch.int32, device="cuda")
    dst = torch.full((max(pairs, 1),), -7, dtype=torch.int32, device="cuda")
    wsb = lib.esmoe_route_workspace_bytes(pairs, experts)
    ws = torch.empty((wsb,), dtype=torch.uint8, device="cuda")
    rc = lib.esmoe_route_metadata(H.ptr(d_ids) if pairs else None, pairs, first, experts, n, k, H.ptr(ps), H.ptr(eo), H.ptr(bso),
                                  H.ptr(dst) if pairs else None, H.ptr(ws), wsb, H.stream_ptr())
    assert rc == 0, native.last_error()
    torch.cuda.synchronize()
    return ps.cpu().numpy(), eo.cpu().numpy(), bso.cpu().numpy(), dst.cpu().numpy()[:pairs]


@pytest.mark.parametrize("seed,pairs,experts,first,span", [(0, 0, 4, 0, 4), (1, 1, 1, 0, 1), (2, 777, 8, 16, 40), (3, 1024, 32, 0, 32),
                                                            (4, 1025, 32, 0, 256), (5, 32768, 32, 64, 256),
                                                            (6, 131072, 128, 0, 128), (7, 5000, 1024, 0, 1024),
                                                            (8, 4096, 3, 5, 6), (9, 16384, 256, 0, 300), (10, 16385, 256, 0, 300),
                                                            (11, 6579, 32, 0, 256), (12, 16384, 257, 0, 257)])
def test_route_metadata_bit_exact(esmoe, seed, pairs, experts, first, span):
    from expert_specialization_moe_amd import _native

    rng = np.random.default_rng(seed)
    ids = rng.integers(0, span, size=pairs).astype(np.int32)
    if pairs > 100:
        ids[:70] = first            # a long run of one expert inside one wavefront step
    got = _capi_route(_native, ids, first, experts, 4096, 7168)
    ref = oroute.route_metadata(ids, first, experts, 4096, 7168)
    for name, g, r in zip(("problem_sizes", "expert_offsets", "blockscale_offsets", "dst_row"), got, ref):
        assert np.array_equal(g, r), name


def test_route_rejects(esmoe):
    from expert_specialization_moe_amd import _native

    p = ctypes.c_void_p(256)
    lib = _native.lib
    assert lib.esmoe_route_metadata(p, 10, 0, 0, 1, 1, p, p, p, p, p, 1 << 20, None) == -1
    assert lib.esmoe_route_metadata(p, 10, 0, 4, 1, 1, p, p, p, p, p, 4, None) == -2
    assert lib.esmoe_permute_rows(p, p, 4, 1, 24, p, None) == -1


@pytest.mark.parametrize("topk,row_elems", [(8, 4096 + 8), (2, 7168), (64, 128), (65, 64), (1, 4104)])
def test_permute_rows_of_topk_pairs(esmoe, topk, row_elems):
    """Row packing for top-k routing (a token's row goes to each of its local pairs' rows, remote pairs skipped),
    rows longer than one 4 KB pass and not a multiple of it; bit-exact against the oracle."""
    tokens, experts = 77, 96
    rng = np.random.default_rng(topk)
    ids = np.stack([rng.permutation(128)[:topk] for _ in range(tokens)]).astype(np.int32)   # experts 96..127 are remote
    x = torch.randn((tokens, row_elems), generator=torch.Generator().manual_seed(topk)).to(torch.bfloat16)
    ps, eo, bso, dst = esmoe.es_route_metadata(torch.from_numpy(ids).cuda(), 0, experts, 256, 128)
    total = int(eo[-1].item())
    packed = torch.full((total, row_elems), float("nan"), dtype=torch.bfloat16, device="cuda")
    esmoe.es_permute_rows(x.cuda(), dst, topk, packed)
    torch.cuda.synchronize()
    ps_r, eo_r, bso_r, dst_r = oroute.route_metadata(ids, 0, experts, 256, 128)
    assert np.array_equal(dst.cpu().numpy(), dst_r)
    assert np.array_equal(H.hp_to_f32(packed.cpu()), oroute.permute_rows(H.hp_to_f32(x), dst_r, topk, total))


def test_routed_fp8_layer_on_device(esmoe):
    """ids -> metadata -> packed rows -> 1x128 quant -> grouped GEMM, all on the device, against the oracle chain."""
    from expert_specialization_moe_amd import workloads as W

    tokens, topk, experts, n, k = 300, 4, 8, 256, 512
    rng = np.random.default_rng(17)
    ids = np.stack([rng.permutation(12)[:topk] for _ in range(tokens)]).astype(np.int32)   # experts 8..11 are remote
    gen = torch.Generator().manual_seed(17)
    x = torch.randn((tokens, k), generator=gen).to(torch.bfloat16)
    w = (torch.randn((experts, n, k), generator=gen) * 0.05).to(torch.bfloat16)
    d_ids = torch.from_numpy(ids).cuda()
    ps, eo, bso, dst = esmoe.es_route_metadata(d_ids, 0, experts, n, k)
    total = int(eo[-1].item())
    packed = torch.full((total, k), float("nan"), dtype=torch.bfloat16, device="cuda")
    esmoe.es_permute_rows(x.cuda(), dst, topk, packed)
    qa, sa = esmoe.es_fp8_quant_act_1x128(packed)
    qw, sw = esmoe.es_fp8_quant_weight_128x128(w.cuda())
    out = torch.full((total, n), float("nan"), dtype=torch.bfloat16, device="cuda")
    stride = torch.full((experts,), k, dtype=torch.int64, device="cuda")
    stride_d = torch.full((experts,), n, dtype=torch.int64, device="cuda")
    esmoe.es_fp8_blockwise_scaled_grouped_mm(out, qa, qw.transpose(1, 2), sa, sw.transpose(1, 2), stride, stride, stride_d,
                                             ps, eo[:experts].contiguous(), torch.empty((0,), dtype=torch.uint8, device="cuda"))
    torch.cuda.synchronize()
    # oracle chain on the host
    ps_r, eo_r, bso_r, dst_r = oroute.route_metadata(ids, 0, experts, n, k)
    assert np.array_equal(ps.cpu().numpy(), ps_r) and np.array_equal(dst.cpu().numpy(), dst_r)
    assert np.array_equal(bso.cpu().numpy(), bso_r)
    packed_r = oroute.permute_rows(H.hp_to_f32(x), dst_r, topk, total)
    assert np.array_equal(H.hp_to_f32(packed.cpu()), packed_r)
    qa_r, sa_r = ofp8.quant_act_1x128(packed_r, scale_via_reciprocal=True)
    assert np.array_equal(qa.view(torch.uint8).cpu().numpy(), qa_r)
    qw_r = np.stack([ofp8.quant_weight_128x128(H.hp_to_f32(w[e]), scale_via_reciprocal=True)[0] for e in range(experts)])
    sw_r = np.stack([ofp8.quant_weight_128x128(H.hp_to_f32(w[e]), scale_via_reciprocal=True)[1] for e in range(experts)])
    ref = ofp8.grouped_mm(qa_r, qw_r, sa_r, sw_r, ps_r, eo_r[:experts])
    rows = [int(v) for v in ps_r[:, 0]]
    H.check_grouped(H.f32(out), ref, rows, [int(v) for v in eo_r[:experts]], "routed layer")
