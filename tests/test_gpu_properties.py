"""GPU checks that do not need the oracle at full size: exact special cases, untouched rows,
size-independent properties at the benchmark configurations' real shapes."""
import numpy as np
import pytest
import torch

from oracle import fp8
from oracle import fp8_blockwise as ofp8
from tests import helpers as H

pytestmark = pytest.mark.gpu


def _int_operands(rows, n, k, seed, dev="cuda"):
    """Small-integer fp8 operands with unit scales: the GEMM result is an exact integer matmul."""
    from expert_specialization_moe_amd import workloads as W

    rng = np.random.default_rng(seed)
    e, total = len(rows), sum(rows)
    ai = rng.integers(-3, 4, size=(total, k)).astype(np.float32)
    bi = rng.integers(-3, 4, size=(e, n, k)).astype(np.float32)
    ops = {
        "a": torch.from_numpy(fp8.e4m3fn_encode_rne(ai)).to(dev).view(torch.float8_e4m3fn),
        "b_phys": torch.from_numpy(fp8.e4m3fn_encode_rne(bi)).to(dev).view(torch.float8_e4m3fn),
        "scales_a": torch.ones((total, k // 128), device=dev),
        "scales_b_phys": torch.ones((e, n // 128, k // 128), device=dev),
        "problem_sizes": torch.tensor([[m, n, k] for m in rows], dtype=torch.int32, device=dev),
        "expert_offsets": torch.tensor(W.offsets_of(rows), dtype=torch.int32, device=dev),
        "output": torch.full((total, n), float("nan"), dtype=torch.bfloat16, device=dev),
    }
    return ops, ai, bi


@pytest.mark.parametrize("force_bm", [0, 16, 128, 192])
def test_exact_integer_gemm(esmoe, force_bm):
    from expert_specialization_moe_amd import _native
    from expert_specialization_moe_amd import workloads as W

    rows, n, k = [40, 0, 3, 200], 256, 256   # |sum| <= 9 * 256 = 2304: not all bf16-exact, so compare after rounding
    ops, ai, bi = _int_operands(rows, n, k, seed=11)
    y = H.f32(H.capi_fp8_mm(_native, ops, force_bm=force_bm))
    for e, (m, off) in enumerate(zip(rows, W.offsets_of(rows))):
        if m:
            exact = ai[off:off + m] @ bi[e].T
            assert np.array_equal(y[off:off + m], fp8.bf16_round(exact.astype(np.float32))), f"expert {e}"


def test_rows_of_no_expert_are_not_written(esmoe):
    from expert_specialization_moe_amd import _native

    rows, n, k = [5, 0, 17], 128, 128
    ops, _, _ = _int_operands(rows, n, k, seed=12)
    # 7 spare rows after the last expert in the same buffers
    spare = 7
    big_out = torch.full((sum(rows) + spare, n), float("nan"), dtype=torch.bfloat16, device="cuda")
    ops["a"] = torch.cat([ops["a"].view(torch.uint8), torch.zeros((spare, k), dtype=torch.uint8, device="cuda")]).view(torch.float8_e4m3fn)
    ops["scales_a"] = torch.cat([ops["scales_a"], torch.ones((spare, k // 128), device="cuda")])
    y = H.capi_fp8_mm(_native, ops, out=big_out)
    assert torch.isnan(y[-spare:]).all() and not torch.isnan(y[:-spare]).any()


def test_power_of_two_scale_shift_and_expert_permutation(esmoe):
    from expert_specialization_moe_amd import _native
    from expert_specialization_moe_amd import workloads as W

    prob = W.Problem("p", 256, 384, [70, 9, 131])
    ops = W.make_fp8_blockwise_operands(prob, "cuda", seed=13)
    y1 = H.capi_fp8_mm(_native, ops).clone()
    ops2 = dict(ops, scales_a=ops["scales_a"] * 4.0, output=torch.empty_like(ops["output"]))
    y2 = H.capi_fp8_mm(_native, ops2)
    assert torch.equal(y2.float(), y1.float() * 4.0)
    # experts listed in another order (same rows, same weights): identical bits per expert
    perm = [2, 0, 1]
    offs = W.offsets_of(prob.rows)
    ops3 = dict(ops, b_phys=ops["b_phys"][perm].contiguous(), scales_b_phys=ops["scales_b_phys"][perm].contiguous(),
                problem_sizes=ops["problem_sizes"][perm].contiguous(),
                expert_offsets=torch.tensor([offs[i] for i in perm], dtype=torch.int32, device="cuda"),
                output=torch.empty_like(ops["output"]))
    y3 = H.capi_fp8_mm(_native, ops3)
    assert torch.equal(y3, y1)


@pytest.mark.parametrize("cfg", ["c1", "c2"] + [f"c3:{t}:{r}" for t in (64, 512, 2048, 8192, 16384) for r in ("zipf", "uniform")])
def test_benchmark_shapes_sampled_against_oracle(esmoe, cfg):
    """Real shapes of the benchmark configurations; the oracle checks a sample of experts and columns."""
    from expert_specialization_moe_amd import workloads as W

    if cfg.startswith("c3"):
        _, tokens, routing = cfg.split(":")
        prob = W.config_problem("c3", seed=0, tokens=int(tokens), routing=routing)
    else:
        prob = W.config_problem(cfg, seed=0)
    ops = W.make_fp8_blockwise_operands(prob, "cuda", seed=0)
    ops["output"].fill_(float("nan"))
    esmoe.es_fp8_blockwise_scaled_grouped_mm(ops["output"], ops["a"], ops["b"], ops["scales_a"], ops["scales_b"],
                                             ops["stride_a"], ops["stride_b"], ops["stride_d"], ops["problem_sizes"],
                                             ops["expert_offsets"], ops["workspace"])
    torch.cuda.synchronize()
    out = ops["output"]
    assert not torch.isnan(out).any()
    offs = W.offsets_of(prob.rows)
    order = np.argsort(prob.rows)
    picks = [int(order[-1]), int(order[len(order) // 2]), int(next(i for i in order if prob.rows[i] > 0))]
    for e in picks:
        m, off = prob.rows[e], int(offs[e])
        m_s = min(m, 300)                      # first rows and last rows of the expert
        rows_idx = np.unique(np.concatenate([np.arange(min(m_s, m)), np.arange(max(0, m - 40), m)]))
        cols = slice(prob.n - 384, prob.n)     # last three 128-column blocks
        a = H.codes(ops["a"][off:off + m])[rows_idx]
        sa = H.f32(ops["scales_a"][off:off + m])[rows_idx]
        b = H.codes(ops["b_phys"][e, cols])[None]
        sb = H.f32(ops["scales_b_phys"][e, (prob.n - 384) // 128:])[None]
        ref = ofp8.grouped_mm(a, b, sa, sb, [[len(rows_idx), 384, prob.k]], [0])
        y = H.f32(out[off:off + m, cols])[rows_idx]
        H.check_close(y, ref, f"{cfg} expert {e}")


def test_c4_shape_quant_bit_exact_and_gemm_sampled_against_oracle(esmoe):
    """MXFP8 benchmark configuration at its real size: stage 1 (grouped quantisation of activations, and of the weights
    through the transposed problem list) bit-exact and stage 2 (block-scaled GEMM) within tolerance, on a sample of
    experts, rows and columns that the oracle finishes in seconds."""
    from expert_specialization_moe_amd import workloads as W
    from oracle import mxfp8 as omx

    prob = W.config_problem("c4", seed=0)
    ops = W.make_mxfp8_operands(prob, "cuda", seed=0)
    ops["output"].fill_(float("nan"))
    esmoe.es_sm100_mxfp8_blockscaled_grouped_mm(ops["output"], ops["a"], ops["b"], ops["sfa"], ops["sfb"],
                                                ops["problem_sizes"], ops["expert_offsets"], ops["blockscale_offsets"])
    torch.cuda.synchronize()
    out = ops["output"]
    assert not torch.isnan(out).any()
    n, k, kc = prob.n, prob.k, prob.k // 32
    offs = W.offsets_of(prob.rows)
    bso = ops["blockscale_offsets"].cpu().numpy()
    sfa_flat = ops["sfa"].cpu().numpy().reshape(-1)
    order = np.argsort(prob.rows)
    for e in [int(order[-1]), int(order[len(order) // 2]), int(order[0])]:
        m, off = prob.rows[e], int(offs[e])
        rows_idx = np.unique(np.concatenate([np.arange(min(200, m)), np.arange(max(0, m - 40), m)]))
        cols = slice(n - 384, n)
        # stage 1, activations: bytes and scale codes of the sampled rows
        x = H.hp_to_f32(ops["a_hp"][off:off + m].cpu())[rows_idx]
        q_ref, sc_ref = omx.quant_rows(x)
        a_codes = H.codes(ops["a"][off:off + m])[rows_idx]
        sa = omx.unswizzle_scales(sfa_flat, m, k, base=int(bso[e]) * kc)[rows_idx]
        assert np.array_equal(a_codes, q_ref) and np.array_equal(sa, sc_ref), f"c4 activation quant, expert {e}"
        # stage 1, weights: the last 384 weight rows of the expert
        w = H.hp_to_f32(ops["w_hp"][e * n + n - 384:(e + 1) * n].cpu())
        wq_ref, wsc_ref = omx.quant_rows(w)
        b_codes = H.codes(ops["b_phys"][e, cols])
        sb = omx.unswizzle_scales(ops["sfb_phys"][e].cpu().numpy().reshape(-1), n, k)[cols]
        assert np.array_equal(b_codes, wq_ref) and np.array_equal(sb, wsc_ref), f"c4 weight quant, expert {e}"
        # stage 2
        ref = omx.dequant_rows(a_codes, sa) @ omx.dequant_rows(b_codes, sb).T
        ref = torch.from_numpy(ref).to(torch.bfloat16).to(torch.float32).numpy()
        y = H.f32(out[off:off + m, cols])[rows_idx]
        H.check_close(y, ref, f"c4 expert {e}")


def test_reference_style_diff_against_unquantised_product(esmoe):
    """The reference's own acceptance test: calc_diff(actual, a @ b) < 1e-3 per expert
    (test/test_es_grouped_gemm.py:195-199), both output dtypes."""
    from expert_specialization_moe_amd import quant

    for out_dtype in (torch.bfloat16, torch.half):
        gen = torch.Generator(device="cuda").manual_seed(21)
        e, n, k = 8, 384, 640
        rows = [int(v) for v in torch.randint(1, 257, (e,), generator=torch.Generator().manual_seed(3))]
        total = sum(rows)
        a = torch.randn((total, k), device="cuda", dtype=out_dtype, generator=gen)
        w = torch.randn((e, n, k), device="cuda", dtype=out_dtype, generator=gen)
        a_q, sa = quant.quant_act_1x128(a)
        b_q, sb = quant.quant_weight_128x128(w)
        offs = np.concatenate([[0], np.cumsum(rows)[:-1]])
        ps = torch.tensor([[m, n, k] for m in rows], dtype=torch.int32, device="cuda")
        eo = torch.tensor(offs, dtype=torch.int32, device="cuda")
        out = torch.empty((total, n), dtype=out_dtype, device="cuda")
        st = torch.full((e,), k, dtype=torch.int64, device="cuda")
        esmoe.es_fp8_blockwise_scaled_grouped_mm(out, a_q.contiguous(), b_q.transpose(1, 2), sa.contiguous(),
                                                 sb.transpose(1, 2), st, st,
                                                 torch.full((e,), n, dtype=torch.int64, device="cuda"), ps, eo,
                                                 torch.empty((1024,), dtype=torch.uint8, device="cuda"))
        torch.cuda.synchronize()
        for g, (m, off) in enumerate(zip(rows, offs)):
            base = (a[off:off + m].float() @ w[g].float().t()).cpu().numpy()
            assert ofp8.calc_diff(H.f32(out[off:off + m]), base) < 1e-3


def test_small_k_and_many_experts(esmoe):
    """K = 256 / 384 (fewer than 4 K blocks: per-block activation scales path) and 128 experts."""
    from expert_specialization_moe_amd import _native
    from expert_specialization_moe_amd import workloads as W
    from oracle import fp8_blockwise as o

    rng = np.random.default_rng(5)
    for k in (128, 256, 384):
        rows = [int(v) for v in rng.integers(0, 40, size=128)]
        prob = W.Problem("many", 256, k, rows)
        ops = W.make_fp8_blockwise_operands(prob, "cuda", seed=k)
        y = H.f32(H.capi_fp8_mm(_native, ops))
        ref = o.grouped_mm(H.codes(ops["a"]), H.codes(ops["b_phys"]), H.f32(ops["scales_a"]), H.f32(ops["scales_b_phys"]),
                           [[m, 256, k] for m in rows], W.offsets_of(rows))
        H.check_grouped(y, ref, rows, W.offsets_of(rows), f"k={k}")


@pytest.mark.parametrize("experts", [5, 128, 129, 300])
def test_workspace_contents_do_not_matter(esmoe, experts):
    """The schedule records and the hand-out counters live in the caller's workspace, and every call writes them anew:
    whatever the workspace holds (all ones, random bytes, what a previous call left), the result is the same."""
    from expert_specialization_moe_amd import _native
    from expert_specialization_moe_amd import workloads as W
    from oracle import fp8_blockwise as o

    rng = np.random.default_rng(experts)
    rows = [int(v) for v in rng.integers(0, 50, size=experts)]
    rows[1], rows[3] = 200, 70
    prob = W.Problem("ws", 256, 256, rows)
    ops = W.make_fp8_blockwise_operands(prob, "cuda", seed=experts)
    lib = _native.lib
    need = lib.esmoe_gemm_workspace_bytes(experts)
    ref = o.grouped_mm(H.codes(ops["a"]), H.codes(ops["b_phys"]), H.f32(ops["scales_a"]), H.f32(ops["scales_b_phys"]),
                       [[m, 256, 256] for m in rows], W.offsets_of(rows))
    gen = torch.Generator(device="cuda").manual_seed(1)
    fills = [torch.full((need,), 0xFF, dtype=torch.uint8, device="cuda"),
             torch.randint(0, 256, (need,), dtype=torch.uint8, device="cuda", generator=gen),
             torch.zeros((need,), dtype=torch.uint8, device="cuda")]
    first = None
    for ws in fills:
        for rep in range(2):    # the second call finds the counters the first one left
            out = torch.full_like(ops["output"], float("nan"))
            rc = lib.esmoe_fp8_blockwise_grouped_mm(
                H.ptr(out), 0, H.ptr(ops["a"]), H.ptr(ops["b_phys"]), H.ptr(ops["scales_a"]), H.ptr(ops["scales_b_phys"]),
                H.ptr(ops["problem_sizes"]), H.ptr(ops["expert_offsets"]), experts, prob.total_rows, 256, 256, 0, H.ptr(ws),
                need, H.stream_ptr())
            assert rc == 0, _native.last_error()
            torch.cuda.synchronize()
            if first is None:
                first = out.clone()
                H.check_grouped(H.f32(out), ref, rows, W.offsets_of(rows), f"E={experts}")
            assert torch.equal(out.view(torch.int16), first.view(torch.int16))


@pytest.mark.parametrize("kind", ["fp8_blockwise", "mxfp8"])
def test_graph_capture_replays_match_eager(esmoe, kind):
    """The operators enqueue kernels only (no memset nodes, no host reads), so a HIP graph of them can be
    replayed: every replay, with eager work and synchronisations in between, must reproduce the eager result."""
    from expert_specialization_moe_amd import workloads as W

    prob = W.Problem("graph", 384, 512, [33, 0, 200, 7, 129], kind=kind)
    make = W.make_mxfp8_operands if kind == "mxfp8" else W.make_fp8_blockwise_operands
    ops = make(prob, "cuda", seed=21)
    # a workspace large enough that the FP8 operator allocates nothing while the graph is recorded
    ops["workspace"] = torch.zeros((4096,), dtype=torch.uint8, device="cuda")

    def call(out):
        if kind == "mxfp8":
            esmoe.es_sm100_mxfp8_blockscaled_grouped_mm(out, ops["a"], ops["b"], ops["sfa"], ops["sfb"], ops["problem_sizes"],
                                                        ops["expert_offsets"], ops["blockscale_offsets"])
        else:
            esmoe.es_fp8_blockwise_scaled_grouped_mm(out, ops["a"], ops["b"], ops["scales_a"], ops["scales_b"],
                                                     ops["stride_a"], ops["stride_b"], ops["stride_d"], ops["problem_sizes"],
                                                     ops["expert_offsets"], ops["workspace"])

    eager = torch.zeros_like(ops["output"])
    call(eager)
    torch.cuda.synchronize()
    out = torch.zeros_like(ops["output"])
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        call(out)                      # warm-up on the capture stream
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        call(out)
    for rep in range(3):
        out.fill_(float("nan"))
        torch.cuda.synchronize()
        graph.replay()
        scratch = torch.randn(1024, device="cuda").sum().item()   # eager work between replays
        assert np.isfinite(scratch)
        torch.cuda.synchronize()
        assert torch.equal(out, eager), f"replay {rep} differs from the eager result"


@pytest.mark.parametrize("kind", ["fp8", "mx"])
@pytest.mark.parametrize("n", [1024, 1152])
def test_half_items_give_the_bytes_of_whole_items(esmoe, kind, n):
    """A plain launch hands its last 128 light items out as 128-column halves; a launch with a forced tile height hands out
    whole tiles only.  On experts of at most 16 rows both use 16-row tiles with the same K order, so the outputs must be
    identical bit for bit.  44 experts x 4-5 column tiles: whole items, then halves; n = 1152 ends on a 128-column tile
    whose second half is skipped."""
    from expert_specialization_moe_amd import _native
    from expert_specialization_moe_amd import workloads as W

    rows = [1 + (7 * i) % 16 for i in range(44)]
    rows[5] = 0
    prob = W.Problem("halves", n, 768, rows, kind="mxfp8" if kind == "mx" else "fp8_blockwise")
    if kind == "mx":
        ops = W.make_mxfp8_operands(prob, "cuda", seed=21, weight_std=0.05)
        mm = H.capi_mx_mm
    else:
        ops = W.make_fp8_blockwise_operands(prob, "cuda", seed=21, weight_std=0.05)
        mm = H.capi_fp8_mm
    y0 = mm(_native, ops, 0, out=torch.full_like(ops["output"], 7.0)).clone()
    y16 = mm(_native, ops, 16, out=torch.full_like(ops["output"], 7.0)).clone()
    assert torch.equal(y0.view(torch.int16), y16.view(torch.int16))
    assert not (y0 == 7.0).all(dim=1).any()      # every row of an expert was written
