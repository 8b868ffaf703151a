"""One launch per call: the GEMM entry points called without a workspace use a workspace of the library whose hand-out
counters are zero between launches, and the GEMM kernel builds the schedule itself (no schedule kernel in front).
Same tiles, same K order: the output bits must equal those of the same call with a caller workspace (two launches)."""
import ctypes

import numpy as np
import pytest
import torch

from tests import helpers as H

pytestmark = pytest.mark.gpu


def _mm(native, ops, kind, ws, out, force_bm=0):
    lib = native.lib
    e = ops["problem_sizes"].size(0)
    total, k = ops["a"].shape
    n = ops["b_phys"].size(1)
    wp, wb = (H.ptr(ws), ws.numel()) if ws is not None else (None, 0)
    dt = 0 if out.dtype == torch.bfloat16 else 1
    if kind == "mx":
        rc = lib.esmoe_mxfp8_grouped_mm(H.ptr(out), dt, H.ptr(ops["a"]), H.ptr(ops["b_phys"]), H.ptr(ops["sfa"]), H.ptr(ops["sfb_phys"]),
                                        H.ptr(ops["problem_sizes"]), H.ptr(ops["expert_offsets"]), H.ptr(ops["blockscale_offsets"]),
                                        e, total, n, k, force_bm, wp, wb, H.stream_ptr())
    else:
        rc = lib.esmoe_fp8_blockwise_grouped_mm(H.ptr(out), dt, H.ptr(ops["a"]), H.ptr(ops["b_phys"]), H.ptr(ops["scales_a"]),
                                                H.ptr(ops["scales_b_phys"]), H.ptr(ops["problem_sizes"]), H.ptr(ops["expert_offsets"]),
                                                e, total, n, k, force_bm, wp, wb, H.stream_ptr())
    assert rc == 0, (rc, native.last_error())
    torch.cuda.synchronize()
    return out


def _read_stream_workspace(native, words):
    """The library's workspace of the current stream, copied to the host."""
    p, nbytes = ctypes.c_void_p(), ctypes.c_size_t()
    rc = native.lib.esmoe_stream_workspace(H.stream_ptr(), ctypes.byref(p), ctypes.byref(nbytes))
    assert rc == 0, native.last_error()
    assert nbytes.value >= words * 4
    hip = ctypes.CDLL("libamdhip64.so")
    host = np.zeros(words, dtype=np.int32)
    torch.cuda.synchronize()
    rc = hip.hipMemcpy(host.ctypes.data_as(ctypes.c_void_p), p, ctypes.c_size_t(words * 4), 2)   # device to host
    assert rc == 0
    return host


def _rows(experts, seed):
    rng = np.random.default_rng(seed)
    rows = [int(v) for v in rng.integers(0, 50, size=experts)]
    rows[0], rows[experts // 2], rows[-1] = 200, 70, 0
    if experts > 3:
        rows[2] = 400
    return rows


@pytest.mark.parametrize("kind", ["fp8", "mx"])
def test_library_workspace_gives_the_bits_of_a_caller_workspace(esmoe, kind):
    """Calls in a row on one stream, problems growing and shrinking, experts from 1 to more than a workgroup has threads
    (above 512 the library falls back to the schedule kernel, on its own workspace); every forced height on one of them."""
    from expert_specialization_moe_amd import _native
    from expert_specialization_moe_amd import workloads as W

    make = W.make_mxfp8_operands if kind == "mx" else W.make_fp8_blockwise_operands
    for experts, n, k in ((37, 512, 640), (600, 256, 256), (3, 384, 384), (300, 256, 128), (1, 256, 256), (512, 128, 256), (64, 1152, 512)):
        rows = _rows(experts, experts) if experts > 1 else [333]
        prob = W.Problem("one", n, k, rows, kind="mxfp8" if kind == "mx" else "fp8_blockwise")
        ops = make(prob, "cuda", seed=experts, weight_std=0.05)
        ws = torch.randint(0, 256, (_native.lib.esmoe_gemm_workspace_bytes(experts),), dtype=torch.uint8, device="cuda")
        for force_bm in ((0, 16, 32, 64, 128, 192) if experts == 37 else (0,)):
            print(f"{kind} E={experts} n={n} k={k} force_bm={force_bm}", flush=True)
            want = _mm(_native, ops, kind, ws, torch.full_like(ops["output"], float("nan")), force_bm).clone()
            for rep in range(2):
                got = _mm(_native, ops, kind, None, torch.full_like(ops["output"], float("nan")), force_bm)
                assert torch.equal(got.view(torch.int16), want.view(torch.int16)), (experts, force_bm, rep)


@pytest.mark.parametrize("experts,force_bm,kind", [(40, 0, "fp8"), (40, 64, "fp8"), (129, 0, "mx"), (512, 0, "fp8")])
def test_records_built_by_the_gemm_kernel_equal_the_host_mirror(esmoe, experts, force_bm, kind):
    """After a one-launch call the library's workspace holds the records every workgroup wrote: they must be the host
    mirror's (which is also what the schedule kernel writes), and every counter must be back at zero."""
    from expert_specialization_moe_amd import _native
    from expert_specialization_moe_amd import workloads as W

    lib = _native.lib
    rows = _rows(experts, 7 * experts)
    n, k = 768, 256
    prob = W.Problem("rec", n, k, rows, kind="mxfp8" if kind == "mx" else "fp8_blockwise")
    ops = (W.make_mxfp8_operands if kind == "mx" else W.make_fp8_blockwise_operands)(prob, "cuda", seed=1, weight_std=0.05)
    _mm(_native, ops, kind, None, torch.full_like(ops["output"], float("nan")), force_bm)
    words = lib.esmoe_gemm_workspace_bytes(experts) // 4
    dev = _read_stream_workspace(_native, words)
    ps = np.array([[m, n, k] for m in rows], dtype=np.int32)
    host = np.zeros(words, dtype=np.int32)
    rc = lib.esmoe_host_schedule(ps.ctypes.data_as(ctypes.c_void_p), experts, n, force_bm, 1 if kind == "mx" else 0,
                                 host.ctypes.data_as(ctypes.c_void_p))
    assert rc == 0
    first_rec = 64 + 32 * 8
    assert np.array_equal(dev[first_rec:first_rec + 4 * (experts + 1)], host[first_rec:first_rec + 4 * (experts + 1)])
    counters = [16, 32] + [64 + 32 * x for x in range(8)]     # exit counter, light counter, the eight XCD queues
    assert not dev[counters].any(), dev[counters]


def test_two_streams_use_two_library_workspaces(esmoe):
    """Calls in flight on two streams at once, each without a workspace: every stream has its own."""
    from expert_specialization_moe_amd import _native
    from expert_specialization_moe_amd import workloads as W

    probs = [W.Problem("s0", 512, 1024, [300, 0, 17, 700, 64, 5]), W.Problem("s1", 384, 768, [40, 129, 0, 260, 33])]
    opss = [W.make_fp8_blockwise_operands(p, "cuda", seed=50 + i) for i, p in enumerate(probs)]
    wants = [H.capi_fp8_mm(_native, ops, out=torch.full_like(ops["output"], float("nan"))).clone() for ops in opss]
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    ptrs = []
    for st in streams:
        with torch.cuda.stream(st):
            p, nb = ctypes.c_void_p(), ctypes.c_size_t()
            assert _native.lib.esmoe_stream_workspace(H.stream_ptr(), ctypes.byref(p), ctypes.byref(nb)) == 0
            ptrs.append(p.value)
    assert ptrs[0] != ptrs[1]
    outs = [torch.empty_like(ops["output"]) for ops in opss]
    for rep in range(4):
        for o in outs:
            o.fill_(float("nan"))
        torch.cuda.synchronize()
        for ops, st, o in zip(opss, streams, outs):
            with torch.cuda.stream(st):
                for _ in range(3):
                    esmoe.es_fp8_blockwise_scaled_grouped_mm(
                        o, ops["a"], ops["b"], ops["scales_a"], ops["scales_b"], ops["stride_a"], ops["stride_b"],
                        ops["stride_d"], ops["problem_sizes"], ops["expert_offsets"], ops["workspace"])
        torch.cuda.synchronize()
        for o, want in zip(outs, wants):
            assert torch.equal(o.view(torch.int16), want.view(torch.int16)), rep
