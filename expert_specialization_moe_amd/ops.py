"""Python entry points with the reference's names and positional orders
(expert_specialization/ops.py:4-50).  Each forwards to the operator registered
under ``torch.ops.expert_specialization`` and returns None; results are written
into the caller's output tensor.
"""
import torch

_ns = torch.ops.expert_specialization


def es_fp8_blockwise_scaled_grouped_mm(output, a, b, scales_a, scales_b, stride_a, stride_b, stride_d,
                                       problem_sizes, expert_offsets, workspace):
    """output[off_e:off_e+M_e] = (scales_a * a)[rows of e] @ (scales_b * b)[e]  (ops.py:4-29)."""
    _ns.es_fp8_blockwise_scaled_grouped_mm.default(
        output, a, b, scales_a, scales_b, stride_a, stride_b, stride_d, problem_sizes, expert_offsets, workspace)


def es_sm100_mxfp8_blockscaled_grouped_mm(output, a, b, sfa, sfb, problem_sizes, expert_offsets, blockscale_offsets):
    """MXFP8 grouped GEMM; note the operator takes ``output`` fifth (ops.py:32-37)."""
    _ns.es_sm100_mxfp8_blockscaled_grouped_mm.default(
        a, b, sfa, sfb, output, problem_sizes, expert_offsets, blockscale_offsets)


def es_sm100_mxfp8_blockscaled_grouped_quant(input, problem_sizes, expert_offsets, blockscale_offsets,
                                             quant_output, scale_factor):
    """bf16/fp16 rows -> e4m3 bytes + swizzled E8M0 scales (ops.py:40-50)."""
    _ns.es_sm100_mxfp8_blockscaled_grouped_quant.default(
        input, problem_sizes, expert_offsets, blockscale_offsets, quant_output, scale_factor)


def es_fp8_quant_act_1x128(input, quant_output=None, scales=None):
    """bf16/fp16 [M, K] -> (e4m3fn [M, K], fp32 scales [M, K/128]) on the device.

    No counterpart among the reference's operators: it is the torch helper its callers use to
    prepare ``a`` / ``scales_a`` (per_token_cast_to_fp8, test/test_es_grouped_gemm.py:36-44),
    reproduced bit for bit by a HIP kernel.  Allocates the outputs when they are not given.
    """
    m, k = input.shape
    if quant_output is None:
        quant_output = torch.empty((m, k), dtype=torch.float8_e4m3fn, device=input.device)
    if scales is None:
        scales = torch.empty((m, k // 128), dtype=torch.float32, device=input.device)
    _ns.es_fp8_quant_act_1x128.default(input, quant_output, scales)
    return quant_output, scales


def es_fp8_quant_weight_128x128(input, quant_output=None, scales=None):
    """bf16/fp16 [..., N, K] -> (e4m3fn [..., N, K], fp32 scales [..., N/128, K/128]) on the device.

    The weight-side torch helper of the reference's callers (per_block_cast_to_fp8,
    test/test_es_grouped_gemm.py:47-59) on the physical weight layout, bit for bit.
    """
    lead, n, k = input.shape[:-2], input.shape[-2], input.shape[-1]
    if quant_output is None:
        quant_output = torch.empty(input.shape, dtype=torch.float8_e4m3fn, device=input.device)
    if scales is None:
        scales = torch.empty((*lead, n // 128, k // 128), dtype=torch.float32, device=input.device)
    _ns.es_fp8_quant_weight_128x128.default(input, quant_output, scales)
    return quant_output, scales


def es_route_metadata(topk_ids, first_expert, num_experts, n, k):
    """int32 top-k expert ids [T, topk] -> (problem_sizes [E,3], expert_offsets [E+1], blockscale_offsets [E+1],
    dst_row [T*topk]) on the device, never touching the host.

    The reference's callers compute these with Python loops on the host
    (benchmark/benchmark_es_fp8_blockwise_moe.py:44-56,72-88).  Pass ``expert_offsets[:E]`` and
    ``blockscale_offsets[:E]`` to the grouped operators; the last entries are the packed row totals.
    """
    return _ns.es_route_metadata.default(topk_ids.reshape(-1), first_expert, num_experts, n, k)


def es_permute_rows(input, dst_row, topk, output):
    """output[dst_row[p]] = input[p // topk] for every pair with dst_row[p] >= 0 (rows packed by expert)."""
    _ns.es_permute_rows.default(input, dst_row, topk, output)


def es_swiglu_quant_1x128(input, quant_output=None, scales=None):
    """bf16/fp16 gate_up output [M, 2*I] -> (e4m3fn [M, I], fp32 scales [M, I/128]) of silu(gate) * up:
    the down projection's ``a`` / ``scales_a`` in one pass (no counterpart in the reference)."""
    m, two_i = input.shape
    inter = two_i // 2
    if quant_output is None:
        quant_output = torch.empty((m, inter), dtype=torch.float8_e4m3fn, device=input.device)
    if scales is None:
        scales = torch.empty((m, inter // 128), dtype=torch.float32, device=input.device)
    _ns.es_swiglu_quant_1x128.default(input, quant_output, scales)
    return quant_output, scales


def es_swiglu_mxfp8_grouped_quant(input, problem_sizes, expert_offsets, blockscale_offsets, quant_output, scale_factor):
    """bf16/fp16 gate_up output [M, 2*I] -> MXFP8 operands of the down projection (e4m3 [M, I] + swizzled E8M0
    scales) of silu(gate) * up in one pass; metadata and layouts as es_sm100_mxfp8_blockscaled_grouped_quant with
    K = I (no counterpart in the reference)."""
    _ns.es_swiglu_mxfp8_grouped_quant.default(input, problem_sizes, expert_offsets, blockscale_offsets, quant_output,
                                              scale_factor)


def es_mxfp8_quant_weight(input, quant_output=None, scale_factor=None):
    """bf16/fp16 weights [..., N, K] -> (e4m3fn [..., N, K], uint8 swizzled E8M0 scales [..., N, K/32]) in the
    layout es_sm100_mxfp8_blockscaled_grouped_mm reads as ``sfb``.  Same bytes as the reference's way of
    quantising weights (the activation operator with the transposed problem list [N, M, K] and offsets e*N,
    test/test_es_sm100_mxfp8_blockscaled_grouped_quant.py:53,87-96), without the metadata tensors."""
    if quant_output is None:
        quant_output = torch.empty(input.shape, dtype=torch.float8_e4m3fn, device=input.device)
    if scale_factor is None:
        scale_factor = torch.empty((*input.shape[:-1], input.shape[-1] // 32), dtype=torch.uint8, device=input.device)
    _ns.es_mxfp8_quant_weight.default(input, quant_output, scale_factor)
    return quant_output, scale_factor


def es_fp8_blockwise_scaled_grouped_mm_swiglu_quant(quant_output, scales_out, a, b, scales_a, scales_b, problem_sizes,
                                                    expert_offsets, workspace, mid_dtype=torch.bfloat16):
    """gate_up projection + SwiGLU + 1x128 re-quantisation in one kernel: writes the down projection's ``a``
    (e4m3fn [M, I]) and ``scales_a`` (fp32 [M, I/128]) where ``b`` is the (E, K, 2I) view of gate_up weights
    [E, 2I, K] (gate rows first).  Same bytes as es_fp8_blockwise_scaled_grouped_mm (output of ``mid_dtype``)
    followed by es_swiglu_quant_1x128; no counterpart in the reference."""
    _ns.es_fp8_blockwise_scaled_grouped_mm_swiglu_quant.default(quant_output, scales_out, a, b, scales_a, scales_b,
                                                                problem_sizes, expert_offsets, workspace,
                                                                mid_dtype == torch.bfloat16)


def es_mxfp8_blockscaled_grouped_mm_swiglu_quant(quant_output, scale_factor, a, b, sfa, sfb, problem_sizes, expert_offsets,
                                                 blockscale_offsets, mid_dtype=torch.bfloat16):
    """gate_up projection + SwiGLU + 1x32 E8M0 re-quantisation in one kernel: writes the down projection's ``a``
    (e4m3 bytes [M, I]) and ``sfa`` (swizzled scale tiles for K = I, in the layout of
    es_sm100_mxfp8_blockscaled_grouped_quant) where ``b`` is the (E, K, 2I) view of gate_up weights [E, 2I, K]
    (gate rows first).  Same bytes as es_sm100_mxfp8_blockscaled_grouped_mm (output of ``mid_dtype``) followed by
    es_swiglu_mxfp8_grouped_quant; no counterpart in the reference."""
    _ns.es_mxfp8_blockscaled_grouped_mm_swiglu_quant.default(quant_output, scale_factor, a, b, sfa, sfb, problem_sizes,
                                                             expert_offsets, blockscale_offsets,
                                                             mid_dtype == torch.bfloat16)
