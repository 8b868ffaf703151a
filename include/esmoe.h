/*
 * C ABI of the MI355X (gfx950) expert-specialized grouped-GEMM library (libesmoe.so).
 *
 * Plain pointers and sizes only; every pointer is device memory unless stated.
 * All entry points enqueue work on `stream` (a hipStream_t passed as void*) and
 * return without synchronising.  Return value: 0 on success, a negative
 * ESMOE_ERR_* for rejected arguments, a positive hipError_t if a launch failed.
 * esmoe_last_error() gives a message for the calling thread's last failure.
 *
 * Per-expert metadata follows the reference operators exactly:
 *   problem_sizes     int32 [E,3] rows (M_e, N, K)      (N and K equal for all experts)
 *   expert_offsets    int32 [E]   first row of expert e in the packed [sum M, .] tensors
 *   blockscale_offsets int32 [E]  first row of expert e in the swizzled scale tensor
 *                                 (prefix sum of M_e rounded up to 128)
 * They are read on the device only; no entry point copies them to the host.
 */
#ifndef ESMOE_H_
#define ESMOE_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define ESMOE_OUT_BF16 0
#define ESMOE_OUT_FP16 1
#define ESMOE_IN_BF16 0
#define ESMOE_IN_FP16 1

#define ESMOE_ERR_INVALID_ARGUMENT (-1)
#define ESMOE_ERR_WORKSPACE_TOO_SMALL (-2)
#define ESMOE_ERR_UNSUPPORTED_DEVICE (-3)

#define ESMOE_MAX_EXPERTS 1024 /* same limit as the reference, es_fp8_blockwise_launcher.cuh:53 */

/* ABI revision of this header; esmoe_version() of a matching library reads "esmoe 0.<ESMOE_ABI> (gfx950)".
 * 3: a null `workspace` selects the library's own; esmoe_stream_workspace added; the workspace layout gained an exit
 *    counter (same size).  2: the esmoe_host_* mirrors gained `kind` after `force_bm`; esmoe_gemm_workspace_bytes
 *    grew from 16 E + 80 to 16 E + 1296 bytes and the workspace must be 16-byte aligned. */
#define ESMOE_ABI 3

/* Bytes of device scratch the GEMM entry points need for `num_experts` experts
 * (the device-built tile schedule and its hand-out counters).  The scratch must be 16-byte aligned (device allocations
 * are); its contents before a call do not matter: a one-workgroup schedule kernel in front of the GEMM kernel writes
 * every word the GEMM kernel reads.
 *
 * Every GEMM entry point below also accepts workspace == NULL with workspace_bytes == 0: the library then uses a
 * workspace of its own, one per (device, stream), whose counters it knows to be zero between launches (zeroed when
 * allocated; the last workgroup of every launch zeroes them again).  Such a call is ONE kernel launch: every workgroup
 * builds the schedule records itself (up to 512 experts; more fall back to the schedule kernel).  This replaces the
 * reference's pre-compute launch and its twelve per-call scratch tensors (es_fp8_blockwise_launcher.cuh:18-86,
 * es_fp8_blockwise.cu:58-75) by nothing.  The library's workspaces are allocated 16 at a time (hipMalloc + hipMemset):
 * by the first such call on a device, and again by the first call of a 17th, 33rd, ... distinct stream handle; those
 * calls must not happen during graph capture.  A slot stays with its stream handle until the process ends; calls on
 * one stream are ordered and safe, a graph captured on a stream keeps that stream's workspace. */
size_t esmoe_gemm_workspace_bytes(int num_experts);

/* The library's own schedule workspace of `stream` on the current device (allocated on first use, see above), for
 * tools and tests that inspect the schedule records a launch left there.  No counterpart in the reference. */
int esmoe_stream_workspace(void* stream, void** workspace, size_t* bytes);

/*
 * FP8-blockwise scaled grouped GEMM.
 * Replaces es_fp8_blockwise_scaled_grouped_mm
 *   (expert_specialization/csrc/cuda/es_fp8_blockwise.cu:34-193, schema
 *    expert_specialization/csrc/expert_specialization.cpp:57-60).
 *
 *   out[off_e + m, n] = cast( sum_kb sa[off_e + m, kb] * sb[e, n/128, kb]
 *                               * sum_{k in kb} a[off_e + m, k] * b[e, n, k] )
 *
 *   out  [total_rows, N] bf16 or fp16 (out_dtype), row-major
 *   a    [total_rows, K] e4m3fn bytes, row-major
 *   b    [E, N, K] e4m3fn bytes (the physical layout behind the reference's (E,K,N) view)
 *   sa   [total_rows, K/128] fp32;  sb [E, N/128, K/128] fp32
 * N % 128 == 0, K % 128 == 0, 1 <= E <= ESMOE_MAX_EXPERTS.
 * force_bm: 0 lets the device-side schedule pick an M-tile shape per expert;
 *           16/32/64/128/192 forces that single shape for every tile (benchmarking).
 * Rows of `out` that belong to no expert (M_e == 0) are not written.
 */
int esmoe_fp8_blockwise_grouped_mm(void* out, int out_dtype, const void* a, const void* b, const float* sa,
                                   const float* sb, const int32_t* problem_sizes, const int32_t* expert_offsets,
                                   int num_experts, int total_rows, int n, int k, int force_bm, void* workspace,
                                   size_t workspace_bytes, void* stream);

/*
 * esmoe_fp8_blockwise_grouped_mm for callers that cannot allocate device memory (code under HIP graph capture,
 * serving loops and harnesses that forbid hipMalloc): same arguments without the workspace, same kernels, same
 * results.  No counterpart in the reference, whose operator allocates its scratch tensors on every call
 * (es_fp8_blockwise.cu:58-75).  The schedule workspace is a static array inside the library, one copy per GPU,
 * ESMOE_STATIC_MAX_EXPERTS experts at most (more are rejected with ESMOE_ERR_INVALID_ARGUMENT); the call allocates
 * and frees nothing.  The array is zero when the library is loaded and every launch leaves its counters zero, so up to
 * 512 experts the call is one kernel launch.  The first call on a device looks the array's address up
 * (hipGetSymbolAddress) and reads the device's properties: make it outside graph capture.  All calls on one GPU share that array: calls that overlap in time on one GPU (two streams,
 * two threads) race on it and must be serialised by the caller; calls ordered on one stream are safe.
 */
#define ESMOE_STATIC_MAX_EXPERTS 1024
int esmoe_fp8_blockwise_grouped_mm_static(void* out, int out_dtype, const void* a, const void* b, const float* sa,
                                          const float* sb, const int32_t* problem_sizes,
                                          const int32_t* expert_offsets, int num_experts, int total_rows, int n, int k,
                                          int force_bm, void* stream);

/*
 * MXFP8 block-scaled grouped GEMM (e4m3 data, E8M0 scale per 1x32 block along K).
 * Replaces es_sm100_mxfp8_blockscaled_grouped_mm
 *   (expert_specialization/csrc/cuda/es_sm100_mxfp8_blockscaled.cu:5-40, schema
 *    expert_specialization/csrc/expert_specialization.cpp:61-63).
 *
 *   d[off_e + m, n] = cast( sum_k a[off_e+m,k] 2^(sfa-127) * b[e,n,k] 2^(sfb-127) )
 *
 *   sfa: swizzled 128x4 scale tiles, expert e at byte blockscale_offsets[e]*(K/32)
 *   sfb: swizzled 128x4 scale tiles, expert e at byte e*N*(K/32), N rows
 *   (tile layout: es_sm100_mxfp8_blockscaled_group_quant.cuh:25,294-307)
 */
int esmoe_mxfp8_grouped_mm(void* d, int out_dtype, const void* a, const void* b, const uint8_t* sfa,
                           const uint8_t* sfb, const int32_t* problem_sizes, const int32_t* expert_offsets,
                           const int32_t* blockscale_offsets, int num_experts, int total_rows, int n, int k,
                           int force_bm, void* workspace, size_t workspace_bytes, void* stream);

/*
 * FP8-blockwise grouped GEMM of a gate_up projection with the SwiGLU and the 1x128 re-quantisation fused into its
 * epilogue: produces the `a` / `scales_a` operands of the down projection directly, without the bf16 [total_rows, n]
 * intermediate.  No counterpart in the reference (its callers run projection, activation and quantisation as
 * separate steps); the arithmetic is that of esmoe_fp8_blockwise_grouped_mm followed by esmoe_swiglu_quant_1x128,
 * step for step, so the two routes give the same bytes.
 *
 *   b [E, n, K] with n = 2 * inter: weight rows [0, inter) are the gate, [inter, 2 * inter) the up projection
 *   (inter % 128 == 0); sb [E, n/128, K/128] as usual.
 *   q [total_rows, inter] e4m3fn;  scales [total_rows, inter/128] fp32.
 *   mid_dtype: ESMOE_OUT_BF16 / ESMOE_OUT_FP16, the type the projection and the activation are rounded to on the
 *   way (what `out_dtype` and the activation's input type would be on the separate route).
 * The other arguments are those of esmoe_fp8_blockwise_grouped_mm.
 */
int esmoe_fp8_blockwise_grouped_mm_swiglu_quant(void* q, float* scales, int mid_dtype, const void* a, const void* b,
                                                const float* sa, const float* sb, const int32_t* problem_sizes,
                                                const int32_t* expert_offsets, int num_experts, int total_rows, int n,
                                                int k, int force_bm, void* workspace, size_t workspace_bytes,
                                                void* stream);

/*
 * MXFP8 grouped GEMM of a gate_up projection with the SwiGLU and the 1x32 E8M0 re-quantisation fused into its
 * epilogue: produces the `a` / `sfa` operands of the down projection directly, without the bf16 [total_rows, n]
 * intermediate.  No counterpart in the reference (its callers run projection, activation and quantisation as
 * separate steps); the arithmetic is that of esmoe_mxfp8_grouped_mm followed by esmoe_swiglu_mxfp8_grouped_quant,
 * step for step, so the two routes give the same bytes.
 *
 *   b [E, n, K] with n = 2 * inter: weight rows [0, inter) are the gate, [inter, 2 * inter) the up projection
 *   (inter % 128 == 0); sfb as for esmoe_mxfp8_grouped_mm.
 *   q [total_rows, inter] e4m3 bytes;  sf: `sf_rows` rows of inter/32 scale bytes in the layout
 *   esmoe_mxfp8_grouped_quant writes for K = inter (expert e at byte blockscale_offsets[e] * inter/32, padding
 *   rows of an expert's last 128-row tile written as 0); sf_rows as there.
 *   mid_dtype: ESMOE_OUT_BF16 / ESMOE_OUT_FP16, the type the projection and the activation are rounded to on the way.
 * The other arguments are those of esmoe_mxfp8_grouped_mm.
 */
int esmoe_mxfp8_grouped_mm_swiglu_quant(void* q, uint8_t* sf, int mid_dtype, const void* a, const void* b,
                                        const uint8_t* sfa, const uint8_t* sfb, const int32_t* problem_sizes,
                                        const int32_t* expert_offsets, const int32_t* blockscale_offsets,
                                        int num_experts, int total_rows, int sf_rows, int n, int k, int force_bm,
                                        void* workspace, size_t workspace_bytes, void* stream);

/*
 * MXFP8 grouped quantisation: bf16/fp16 rows -> e4m3 bytes + swizzled E8M0 scales.
 * Replaces es_sm100_mxfp8_blockscaled_grouped_quant
 *   (expert_specialization/csrc/cuda/es_sm100_mxfp8_blockscaled_group_quant.cu:5-39,
 *    ..._group_quant.cuh:261-405, schema expert_specialization.cpp:64-66).
 *
 *   in [total_rows, K] bf16 or fp16 (in_dtype);  q [total_rows, K] bytes;
 *   sf: `sf_rows` rows of K/32 scale bytes (sf_rows % 128 == 0, >= the largest
 *       blockscale_offsets[e] + M_e rounded up to 128); expert e's scales start at byte
 *       blockscale_offsets[e]*(K/32); rows < M_e are defined, padding rows of an expert's
 *       last 128-row tile are written as 0 (the reference leaves them unspecified).
 *   blockscale_offsets must be non-decreasing multiples of 128 (the reference's callers
 *   build them as the prefix sum of M_e rounded up to 128).
 * Only columns 0 (M_e) and 2 (K) of problem_sizes are used, as in the reference (:281-282).
 */
int esmoe_mxfp8_grouped_quant(const void* in, int in_dtype, const int32_t* problem_sizes,
                              const int32_t* expert_offsets, const int32_t* blockscale_offsets, void* q,
                              uint8_t* sf, int num_experts, int total_rows, int sf_rows, int k, void* stream);

/*
 * MXFP8 quantisation of a weight tensor [E, N, K] (N % 128 == 0), passed as rows = E*N rows of K: e4m3 bytes and the
 * swizzled E8M0 scales in the layout esmoe_mxfp8_grouped_mm reads as `sfb` (expert e at byte e*N*(K/32)).  The
 * reference has no weight entry point: its test passes the activation operator a transposed problem list
 * [N, M, K] with offsets e*N (test/test_es_sm100_mxfp8_blockscaled_grouped_quant.py:53,87-96); this call produces
 * the same bytes without the metadata.
 */
int esmoe_mxfp8_quant_weight(const void* in, int in_dtype, void* q, uint8_t* sf, long rows, int k, void* stream);

/*
 * Fused SwiGLU + MXFP8 grouped quantisation between the gate_up and the down projection: `in` is the gate_up
 * output [total_rows, 2*inter]; x = silu(gate) * up (gate = first half of a row), formed in fp32 and rounded once
 * to the input type, is quantised exactly as esmoe_mxfp8_grouped_quant quantises a [total_rows, inter] tensor
 * (same q / sf layouts, same metadata, K = inter).  No counterpart in the reference, whose callers run the
 * activation and the quantisation as separate steps.
 */
int esmoe_swiglu_mxfp8_grouped_quant(const void* in, int in_dtype, const int32_t* problem_sizes,
                                     const int32_t* expert_offsets, const int32_t* blockscale_offsets, void* q,
                                     uint8_t* sf, int num_experts, int total_rows, int sf_rows, int inter,
                                     void* stream);

/*
 * FP8 1x128 activation quantisation: bf16/fp16 rows -> e4m3fn bytes + fp32 scale per 128-wide block,
 * the `a` / `scales_a` operands of esmoe_fp8_blockwise_grouped_mm.
 * The reference has no operator for this step: its callers run the torch helper per_token_cast_to_fp8
 * (test/test_es_grouped_gemm.py:36-44, again in benchmark/benchmark_es_fp8_blockwise_moe.py:18-26);
 * this entry point reproduces that helper's arithmetic bit for bit on the device.
 *
 *   in [total_rows, K] bf16 or fp16 (in_dtype), K % 128 == 0;  q [total_rows, K] bytes;
 *   scales [total_rows, K/128] fp32.   amax = max(|x|, 1e-4) per block, q = e4m3(x * (448/amax)),
 *   scale = amax * fl(1/448) (torch's GPU evaluation of amax / 448.0).  Rows are independent, so the
 *   grouped layout needs no metadata.
 */
int esmoe_fp8_quant_act_1x128(const void* in, int in_dtype, void* q, float* scales, long total_rows, int k,
                              void* stream);

/*
 * FP8 128x128 weight quantisation: bf16/fp16 [rows, K] (rows = E * N, the physical [E, N, K] weight
 * tensor) -> e4m3fn bytes + one fp32 scale per 128x128 block, the `b` / `scales_b` operands of
 * esmoe_fp8_blockwise_grouped_mm in their physical layouts ([E, N, K] and [E, N/128, K/128]).
 * Like the activation quantiser it replaces a torch helper of the reference's callers,
 * per_block_cast_to_fp8 (test/test_es_grouped_gemm.py:47-59, applied through the transposed view at
 * :127,132-134,160,166-168), bit for bit.  rows % 128 == 0, K % 128 == 0, rows <= 128 * 65535.
 */
int esmoe_fp8_quant_weight_128x128(const void* in, int in_dtype, void* q, float* scales, long rows, int k,
                                   void* stream);

/*
 * Fused SwiGLU + 1x128 quantisation between the gate_up and the down projection:
 *   in [total_rows, 2*inter] bf16/fp16 (gate = first half of a row, up = second half)
 *   h = cast_to_in_dtype(silu(gate) * up)   (fp32 product, one rounding; silu(x) = x / (1 + exp(-x)))
 *   q [total_rows, inter], scales [total_rows, inter/128] = the 1x128 quantisation of h, as
 *   esmoe_fp8_quant_act_1x128 computes it.   inter % 128 == 0.
 * No counterpart in the reference (its benchmark shapes pair a gate_up N = 2*inter with a down
 * K = inter, benchmark/benchmark_es_fp8_blockwise_moe.py:349-364, and leave the step between to the caller).
 * exp() is the device's fp32 routine, so bytes can differ from a host evaluation where a product
 * falls within an ulp of a rounding boundary; the parity test states the tolerance.
 */
int esmoe_swiglu_quant_1x128(const void* in, int in_dtype, void* q, float* scales, long total_rows, int inter,
                             void* stream);

/*
 * Routing metadata on the device: top-k expert ids -> the per-expert tensors the operators above take.
 * The reference's callers build these on the host (counts and their prefix sum:
 * benchmark/benchmark_es_fp8_blockwise_moe.py:44-56,72-88; blockscale_offsets as the prefix sum of the
 * counts rounded up to 128: test/test_es_sm100_mxfp8_blockscaled_grouped_quant.py:42-60); there is no
 * operator for it in the reference.
 *
 *   topk_ids [num_pairs] int32: expert id of pair p = (token p / topk, choice p % topk); ids outside
 *            [first_expert, first_expert + num_experts) belong to other devices and are skipped
 *   problem_sizes [E,3] = (count_e, n, k);  expert_offsets [E+1], blockscale_offsets [E+1]: exclusive prefix
 *            sums of the counts and of the counts rounded up to 128, last entry = total
 *   dst_row [num_pairs]: row of pair p in the packed [sum count, .] tensors (pairs of one expert keep
 *            their order, so the result is deterministic), -1 for skipped pairs
 *   workspace: esmoe_route_workspace_bytes(num_pairs, num_experts) bytes of device scratch
 */
size_t esmoe_route_workspace_bytes(long num_pairs, int num_experts);
int esmoe_route_metadata(const int32_t* topk_ids, long num_pairs, int first_expert, int num_experts, int n, int k,
                         int32_t* problem_sizes, int32_t* expert_offsets, int32_t* blockscale_offsets,
                         int32_t* dst_row, void* workspace, size_t workspace_bytes, void* stream);

/* out[dst_row[p], :] = in[p / topk, :] for every pair with dst_row[p] >= 0; rows of row_bytes bytes
 * (a multiple of 16), `in` and `out` 16-byte aligned.  No counterpart in the reference. */
int esmoe_permute_rows(const void* in, const int32_t* dst_row, long num_pairs, int topk, long row_bytes, void* out,
                       void* stream);

/*
 * Host mirrors of the device-side tile schedule, for inspection and CPU tests; they touch no GPU.
 * No counterpart in the reference (its schedule lives inside CUTLASS's grouped tile scheduler).
 * esmoe_host_schedule fills `ws_host` (esmoe_gemm_workspace_bytes(E) bytes of host memory) from host
 * copies of problem_sizes exactly as the schedule kernel fills the device workspace: words 1 and 2 are
 * the number of light items and of heavy blocks.
 * Experts with more than 64 rows are "heavy": their tiles are handed out in blocks of 8 x 4 tiles, block b
 * to XCD b % 8, through one ticket counter per XCD; esmoe_host_decode_heavy maps ticket `ticket` of XCD `xcd`
 * to out5 = {expert, tile rows, tile cols, m0, n0} and returns 0, or 1 if the ticket falls outside the
 * expert's tile grid (the kernel skips it), or 2 if that XCD's queue is exhausted.
 * The other experts are "light": one short tile per 256 columns from a launch-wide counter, except that the last 128
 * light items of a launch go out as two 128-column halves each (word 4 of the workspace is the first ticket that is a
 * half, word 1 the number of light tickets); esmoe_host_decode_light maps ticket `item` (< word 1) to out5 and returns
 * 0, or 1 for the second half of a last column tile that is only 128 columns wide (the kernel skips it).
 * kind: bit 0 clear describes the FP8-blockwise launch, set the MXFP8 launch (both cut experts into full tiles of 192
 * rows today); bit 1 set describes a launch with a fused SwiGLU epilogue, whose items all stay 256 columns wide, as do
 * those of a launch with a forced tile height.
 * The mirrors describe the default policy; the ESMOE_* environment variables, which a launch reads once per process, do not
 * reach them.
 */
int esmoe_host_schedule(const int32_t* problem_sizes_host, int num_experts, int n, int force_bm, int kind,
                        int32_t* ws_host);
int esmoe_host_decode_heavy(const int32_t* problem_sizes_host, const int32_t* ws_host, int num_experts, int n,
                            int force_bm, int kind, int xcd, int ticket, int32_t* out5);
int esmoe_host_decode_light(const int32_t* problem_sizes_host, const int32_t* ws_host, int num_experts, int n,
                            int force_bm, int kind, int item, int32_t* out5);

/* Message describing the calling thread's most recent failure ("" if none). */
const char* esmoe_last_error(void);

/* Library version string. */
const char* esmoe_version(void);

#ifdef __cplusplus
}
#endif
#endif /* ESMOE_H_ */
