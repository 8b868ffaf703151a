// PyTorch-ROCm operator registration for the three expert_specialization ops.
//
// Same library name, schemas and dispatch key as the reference
// (expert_specialization/csrc/expert_specialization.cpp:56-73); the argument
// checks mirror its TORCH_CHECKs (es_fp8_blockwise.cu:47-56,
// es_sm100_mxfp8_blockscaled.cu:15-25, es_sm100_mxfp8_blockscaled_group_quant.cu:13-24,
// es_fp8_blockwise_launcher.cuh:53).  Everything below the checks is the C ABI of
// libesmoe.so (include/esmoe.h): this file only unwraps tensors.
//
// Validation is also registered for CPU tensors so that it can be exercised on a
// machine without a GPU; after the checks pass a CPU call fails loudly, there is
// no CPU implementation of the ops.
#include <Python.h>
#include <c10/hip/HIPStream.h>
#include <torch/all.h>

#include "esmoe.h"

extern "C" {
// Empty module so that `import ..._C` loads this library and runs the static
// registrations below (same device as the reference, expert_specialization.cpp:4-21).
PyObject* PyInit__C(void) {
  static struct PyModuleDef module_def = {PyModuleDef_HEAD_INIT, "_C", NULL, -1, NULL};
  return PyModule_Create(&module_def);
}
}

namespace {

void* current_stream(const torch::Tensor& t) {
  return (void*)c10::hip::getCurrentHIPStream(t.device().index()).stream();
}

void require_device(const torch::Tensor& t, const char* op) {
  TORCH_CHECK(t.is_cuda(), op, ": tensors must live on a HIP device (MI355X); there is no CPU implementation");
}

void check_rc(int rc, const char* op) { TORCH_CHECK(rc == 0, op, " failed (", rc, "): ", esmoe_last_error()); }

int out_dtype_of(const torch::Tensor& t) { return t.scalar_type() == torch::kBFloat16 ? ESMOE_OUT_BF16 : ESMOE_OUT_FP16; }

// Scratch for the device-built schedule: the operators pass no workspace to the library, which then uses its own
// workspace of the current stream (zeroed once, left clean by every launch) and needs one launch per call instead of
// two.  The `workspace` tensor of the reference's signature is accepted and not used: its contents are the caller's,
// and a schedule built in it would need a kernel of its own in front of the GEMM to clear the counters.
}  // namespace

void es_fp8_blockwise_scaled_grouped_mm(torch::Tensor& output, const torch::Tensor& a, const torch::Tensor& b,
                                        const torch::Tensor& scales_a, const torch::Tensor& scales_b,
                                        const torch::Tensor& stride_a, const torch::Tensor& stride_b,
                                        const torch::Tensor& stride_d, const torch::Tensor& problem_sizes,
                                        const torch::Tensor& expert_offsets, const torch::Tensor& workspace) {
  TORCH_CHECK(problem_sizes.dim() == 2, "problem_sizes must be 2D tensor");
  TORCH_CHECK(problem_sizes.size(1) == 3, "problem_sizes must have shape (num_experts, 3)");
  TORCH_CHECK(problem_sizes.size(0) == expert_offsets.size(0),
              "Number of experts in problem_sizes must match expert_offsets");
  TORCH_CHECK(problem_sizes.dtype() == torch::kInt32, "problem_sizes must be int32");
  TORCH_CHECK(expert_offsets.dtype() == torch::kInt32, "expert_offsets must be int32");
  TORCH_CHECK(a.scalar_type() == torch::kFloat8_e4m3fn, "a must be kFloat8_e4m3fn");
  TORCH_CHECK(b.scalar_type() == torch::kFloat8_e4m3fn, "b must be kFloat8_e4m3fn");
  TORCH_CHECK(output.scalar_type() == torch::kBFloat16 || output.scalar_type() == torch::kHalf,
              "output must be bfloat16 or half");
  const int64_t num_experts = problem_sizes.size(0);
  TORCH_CHECK(num_experts >= 1 && num_experts <= ESMOE_MAX_EXPERTS, "Number of experts cannot exceed 1024");
  // Layout contract (the reference only ever dereferences data_ptr(), so the views below are the
  // ones its callers build: test/test_es_grouped_gemm.py:145-170).
  TORCH_CHECK(a.dim() == 2 && a.stride(1) == 1 && a.stride(0) == a.size(1), "a must be a packed row-major (rows, k) tensor");
  TORCH_CHECK(b.dim() == 3 && b.size(0) == num_experts, "b must be a (num_experts, k, n) tensor");
  TORCH_CHECK(b.stride(1) == 1 && b.stride(2) == b.size(1) && b.stride(0) == b.size(1) * b.size(2),
              "b must be the column-major (num_experts, k, n) view of a packed (num_experts, n, k) tensor");
  const int64_t total_rows = a.size(0), k = a.size(1), n = b.size(2);
  TORCH_CHECK(b.size(1) == k, "a and b disagree on k");
  TORCH_CHECK(k % 128 == 0 && n % 128 == 0, "n and k must be multiples of 128");
  TORCH_CHECK(output.dim() == 2 && output.size(0) == total_rows && output.size(1) == n && output.is_contiguous(),
              "output must be a contiguous (rows, n) tensor");
  TORCH_CHECK(scales_a.scalar_type() == torch::kFloat32 && scales_b.scalar_type() == torch::kFloat32,
              "scales must be float32");
  TORCH_CHECK(scales_a.dim() == 2 && scales_a.size(0) == total_rows && scales_a.size(1) == k / 128 &&
                  scales_a.is_contiguous(),
              "scales_a must be a contiguous (rows, k/128) tensor");
  TORCH_CHECK(scales_b.dim() == 3 && scales_b.size(0) == num_experts && scales_b.size(1) == k / 128 &&
                  scales_b.size(2) == n / 128 && scales_b.stride(1) == 1 &&
                  (scales_b.size(2) == 1 || scales_b.stride(2) == k / 128),
              "scales_b must be the (num_experts, k/128, n/128) view of a packed (num_experts, n/128, k/128) tensor");
  for (const torch::Tensor* s : {&stride_a, &stride_b, &stride_d}) {
    TORCH_CHECK(s->dim() == 1 && s->size(0) == num_experts, "stride tensors must have one entry per expert");
  }
  TORCH_CHECK(total_rows < (int64_t(1) << 31) && n < (int64_t(1) << 31) && k < (int64_t(1) << 31), "tensor too large");

  require_device(a, "es_fp8_blockwise_scaled_grouped_mm");
  for (const torch::Tensor* t :
       {(const torch::Tensor*)&output, &b, &scales_a, &scales_b, &problem_sizes, &expert_offsets}) {
    TORCH_CHECK(t->device() == a.device(), "all tensors must be on the same device");
  }
  TORCH_CHECK(problem_sizes.is_contiguous() && expert_offsets.is_contiguous(), "metadata tensors must be contiguous");
  if (total_rows == 0) return;
  c10::DeviceGuard guard(a.device());
  int rc = esmoe_fp8_blockwise_grouped_mm(
      output.data_ptr(), out_dtype_of(output), a.data_ptr(), b.data_ptr(), scales_a.data_ptr<float>(),
      scales_b.data_ptr<float>(), problem_sizes.data_ptr<int32_t>(), expert_offsets.data_ptr<int32_t>(),
      (int)num_experts, (int)total_rows, (int)n, (int)k, /*force_bm=*/0, /*workspace=*/nullptr, 0, current_stream(a));
  check_rc(rc, "es_fp8_blockwise_scaled_grouped_mm");
}

// The gate_up projection with SwiGLU and 1x128 re-quantisation fused into its epilogue (no counterpart in the
// reference).  Operand layouts as es_fp8_blockwise_scaled_grouped_mm with n = 2 * inter; `mid_dtype_bf16` selects the
// type the projection and the activation are rounded to on the way (true: bfloat16, false: half).
void es_fp8_blockwise_scaled_grouped_mm_swiglu_quant(torch::Tensor& quant_output, torch::Tensor& scales_out,
                                                     const torch::Tensor& a, const torch::Tensor& b,
                                                     const torch::Tensor& scales_a, const torch::Tensor& scales_b,
                                                     const torch::Tensor& problem_sizes,
                                                     const torch::Tensor& expert_offsets, const torch::Tensor& workspace,
                                                     bool mid_dtype_bf16) {
  TORCH_CHECK(problem_sizes.dim() == 2 && problem_sizes.size(1) == 3, "problem_sizes must have shape (num_experts, 3)");
  TORCH_CHECK(expert_offsets.dim() == 1 && problem_sizes.size(0) == expert_offsets.size(0),
              "Number of experts in problem_sizes must match expert_offsets");
  TORCH_CHECK(problem_sizes.dtype() == torch::kInt32 && expert_offsets.dtype() == torch::kInt32,
              "problem_sizes and expert_offsets must be int32");
  TORCH_CHECK(a.scalar_type() == torch::kFloat8_e4m3fn && b.scalar_type() == torch::kFloat8_e4m3fn,
              "a and b must be kFloat8_e4m3fn");
  const int64_t num_experts = problem_sizes.size(0);
  TORCH_CHECK(num_experts >= 1 && num_experts <= ESMOE_MAX_EXPERTS, "Number of experts cannot exceed 1024");
  TORCH_CHECK(a.dim() == 2 && a.stride(1) == 1 && a.stride(0) == a.size(1), "a must be a packed row-major (rows, k) tensor");
  TORCH_CHECK(b.dim() == 3 && b.size(0) == num_experts, "b must be a (num_experts, k, n) tensor");
  TORCH_CHECK(b.stride(1) == 1 && b.stride(2) == b.size(1) && b.stride(0) == b.size(1) * b.size(2),
              "b must be the column-major (num_experts, k, n) view of a packed (num_experts, n, k) tensor");
  const int64_t total_rows = a.size(0), k = a.size(1), n = b.size(2);
  TORCH_CHECK(b.size(1) == k, "a and b disagree on k");
  TORCH_CHECK(k % 128 == 0 && n % 256 == 0, "k must be a multiple of 128 and n = 2 * inter a multiple of 256");
  const int64_t inter = n / 2;
  TORCH_CHECK(quant_output.is_contiguous() && quant_output.element_size() == 1 && quant_output.numel() == total_rows * inter,
              "quant_output must be a contiguous 1-byte tensor of rows * n / 2 elements");
  TORCH_CHECK(scales_out.is_contiguous() && scales_out.scalar_type() == torch::kFloat32 &&
                  scales_out.numel() == total_rows * (inter / 128),
              "scales_out must be a contiguous float32 tensor of rows * n / 256 elements");
  TORCH_CHECK(scales_a.scalar_type() == torch::kFloat32 && scales_b.scalar_type() == torch::kFloat32,
              "scales must be float32");
  TORCH_CHECK(scales_a.dim() == 2 && scales_a.size(0) == total_rows && scales_a.size(1) == k / 128 &&
                  scales_a.is_contiguous(),
              "scales_a must be a contiguous (rows, k/128) tensor");
  TORCH_CHECK(scales_b.dim() == 3 && scales_b.size(0) == num_experts && scales_b.size(1) == k / 128 &&
                  scales_b.size(2) == n / 128 && scales_b.stride(1) == 1 && scales_b.stride(2) == k / 128,
              "scales_b must be the (num_experts, k/128, n/128) view of a packed (num_experts, n/128, k/128) tensor");
  TORCH_CHECK(total_rows < (int64_t(1) << 31) && n < (int64_t(1) << 31) && k < (int64_t(1) << 31), "tensor too large");
  require_device(a, "es_fp8_blockwise_scaled_grouped_mm_swiglu_quant");
  for (const torch::Tensor* t : {(const torch::Tensor*)&quant_output, (const torch::Tensor*)&scales_out, &b, &scales_a,
                                 &scales_b, &problem_sizes, &expert_offsets}) {
    TORCH_CHECK(t->device() == a.device(), "all tensors must be on the same device");
  }
  TORCH_CHECK(problem_sizes.is_contiguous() && expert_offsets.is_contiguous(), "metadata tensors must be contiguous");
  if (total_rows == 0) return;
  c10::DeviceGuard guard(a.device());
  int rc = esmoe_fp8_blockwise_grouped_mm_swiglu_quant(
      quant_output.data_ptr(), scales_out.data_ptr<float>(), mid_dtype_bf16 ? ESMOE_OUT_BF16 : ESMOE_OUT_FP16, a.data_ptr(),
      b.data_ptr(), scales_a.data_ptr<float>(), scales_b.data_ptr<float>(), problem_sizes.data_ptr<int32_t>(),
      expert_offsets.data_ptr<int32_t>(), (int)num_experts, (int)total_rows, (int)n, (int)k, /*force_bm=*/0, /*workspace=*/nullptr, 0, current_stream(a));
  check_rc(rc, "es_fp8_blockwise_scaled_grouped_mm_swiglu_quant");
}

void es_sm100_mxfp8_blockscaled_grouped_mm(const torch::Tensor& a, const torch::Tensor& b, const torch::Tensor& sfa,
                                           const torch::Tensor& sfb, torch::Tensor& d,
                                           const torch::Tensor& problem_sizes, const torch::Tensor& expert_offsets,
                                           const torch::Tensor& blockscale_offsets) {
  TORCH_CHECK(problem_sizes.dim() == 2, "problem_sizes must be 2D tensor");
  TORCH_CHECK(problem_sizes.size(1) == 3, "problem_sizes must have shape (num_experts, 3)");
  TORCH_CHECK(problem_sizes.size(0) == expert_offsets.size(0),
              "Number of experts in problem_sizes must match expert_offsets");
  TORCH_CHECK(problem_sizes.dtype() == torch::kInt32, "problem_sizes must be int32");
  TORCH_CHECK(a.dim() == 2, "a must be a 2D tensor of shape (num_tokens, k)");
  TORCH_CHECK(b.dim() == 3, "b must be a 3D tensor of shape (num_experts, k, n)");
  TORCH_CHECK(a.size(1) == b.size(1) && a.size(1) % 128 == 0, "k should align 128");
  TORCH_CHECK(b.size(2) % 128 == 0, "n should align 128");
  TORCH_CHECK(a.strides()[1] == 1, "a must be row major");
  TORCH_CHECK(b.strides()[1] == 1, "b must be column major");
  TORCH_CHECK(d.scalar_type() == torch::kBFloat16 || d.scalar_type() == torch::kHalf,
              "dtype must be kFloat16 or kBFloat16");
  const int64_t num_experts = problem_sizes.size(0);
  TORCH_CHECK(num_experts >= 1 && num_experts <= ESMOE_MAX_EXPERTS,
              "Number of experts cannot exceed 1024, the maximum number of threads per block.");
  // a and b are read through data_ptr() as e4m3 bytes whatever their dtype: the reference's own test
  // passes 2-byte tensors that the quant op filled with bytes
  // (test/test_es_sm100_mxfp8_blockscaled_grouped_quant.py:72-76,95-101).
  TORCH_CHECK(a.stride(0) == a.size(1), "a must be packed");
  TORCH_CHECK(b.size(0) == num_experts && b.stride(2) == b.size(1) && b.stride(0) == b.size(1) * b.size(2),
              "b must be the column-major (num_experts, k, n) view of a packed (num_experts, n, k) tensor");
  const int64_t total_rows = a.size(0), k = a.size(1), n = b.size(2);
  TORCH_CHECK(d.dim() == 2 && d.size(0) == total_rows && d.size(1) == n && d.is_contiguous(),
              "d must be a contiguous (num_tokens, n) tensor");
  TORCH_CHECK(sfa.element_size() == 1 && sfb.element_size() == 1, "scale factors must be 1-byte E8M0");
  TORCH_CHECK(sfb.numel() >= num_experts * n * (k / 32), "sfb is smaller than num_experts * n * k / 32 bytes");
  // every expert's scale rows are padded to 128, so the tensor holds at least the row total rounded up (a bound that
  // needs no look at the device-side metadata)
  TORCH_CHECK(sfa.numel() >= (total_rows + 127) / 128 * 128 * (k / 32),
              "sfa is smaller than the rows rounded up to 128 times k / 32 bytes");
  TORCH_CHECK(expert_offsets.dtype() == torch::kInt32 && blockscale_offsets.dtype() == torch::kInt32,
              "offset tensors must be int32");
  TORCH_CHECK(blockscale_offsets.dim() == 1 && blockscale_offsets.size(0) == num_experts,
              "blockscale_offsets must be 1D and have size equal to the number of experts");
  TORCH_CHECK(total_rows < (int64_t(1) << 31), "tensor too large");

  require_device(a, "es_sm100_mxfp8_blockscaled_grouped_mm");
  for (const torch::Tensor* t :
       {&b, &sfa, &sfb, (const torch::Tensor*)&d, &problem_sizes, &expert_offsets, &blockscale_offsets}) {
    TORCH_CHECK(t->device() == a.device(), "all tensors must be on the same device");
  }
  TORCH_CHECK(problem_sizes.is_contiguous() && expert_offsets.is_contiguous() && blockscale_offsets.is_contiguous(),
              "metadata tensors must be contiguous");
  if (total_rows == 0) return;
  c10::DeviceGuard guard(a.device());
  int rc = esmoe_mxfp8_grouped_mm(d.data_ptr(), out_dtype_of(d), a.data_ptr(), b.data_ptr(),
                                  (const uint8_t*)sfa.data_ptr(), (const uint8_t*)sfb.data_ptr(),
                                  problem_sizes.data_ptr<int32_t>(), expert_offsets.data_ptr<int32_t>(),
                                  blockscale_offsets.data_ptr<int32_t>(), (int)num_experts, (int)total_rows, (int)n,
                                  (int)k, /*force_bm=*/0, /*workspace=*/nullptr, 0, current_stream(a));
  check_rc(rc, "es_sm100_mxfp8_blockscaled_grouped_mm");
}

// The mxfp8 gate_up projection with SwiGLU and the 1x32 E8M0 re-quantisation fused into its epilogue (no counterpart
// in the reference).  Operand layouts as es_sm100_mxfp8_blockscaled_grouped_mm with n = 2 * inter; the outputs are what
// es_sm100_mxfp8_blockscaled_grouped_quant would write for a (rows, inter) input.
void es_mxfp8_blockscaled_grouped_mm_swiglu_quant(torch::Tensor& quant_output, torch::Tensor& scale_factor,
                                                  const torch::Tensor& a, const torch::Tensor& b,
                                                  const torch::Tensor& sfa, const torch::Tensor& sfb,
                                                  const torch::Tensor& problem_sizes, const torch::Tensor& expert_offsets,
                                                  const torch::Tensor& blockscale_offsets, bool mid_dtype_bf16) {
  TORCH_CHECK(problem_sizes.dim() == 2 && problem_sizes.size(1) == 3, "problem_sizes must have shape (num_experts, 3)");
  const int64_t num_experts = problem_sizes.size(0);
  TORCH_CHECK(expert_offsets.dim() == 1 && expert_offsets.size(0) == num_experts && blockscale_offsets.dim() == 1 &&
                  blockscale_offsets.size(0) == num_experts,
              "expert_offsets and blockscale_offsets must be 1D and have size equal to the number of experts");
  TORCH_CHECK(problem_sizes.dtype() == torch::kInt32 && expert_offsets.dtype() == torch::kInt32 &&
                  blockscale_offsets.dtype() == torch::kInt32,
              "problem_sizes, expert_offsets and blockscale_offsets must be int32");
  TORCH_CHECK(num_experts >= 1 && num_experts <= ESMOE_MAX_EXPERTS, "Number of experts cannot exceed 1024");
  TORCH_CHECK(a.dim() == 2 && a.stride(1) == 1 && a.stride(0) == a.size(1), "a must be a packed row-major (rows, k) tensor");
  TORCH_CHECK(b.dim() == 3 && b.size(0) == num_experts, "b must be a (num_experts, k, n) tensor");
  TORCH_CHECK(b.stride(1) == 1 && b.stride(2) == b.size(1) && b.stride(0) == b.size(1) * b.size(2),
              "b must be the column-major (num_experts, k, n) view of a packed (num_experts, n, k) tensor");
  TORCH_CHECK(a.element_size() == 1 && b.element_size() == 1, "a and b must be 1-byte e4m3 tensors");
  const int64_t total_rows = a.size(0), k = a.size(1), n = b.size(2);
  TORCH_CHECK(b.size(1) == k, "a and b disagree on k");
  TORCH_CHECK(k % 128 == 0 && n % 256 == 0, "k must be a multiple of 128 and n = 2 * inter a multiple of 256");
  const int64_t inter = n / 2;
  TORCH_CHECK(quant_output.is_contiguous() && quant_output.element_size() == 1 && quant_output.numel() == total_rows * inter,
              "quant_output must be a contiguous 1-byte tensor of rows * n / 2 elements");
  TORCH_CHECK(scale_factor.is_contiguous() && scale_factor.element_size() == 1,
              "scale_factor must be a contiguous 1-byte tensor");
  const int64_t sf_rows = (scale_factor.numel() / (inter / 32)) / 128 * 128;
  TORCH_CHECK(sf_rows >= (total_rows + 127) / 128 * 128,
              "scale_factor is smaller than the rows rounded up to 128 times n / 64 bytes");
  TORCH_CHECK(sfa.element_size() == 1 && sfb.element_size() == 1, "scale factors must be 1-byte E8M0");
  TORCH_CHECK(sfb.numel() >= num_experts * n * (k / 32), "sfb is smaller than num_experts * n * k / 32 bytes");
  TORCH_CHECK(sfa.numel() >= (total_rows + 127) / 128 * 128 * (k / 32),
              "sfa is smaller than the rows rounded up to 128 times k / 32 bytes");
  TORCH_CHECK(total_rows < (int64_t(1) << 31) && sf_rows < (int64_t(1) << 31) && n < (int64_t(1) << 31) &&
                  k < (int64_t(1) << 31),
              "tensor too large");
  require_device(a, "es_mxfp8_blockscaled_grouped_mm_swiglu_quant");
  for (const torch::Tensor* t : {(const torch::Tensor*)&quant_output, (const torch::Tensor*)&scale_factor, &b, &sfa, &sfb,
                                 &problem_sizes, &expert_offsets, &blockscale_offsets}) {
    TORCH_CHECK(t->device() == a.device(), "all tensors must be on the same device");
  }
  TORCH_CHECK(problem_sizes.is_contiguous() && expert_offsets.is_contiguous() && blockscale_offsets.is_contiguous(),
              "metadata tensors must be contiguous");
  if (total_rows == 0) return;
  c10::DeviceGuard guard(a.device());
  int rc = esmoe_mxfp8_grouped_mm_swiglu_quant(
      quant_output.data_ptr(), (uint8_t*)scale_factor.data_ptr(), mid_dtype_bf16 ? ESMOE_OUT_BF16 : ESMOE_OUT_FP16,
      a.data_ptr(), b.data_ptr(), (const uint8_t*)sfa.data_ptr(), (const uint8_t*)sfb.data_ptr(),
      problem_sizes.data_ptr<int32_t>(), expert_offsets.data_ptr<int32_t>(), blockscale_offsets.data_ptr<int32_t>(),
      (int)num_experts, (int)total_rows, (int)sf_rows, (int)n, (int)k, /*force_bm=*/0, /*workspace=*/nullptr, 0,
      current_stream(a));
  check_rc(rc, "es_mxfp8_blockscaled_grouped_mm_swiglu_quant");
}

void es_sm100_mxfp8_blockscaled_grouped_quant(const torch::Tensor& input, const torch::Tensor& problem_sizes,
                                              const torch::Tensor& expert_offsets,
                                              const torch::Tensor& blockscale_offsets, torch::Tensor& quant_output,
                                              torch::Tensor& scale_factor) {
  TORCH_CHECK(input.dim() == 2, "input must be 2D tensor");
  TORCH_CHECK(input.size(1) % 128 == 0, "k must align to 128");
  TORCH_CHECK(input.strides()[1] == 1, "input must be row major");
  TORCH_CHECK(problem_sizes.dim() == 2, "problem_sizes must be 2D tensor");
  const int64_t groups = problem_sizes.size(0);
  TORCH_CHECK(expert_offsets.dim() == 1 && expert_offsets.size(0) == groups,
              "expert_offsets must be 1D and have size equal to the number of groups");
  TORCH_CHECK(blockscale_offsets.dim() == 1 && blockscale_offsets.size(0) == groups,
              "blockscale_offsets must be 1D and have size equal to the number of groups");
  TORCH_CHECK(input.scalar_type() == torch::kBFloat16 || input.scalar_type() == torch::kHalf,
              "dtype must be kFloat16 or kBFloat16");
  TORCH_CHECK(problem_sizes.size(1) == 3 && problem_sizes.dtype() == torch::kInt32 &&
                  expert_offsets.dtype() == torch::kInt32 && blockscale_offsets.dtype() == torch::kInt32,
              "problem_sizes (groups, 3), expert_offsets and blockscale_offsets must be int32");
  TORCH_CHECK(groups >= 1 && groups <= ESMOE_MAX_EXPERTS, "number of groups must be in [1, 1024]");
  TORCH_CHECK(input.stride(0) == input.size(1), "input must be packed");
  const int64_t total_rows = input.size(0), k = input.size(1);
  // The reference's test hands over zeros_like(input) (2-byte elements) and lets the kernel write
  // bytes into it (test/test_es_sm100_mxfp8_blockscaled_grouped_quant.py:72); any contiguous
  // tensor with room for rows*k bytes is accepted.
  TORCH_CHECK(quant_output.is_contiguous() && (int64_t)quant_output.nbytes() >= total_rows * k,
              "quant_output must be contiguous and hold at least rows * k bytes");
  TORCH_CHECK(scale_factor.is_contiguous() && scale_factor.element_size() == 1,
              "scale_factor must be a contiguous 1-byte tensor");
  const int64_t sf_rows = (scale_factor.numel() / (k / 32)) / 128 * 128;
  TORCH_CHECK(sf_rows >= (total_rows + 127) / 128 * 128,
              "scale_factor is smaller than the rows rounded up to 128 times k / 32 bytes");
  TORCH_CHECK(total_rows < (int64_t(1) << 31) && sf_rows < (int64_t(1) << 31), "tensor too large");

  require_device(input, "es_sm100_mxfp8_blockscaled_grouped_quant");
  for (const torch::Tensor* t : {&problem_sizes, &expert_offsets, &blockscale_offsets, (const torch::Tensor*)&quant_output,
                                 (const torch::Tensor*)&scale_factor}) {
    TORCH_CHECK(t->device() == input.device(), "all tensors must be on the same device");
  }
  TORCH_CHECK(problem_sizes.is_contiguous() && expert_offsets.is_contiguous() && blockscale_offsets.is_contiguous(),
              "metadata tensors must be contiguous");
  if (total_rows == 0) return;
  c10::DeviceGuard guard(input.device());
  int rc = esmoe_mxfp8_grouped_quant(
      input.data_ptr(), input.scalar_type() == torch::kBFloat16 ? ESMOE_IN_BF16 : ESMOE_IN_FP16,
      problem_sizes.data_ptr<int32_t>(), expert_offsets.data_ptr<int32_t>(), blockscale_offsets.data_ptr<int32_t>(),
      quant_output.data_ptr(), (uint8_t*)scale_factor.data_ptr(), (int)groups, (int)total_rows, (int)sf_rows, (int)k,
      current_stream(input));
  check_rc(rc, "es_sm100_mxfp8_blockscaled_grouped_quant");
}

// Extension beyond the reference's three operators: the 1x128 activation quantiser its callers run in
// torch (per_token_cast_to_fp8, test/test_es_grouped_gemm.py:36-44), as a device operator.
void es_fp8_quant_act_1x128(const torch::Tensor& input, torch::Tensor& quant_output, torch::Tensor& scales) {
  TORCH_CHECK(input.dim() == 2, "input must be 2D tensor");
  TORCH_CHECK(input.size(1) % 128 == 0, "k must align to 128");
  TORCH_CHECK(input.scalar_type() == torch::kBFloat16 || input.scalar_type() == torch::kHalf,
              "dtype must be kFloat16 or kBFloat16");
  TORCH_CHECK(input.is_contiguous(), "input must be packed row major");
  const int64_t total_rows = input.size(0), k = input.size(1);
  TORCH_CHECK(quant_output.is_contiguous() && quant_output.element_size() == 1 && quant_output.numel() == total_rows * k,
              "quant_output must be a contiguous 1-byte tensor of rows * k elements");
  TORCH_CHECK(scales.is_contiguous() && scales.scalar_type() == torch::kFloat32 && scales.numel() == total_rows * (k / 128),
              "scales must be a contiguous float32 tensor of rows * k / 128 elements");
  require_device(input, "es_fp8_quant_act_1x128");
  TORCH_CHECK(quant_output.device() == input.device() && scales.device() == input.device(),
              "all tensors must be on the same device");
  if (total_rows == 0) return;
  c10::DeviceGuard guard(input.device());
  int rc = esmoe_fp8_quant_act_1x128(input.data_ptr(), input.scalar_type() == torch::kBFloat16 ? ESMOE_IN_BF16 : ESMOE_IN_FP16,
                                     quant_output.data_ptr(), scales.data_ptr<float>(), (long)total_rows, (int)k,
                                     current_stream(input));
  check_rc(rc, "es_fp8_quant_act_1x128");
}

// Fused SwiGLU + 1x128 quantisation (no counterpart in the reference).
void es_swiglu_quant_1x128(const torch::Tensor& input, torch::Tensor& quant_output, torch::Tensor& scales) {
  TORCH_CHECK(input.dim() == 2 && input.is_contiguous(), "input must be a contiguous 2D tensor");
  TORCH_CHECK(input.size(1) % 256 == 0, "the row length must be 2 * inter with inter aligned to 128");
  TORCH_CHECK(input.scalar_type() == torch::kBFloat16 || input.scalar_type() == torch::kHalf,
              "dtype must be kFloat16 or kBFloat16");
  const int64_t rows = input.size(0), inter = input.size(1) / 2;
  TORCH_CHECK(quant_output.is_contiguous() && quant_output.element_size() == 1 && quant_output.numel() == rows * inter,
              "quant_output must be a contiguous 1-byte tensor of rows * inter elements");
  TORCH_CHECK(scales.is_contiguous() && scales.scalar_type() == torch::kFloat32 && scales.numel() == rows * (inter / 128),
              "scales must be a contiguous float32 tensor of rows * inter / 128 elements");
  require_device(input, "es_swiglu_quant_1x128");
  TORCH_CHECK(quant_output.device() == input.device() && scales.device() == input.device(),
              "all tensors must be on the same device");
  if (rows == 0) return;
  c10::DeviceGuard guard(input.device());
  int rc = esmoe_swiglu_quant_1x128(input.data_ptr(), input.scalar_type() == torch::kBFloat16 ? ESMOE_IN_BF16 : ESMOE_IN_FP16,
                                    quant_output.data_ptr(), scales.data_ptr<float>(), (long)rows, (int)inter,
                                    current_stream(input));
  check_rc(rc, "es_swiglu_quant_1x128");
}

// Routing metadata and row packing on the device (no counterpart among the reference's operators; its
// callers build these tensors on the host, benchmark/benchmark_es_fp8_blockwise_moe.py:44-56,72-88).
std::tuple<torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor> es_route_metadata(const torch::Tensor& topk_ids,
                                                                                         int64_t first_expert,
                                                                                         int64_t num_experts, int64_t n,
                                                                                         int64_t k) {
  TORCH_CHECK(topk_ids.scalar_type() == torch::kInt32 && topk_ids.is_contiguous(), "topk_ids must be contiguous int32");
  TORCH_CHECK(num_experts >= 1 && num_experts <= ESMOE_MAX_EXPERTS, "num_experts must be in [1, 1024]");
  require_device(topk_ids, "es_route_metadata");
  c10::DeviceGuard guard(topk_ids.device());
  const int64_t pairs = topk_ids.numel();
  auto opts = topk_ids.options();
  torch::Tensor ps = torch::empty({num_experts, 3}, opts), eo = torch::empty({num_experts + 1}, opts),
                bso = torch::empty({num_experts + 1}, opts), dst = torch::empty({pairs}, opts);
  torch::Tensor ws = torch::empty({(int64_t)esmoe_route_workspace_bytes((long)pairs, (int)num_experts)},
                                  opts.dtype(torch::kUInt8));
  int rc = esmoe_route_metadata(pairs ? topk_ids.data_ptr<int32_t>() : nullptr, (long)pairs, (int)first_expert,
                                (int)num_experts, (int)n, (int)k, ps.data_ptr<int32_t>(), eo.data_ptr<int32_t>(),
                                bso.data_ptr<int32_t>(), pairs ? dst.data_ptr<int32_t>() : nullptr, ws.data_ptr(),
                                ws.nbytes(), current_stream(topk_ids));
  check_rc(rc, "es_route_metadata");
  return {ps, eo, bso, dst};
}

void es_permute_rows(const torch::Tensor& input, const torch::Tensor& dst_row, int64_t topk, torch::Tensor& output) {
  TORCH_CHECK(input.dim() == 2 && output.dim() == 2 && input.is_contiguous() && output.is_contiguous(),
              "input and output must be contiguous 2D tensors");
  TORCH_CHECK(input.size(1) == output.size(1) && input.scalar_type() == output.scalar_type(),
              "input and output must have the same row length and dtype");
  TORCH_CHECK(dst_row.scalar_type() == torch::kInt32 && dst_row.is_contiguous(), "dst_row must be contiguous int32");
  TORCH_CHECK(topk >= 1 && dst_row.numel() == input.size(0) * topk, "dst_row must have rows * topk entries");
  const int64_t row_bytes = input.size(1) * input.element_size();
  TORCH_CHECK(row_bytes % 16 == 0, "rows must be a multiple of 16 bytes");
  require_device(input, "es_permute_rows");
  TORCH_CHECK(dst_row.device() == input.device() && output.device() == input.device(),
              "all tensors must be on the same device");
  if (dst_row.numel() == 0) return;
  c10::DeviceGuard guard(input.device());
  int rc = esmoe_permute_rows(input.data_ptr(), dst_row.data_ptr<int32_t>(), (long)dst_row.numel(), (int)topk,
                              (long)row_bytes, output.data_ptr(), current_stream(input));
  check_rc(rc, "es_permute_rows");
}

// Weight-side companion of es_fp8_quant_act_1x128: per_block_cast_to_fp8
// (test/test_es_grouped_gemm.py:47-59) on the physical [..., N, K] weight tensor.
void es_fp8_quant_weight_128x128(const torch::Tensor& input, torch::Tensor& quant_output, torch::Tensor& scales) {
  TORCH_CHECK(input.dim() >= 2, "input must have at least 2 dimensions");
  const int64_t k = input.size(-1), n = input.size(-2);
  TORCH_CHECK(k % 128 == 0 && n % 128 == 0, "n and k must align to 128");
  TORCH_CHECK(input.scalar_type() == torch::kBFloat16 || input.scalar_type() == torch::kHalf,
              "dtype must be kFloat16 or kBFloat16");
  TORCH_CHECK(input.is_contiguous(), "input must be contiguous");
  const int64_t rows = input.numel() / k;
  TORCH_CHECK(quant_output.is_contiguous() && quant_output.element_size() == 1 && quant_output.numel() == rows * k,
              "quant_output must be a contiguous 1-byte tensor with the input's number of elements");
  TORCH_CHECK(scales.is_contiguous() && scales.scalar_type() == torch::kFloat32 &&
                  scales.numel() == (rows / 128) * (k / 128),
              "scales must be a contiguous float32 tensor with one element per 128x128 block");
  require_device(input, "es_fp8_quant_weight_128x128");
  TORCH_CHECK(quant_output.device() == input.device() && scales.device() == input.device(),
              "all tensors must be on the same device");
  if (rows == 0) return;
  c10::DeviceGuard guard(input.device());
  int rc = esmoe_fp8_quant_weight_128x128(input.data_ptr(),
                                          input.scalar_type() == torch::kBFloat16 ? ESMOE_IN_BF16 : ESMOE_IN_FP16,
                                          quant_output.data_ptr(), scales.data_ptr<float>(), (long)rows, (int)k,
                                          current_stream(input));
  check_rc(rc, "es_fp8_quant_weight_128x128");
}

// Fused SwiGLU + MXFP8 grouped quantisation: the gate_up output [rows, 2*inter] -> the down projection's operands
// (no counterpart in the reference; metadata and output layouts as es_sm100_mxfp8_blockscaled_grouped_quant with K = inter).
void es_swiglu_mxfp8_grouped_quant(const torch::Tensor& input, const torch::Tensor& problem_sizes,
                                   const torch::Tensor& expert_offsets, const torch::Tensor& blockscale_offsets,
                                   torch::Tensor& quant_output, torch::Tensor& scale_factor) {
  TORCH_CHECK(input.dim() == 2 && input.is_contiguous(), "input must be a contiguous 2D tensor");
  TORCH_CHECK(input.size(1) % 256 == 0, "the row length must be 2 * inter with inter aligned to 128");
  TORCH_CHECK(input.scalar_type() == torch::kBFloat16 || input.scalar_type() == torch::kHalf,
              "dtype must be kFloat16 or kBFloat16");
  TORCH_CHECK(problem_sizes.dim() == 2 && problem_sizes.size(1) == 3, "problem_sizes must be (groups, 3)");
  const int64_t groups = problem_sizes.size(0);
  TORCH_CHECK(expert_offsets.dim() == 1 && expert_offsets.size(0) == groups && blockscale_offsets.dim() == 1 &&
                  blockscale_offsets.size(0) == groups,
              "expert_offsets and blockscale_offsets must be 1D and have size equal to the number of groups");
  TORCH_CHECK(problem_sizes.dtype() == torch::kInt32 && expert_offsets.dtype() == torch::kInt32 &&
                  blockscale_offsets.dtype() == torch::kInt32,
              "problem_sizes, expert_offsets and blockscale_offsets must be int32");
  TORCH_CHECK(groups >= 1 && groups <= ESMOE_MAX_EXPERTS, "number of groups must be in [1, 1024]");
  const int64_t total_rows = input.size(0), inter = input.size(1) / 2;
  TORCH_CHECK(quant_output.is_contiguous() && (int64_t)quant_output.nbytes() >= total_rows * inter,
              "quant_output must be contiguous and hold at least rows * inter bytes");
  TORCH_CHECK(scale_factor.is_contiguous() && scale_factor.element_size() == 1,
              "scale_factor must be a contiguous 1-byte tensor");
  const int64_t sf_rows = (scale_factor.numel() / (inter / 32)) / 128 * 128;
  TORCH_CHECK(sf_rows >= (total_rows + 127) / 128 * 128,
              "scale_factor is smaller than the rows rounded up to 128 times inter / 32 bytes");
  TORCH_CHECK(total_rows < (int64_t(1) << 31) && sf_rows < (int64_t(1) << 31), "tensor too large");
  require_device(input, "es_swiglu_mxfp8_grouped_quant");
  for (const torch::Tensor* t : {&problem_sizes, &expert_offsets, &blockscale_offsets, (const torch::Tensor*)&quant_output,
                                 (const torch::Tensor*)&scale_factor}) {
    TORCH_CHECK(t->device() == input.device(), "all tensors must be on the same device");
  }
  TORCH_CHECK(problem_sizes.is_contiguous() && expert_offsets.is_contiguous() && blockscale_offsets.is_contiguous(),
              "metadata tensors must be contiguous");
  if (total_rows == 0) return;
  c10::DeviceGuard guard(input.device());
  int rc = esmoe_swiglu_mxfp8_grouped_quant(
      input.data_ptr(), input.scalar_type() == torch::kBFloat16 ? ESMOE_IN_BF16 : ESMOE_IN_FP16,
      problem_sizes.data_ptr<int32_t>(), expert_offsets.data_ptr<int32_t>(), blockscale_offsets.data_ptr<int32_t>(),
      quant_output.data_ptr(), (uint8_t*)scale_factor.data_ptr(), (int)groups, (int)total_rows, (int)sf_rows, (int)inter,
      current_stream(input));
  check_rc(rc, "es_swiglu_mxfp8_grouped_quant");
}

// MXFP8 quantisation of a weight tensor [..., N, K] (no counterpart among the reference's operators: its test
// passes the activation operator a transposed problem list, test/test_es_sm100_mxfp8_blockscaled_grouped_quant.py:87-96).
void es_mxfp8_quant_weight(const torch::Tensor& input, torch::Tensor& quant_output, torch::Tensor& scale_factor) {
  TORCH_CHECK(input.dim() >= 2, "input must have at least 2 dimensions");
  const int64_t k = input.size(-1), n = input.size(-2);
  TORCH_CHECK(k % 128 == 0 && n % 128 == 0, "n and k must align to 128");
  TORCH_CHECK(input.scalar_type() == torch::kBFloat16 || input.scalar_type() == torch::kHalf,
              "dtype must be kFloat16 or kBFloat16");
  TORCH_CHECK(input.is_contiguous(), "input must be contiguous");
  const int64_t rows = input.numel() / k;
  TORCH_CHECK(quant_output.is_contiguous() && quant_output.element_size() == 1 && quant_output.numel() == rows * k,
              "quant_output must be a contiguous 1-byte tensor with the input's number of elements");
  TORCH_CHECK(scale_factor.is_contiguous() && scale_factor.element_size() == 1 && scale_factor.numel() == rows * (k / 32),
              "scale_factor must be a contiguous 1-byte tensor of rows * k / 32 elements");
  require_device(input, "es_mxfp8_quant_weight");
  TORCH_CHECK(quant_output.device() == input.device() && scale_factor.device() == input.device(),
              "all tensors must be on the same device");
  if (rows == 0) return;
  c10::DeviceGuard guard(input.device());
  int rc = esmoe_mxfp8_quant_weight(input.data_ptr(), input.scalar_type() == torch::kBFloat16 ? ESMOE_IN_BF16 : ESMOE_IN_FP16,
                                    quant_output.data_ptr(), (uint8_t*)scale_factor.data_ptr(), (long)rows, (int)k,
                                    current_stream(input));
  check_rc(rc, "es_mxfp8_quant_weight");
}

TORCH_LIBRARY(expert_specialization, m) {
  m.def(
      "es_fp8_blockwise_scaled_grouped_mm(Tensor output, Tensor a, Tensor b, Tensor scales_a, Tensor scales_b, Tensor "
      "stride_a, Tensor stride_b, Tensor stride_d, Tensor problem_sizes, Tensor expert_offsets, Tensor workspace) -> "
      "()");
  m.def(
      "es_sm100_mxfp8_blockscaled_grouped_mm(Tensor a, Tensor b, Tensor sfa, Tensor sfb, Tensor d, Tensor "
      "problem_sizes, Tensor expert_offsets, Tensor blockscale_offsets) -> ()");
  m.def(
      "es_sm100_mxfp8_blockscaled_grouped_quant(Tensor input, Tensor problem_sizes, Tensor expert_offsets, Tensor "
      "blockscale_offsets, Tensor quant_output, Tensor scale_factor) -> () ");
  m.def(
      "es_fp8_blockwise_scaled_grouped_mm_swiglu_quant(Tensor quant_output, Tensor scales_out, Tensor a, Tensor b, Tensor "
      "scales_a, Tensor scales_b, Tensor problem_sizes, Tensor expert_offsets, Tensor workspace, bool mid_dtype_bf16) -> ()");
  m.def("es_fp8_quant_act_1x128(Tensor input, Tensor quant_output, Tensor scales) -> ()");
  m.def("es_fp8_quant_weight_128x128(Tensor input, Tensor quant_output, Tensor scales) -> ()");
  m.def("es_swiglu_quant_1x128(Tensor input, Tensor quant_output, Tensor scales) -> ()");
  m.def(
      "es_mxfp8_blockscaled_grouped_mm_swiglu_quant(Tensor quant_output, Tensor scale_factor, Tensor a, Tensor b, Tensor "
      "sfa, Tensor sfb, Tensor problem_sizes, Tensor expert_offsets, Tensor blockscale_offsets, bool mid_dtype_bf16) -> ()");
  m.def(
      "es_swiglu_mxfp8_grouped_quant(Tensor input, Tensor problem_sizes, Tensor expert_offsets, Tensor "
      "blockscale_offsets, Tensor quant_output, Tensor scale_factor) -> ()");
  m.def("es_mxfp8_quant_weight(Tensor input, Tensor quant_output, Tensor scale_factor) -> ()");
  m.def("es_route_metadata(Tensor topk_ids, int first_expert, int num_experts, int n, int k) -> (Tensor, Tensor, Tensor, Tensor)");
  m.def("es_permute_rows(Tensor input, Tensor dst_row, int topk, Tensor output) -> ()");
}

TORCH_LIBRARY_IMPL(expert_specialization, CUDA, m) {
  m.impl("es_fp8_blockwise_scaled_grouped_mm", &es_fp8_blockwise_scaled_grouped_mm);
  m.impl("es_sm100_mxfp8_blockscaled_grouped_mm", &es_sm100_mxfp8_blockscaled_grouped_mm);
  m.impl("es_sm100_mxfp8_blockscaled_grouped_quant", &es_sm100_mxfp8_blockscaled_grouped_quant);
  m.impl("es_fp8_blockwise_scaled_grouped_mm_swiglu_quant", &es_fp8_blockwise_scaled_grouped_mm_swiglu_quant);
  m.impl("es_fp8_quant_act_1x128", &es_fp8_quant_act_1x128);
  m.impl("es_fp8_quant_weight_128x128", &es_fp8_quant_weight_128x128);
  m.impl("es_swiglu_quant_1x128", &es_swiglu_quant_1x128);
  m.impl("es_mxfp8_blockscaled_grouped_mm_swiglu_quant", &es_mxfp8_blockscaled_grouped_mm_swiglu_quant);
  m.impl("es_swiglu_mxfp8_grouped_quant", &es_swiglu_mxfp8_grouped_quant);
  m.impl("es_mxfp8_quant_weight", &es_mxfp8_quant_weight);
  m.impl("es_route_metadata", &es_route_metadata);
  m.impl("es_permute_rows", &es_permute_rows);
}

// Same functions on the CPU key: the checks run, then require_device() raises.
TORCH_LIBRARY_IMPL(expert_specialization, CPU, m) {
  m.impl("es_fp8_blockwise_scaled_grouped_mm", &es_fp8_blockwise_scaled_grouped_mm);
  m.impl("es_sm100_mxfp8_blockscaled_grouped_mm", &es_sm100_mxfp8_blockscaled_grouped_mm);
  m.impl("es_sm100_mxfp8_blockscaled_grouped_quant", &es_sm100_mxfp8_blockscaled_grouped_quant);
  m.impl("es_fp8_blockwise_scaled_grouped_mm_swiglu_quant", &es_fp8_blockwise_scaled_grouped_mm_swiglu_quant);
  m.impl("es_fp8_quant_act_1x128", &es_fp8_quant_act_1x128);
  m.impl("es_fp8_quant_weight_128x128", &es_fp8_quant_weight_128x128);
  m.impl("es_swiglu_quant_1x128", &es_swiglu_quant_1x128);
  m.impl("es_mxfp8_blockscaled_grouped_mm_swiglu_quant", &es_mxfp8_blockscaled_grouped_mm_swiglu_quant);
  m.impl("es_swiglu_mxfp8_grouped_quant", &es_swiglu_mxfp8_grouped_quant);
  m.impl("es_mxfp8_quant_weight", &es_mxfp8_quant_weight);
  m.impl("es_route_metadata", &es_route_metadata);
  m.impl("es_permute_rows", &es_permute_rows);
}
