// Kernel argument block shared by the host launcher and the grouped GEMM kernels.
#pragma once
#include <stdint.h>

#include "schedule.h"

namespace esmoe {

struct GemmArgs {
  const void* a;        // [total_rows, K] e4m3
  const void* b;        // [E, N, K] e4m3
  const float* sa;      // fp8-blockwise: [total_rows, K/128]
  const float* sb;      // fp8-blockwise: [E, N/128, K/128]
  const uint8_t* sfa;   // mxfp8: swizzled E8M0, expert base blockscale_offsets[e] * K/32
  const uint8_t* sfb;   // mxfp8: swizzled E8M0, expert base e * N * K/32
  void* out;            // [total_rows, N]
  void* q_out;          // fused SwiGLU + quantisation: e4m3 [total_rows, N/2]; null = plain projection
  float* scales_out;    //   fp8-blockwise: its fp32 scales [total_rows, N/256]
  uint8_t* sf_out;      //   mxfp8: its swizzled E8M0 scales, expert base blockscale_offsets[e] * N/64
  const int32_t* problem_sizes;
  const int32_t* expert_offsets;
  const int32_t* blockscale_offsets;
  int32_t* ws;          // schedule workspace, ws_words(num_experts) int32
  int num_experts;
  int total_rows;
  int n;
  int k;
  int out_dtype;        // 0 bf16, 1 fp16
  int self_schedule;    // 1: no schedule kernel ran; ws counters are zero and every workgroup builds the records itself
  SchedPolicy policy;
};

}  // namespace esmoe
