// E8M0 scale code of an MXFP8 1x32 block, shared by the quantisation kernels and the fused GEMM epilogue.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace esmoe {

// E8M0 code of the smallest power of two >= amax / 448 (amax >= 0, finite), from the bit pattern of amax:
// 448 = 1.75 * 2^8  =>  code = exponent(amax) - 8 + (mantissa > .75).  Equals the float route of
// cvt_warp_fp16_to_mxfp8 (expert_specialization/csrc/cuda/es_sm100_mxfp8_blockscaled_group_quant.cuh:36-134)
// with a correctly rounded 1/448.
__device__ __forceinline__ int mx_scale_code(float amax) {
  uint32_t bits = __builtin_bit_cast(uint32_t, amax);
  int code = (int)((bits >> 23) & 0xff) - 8 + ((bits & 0x7fffffu) > 0x600000u ? 1 : 0);
  code = code < 0 ? 0 : (code > 254 ? 254 : code);
  return amax == 0.f ? 0 : code;
}

// Multiplier 2^(127 - code) that maps the block into e4m3 range (0 for an all-zero block).
__device__ __forceinline__ float mx_scale_inverse(float amax, int code) {
  return amax == 0.f ? 0.f : __builtin_bit_cast(float, (uint32_t)(254 - code) << 23);
}

}  // namespace esmoe
