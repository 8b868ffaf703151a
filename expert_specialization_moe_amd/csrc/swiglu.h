// silu(gate) * up in fp32, the one form every SwiGLU path of this library uses (the stand-alone fused
// quantisation kernels and the GEMM epilogue), so that their results are identical byte for byte.
// silu(g) = g / (1 + exp(-g)) through the hardware's base-2 exponential and reciprocal (about 1 ulp each):
// the product is rounded to bf16/fp16 right after, which hides those ulps in all but ~1e-4 of the elements;
// the library's exp and an IEEE division cost four times the instructions and made the kernels ALU-bound.
#pragma once
#include <hip/hip_runtime.h>

namespace esmoe {

__device__ __forceinline__ float swiglu_f32(float gate, float up) {
  const float e = __builtin_amdgcn_exp2f(gate * -1.44269504088896340736f);   // exp(-gate); overflows to +inf
  return (gate * __builtin_amdgcn_rcpf(1.0f + e)) * up;
}

}  // namespace esmoe
