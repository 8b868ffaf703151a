// FP8 operand quantisers for gfx950 (activations 1x128, weights 128x128).
//
// Activations: bf16/fp16 rows -> e4m3fn bytes + one fp32 scale
// per 128-wide block of a row (the operand format of the FP8-blockwise grouped GEMM).
//
// Arithmetic follows the torch helper the reference's callers use, per_token_cast_to_fp8
// (test/test_es_grouped_gemm.py:36-44), rounding for rounding:
//   amax  = max(|x| over the block, 1e-4)              (fp32)
//   mult  = fl(fl(1 / amax) * 448)                     (torch evaluates 448.0 / t as reciprocal(t) * 448)
//   q     = e4m3fn_rne(fl(float(x) * mult))
//   scale = fl(amax * fl(1 / 448))                     (how torch divides a GPU tensor by a Python scalar;
//                                                       the CPU path's true division differs by one ulp
//                                                       for some values)
// [M, K] row-major with K % 128 == 0 makes the blocks one flat sequence: block b covers elements
// [128 b, 128 b + 128) of input and output and owns scales[b], so the kernel is one-dimensional.
// 16 lanes take one block (16 bytes of input each, a 256-byte coalesced segment); the block maximum
// is reduced with four lane swaps.  Pure streaming: 2 + 1 + 4/128 bytes per element.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "swiglu.h"

namespace esmoe {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v2i __attribute__((ext_vector_type(2)));

constexpr int kActQuantThreads = 256;
constexpr int kActQuantUnroll = 4;   // 16-byte loads in flight per lane

template <bool FP16>
__global__ void __launch_bounds__(kActQuantThreads) __attribute__((amdgpu_waves_per_eu(6, 8)))
fp8_quant_act_kernel(const uint16_t* __restrict__ in, uint8_t* __restrict__ q, float* __restrict__ scales, long chunks) {
  // chunk c = 8 consecutive elements; 16 consecutive chunks form one 1x128 block
  const long first = ((long)blockIdx.x * kActQuantUnroll) * kActQuantThreads + threadIdx.x;
  v4i raw[kActQuantUnroll];
#pragma unroll
  for (int u = 0; u < kActQuantUnroll; u++) {
    const long c = first + (long)u * kActQuantThreads;
    raw[u] = v4i{0, 0, 0, 0};
    if (c < chunks) raw[u] = __builtin_nontemporal_load((const v4i*)(in + c * 8));
  }
#pragma unroll
  for (int u = 0; u < kActQuantUnroll; u++) {
    const long c = first + (long)u * kActQuantThreads;
    float x[8];
#pragma unroll
    for (int i = 0; i < 4; i++) {
      uint32_t w = (uint32_t)raw[u][i];
      if constexpr (FP16) {
        x[2 * i] = (float)__builtin_bit_cast(_Float16, (uint16_t)(w & 0xffffu));
        x[2 * i + 1] = (float)__builtin_bit_cast(_Float16, (uint16_t)(w >> 16));
      } else {
        x[2 * i] = __builtin_bit_cast(float, w << 16);
        x[2 * i + 1] = __builtin_bit_cast(float, w & 0xffff0000u);
      }
    }
    float amax = 0.f;
#pragma unroll
    for (int i = 0; i < 8; i++) amax = __builtin_fmaxf(amax, __builtin_fabsf(x[i]));
    amax = __builtin_fmaxf(amax, __shfl_xor(amax, 1));
    amax = __builtin_fmaxf(amax, __shfl_xor(amax, 2));
    amax = __builtin_fmaxf(amax, __shfl_xor(amax, 4));
    amax = __builtin_fmaxf(amax, __shfl_xor(amax, 8));
    amax = __builtin_fmaxf(amax, 1e-4f);
    const float mult = (1.0f / amax) * 448.0f;   // two roundings, as torch does
    float y[8];
#pragma unroll
    for (int i = 0; i < 8; i++) y[i] = __builtin_amdgcn_fmed3f(x[i] * mult, -448.f, 448.f);
    int w0 = __builtin_amdgcn_cvt_pk_fp8_f32(y[0], y[1], 0, false);
    w0 = __builtin_amdgcn_cvt_pk_fp8_f32(y[2], y[3], w0, true);
    int w1 = __builtin_amdgcn_cvt_pk_fp8_f32(y[4], y[5], 0, false);
    w1 = __builtin_amdgcn_cvt_pk_fp8_f32(y[6], y[7], w1, true);
    if (c < chunks) {
      __builtin_nontemporal_store(v2i{w0, w1}, (v2i*)(q + c * 8));
      if ((threadIdx.x & 15) == 0) scales[c >> 4] = amax * (1.0f / 448.0f);
    }
  }
}

// Fused SwiGLU + 1x128 quantisation: the glue between the gate_up and the down projection of an
// expert MLP.  in [M, 2*I]: gate = in[:, :I], up = in[:, I:];  h = cast(silu(gate) * up) with the
// product formed in fp32 and rounded once to the input type (what a fused silu-and-mul kernel
// stores), silu(x) = x / (1 + exp(-x)); then h is quantised exactly as fp8_quant_act_kernel does.
// Saves one write and one read of the [M, I] intermediate.  No counterpart in the reference.
template <bool FP16>
__global__ void __launch_bounds__(kActQuantThreads) __attribute__((amdgpu_waves_per_eu(4, 8)))
swiglu_quant_kernel(const uint16_t* __restrict__ in, uint8_t* __restrict__ q, float* __restrict__ scales, long chunks,
                    int inter) {
  const int cpr = inter >> 3;   // 8-element chunks per output row
  const long first = ((long)blockIdx.x * 2) * kActQuantThreads + threadIdx.x;
  v4i rg[2], ru[2];
#pragma unroll
  for (int u = 0; u < 2; u++) {
    const long c = first + (long)u * kActQuantThreads;
    rg[u] = v4i{0, 0, 0, 0};
    ru[u] = v4i{0, 0, 0, 0};
    if (c < chunks) {
      const long row = c / cpr;
      const long col = (c - row * cpr) * 8;
      const uint16_t* g = in + row * 2 * inter + col;
      rg[u] = __builtin_nontemporal_load((const v4i*)g);
      ru[u] = __builtin_nontemporal_load((const v4i*)(g + inter));
    }
  }
#pragma unroll
  for (int u = 0; u < 2; u++) {
    const long c = first + (long)u * kActQuantThreads;
    float x[8];
#pragma unroll
    for (int i = 0; i < 4; i++) {
      const uint32_t wg = (uint32_t)rg[u][i], wu = (uint32_t)ru[u][i];
      float g0, g1, u0, u1;
      if constexpr (FP16) {
        g0 = (float)__builtin_bit_cast(_Float16, (uint16_t)(wg & 0xffffu));
        g1 = (float)__builtin_bit_cast(_Float16, (uint16_t)(wg >> 16));
        u0 = (float)__builtin_bit_cast(_Float16, (uint16_t)(wu & 0xffffu));
        u1 = (float)__builtin_bit_cast(_Float16, (uint16_t)(wu >> 16));
      } else {
        g0 = __builtin_bit_cast(float, wg << 16);
        g1 = __builtin_bit_cast(float, wg & 0xffff0000u);
        u0 = __builtin_bit_cast(float, wu << 16);
        u1 = __builtin_bit_cast(float, wu & 0xffff0000u);
      }
      const float h0 = swiglu_f32(g0, u0), h1 = swiglu_f32(g1, u1);
      if constexpr (FP16) {
        x[2 * i] = (float)(_Float16)h0;
        x[2 * i + 1] = (float)(_Float16)h1;
      } else {
        x[2 * i] = (float)(__bf16)h0;
        x[2 * i + 1] = (float)(__bf16)h1;
      }
    }
    float amax = 0.f;
#pragma unroll
    for (int i = 0; i < 8; i++) amax = __builtin_fmaxf(amax, __builtin_fabsf(x[i]));
    amax = __builtin_fmaxf(amax, __shfl_xor(amax, 1));
    amax = __builtin_fmaxf(amax, __shfl_xor(amax, 2));
    amax = __builtin_fmaxf(amax, __shfl_xor(amax, 4));
    amax = __builtin_fmaxf(amax, __shfl_xor(amax, 8));
    amax = __builtin_fmaxf(amax, 1e-4f);
    const float mult = (1.0f / amax) * 448.0f;
    float y[8];
#pragma unroll
    for (int i = 0; i < 8; i++) y[i] = __builtin_amdgcn_fmed3f(x[i] * mult, -448.f, 448.f);
    int w0 = __builtin_amdgcn_cvt_pk_fp8_f32(y[0], y[1], 0, false);
    w0 = __builtin_amdgcn_cvt_pk_fp8_f32(y[2], y[3], w0, true);
    int w1 = __builtin_amdgcn_cvt_pk_fp8_f32(y[4], y[5], 0, false);
    w1 = __builtin_amdgcn_cvt_pk_fp8_f32(y[6], y[7], w1, true);
    if (c < chunks) {
      __builtin_nontemporal_store(v2i{w0, w1}, (v2i*)(q + c * 8));
      if ((threadIdx.x & 15) == 0) scales[c >> 4] = amax * (1.0f / 448.0f);
    }
  }
}

// 128x128 weight quantisation: the torch helper per_block_cast_to_fp8 (test/test_es_grouped_gemm.py:47-59)
// applied to the physical [rows, K] matrix (rows = E * N), which equals the reference's route through
// the transposed (K, N) view (:127,132-134).  One workgroup per pair of 128x128 blocks that are neighbours
// along K: 32 lanes per 512-byte row segment (which streams 8 % faster than one block's 256 bytes), 8 passes of 16
// rows; each block's maximum goes through lane swaps and a few words of LDS.
constexpr int kWeightQuantThreads = 512;
template <bool FP16>
__global__ void __launch_bounds__(kWeightQuantThreads) __attribute__((amdgpu_waves_per_eu(4, 8)))
fp8_quant_weight_kernel(const uint16_t* __restrict__ in, uint8_t* __restrict__ q, float* __restrict__ scales, int k) {
  // Two 128x128 blocks side by side per workgroup (the second absent when k % 256 == 128): 32 lanes read one 512-byte
  // row segment, lanes 0-15 of it the left block and 16-31 the right one; a wavefront holds two rows.
  __shared__ float s_max[kWeightQuantThreads / 64][2];
  const int kt = blockIdx.x, rb = blockIdx.y, tid = threadIdx.x;
  const int sub = tid & 31, rrow = tid >> 5, half = sub >> 4;
  const bool col_ok = kt * 256 + sub * 8 < k;
  const long base = ((long)rb * 128 + rrow) * k + kt * 256 + sub * 8;
  v4i raw[8];
#pragma unroll
  for (int p = 0; p < 8; p++) {
    raw[p] = v4i{0, 0, 0, 0};
    if (col_ok) raw[p] = __builtin_nontemporal_load((const v4i*)(in + base + (long)p * 16 * k));
  }
  float amax = 0.f;
#pragma unroll
  for (int p = 0; p < 8; p++) {
#pragma unroll
    for (int i = 0; i < 4; i++) {
      uint32_t w = (uint32_t)raw[p][i];
      float a, b;
      if constexpr (FP16) {
        a = (float)__builtin_bit_cast(_Float16, (uint16_t)(w & 0xffffu));
        b = (float)__builtin_bit_cast(_Float16, (uint16_t)(w >> 16));
      } else {
        a = __builtin_bit_cast(float, w << 16);
        b = __builtin_bit_cast(float, w & 0xffff0000u);
      }
      amax = __builtin_fmaxf(amax, __builtin_fmaxf(__builtin_fabsf(a), __builtin_fabsf(b)));
    }
  }
  // over the 16 lanes of the block's row segment, then over the wavefront's two rows (lane ^ 32: same block)
  amax = __builtin_fmaxf(amax, __shfl_xor(amax, 1));
  amax = __builtin_fmaxf(amax, __shfl_xor(amax, 2));
  amax = __builtin_fmaxf(amax, __shfl_xor(amax, 4));
  amax = __builtin_fmaxf(amax, __shfl_xor(amax, 8));
  amax = __builtin_fmaxf(amax, __shfl_xor(amax, 32));
  if ((tid & 47) == 0) s_max[tid >> 6][half] = amax;   // lanes 0 and 16 of every wavefront
  __syncthreads();
  amax = s_max[0][half];
#pragma unroll
  for (int w = 1; w < kWeightQuantThreads / 64; w++) amax = __builtin_fmaxf(amax, s_max[w][half]);
  amax = __builtin_fmaxf(amax, 1e-4f);
  const float mult = (1.0f / amax) * 448.0f;
#pragma unroll
  for (int p = 0; p < 8; p++) {
    float x[8];
#pragma unroll
    for (int i = 0; i < 4; i++) {
      uint32_t w = (uint32_t)raw[p][i];
      if constexpr (FP16) {
        x[2 * i] = (float)__builtin_bit_cast(_Float16, (uint16_t)(w & 0xffffu));
        x[2 * i + 1] = (float)__builtin_bit_cast(_Float16, (uint16_t)(w >> 16));
      } else {
        x[2 * i] = __builtin_bit_cast(float, w << 16);
        x[2 * i + 1] = __builtin_bit_cast(float, w & 0xffff0000u);
      }
    }
    float y[8];
#pragma unroll
    for (int i = 0; i < 8; i++) y[i] = __builtin_amdgcn_fmed3f(x[i] * mult, -448.f, 448.f);
    int w0 = __builtin_amdgcn_cvt_pk_fp8_f32(y[0], y[1], 0, false);
    w0 = __builtin_amdgcn_cvt_pk_fp8_f32(y[2], y[3], w0, true);
    int w1 = __builtin_amdgcn_cvt_pk_fp8_f32(y[4], y[5], 0, false);
    w1 = __builtin_amdgcn_cvt_pk_fp8_f32(y[6], y[7], w1, true);
    if (col_ok) __builtin_nontemporal_store(v2i{w0, w1}, (v2i*)(q + base + (long)p * 16 * k));
  }
  if ((tid == 0 || tid == 16) && col_ok) scales[(long)rb * (k >> 7) + kt * 2 + half] = amax * (1.0f / 448.0f);
}

}  // namespace esmoe

extern "C" int esmoe_launch_fp8_quant_weight(const void* in, int in_dtype, void* q, float* scales, long rows, int k,
                                             hipStream_t stream) {
  using namespace esmoe;
  if (rows == 0) return 0;
  dim3 grid((k + 255) / 256, (unsigned)(rows / 128));
  if (in_dtype == 1)
    hipLaunchKernelGGL(fp8_quant_weight_kernel<true>, grid, dim3(kWeightQuantThreads), 0, stream, (const uint16_t*)in,
                       (uint8_t*)q, scales, k);
  else
    hipLaunchKernelGGL(fp8_quant_weight_kernel<false>, grid, dim3(kWeightQuantThreads), 0, stream, (const uint16_t*)in,
                       (uint8_t*)q, scales, k);
  return (int)hipGetLastError();
}

extern "C" int esmoe_launch_swiglu_quant(const void* in, int in_dtype, void* q, float* scales, long total_rows, int inter,
                                        hipStream_t stream) {
  using namespace esmoe;
  const long chunks = total_rows * (long)inter / 8;
  if (chunks == 0) return 0;
  const long per_wg = (long)kActQuantThreads * 2;
  const long grid = (chunks + per_wg - 1) / per_wg;
  if (in_dtype == 1)
    hipLaunchKernelGGL(swiglu_quant_kernel<true>, dim3((unsigned)grid), dim3(kActQuantThreads), 0, stream,
                       (const uint16_t*)in, (uint8_t*)q, scales, chunks, inter);
  else
    hipLaunchKernelGGL(swiglu_quant_kernel<false>, dim3((unsigned)grid), dim3(kActQuantThreads), 0, stream,
                       (const uint16_t*)in, (uint8_t*)q, scales, chunks, inter);
  return (int)hipGetLastError();
}

extern "C" int esmoe_launch_fp8_quant_act(const void* in, int in_dtype, void* q, float* scales, long total_rows, int k,
                                          hipStream_t stream) {
  using namespace esmoe;
  const long chunks = total_rows * (long)k / 8;
  if (chunks == 0) return 0;
  const long per_wg = (long)kActQuantThreads * kActQuantUnroll;
  const long grid = (chunks + per_wg - 1) / per_wg;
  if (in_dtype == 1)
    hipLaunchKernelGGL(fp8_quant_act_kernel<true>, dim3((unsigned)grid), dim3(kActQuantThreads), 0, stream,
                       (const uint16_t*)in, (uint8_t*)q, scales, chunks);
  else
    hipLaunchKernelGGL(fp8_quant_act_kernel<false>, dim3((unsigned)grid), dim3(kActQuantThreads), 0, stream,
                       (const uint16_t*)in, (uint8_t*)q, scales, chunks);
  return (int)hipGetLastError();
}
