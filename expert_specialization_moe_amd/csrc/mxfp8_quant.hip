// MXFP8 grouped quantisation for gfx950: bf16/fp16 rows -> e4m3 bytes + swizzled E8M0 scales.
//
// Arithmetic follows cvt_warp_fp16_to_mxfp8
// (expert_specialization/csrc/cuda/es_sm100_mxfp8_blockscaled_group_quant.cuh:36-134):
// per 1x32 block  amax = max|x|,  scale = smallest power of two >= amax/448,
// q = e4m3_rne(x / scale).  The scale exponent is taken from the bit pattern of
// amax (448 = 1.75 * 2^8  =>  E = exponent(amax) - 8 + (mantissa > .75)), which equals
// the reference's float route with a correctly rounded 1/448.
//
// Work decomposition: one workgroup per 128 rows of the *scale* row space
// (blockscale_offsets are multiples of 128, so the rows belong to one expert) x 256
// columns (128 in the SwiGLU form).  32 (16) lanes read one row segment (16 bytes each,
// a 512-byte coalesced segment), 4 lanes share one 32-wide block and reduce amax with
// two lane swaps.  The 512-byte scale tiles (128 rows x 4 scale columns, layout
// ((32,4),4):((16,4),1), group_quant.cuh:25; tiles of consecutive 128-column blocks are
// consecutive in memory) are assembled in LDS and written with 16-byte stores.
//
// Two more forms of the same kernel (no counterpart in the reference, which quantises weights by passing
// the activation operator a transposed problem list, test/test_es_sm100_mxfp8_blockscaled_grouped_quant.py:53,87-96,
// and leaves the activation function to its callers):
//   * dense: no metadata, all `dense_rows` rows (a multiple of 128) belong to one problem.  That is the
//     weight tensor [E, N, K] with N % 128 == 0, whose scale layout is the concatenation of the experts';
//   * SwiGLU: the input is the gate_up projection [rows, 2K]; x = silu(gate) * up with gate the first half of
//     a row, the product formed in fp32 and rounded once to the input type, then quantised as above.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "mx_scale.h"
#include "swiglu.h"

namespace esmoe {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v2i __attribute__((ext_vector_type(2)));

// A workgroup covers 128 rows x 256 columns (32 lanes per row segment, 16 rows per pass, 512 threads): 512-byte row
// segments stream 8 % faster than 256-byte ones on the large inputs.  The SwiGLU form, whose inputs are small and whose
// lanes hold twice the registers, keeps 128 columns and 256 threads.
template <bool SWIGLU> constexpr int quant_cols() { return SWIGLU ? 128 : 256; }
template <bool SWIGLU> constexpr int quant_threads() { return quant_cols<SWIGLU>() * 2; }

template <bool FP16>
__device__ __forceinline__ void unpack8(v4i raw, float* x) {
#pragma unroll
  for (int i = 0; i < 4; i++) {
    uint32_t w = (uint32_t)raw[i];
    if constexpr (FP16) {
      x[2 * i] = (float)__builtin_bit_cast(_Float16, (uint16_t)(w & 0xffffu));
      x[2 * i + 1] = (float)__builtin_bit_cast(_Float16, (uint16_t)(w >> 16));
    } else {
      x[2 * i] = __builtin_bit_cast(float, w << 16);
      x[2 * i + 1] = __builtin_bit_cast(float, w & 0xffff0000u);
    }
  }
}

template <bool FP16>
__device__ __forceinline__ float round_to_input_type(float h) {
  if constexpr (FP16) return (float)(_Float16)h;
  else return (float)(__bf16)h;
}

template <bool FP16, bool SWIGLU>
__global__ void __launch_bounds__(quant_threads<SWIGLU>()) __attribute__((amdgpu_waves_per_eu(SWIGLU ? 4 : 6, 8))) mxfp8_quant_kernel(const uint16_t* __restrict__ in,
                                                                    const int* __restrict__ problem_sizes,
                                                                    const int* __restrict__ expert_offsets,
                                                                    const int* __restrict__ blockscale_offsets,
                                                                    uint8_t* __restrict__ q, uint8_t* __restrict__ sf,
                                                                    int num_experts, int k, long dense_rows) {
  constexpr int kCols = quant_cols<SWIGLU>(), kLanes = kCols / 8, kTiles = kCols / 128;
  __shared__ __attribute__((aligned(16))) uint8_t s_sf[512 * kTiles];   // the 512-byte scale tiles of the workgroup's columns
  const int kt = blockIdx.x;               // tile of kCols columns (the last one may be 128 wide)
  const int sf_row0 = blockIdx.y * 128;    // first row of this tile in scale-row space
  const int tid = threadIdx.x;

  int m_e, r0;
  long row_base, sf_base;
  if (dense_rows > 0) {
    m_e = (int)dense_rows;
    r0 = sf_row0;
    row_base = 0;
    sf_base = 0;
  } else {
    // expert owning scale row sf_row0: last e with blockscale_offsets[e] <= sf_row0
    int lo = 0, hi = num_experts;
    while (hi - lo > 1) {
      int mid = (lo + hi) >> 1;
      if (blockscale_offsets[mid] <= sf_row0) lo = mid; else hi = mid;
    }
    const int e = lo;
    m_e = problem_sizes[e * 3];
    r0 = sf_row0 - blockscale_offsets[e];  // first row of the tile inside the expert
    row_base = expert_offsets[e];
    sf_base = blockscale_offsets[e];
  }
  if (r0 < 0 || r0 >= m_e) return;           // tile past the expert's rows: nothing defined there
  const int kcols = k >> 5;
  const long in_stride = SWIGLU ? 2L * k : k;   // SwiGLU reads [rows, 2K]: gate | up

  const int sub = tid % kLanes;    // 16-byte column of the row segment: elements [8*sub, 8*sub + 8)
  const int rrow = tid / kLanes;   // row within a 16-row pass
  const bool col_ok = kt * kCols + sub * 8 < k;
  v4i raw[8], rup[SWIGLU ? 8 : 1];
#pragma unroll
  for (int p = 0; p < 8; p++) {
    int r = r0 + p * 16 + rrow;
    raw[p] = v4i{0, 0, 0, 0};
    if constexpr (SWIGLU) rup[p] = v4i{0, 0, 0, 0};
    if (r < m_e && col_ok) {
      const uint16_t* src = in + (row_base + r) * in_stride + kt * kCols + sub * 8;
      raw[p] = __builtin_nontemporal_load((const v4i*)src);
      if constexpr (SWIGLU) rup[p] = __builtin_nontemporal_load((const v4i*)(src + k));
    }
  }
#pragma unroll
  for (int p = 0; p < 8; p++) {
    const int rt = p * 16 + rrow;  // row within the tile
    const int r = r0 + rt;
    float x[8];
    unpack8<FP16>(raw[p], x);
    if constexpr (SWIGLU) {
      float u[8];
      unpack8<FP16>(rup[p], u);
#pragma unroll
      for (int i = 0; i < 8; i++) x[i] = round_to_input_type<FP16>(swiglu_f32(x[i], u[i]));
    }
    float amax = 0.f;
#pragma unroll
    for (int i = 0; i < 8; i++) amax = __builtin_fmaxf(amax, __builtin_fabsf(x[i]));
    amax = __builtin_fmaxf(amax, __shfl_xor(amax, 1));
    amax = __builtin_fmaxf(amax, __shfl_xor(amax, 2));
    const int code = mx_scale_code(amax);
    const float inv = mx_scale_inverse(amax, code);
    float y[8];
#pragma unroll
    for (int i = 0; i < 8; i++) y[i] = __builtin_amdgcn_fmed3f(x[i] * inv, -448.f, 448.f);
    int w0 = __builtin_amdgcn_cvt_pk_fp8_f32(y[0], y[1], 0, false);
    w0 = __builtin_amdgcn_cvt_pk_fp8_f32(y[2], y[3], w0, true);
    int w1 = __builtin_amdgcn_cvt_pk_fp8_f32(y[4], y[5], 0, false);
    w1 = __builtin_amdgcn_cvt_pk_fp8_f32(y[6], y[7], w1, true);
    if (r < m_e && col_ok) {
      __builtin_nontemporal_store(v2i{w0, w1}, (v2i*)(q + (row_base + r) * k + kt * kCols + sub * 8));
    }
    if ((sub & 3) == 0) s_sf[(sub >> 4) * 512 + (rt & 31) * 16 + (rt >> 5) * 4 + ((sub >> 2) & 3)] = (uint8_t)(r < m_e ? code : 0);
  }
  __syncthreads();
  if (tid < 32 * kTiles && kt * kTiles + (tid >> 5) < (k >> 7)) {   // consecutive 128-column tiles are consecutive 512-byte tiles
    uint8_t* dst = sf + sf_base * kcols + ((long)(r0 >> 7) * (k >> 7) + kt * kTiles) * 512;
    *(v4i*)(dst + tid * 16) = *(const v4i*)(s_sf + tid * 16);
  }
}

}  // namespace esmoe

// swiglu != 0: `in` is [rows, 2k].  dense_rows > 0: no metadata (the three pointers may be null).
extern "C" int esmoe_launch_mxfp8_quant(const void* in, int in_dtype, const int* problem_sizes,
                                        const int* expert_offsets, const int* blockscale_offsets, void* q, uint8_t* sf,
                                        int num_experts, long sf_rows, int k, int swiglu, long dense_rows,
                                        hipStream_t stream) {
  using namespace esmoe;
  const unsigned rows128 = (unsigned)(sf_rows / 128);
  if (k < 128 || rows128 == 0) return 0;
#define ESMOE_LAUNCH_QUANT(F16_, SW_)                                                                               \
  hipLaunchKernelGGL((mxfp8_quant_kernel<F16_, SW_>), dim3((k + quant_cols<SW_>() - 1) / quant_cols<SW_>(), rows128), \
                     dim3(quant_threads<SW_>()), 0, stream, (const uint16_t*)in,                                   \
                     problem_sizes, expert_offsets, blockscale_offsets, (uint8_t*)q, sf, num_experts, k, dense_rows)
  if (in_dtype == 1) {
    if (swiglu) ESMOE_LAUNCH_QUANT(true, true); else ESMOE_LAUNCH_QUANT(true, false);
  } else {
    if (swiglu) ESMOE_LAUNCH_QUANT(false, true); else ESMOE_LAUNCH_QUANT(false, false);
  }
#undef ESMOE_LAUNCH_QUANT
  return (int)hipGetLastError();
}
