// MXFP8 grouped quantisation for gfx950: bf16/fp16 rows -> e4m3 bytes + swizzled E8M0 scales.
//
// Arithmetic follows cvt_warp_fp16_to_mxfp8
// (expert_specialization/csrc/cuda/es_sm100_mxfp8_blockscaled_group_quant.cuh:36-134):
// per 1x32 block  amax = max|x|,  scale = smallest power of two >= amax/448,
// q = e4m3_rne(x / scale).  The scale exponent is taken from the bit pattern of
// amax (448 = 1.75 * 2^8  =>  E = exponent(amax) - 8 + (mantissa > .75)), which equals
// the reference's float route with a correctly rounded 1/448.
//
// Work decomposition.  A 512-byte scale tile (128 rows x 4 scale columns, layout ((32,4),4):((16,4),1),
// group_quant.cuh:25) keeps the four scale bytes of row r (one dword per 128 columns) at (r % 32) * 16 + (r / 32) * 4:
// rows r, r + 32, r + 64 and r + 96 of a tile share one 16-byte unit, and eight neighbouring rows a 128-byte line.
// Scale bytes that reach memory as scattered dwords cost 4 us of 31 on 8192 x 7168 rows (lines that are filled piece by
// piece from several L2s; one store instruction instead of four for the same dwords changes nothing); whole units
// side by side cost a tenth of that.  (Flat 4 KB runs of consecutive rows per load instruction, the shape of the FP8
// 1x128 quantiser of fp8_quant.hip, would stream 8 % faster than 512-byte row segments, but their scale bytes can only
// leave as scattered dwords; 16-byte units from rows 32 apart with 4 KB runs lose the gain to the row stride.)
// So a workgroup of 256 threads takes the rows
// {s * 8 + i + 32 * j : i < 8, j < 4} of one 128-row slab of the *scale* row space (blockscale_offsets are multiples of
// 128: a slab belongs to one expert) x 256 columns (128 in the SwiGLU form): 32 (16) lanes read one 512-byte row
// segment, 8 (16) rows per pass, one pass per quarter j, four (SwiGLU: two, of two loads) 16-byte loads in flight
// per lane; 4 lanes share one 32-wide block and reduce amax with two lane swaps, the four codes of a row's 128-column
// group are gathered with two more, and after the passes the group's first lane holds the row's whole 16-byte unit:
// the workgroup writes whole 128-byte lines of the scale tiles.  Rows between the expert's last row and the end of
// its last 128-row tile get scale bytes 0 (the reference leaves them unspecified).
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

// (measured on 8192 x 7168 rows: 128 ... 1024 columns per workgroup of 256 or 512 threads are within 1 % of one another)
template <bool SWIGLU> constexpr int quant_cols() { return SWIGLU ? 128 : 256; }   // columns per workgroup
template <bool SWIGLU> constexpr int quant_threads() { return 256; }

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

// Value of another lane through DPP (inside the VALU, no LDS trip).  CTRL 0xB1 / 0x4E: lane ^ 1 / lane ^ 2 inside
// each group of four; 0x100 + n: lane + n inside each row of 16 lanes (0 from past the row's end).
template <int CTRL>
__device__ __forceinline__ int dpp_i32(int v) { return __builtin_amdgcn_update_dpp(0, v, CTRL, 0xF, 0xF, true); }
template <int CTRL>
__device__ __forceinline__ float dpp_f32(float v) { return __builtin_bit_cast(float, dpp_i32<CTRL>(__builtin_bit_cast(int, v))); }

template <bool FP16, bool SWIGLU>
__global__ void __launch_bounds__(quant_threads<SWIGLU>()) __attribute__((amdgpu_waves_per_eu(6, 8))) mxfp8_quant_kernel(
    const uint16_t* __restrict__ in, const int* __restrict__ problem_sizes, const int* __restrict__ expert_offsets,
    const int* __restrict__ blockscale_offsets, uint8_t* __restrict__ q, uint8_t* __restrict__ sf, int num_experts, int k,
    long dense_rows, int ktiles) {
  constexpr int kCols = quant_cols<SWIGLU>(), kLanes = kCols / 8, kRowsPerPass = quant_threads<SWIGLU>() / kLanes, kSubs = 32 / kRowsPerPass;
  // consecutive workgroups: consecutive column tiles of the same rows, then the next rows of the slab
  const int kt = blockIdx.x % ktiles;                                       // tile of kCols columns (the last one may be 128 wide)
  const int s = (blockIdx.x / ktiles) % kSubs;
  const int sf_row0 = (int)((long)(blockIdx.x / (ktiles * kSubs)) * 128);   // first row of the slab in scale-row space
  const int tid = threadIdx.x;

  int m_e, r0;
  long row_base, sf_base;
  if (dense_rows > 0) {
    m_e = (int)dense_rows;
    r0 = sf_row0;
    row_base = 0;
    sf_base = 0;
  } else {
    // expert owning scale row sf_row0: the last e with blockscale_offsets[e] <= sf_row0 (the offsets never decrease),
    // counted by the wavefront 64 offsets at a time: one trip to memory where a bisection makes one per step
    int cnt = 0;
    for (int base = 0; base < num_experts; base += 64) {
      const int idx = base + (tid & 63);
      const int b = idx < num_experts ? blockscale_offsets[idx] : 0x7fffffff;
      cnt += __popcll(__ballot(b <= sf_row0));
    }
    const int e = __builtin_amdgcn_readfirstlane(cnt) - 1;
    if (e < 0) return;
    m_e = problem_sizes[e * 3];
    if (m_e < 0) m_e = 0;
    r0 = sf_row0 - blockscale_offsets[e];  // first row of the slab inside the expert
    row_base = expert_offsets[e];
    sf_base = blockscale_offsets[e];
  }
  // slabs past the expert's rows (an empty expert has none; the launch's scale rows may run past the last expert's)
  if (r0 < 0 || r0 >= m_e) return;
  const int sub = tid % kLanes;    // 16-byte column of the row segment: elements [8*sub, 8*sub + 8)
  const int rrow = tid / kLanes;   // row within a pass
  const bool col_ok = kt * kCols + sub * 8 < k;
  // wave-uniform 64-bit bases, 32-bit lane offsets (SwiGLU reads [rows, 2K]: gate | up)
  const uint32_t row_pitch = (SWIGLU ? 2u : 1u) * (uint32_t)k * 2u;   // bytes
  const char* const in_b = (const char*)(in + (row_base + r0) * (SWIGLU ? 2L * k : (long)k) + kt * kCols);
  uint8_t* const q_b = q + (row_base + r0) * (long)k + kt * kCols;
  const int rl0 = s * kRowsPerPass + rrow;   // this lane's row of quarter 0; quarter j: + 32 j

  v4i raw[4], rup[SWIGLU ? 4 : 1];
#pragma unroll
  for (int j = 0; j < 4; j++) {
    const int rl = rl0 + 32 * j;
    raw[j] = v4i{0, 0, 0, 0};
    if constexpr (SWIGLU) rup[j] = v4i{0, 0, 0, 0};
    if (r0 + rl < m_e && col_ok) {
      const char* src = in_b + (uint32_t)rl * row_pitch + sub * 16;
      raw[j] = __builtin_nontemporal_load((const v4i*)src);
      if constexpr (SWIGLU) rup[j] = __builtin_nontemporal_load((const v4i*)(src + 2 * (uint32_t)k));
    }
  }
  v4i unit;   // the 16-byte unit of row rl0, 128-column group sub / 16 (in the group's first lane)
#pragma unroll
  for (int j = 0; j < 4; j++) {
    const int rl = rl0 + 32 * j;
    const bool live = r0 + rl < m_e && col_ok;
    float x[8];
    unpack8<FP16>(raw[j], x);
    if constexpr (SWIGLU) {
      float up[8];
      unpack8<FP16>(rup[j], up);
#pragma unroll
      for (int t = 0; t < 8; t++) x[t] = round_to_input_type<FP16>(swiglu_f32(x[t], up[t]));
    }
    float amax = 0.f;
#pragma unroll
    for (int t = 0; t < 8; t++) amax = __builtin_fmaxf(amax, __builtin_fabsf(x[t]));
    amax = __builtin_fmaxf(amax, dpp_f32<0xB1>(amax));   // lane ^ 1
    amax = __builtin_fmaxf(amax, dpp_f32<0x4E>(amax));   // lane ^ 2
    const int code = mx_scale_code(amax);
    const float inv = mx_scale_inverse(amax, code);
    // |x| * inv <= 448 for every finite input (the scale is the smallest power of two >= amax / 448), so the
    // conversion needs no clamp
    int w0 = __builtin_amdgcn_cvt_pk_fp8_f32(x[0] * inv, x[1] * inv, 0, false);
    w0 = __builtin_amdgcn_cvt_pk_fp8_f32(x[2] * inv, x[3] * inv, w0, true);
    int w1 = __builtin_amdgcn_cvt_pk_fp8_f32(x[4] * inv, x[5] * inv, 0, false);
    w1 = __builtin_amdgcn_cvt_pk_fp8_f32(x[6] * inv, x[7] * inv, w1, true);
    if (live) __builtin_nontemporal_store(v2i{w0, w1}, (v2i*)(q_b + (long)rl * k + sub * 8));
    // 16 consecutive lanes hold the row's four blocks of a 128-column scale tile: their codes -> one dword in the
    // first of them (rows past the expert's last: 0, loaded as zeros)
    int codes = live ? code : 0;
    codes |= dpp_i32<0x104>(codes) << 8;     // from lane + 4 of the 16-lane row
    codes |= dpp_i32<0x108>(codes) << 16;    // from lane + 8
    // (the exchanges have to run with every lane active: the empty statement keeps the compiler from moving them into
    // the store's branch below, where their source lanes would be switched off and read as 0)
    asm volatile("" : "+v"(codes));
    unit[j] = codes;
  }
  if ((sub & 15) == 0 && col_ok)
    *(v4i*)(sf + sf_base * (k >> 5) + ((long)(r0 >> 7) * (k >> 7) + kt * (kCols / 128) + (sub >> 4)) * 512 + rl0 * 16) = unit;
}

}  // namespace esmoe

// swiglu != 0: `in` is [rows, 2k].  dense_rows > 0: no metadata (the three pointers may be null).
extern "C" int esmoe_launch_mxfp8_quant(const void* in, int in_dtype, const int* problem_sizes,
                                        const int* expert_offsets, const int* blockscale_offsets, void* q, uint8_t* sf,
                                        int num_experts, long sf_rows, int k, int swiglu, long dense_rows,
                                        hipStream_t stream) {
  using namespace esmoe;
  const long slabs = sf_rows / 128;
  if (k < 128 || slabs == 0) return 0;
#define ESMOE_LAUNCH_QUANT(F16_, SW_)                                                                               \
  do {                                                                                                              \
    const int ktiles = (k + quant_cols<SW_>() - 1) / quant_cols<SW_>();                                             \
    const int subs = 32 / (quant_threads<SW_>() / (quant_cols<SW_>() / 8));                                         \
    hipLaunchKernelGGL((mxfp8_quant_kernel<F16_, SW_>), dim3((unsigned)(slabs * subs * ktiles)), dim3(quant_threads<SW_>()), 0, \
                       stream, (const uint16_t*)in, problem_sizes, expert_offsets, blockscale_offsets, (uint8_t*)q, sf, \
                       num_experts, k, dense_rows, ktiles);                                                          \
  } while (0)
  if (in_dtype == 1) {
    if (swiglu) ESMOE_LAUNCH_QUANT(true, true); else ESMOE_LAUNCH_QUANT(true, false);
  } else {
    if (swiglu) ESMOE_LAUNCH_QUANT(false, true); else ESMOE_LAUNCH_QUANT(false, false);
  }
#undef ESMOE_LAUNCH_QUANT
  return (int)hipGetLastError();
}
