// Persistent grouped GEMM for gfx950 (MI355X): FP8-blockwise and MXFP8 variants.
//
// One launch serves every expert.  A one-workgroup schedule kernel turns
// problem_sizes into a list of workgroup tiles (schedule.h); persistent workgroups
// then pull tiles from an atomic counter.  A workgroup is 4 wavefronts laid out
// along N; a tile is (MT*16) rows x (NT*64) columns and each wavefront owns
// NT*16 columns of it.
//
// MFMA mapping (v_mfma[_scale]_f32_16x16x128_f8f6f4, both operands e4m3):
//   * the weight rows ride on the instruction's "A" side and the token rows on its
//     "B" side, so a lane ends up with 4 consecutive output columns of one token
//     row (one packed 8-byte store);
//   * lane l feeds row (l % 16); its 8 operand registers hold K bytes
//     [16*(l/16), +16) and [64 + 16*(l/16), +16) of the 128-wide K block;
//   * for the scaled form lane l supplies the E8M0 scale of row (l % 16),
//     K sub-block (l / 16) in byte 0 of the scale register.
// Weights stream from global memory straight into registers (each wavefront owns
// its rows, nothing to share); token rows are shared by the 4 wavefronts and are
// staged through double-buffered LDS.
//
// FP8-blockwise arithmetic follows the reference's blockwise mainloop order
// (es_fp8_blockwise_traits.cuh:35,60): each 128-wide K block is multiplied into a
// zeroed temporary and promoted into the fp32 accumulator times sa[row]*sb[nblk].
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "gemm_args.h"
#include "schedule.h"

namespace esmoe {

typedef int v8i __attribute__((ext_vector_type(8)));
typedef int v4i __attribute__((ext_vector_type(4)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));

constexpr int kThreads = 256;
constexpr int kLdsRow = 144;  // 128 data bytes + 16 pad: conflict-free 16-byte reads down a column of rows
constexpr int kMaxMT = 16;
constexpr int kLdsBuf = kMaxMT * 16 * kLdsRow;

__device__ __forceinline__ v8i join(v4i lo, v4i hi) {
  v8i r;
  r[0] = lo[0]; r[1] = lo[1]; r[2] = lo[2]; r[3] = lo[3];
  r[4] = hi[0]; r[5] = hi[1]; r[6] = hi[2]; r[7] = hi[3];
  return r;
}

template <int MT, int NT, bool MX>
struct TileRegs {
  v4i w[NT][2];       // weight fragments of one K block
  float sa[MX ? 1 : MT];  // activation scales of this lane's token row per row tile (fp8-blockwise)
  float sb;               // weight block scale (fp8-blockwise)
  int sfw[MX ? NT : 1];   // E8M0 weight scale, already shifted into byte 0 (mxfp8)
  int sfa[MX ? MT : 1];   // E8M0 activation scale (mxfp8)
};

template <int MT, int NT, bool MX>
__device__ __forceinline__ void gemm_tile(const GemmArgs& g, int e, int M, int m0, int n0, uint8_t* lds) {
  constexpr int BM = MT * 16;
  constexpr int kChunks = BM * 8;  // 16-byte chunks of one K block of the token tile
  constexpr int APASS = (kChunks + kThreads - 1) / kThreads;
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int r = lane & 15;
  const int gq = lane >> 4;
  const int K = g.k, N = g.n, KB = K >> 7;
  const long row_base = g.expert_offsets[e];

  const int nw0 = n0 + wave * (NT * 16);
  const bool wave_active = nw0 < N;
  // weight rows of this lane: nw0 + nt*16 + r  (clamped to stay in bounds for idle wavefronts)
  const int nrow0 = wave_active ? nw0 + r : r;
  const uint8_t* wbase = (const uint8_t*)g.b + ((long)e * N + nrow0) * K + gq * 16;
  const long wstep = 16L * K;

  // token-tile staging: chunk c -> row c/8, 16-byte column c%8
  const uint8_t* asrc[APASS];
  int adst[APASS];
#pragma unroll
  for (int p = 0; p < APASS; p++) {
    int c = tid + p * kThreads;
    int arow = c >> 3, acol = c & 7;
    int grow = m0 + arow;
    if (grow > M - 1) grow = M - 1;
    asrc[p] = (const uint8_t*)g.a + (row_base + grow) * K + acol * 16;
    adst[p] = arow * kLdsRow + acol * 16;
  }
  const int frag_off = r * kLdsRow + gq * 16;

  // per-lane token rows for the scales
  long srow[MT];
#pragma unroll
  for (int mt = 0; mt < MT; mt++) {
    int grow = m0 + mt * 16 + r;
    if (grow > M - 1) grow = M - 1;
    srow[mt] = grow;
  }
  const float* sa_base = nullptr;
  const float* sb_base = nullptr;
  const uint8_t* sfa_base = nullptr;
  const uint8_t* sfw_base = nullptr;
  if constexpr (!MX) {
    sa_base = g.sa + row_base * KB;
    sb_base = g.sb + ((long)e * (N >> 7) + ((wave_active ? nw0 : 0) >> 7)) * KB;
  } else {
    sfa_base = g.sfa + (long)g.blockscale_offsets[e] * (K >> 5);
    sfw_base = g.sfb + (long)e * N * (K >> 5);
  }

  v4f acc[NT][MT];
#pragma unroll
  for (int nt = 0; nt < NT; nt++)
#pragma unroll
    for (int mt = 0; mt < MT; mt++) acc[nt][mt] = v4f{0.f, 0.f, 0.f, 0.f};

  TileRegs<MT, NT, MX> cur, nxt;
  v4i astage[APASS];

  auto load_regs = [&](TileRegs<MT, NT, MX>& t, int kb) {
    const uint8_t* wp = wbase + (long)kb * 128;
#pragma unroll
    for (int nt = 0; nt < NT; nt++) {
      t.w[nt][0] = __builtin_nontemporal_load((const v4i*)(wp + nt * wstep));
      t.w[nt][1] = __builtin_nontemporal_load((const v4i*)(wp + nt * wstep + 64));
    }
    if constexpr (!MX) {
#pragma unroll
      for (int mt = 0; mt < MT; mt++) t.sa[mt] = sa_base[srow[mt] * KB + kb];
      t.sb = sb_base[kb];
    } else {
#pragma unroll
      for (int nt = 0; nt < NT; nt++) {
        int n = nrow0 + nt * 16;
        long off = ((long)(n >> 7) * KB + kb) * 512 + (n & 31) * 16 + ((n & 127) >> 5) * 4;
        t.sfw[nt] = (int)((*(const uint32_t*)(sfw_base + off)) >> (gq * 8));
      }
#pragma unroll
      for (int mt = 0; mt < MT; mt++) {
        long m = srow[mt];
        long off = ((m >> 7) * KB + kb) * 512 + (m & 31) * 16 + ((m & 127) >> 5) * 4;
        t.sfa[mt] = (int)((*(const uint32_t*)(sfa_base + off)) >> (gq * 8));
      }
    }
  };
  auto load_a = [&](int kb) {
#pragma unroll
    for (int p = 0; p < APASS; p++) {
      if (APASS * kThreads == kChunks || tid + p * kThreads < kChunks) astage[p] = *(const v4i*)(asrc[p] + (long)kb * 128);
    }
  };
  auto store_a = [&](int buf) {
#pragma unroll
    for (int p = 0; p < APASS; p++) {
      if (APASS * kThreads == kChunks || tid + p * kThreads < kChunks) *(v4i*)(lds + buf * kLdsBuf + adst[p]) = astage[p];
    }
  };
  auto compute = [&](const TileRegs<MT, NT, MX>& t, int buf) {
    const uint8_t* lb = lds + buf * kLdsBuf + frag_off;
#pragma unroll
    for (int mt = 0; mt < MT; mt++) {
      v4i lo = *(const v4i*)(lb + mt * 16 * kLdsRow);
      v4i hi = *(const v4i*)(lb + mt * 16 * kLdsRow + 64);
      v8i af = join(lo, hi);
      if constexpr (!MX) {
        float s = t.sa[mt] * t.sb;
        v4f tmp[NT];
#pragma unroll
        for (int nt = 0; nt < NT; nt++) {
          tmp[nt] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(join(t.w[nt][0], t.w[nt][1]), af,
                                                                       v4f{0.f, 0.f, 0.f, 0.f}, 0, 0, 0, 0, 0, 0);
        }
#pragma unroll
        for (int nt = 0; nt < NT; nt++) {
#pragma unroll
          for (int i = 0; i < 4; i++) acc[nt][mt][i] = __builtin_fmaf(tmp[nt][i], s, acc[nt][mt][i]);
        }
      } else {
#pragma unroll
        for (int nt = 0; nt < NT; nt++) {
          acc[nt][mt] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(join(t.w[nt][0], t.w[nt][1]), af, acc[nt][mt],
                                                                           0, 0, 0, t.sfw[nt], 0, t.sfa[mt]);
        }
      }
    }
  };

  // prologue
  load_regs(cur, 0);
  load_a(0);
  store_a(0);
  __syncthreads();

  int kb = 0;
  for (; kb + 2 <= KB; kb += 2) {
    load_regs(nxt, kb + 1);
    load_a(kb + 1);
    if (wave_active) compute(cur, 0);
    store_a(1);
    __syncthreads();
    if (kb + 2 < KB) {
      load_regs(cur, kb + 2);
      load_a(kb + 2);
    }
    if (wave_active) compute(nxt, 1);
    if (kb + 2 < KB) store_a(0);
    __syncthreads();
  }
  if (kb < KB) {  // odd number of K blocks: the last one is in `cur` / buffer 0
    if (wave_active) compute(cur, 0);
    __syncthreads();
  }

  // epilogue: lane holds columns nw0 + nt*16 + 4*gq + [0,4) of token row m0 + mt*16 + r
  if (wave_active) {
#pragma unroll
    for (int mt = 0; mt < MT; mt++) {
      int m = m0 + mt * 16 + r;
      if (m < M) {
        long orow = (row_base + m) * (long)N;
#pragma unroll
        for (int nt = 0; nt < NT; nt++) {
          int n = nw0 + nt * 16 + gq * 4;
          if (g.out_dtype == 0) {
            bf16x4 v = __builtin_convertvector(acc[nt][mt], bf16x4);
            *(bf16x4*)((__bf16*)g.out + orow + n) = v;
          } else {
            f16x4 v = __builtin_convertvector(acc[nt][mt], f16x4);
            *(f16x4*)((_Float16*)g.out + orow + n) = v;
          }
        }
      }
    }
  }
}

// ---------------------------------------------------------------------------------------------
// Schedule kernel: one workgroup, thread = expert (E <= 1024, as the reference's pre-compute kernel,
// es_fp8_blockwise_launcher.cuh:53,74).
__global__ void __launch_bounds__(1024) schedule_kernel(const int* __restrict__ problem_sizes, int num_experts, int n,
                                                        SchedPolicy policy, int* __restrict__ ws) {
  __shared__ int s_m[1024];
  __shared__ int s_items[1024];
  const int e = threadIdx.x;
  int m = 0;
  if (e < num_experts) m = problem_sizes[e * 3];
  if (m < 0) m = 0;
  s_m[e] = m;
  __syncthreads();
  int* item_start = ws + ws_item_start(num_experts);
  int* order = ws + ws_order(num_experts);
  if (e < num_experts) {
    int pos = e;
    if (policy.order == 0) {
      pos = 0;
      for (int j = 0; j < num_experts; j++) {
        int mj = s_m[j];
        pos += (mj > m) || (mj == m && j < e);
      }
    }
    order[pos] = e;
    s_items[pos] = sched_items(m, n, policy);
  }
  __syncthreads();
  if (e == 0) {
    int run = 0;
    for (int j = 0; j < num_experts; j++) {
      item_start[j] = run;
      run += s_items[j];
    }
    item_start[num_experts] = run;
    ws[kWsTotal] = run;
    ws[kWsCounter] = 0;
  }
}

// (MT, NT) tile shapes compiled into the persistent kernel.
#ifndef ESMOE_VARIANTS
#define ESMOE_VARIANTS                                 \
  ESMOE_CASE(1, 1) ESMOE_CASE(1, 2) ESMOE_CASE(1, 4)   \
  ESMOE_CASE(2, 1) ESMOE_CASE(2, 2) ESMOE_CASE(2, 4)   \
  ESMOE_CASE(4, 1) ESMOE_CASE(4, 2) ESMOE_CASE(4, 4)   \
  ESMOE_CASE(8, 2) ESMOE_CASE(8, 4)                    \
  ESMOE_CASE(16, 2)
#endif
#ifndef ESMOE_WAVES_PER_SIMD
#define ESMOE_WAVES_PER_SIMD 1
#endif

template <bool MX>
__global__ void __launch_bounds__(kThreads, ESMOE_WAVES_PER_SIMD) grouped_gemm_kernel(GemmArgs g) {
  __shared__ __attribute__((aligned(16))) uint8_t lds[2 * kLdsBuf];
  __shared__ int s_item;
  int* ws = g.ws;
  const int total = ws[kWsTotal];
  const int* item_start = ws + ws_item_start(g.num_experts);
  const int* order = ws + ws_order(g.num_experts);
  for (;;) {
    if (threadIdx.x == 0) s_item = atomicAdd(&ws[kWsCounter], 1);
    __syncthreads();
    const int item = s_item;
    __syncthreads();
    if (item >= total) break;
    // position p with item_start[p] <= item < item_start[p+1]
    int lo = 0, hi = g.num_experts;
    while (hi - lo > 1) {
      int mid = (lo + hi) >> 1;
      if (item_start[mid] <= item) lo = mid; else hi = mid;
    }
    const int e = order[lo];
    const int M = g.problem_sizes[e * 3];
    const TileCoord t = sched_decode(item - item_start[lo], M, g.n, g.policy);
    const int key = t.mt * 8 + t.nt;
#define ESMOE_CASE(MT_, NT_) \
  case (MT_) * 8 + (NT_): gemm_tile<MT_, NT_, MX>(g, e, M, t.m0, t.n0, lds); break;
    switch (key) {
      ESMOE_VARIANTS
      default: break;
    }
#undef ESMOE_CASE
  }
}

}  // namespace esmoe

extern "C" int esmoe_launch_grouped_gemm(const esmoe::GemmArgs* args, int mx, int grid, hipStream_t stream) {
  using namespace esmoe;
  hipLaunchKernelGGL(schedule_kernel, dim3(1), dim3(1024), 0, stream, args->problem_sizes, args->num_experts, args->n,
                     args->policy, args->ws);
  hipError_t err = hipGetLastError();
  if (err != hipSuccess) return (int)err;
  if (mx)
    hipLaunchKernelGGL(grouped_gemm_kernel<true>, dim3(grid), dim3(kThreads), 0, stream, *args);
  else
    hipLaunchKernelGGL(grouped_gemm_kernel<false>, dim3(grid), dim3(kThreads), 0, stream, *args);
  return (int)hipGetLastError();
}
