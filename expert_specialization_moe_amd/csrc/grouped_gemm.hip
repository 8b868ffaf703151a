// Persistent grouped GEMM for gfx950 (MI355X): FP8-blockwise and MXFP8 variants.
//
// One launch serves every expert.  A one-workgroup schedule kernel turns
// problem_sizes into a list of workgroup tiles (schedule.h); persistent workgroups
// then pull tiles from an atomic counter.  A workgroup is 4 wavefronts laid out
// along N; a tile is (MT*16) token rows x (NT*64) weight rows and each wavefront
// owns NT*16 weight rows of it.
//
// Data movement.  Per 128-wide K block the workgroup loads the token rows and the
// weight rows of its tile with lane-contiguous 16-byte loads (8 lanes cover one
// 128-byte row segment, so the texture-address unit sees whole cache lines), keeps
// them in registers for S-1 K blocks (the global prefetch distance) and then writes
// them to a double-buffered LDS tile with 144-byte row pitch.  MFMA operand
// fragments are read back from LDS (16 bytes per lane, conflict-free down a column
// of rows).  Loading fragments straight from global memory is ~4x slower per CU:
// a fragment puts consecutive lanes on different rows, i.e. 64 separate 16-byte
// requests per instruction.
//
// MFMA mapping (v_mfma[_scale]_f32_16x16x128_f8f6f4, both operands e4m3):
//   * the weight rows ride on the instruction's "A" side and the token rows on its
//     "B" side, so a lane ends up with 4 consecutive output columns of one token
//     row (one packed 8-byte store);
//   * lane l feeds row (l % 16); its 8 operand registers hold K bytes
//     [16*(l/16), +16) and [64 + 16*(l/16), +16) of the 128-wide K block;
//   * for the scaled form lane l supplies the E8M0 scale of row (l % 16),
//     K sub-block (l / 16) in byte 0 of the scale register.
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

__device__ __forceinline__ v8i join(v4i lo, v4i hi) {
  v8i r;
  r[0] = lo[0]; r[1] = lo[1]; r[2] = lo[2]; r[3] = lo[3];
  r[4] = hi[0]; r[5] = hi[1]; r[6] = hi[2]; r[7] = hi[3];
  return r;
}

// LDS layout of one K-block buffer of a tile: token rows, weight rows, then the block's scales.
template <int MT, int NT, bool MX>
struct TileGeom {
  static constexpr int BM = MT * 16;
  static constexpr int BN = NT * 64;
  static constexpr int kAChunks = BM * 8;   // 16-byte chunks of the token rows of one K block
  static constexpr int kWChunks = BN * 8;
  static constexpr int kAPass = (kAChunks + kThreads - 1) / kThreads;
  static constexpr int kWPass = kWChunks / kThreads;
  static constexpr int kABytes = BM * kLdsRow;
  static constexpr int kWBytes = BN * kLdsRow;
  // scales: fp8-blockwise -> BM floats (sa of the block); mxfp8 -> verbatim 512-byte swizzled tiles,
  // weight rows first (BN/128 tiles), then token rows (ceil(BM/128) tiles)
  static constexpr int kSfwChunks = MX ? BN / 4 : 0;
  static constexpr int kSfaChunks = MX ? ((BM + 127) / 128) * 32 : 0;
  // every thread stages one scale item (threads past the tile's needs duplicate a valid one), so the
  // region is sized for 256 items and the pipeline stays free of divergent branches
  static constexpr int kScaleBytes = MX ? kThreads * 16 : kThreads * 4;
  static constexpr int kBufBytes = kABytes + kWBytes + ((kScaleBytes + 15) & ~15);
  static_assert(kWChunks % kThreads == 0, "weight tile must fill whole passes");
  static_assert(kSfwChunks + kSfaChunks <= kThreads, "one scale chunk per thread");
};

// Largest LDS footprint over the compiled shapes (two buffers).
constexpr int kLdsBytes = 2 * ((128 + 256) * kLdsRow + 4096);

// One K block of a tile in flight between global memory and LDS.
template <int MT, int NT, bool MX>
struct TileStage {
  using G = TileGeom<MT, NT, MX>;
  v4i a[G::kAPass];
  v4i w[G::kWPass];
  float sa;   // fp8-blockwise: sa[row of this thread][kb] (threads < BM)
  float sb;   // fp8-blockwise: sb[e][n-block of this wavefront][kb]
  v4i sf;     // mxfp8: this thread's 16-byte chunk of the swizzled scale tiles
};

template <int MT, int NT, bool MX, int S>
__device__ __forceinline__ void gemm_tile(const GemmArgs& g, int e, int M, int m0, int n0, uint8_t* lds) {
  using G = TileGeom<MT, NT, MX>;
  static_assert(2 * G::kBufBytes <= kLdsBytes, "LDS budget");
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int r = lane & 15;
  const int gq = lane >> 4;
  const int K = g.k, N = g.n, KB = K >> 7;
  const long row_base = g.expert_offsets[e];
  const int nw0 = n0 + wave * (NT * 16);
  const bool wave_active = nw0 < N;

  // staging map: chunk c -> row c/8, 16-byte column c%8 (8 consecutive lanes = one 128-byte row
  // segment).  Addresses are a wave-uniform 64-bit base plus one 32-bit offset per pass.
  const int srow = tid >> 3, scol = tid & 7;       // pass p handles tile row srow + 32*p
  const uint8_t* a_base = (const uint8_t*)g.a + (row_base + m0) * K;
  const uint8_t* w_base = (const uint8_t*)g.b + ((long)e * N + n0) * K;
  // (a token tile shorter than 32 rows is staged twice by the two halves of the workgroup: same
  // bytes to the same place, which keeps every thread on the same instruction stream)
  const int arow0 = srow & (G::BM < 32 ? G::BM - 1 : 31);
  uint32_t aoff[G::kAPass];
#pragma unroll
  for (int p = 0; p < G::kAPass; p++) {
    int row = arow0 + 32 * p;
    if (row > M - 1 - m0) row = M - 1 - m0;
    aoff[p] = (uint32_t)row * (uint32_t)K + scol * 16;
  }
  uint32_t woff[G::kWPass];
#pragma unroll
  for (int p = 0; p < G::kWPass; p++) {
    int row = srow + 32 * p;
    if (row > N - 1 - n0) row = N - 1 - n0;
    woff[p] = (uint32_t)row * (uint32_t)K + scol * 16;
  }
  const int sdst = srow * kLdsRow + scol * 16;     // LDS offset of pass 0; pass p adds 32 rows
  const int adst = arow0 * kLdsRow + scol * 16;
  constexpr int kScaleOff = G::kABytes + G::kWBytes;
  const float* sa_src = nullptr;
  const float* sb_src = nullptr;
  const uint8_t* sf_src = nullptr;
  if constexpr (!MX) {
    int grow = m0 + tid;
    if (grow > M - 1) grow = M - 1;
    sa_src = g.sa + (row_base + grow) * KB;
    sb_src = g.sb + ((long)e * (N >> 7) + ((wave_active ? nw0 : 0) >> 7)) * KB;
  } else {
    const int kc = K >> 5;
    if (tid < G::kSfwChunks) {
      int blk = (n0 >> 7) + (tid >> 5);
      if (blk * 128 >= N) blk = n0 >> 7;
      sf_src = g.sfb + (long)e * N * kc + (long)blk * KB * 512 + (tid & 31) * 16;
    } else {
      int j = tid - G::kSfwChunks;
      int blk = (m0 >> 7) + (j >> 5);
      if (j >= G::kSfaChunks || blk * 128 >= M) blk = m0 >> 7;
      sf_src = g.sfa + (long)g.blockscale_offsets[e] * kc + (long)blk * KB * 512 + (j & 31) * 16;
    }
  }

  const int frag_off = r * kLdsRow + gq * 16;
  const int wfrag_off = G::kABytes + wave * (NT * 16) * kLdsRow + frag_off;

  v4f acc[NT][MT];
#pragma unroll
  for (int nt = 0; nt < NT; nt++)
#pragma unroll
    for (int mt = 0; mt < MT; mt++) acc[nt][mt] = v4f{0.f, 0.f, 0.f, 0.f};

  TileStage<MT, NT, MX> st[S];

  auto load = [&](TileStage<MT, NT, MX>& t, int kb) {
    const uint8_t* ab = a_base + (long)kb * 128;
    const uint8_t* wb = w_base + (long)kb * 128;
#pragma unroll
    for (int p = 0; p < G::kAPass; p++) {
      t.a[p] = *(const v4i*)(ab + aoff[p]);
    }
#pragma unroll
    for (int p = 0; p < G::kWPass; p++) t.w[p] = *(const v4i*)(wb + woff[p]);
    if constexpr (!MX) {
      t.sa = sa_src[kb];
      t.sb = sb_src[kb];
    } else {
      t.sf = *(const v4i*)(sf_src + (long)kb * 512);
    }
  };
  auto store = [&](const TileStage<MT, NT, MX>& t, int buf) {
    uint8_t* lb = lds + buf * G::kBufBytes;
#pragma unroll
    for (int p = 0; p < G::kAPass; p++) *(v4i*)(lb + adst + p * 32 * kLdsRow) = t.a[p];
#pragma unroll
    for (int p = 0; p < G::kWPass; p++) *(v4i*)(lb + sdst + G::kABytes + p * 32 * kLdsRow) = t.w[p];
    if constexpr (!MX) {
      *(float*)(lb + kScaleOff + tid * 4) = t.sa;
    } else {
      *(v4i*)(lb + kScaleOff + tid * 16) = t.sf;
    }
  };
  auto compute = [&](const TileStage<MT, NT, MX>& t, int buf) {
    const uint8_t* lb = lds + buf * G::kBufBytes;
    v8i wf[NT];
#pragma unroll
    for (int nt = 0; nt < NT; nt++) {
      wf[nt] = join(*(const v4i*)(lb + wfrag_off + nt * 16 * kLdsRow), *(const v4i*)(lb + wfrag_off + nt * 16 * kLdsRow + 64));
    }
    int sfw[MX ? NT : 1];
    if constexpr (MX) {
#pragma unroll
      for (int nt = 0; nt < NT; nt++) {
        int nl = wave * (NT * 16) + nt * 16 + r;  // weight row inside the tile
        uint32_t d = *(const uint32_t*)(lb + kScaleOff + (nl >> 7) * 512 + (nl & 31) * 16 + ((nl & 127) >> 5) * 4);
        sfw[nt] = (int)(d >> (gq * 8));
      }
    }
    v4i af[2][2];
    af[0][0] = *(const v4i*)(lb + frag_off);
    af[0][1] = *(const v4i*)(lb + frag_off + 64);
#pragma unroll
    for (int mt = 0; mt < MT; mt++) {
      if (mt + 1 < MT) {
        af[(mt + 1) & 1][0] = *(const v4i*)(lb + frag_off + (mt + 1) * 16 * kLdsRow);
        af[(mt + 1) & 1][1] = *(const v4i*)(lb + frag_off + (mt + 1) * 16 * kLdsRow + 64);
      }
      v8i afr = join(af[mt & 1][0], af[mt & 1][1]);
      if constexpr (!MX) {
        float sc = *(const float*)(lb + kScaleOff + (mt * 16 + r) * 4) * t.sb;
        v4f tmp[NT];
#pragma unroll
        for (int nt = 0; nt < NT; nt++) {
          tmp[nt] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(wf[nt], afr, v4f{0.f, 0.f, 0.f, 0.f}, 0, 0, 0, 0, 0, 0);
        }
#pragma unroll
        for (int nt = 0; nt < NT; nt++) {
#pragma unroll
          for (int i = 0; i < 4; i++) acc[nt][mt][i] = __builtin_fmaf(tmp[nt][i], sc, acc[nt][mt][i]);
        }
      } else {
        int ml = (m0 & 127) + mt * 16 + r;  // token row inside its 128-row scale tile(s)
        uint32_t d = *(const uint32_t*)(lb + kScaleOff + G::kSfwChunks * 16 + (ml >> 7) * 512 + (ml & 31) * 16 + ((ml & 127) >> 5) * 4);
        int sfa = (int)(d >> (gq * 8));
#pragma unroll
        for (int nt = 0; nt < NT; nt++) {
          acc[nt][mt] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(wf[nt], afr, acc[nt][mt], 0, 0, 0, sfw[nt], 0, sfa);
        }
      }
    }
  };

  // prologue: S-1 K blocks in flight, the first one into LDS buffer 0
#pragma unroll
  for (int j = 0; j < S - 1; j++) {
    if (j < KB) load(st[j], j);
  }
  store(st[0], 0);
  __syncthreads();

  // steady state: branch-free so that the outstanding-load counts stay exact
  int kb0 = 0;
  for (; kb0 + 2 * S - 2 < KB; kb0 += S) {
#pragma unroll
    for (int j = 0; j < S; j++) {
      const int kb = kb0 + j;
      load(st[(j + S - 1) % S], kb + S - 1);
      __builtin_amdgcn_sched_barrier(0);  // keep the phases in program order: the scheduler would
      compute(st[j], kb & 1);             // otherwise overlap all stages' live ranges and spill
      __builtin_amdgcn_sched_barrier(0);
      store(st[(j + 1) % S], (kb + 1) & 1);
      __syncthreads();
      __builtin_amdgcn_sched_barrier(0);
    }
  }
  // drain: at most 2S-2 K blocks left
#pragma unroll
  for (int t = 0; t < 2; t++) {
#pragma unroll
    for (int j = 0; j < S; j++) {
      const int kb = kb0 + t * S + j;
      if (kb < KB) {
        if (kb + S - 1 < KB) load(st[(j + S - 1) % S], kb + S - 1);
        compute(st[j], kb & 1);
        if (kb + 1 < KB) store(st[(j + 1) % S], (kb + 1) & 1);
        __syncthreads();
      }
    }
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
            *(bf16x4*)((__bf16*)g.out + orow + n) = __builtin_convertvector(acc[nt][mt], bf16x4);
          } else {
            *(f16x4*)((_Float16*)g.out + orow + n) = __builtin_convertvector(acc[nt][mt], f16x4);
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
#define ESMOE_VARIANTS \
  ESMOE_CASE(1, 4) ESMOE_CASE(2, 4) ESMOE_CASE(4, 4) ESMOE_CASE(8, 4) ESMOE_CASE(16, 2)
#endif
#ifndef ESMOE_STAGES
#define ESMOE_STAGES 3
#endif
#ifndef ESMOE_WAVES_PER_SIMD
#define ESMOE_WAVES_PER_SIMD 1
#endif

template <bool MX>
__global__ void __launch_bounds__(kThreads, ESMOE_WAVES_PER_SIMD) grouped_gemm_kernel(GemmArgs g) {
  __shared__ __attribute__((aligned(16))) uint8_t lds[kLdsBytes];
  __shared__ int s_item;
  int* ws = g.ws;
  const int total = ws[kWsTotal];
  const int* item_start = ws + ws_item_start(g.num_experts);
  const int* order = ws + ws_order(g.num_experts);
  for (;;) {
    if (threadIdx.x == 0) s_item = atomicAdd(&ws[kWsCounter], 1);
    __syncthreads();
    const int item = __builtin_amdgcn_readfirstlane(s_item);
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
  case (MT_) * 8 + (NT_): gemm_tile<MT_, NT_, MX, ((MT_) >= 16 ? 2 : ESMOE_STAGES)>(g, e, M, t.m0, t.n0, lds); break;
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
