// Persistent grouped GEMM for gfx950 (MI355X): FP8-blockwise and MXFP8 variants.
//
// One launch serves every expert.  A one-workgroup schedule kernel turns problem_sizes into a list of workgroup
// tiles (schedule.h); persistent workgroups of 8 wavefronts then pull tiles from atomic counters.  A tile is
// (MT*16) token rows x 256 weight rows, MT in {1, 2, 4} (short tiles, gemm_tile) or {8, 12} (tall tiles,
// gemm_tile_pp / gemm_tile_pp_mx); the short items that end a launch are handed out as two 128-column halves.
//
// Data movement.  Per 128-wide K block the workgroup copies the token rows, the weight rows and the block's scales
// of its tile from global memory straight into LDS with global_load_lds (no staging registers, no LDS store
// instructions).  One wavefront instruction moves 8 rows x 128 bytes: 8 consecutive lanes read one row's 128
// contiguous bytes, and LDS receives the 64 lanes' 16-byte chunks back to back.  LDS rows are 128 bytes apart; chunk
// c of row r is stored in 16-byte slot c ^ ((r >> 1) & 7), which makes the MFMA fragment reads (16 rows x 16 bytes
// per quarter-wave) bank-conflict free.  Loading fragments straight from global memory is ~4x slower per CU: a
// fragment puts consecutive lanes on different rows, i.e. 64 separate 16-byte requests per instruction.
//
// Short tiles (up to 64 rows, bound by streaming their weight rows from HBM): a ring of up to 4 whole K-block
// stages (148 KB), every wavefront owns all token rows and 32 weight rows, compiler-scheduled K loop.
// Tall tiles (128 and 192 rows, bound by the matrix pipe and its feed): the K block is ONE hand-scheduled statement
// (pp_phase.h, written by gen_pp_phase.py); two groups of four wavefronts, one of each per SIMD, run half a K block
// apart, so that one group's copies and fragment reads overlap the other group's MFMAs; the ring is split by
// operand (three weight stages shared by both groups, two token stages per group).
//
// MFMA mapping (v_mfma[_scale]_f32_16x16x128_f8f6f4, both operands e4m3):
//   * the weight rows ride on the instruction's "A" side and the token rows on its "B" side, so a lane ends up with
//     4 consecutive output columns of one token row (one packed 8-byte store);
//   * lane l feeds row (l % 16); its 8 operand registers hold K bytes [16*(l/16), +16) and [64 + 16*(l/16), +16)
//     of the 128-wide K block;
//   * for the scaled form lane l supplies the E8M0 scale of row (l % 16), K sub-block (l / 16) in byte 0 of the
//     scale register.
//
// FP8-blockwise arithmetic follows the reference's blockwise mainloop order (es_fp8_blockwise_traits.cuh:35,60):
// each 128-wide K block is multiplied into a zeroed temporary and promoted into the fp32 accumulator times
// sa[row]*sb[nblk].
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <mutex>
#include <type_traits>

#include "gemm_args.h"
#include "mx_scale.h"
#include "pp_phase.h"
#include "schedule.h"
#include "swiglu.h"

namespace esmoe {

typedef int v8i __attribute__((ext_vector_type(8)));
typedef int v4i __attribute__((ext_vector_type(4)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));

constexpr int kThreads = 512;  // 8 wavefronts: two per SIMD, 256 registers each
constexpr int kWaves = kThreads / 64;
constexpr int kBN = 256;       // every tile is 256 weight rows wide
constexpr int kRingBytes = 148 * 1024;  // LDS ring of K-block stages
constexpr int kMaxKB = 256;             // K <= 32768: per-tile table of weight block scales
constexpr int kSaChunkBytes = 2 * 256 * 16;  // fp8-blockwise: two buffers of [256 rows][4 K blocks] activation scales
constexpr int kLdsBytes = kRingBytes + 2 * kMaxKB * 4 + kSaChunkBytes;
// mxfp8 keeps nothing outside the ring (its scales travel inside the stages), so its ring takes the whole
// allocation: 158 KB hold three stages of a 128-row tile where 148 KB hold two.
template <bool MX> constexpr int ring_bytes() { return MX ? kLdsBytes : kRingBytes; }

__device__ __forceinline__ v8i join(v4i lo, v4i hi) {
  v8i r;
  r[0] = lo[0]; r[1] = lo[1]; r[2] = lo[2]; r[3] = lo[3];
  r[4] = hi[0]; r[5] = hi[1]; r[6] = hi[2]; r[7] = hi[3];
  return r;
}

// 16-byte slot of chunk c in LDS row r (rows are 128 bytes apart).
__device__ __forceinline__ int swz(int r, int c) { return c ^ ((r >> 1) & 7); }

// Asynchronous global -> LDS copies: lane i's 16 (4) bytes land at lds_addr + 16*i (4*i).
// `base` and `lds_addr` are wave-uniform, `voff` is the lane's byte offset from `base`.
__device__ __forceinline__ void dma16(const void* base, uint32_t voff, uint32_t lds_addr) {
  asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(lds_addr), "v"(voff), "s"(base) : "memory", "m0");
}
__device__ __forceinline__ void dma4(const void* base, uint32_t voff, uint32_t lds_addr) {
  asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dword %1, %2" ::"s"(lds_addr), "v"(voff), "s"(base) : "memory", "m0");
}
// Groups of copies whose LDS destinations are 1024 bytes apart share one write of m0 and one base pointer and use
// the instruction's immediate offset, which the hardware adds to the LDS address and to the global address alike
// (so per-lane offset i must already have i*1024 subtracted).  Writing m0 between two copies costs a wavefront on
// the order of 150 cycles: the write waits until the previous copy has read it.  One scalar base per group keeps the
// scalar work per K block at one 64-bit add: a wavefront issues its scalar instructions 4-5 cycles apart, and a
// pointer per copy put 150 cycles of them between the barrier and the first copy.
#define ESMOE_DMA1(n, nt) "global_load_lds_dwordx4 %" #n ", %1" nt
#define ESMOE_DMAO(n, off, nt) "\n\tglobal_load_lds_dwordx4 %" #n ", %1 offset:" #off nt
template <bool NT, int N>
__device__ __forceinline__ void dma16xn(uint32_t lds_addr, const void* base, const uint32_t (&v)[N]) {
  static_assert(N >= 1 && N <= 4, "copies per group");
  if constexpr (N == 1) {
    if constexpr (NT) asm volatile("s_mov_b32 m0, %0\n\t" ESMOE_DMA1(2, " nt") ::"s"(lds_addr), "s"(base), "v"(v[0]) : "memory", "m0");
    else asm volatile("s_mov_b32 m0, %0\n\t" ESMOE_DMA1(2, "") ::"s"(lds_addr), "s"(base), "v"(v[0]) : "memory", "m0");
  } else if constexpr (N == 2) {
    if constexpr (NT) asm volatile("s_mov_b32 m0, %0\n\t" ESMOE_DMA1(2, " nt") ESMOE_DMAO(3, 1024, " nt")
                                   ::"s"(lds_addr), "s"(base), "v"(v[0]), "v"(v[1]) : "memory", "m0");
    else asm volatile("s_mov_b32 m0, %0\n\t" ESMOE_DMA1(2, "") ESMOE_DMAO(3, 1024, "")
                      ::"s"(lds_addr), "s"(base), "v"(v[0]), "v"(v[1]) : "memory", "m0");
  } else if constexpr (N == 3) {
    if constexpr (NT) asm volatile("s_mov_b32 m0, %0\n\t" ESMOE_DMA1(2, " nt") ESMOE_DMAO(3, 1024, " nt") ESMOE_DMAO(4, 2048, " nt")
                                   ::"s"(lds_addr), "s"(base), "v"(v[0]), "v"(v[1]), "v"(v[2]) : "memory", "m0");
    else asm volatile("s_mov_b32 m0, %0\n\t" ESMOE_DMA1(2, "") ESMOE_DMAO(3, 1024, "") ESMOE_DMAO(4, 2048, "")
                      ::"s"(lds_addr), "s"(base), "v"(v[0]), "v"(v[1]), "v"(v[2]) : "memory", "m0");
  } else {
    if constexpr (NT) asm volatile("s_mov_b32 m0, %0\n\t" ESMOE_DMA1(2, " nt") ESMOE_DMAO(3, 1024, " nt") ESMOE_DMAO(4, 2048, " nt")
                                   ESMOE_DMAO(5, 3072, " nt")
                                   ::"s"(lds_addr), "s"(base), "v"(v[0]), "v"(v[1]), "v"(v[2]), "v"(v[3]) : "memory", "m0");
    else asm volatile("s_mov_b32 m0, %0\n\t" ESMOE_DMA1(2, "") ESMOE_DMAO(3, 1024, "") ESMOE_DMAO(4, 2048, "") ESMOE_DMAO(5, 3072, "")
                      ::"s"(lds_addr), "s"(base), "v"(v[0]), "v"(v[1]), "v"(v[2]), "v"(v[3]) : "memory", "m0");
  }
}
// The non-temporal form (NT) is for lines that no other tile will read again (the weights of an expert that is one
// tile high): they leave L2 to the operands that are shared.  C2, all such tiles, runs 8 % faster with it.
// Read of one dword of read-only data through the scalar cache.
__device__ __forceinline__ int sload(const int* base, int byte_offset) {
  int v;
  asm volatile("s_load_dword %0, %1, %2\n\ts_waitcnt lgkmcnt(0)" : "=s"(v) : "s"(base), "s"(__builtin_amdgcn_readfirstlane(byte_offset)) : "memory");
  return __builtin_amdgcn_readfirstlane(v);
}
__device__ __forceinline__ v4i sload4(const int* base, int byte_offset) {   // 16 bytes, 16-byte aligned
  v4i v;
  asm volatile("s_load_dwordx4 %0, %1, %2\n\ts_waitcnt lgkmcnt(0)" : "=s"(v) : "s"(base), "s"(__builtin_amdgcn_readfirstlane(byte_offset)) : "memory");
  return v;
}
template <int N>
__device__ __forceinline__ void wait_vmcnt() {
  asm volatile("s_waitcnt vmcnt(%0) ; explicit" ::"n"(N) : "memory");
}
__device__ __forceinline__ void block_barrier() {
  asm volatile("" ::: "memory");
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");
}

// Shape of a short tile (MT*16 <= 64 token rows) and the layout of one ring stage (token rows, weight rows, scales):
// each of the 8 wavefronts has all token rows and 32 weight rows.  (Tall tiles: gemm_tile_pp, gemm_tile_pp_mx.)
template <int MT, bool MX, int BN = kBN>
struct TileGeom {
  static_assert(BN == 256 || BN == 128, "tile widths: 256 weight rows, or 128 for the narrow items that end a launch");
  static constexpr int BM = MT * 16;
  static constexpr int kWavesM = 1;
  static constexpr int kWavesN = kWaves / kWavesM;
  static constexpr int MTW = MT / kWavesM;          // row tiles per wavefront
  static constexpr int NTW = BN / 16 / kWavesN;     // weight-row tiles per wavefront
  static constexpr int kABytes = BM * 128;
  static constexpr int kWBytes = BN * 128;
  // scales of one K block: fp8-blockwise -> 256 floats (sa of the tile's rows); mxfp8 -> verbatim
  // 512-byte swizzled scale tiles, 2 for the weight rows then up to 2 for the token rows
  static constexpr int kScaleBytes = MX ? 2048 : 1024;
  static constexpr int kStageBytes = kABytes + kWBytes + kScaleBytes;
  // (a fifth stage for the narrow tile, whose stages are half the bytes; more would let a scale chunk, fetched four K
  // blocks ahead, be younger than the stages the loop's waits leave in flight)
  static constexpr int kMaxBuf = BN == 128 ? 5 : 4;
  static constexpr int kNBuf = ring_bytes<MX>() / kStageBytes >= kMaxBuf ? kMaxBuf : ring_bytes<MX>() / kStageBytes;
  static constexpr int kABlocks = BM / 8;                               // 8-row copy blocks of the token tile
  static constexpr int kACopies = kABlocks >= kWaves ? kABlocks / kWaves : 1;  // per wavefront
  static constexpr int kWCopies = BN / 8 / kWaves;                      // 4 (2 for the narrow tile)
  static constexpr int kCopiesPerStage = kACopies + kWCopies + 1;       // + 1 scale copy
  static_assert(kNBuf >= 2, "ring too small");
};

// The fused epilogues gather a tile's quantised bytes in LDS, BM rows of 128 bytes `stride` apart, and the workgroup
// writes them from there: eight lanes a row, a whole 128-byte line per row where the MFMA layout would give 16-byte
// pieces.  `dst` is the tile's first byte of the expert's row 0 (row pitch `pitch`); rows at or past M are not written.
template <int BM>
__device__ __forceinline__ void store_staged_rows(const uint8_t* stage, int stride, uint8_t* dst, int pitch, int M, int m0) {
  const int tid = threadIdx.x;
#pragma unroll
  for (int row = tid >> 3; row < BM; row += kThreads / 8) {
    const int m = m0 + row;
    if (m < M) __builtin_nontemporal_store(*(const v4i*)(stage + row * stride + (tid & 7) * 16), (v4i*)(dst + (long)m * pitch + (tid & 7) * 16));
  }
}

// Epilogue of a tile: `acc[nt][mt][i]` holds, for this lane, columns n0 + nw + nt*16 + 4*gq + i of token row
// m0 + mw + mt*16 + r (gq = lane / 16, r = lane % 16).  Plain form: convert and store.  FUSE: SwiGLU and the 1x128
// quantisation (the wavefront's first NTW/2 column tiles are gate columns, the rest the matching up columns).
// `lds` is scratch for the fused form and must be free: every wavefront has left the K loop.
template <int BM, int MTW, int NTW, int kWavesN, bool FUSE, typename Acc>
__device__ __forceinline__ void tile_epilogue(const GemmArgs& g, Acc& acc, int M, int m0, int n0, long row_base, int mw,
                                              int nw, int wn, int lane, bool wave_active, uint8_t* lds) {
  const int r = lane & 15, gq = lane >> 4;
  const int N = g.n;
  if constexpr (FUSE) {
    // Lane holds, of token row mw + mt*16 + r, gate (n-tiles 0 .. NTW/2-1) and up (the other half) of the h columns
    // wn*RW/2 + nt*16 + 4*gq + [0,4) of the tile's 128.  Same arithmetic, in the same order, as the unfused
    // sequence: projection rounded to the output type, silu(gate) * up in fp32, rounded to the output type, then
    // the 1x128 quantisation (block maximum floored at 1e-4, multiplier (1/amax)*448, scale amax*(1/448)).
    constexpr int kHalf = NTW / 2, kRW = NTW * 16;
    constexpr int kStageOff = 4096, kStageStride = 144;   // behind s_amax: BM rows of the tile's 128 output bytes
    static_assert(kWavesN * BM * 4 <= kStageOff, "s_amax and the stage overlap");
    const bool f16 = g.out_dtype != 0;
    float* s_amax = (float*)lds;   // [kWavesN][BM]; the ring is free: every wavefront has left the K loop
    float h[MTW][kHalf][4];
#pragma unroll
    for (int mt = 0; mt < MTW; mt++) {
      float amax = 0.f;
#pragma unroll
      for (int nt = 0; nt < kHalf; nt++) {
#pragma unroll
        for (int i = 0; i < 4; i++) {
          float gv, uv;
          if (f16) {
            gv = (float)(_Float16)acc[nt][mt][i];
            uv = (float)(_Float16)acc[nt + kHalf][mt][i];
          } else {
            gv = (float)(__bf16)acc[nt][mt][i];
            uv = (float)(__bf16)acc[nt + kHalf][mt][i];
          }
          float hv = swiglu_f32(gv, uv);
          hv = f16 ? (float)(_Float16)hv : (float)(__bf16)hv;
          h[mt][nt][i] = hv;
          amax = __builtin_fmaxf(amax, __builtin_fabsf(hv));
        }
      }
      amax = __builtin_fmaxf(amax, __shfl_xor(amax, 16));
      amax = __builtin_fmaxf(amax, __shfl_xor(amax, 32));
      if (gq == 0) s_amax[wn * BM + mw + mt * 16 + r] = amax;
    }
    __syncthreads();
    const int inter = N >> 1;
#pragma unroll
    for (int mt = 0; mt < MTW; mt++) {
      const int row = mw + mt * 16 + r;
      float amax = 0.f;
#pragma unroll
      for (int w = 0; w < kWavesN; w++) amax = __builtin_fmaxf(amax, s_amax[w * BM + row]);
      amax = __builtin_fmaxf(amax, 1e-4f);
      const float mult = (1.0f / amax) * 448.0f;
      const int m = m0 + row;
      // the row's 128 quantised bytes are gathered in LDS (a lane holds 4 of them per column tile) and leave as one line
      uint8_t* const qstage = lds + kStageOff + row * kStageStride + wn * (kRW / 2) + gq * 4;
#pragma unroll
      for (int nt = 0; nt < kHalf; nt++) {
        float y[4];
#pragma unroll
        for (int i = 0; i < 4; i++) y[i] = __builtin_amdgcn_fmed3f(h[mt][nt][i] * mult, -448.f, 448.f);
        int w0 = __builtin_amdgcn_cvt_pk_fp8_f32(y[0], y[1], 0, false);
        w0 = __builtin_amdgcn_cvt_pk_fp8_f32(y[2], y[3], w0, true);
        *(int*)(qstage + nt * 16) = w0;
      }
      if (m < M && gq == 0 && wn == 0) g.scales_out[(row_base + m) * (long)(inter >> 7) + (n0 >> 8)] = amax * (1.0f / 448.0f);
    }
    __syncthreads();
    store_staged_rows<BM>(lds + kStageOff, kStageStride, (uint8_t*)g.q_out + row_base * (long)inter + (n0 >> 1), inter, M, m0);
    __syncthreads();   // the stage and s_amax are ring memory: the next tile's copies must not land before they are read
    return;
  }
  // epilogue: lane holds columns n0 + nw + nt*16 + 4*gq + [0,4) of token row m0 + mw + mt*16 + r
  if constexpr (kWavesN == 4 && NTW == 4 && MTW >= 4) {
    // Tall tiles: a wavefront holds 64 columns of its rows, 128 bytes of output per row.  Stored straight from the MFMA
    // layout a store instruction writes 32-byte pieces of sixteen rows; passed through LDS (the ring is free, and each
    // wavefront reads back only what it wrote itself, so no barrier) it writes whole 128-byte lines of eight rows, in half
    // as many instructions.  Rows are 144 bytes apart in LDS to spread the banks.  Whole lines of output are stored with the
    // non-temporal hint: nothing in this launch reads them, and they should not push operand panels out of L2 (C4 -3 %,
    // C1 -1.8 %; the short tiles' 8-byte pieces are better off merging in L2: C2 +0.6 % with the hint).
    constexpr int kRows = MTW * 16, kStride = 144;
    uint8_t* const region = lds + ((mw / kRows) * kWavesN + wn) * (kRows * kStride);
#pragma unroll
    for (int mt = 0; mt < MTW; mt++) {
#pragma unroll
      for (int nt = 0; nt < NTW; nt++) {
        const v4f v = {acc[nt][mt][0], acc[nt][mt][1], acc[nt][mt][2], acc[nt][mt][3]};
        uint8_t* const dst = region + (mt * 16 + r) * kStride + nt * 32 + gq * 8;
        if (g.out_dtype == 0) *(bf16x4*)dst = __builtin_convertvector(v, bf16x4);
        else *(f16x4*)dst = __builtin_convertvector(v, f16x4);
      }
    }
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    const int rr = lane >> 3, ch = lane & 7;
#pragma unroll
    for (int i = 0; i < kRows / 8; i++) {
      const int row = i * 8 + rr;
      const int m = m0 + mw + row;
      const v4i line = *(const v4i*)(region + row * kStride + ch * 16);
      if (wave_active && m < M) __builtin_nontemporal_store(line, (v4i*)((uint8_t*)g.out + ((row_base + m) * (long)N + n0 + nw) * 2 + ch * 16));
    }
    return;
  }
  if (wave_active) {
#pragma unroll
    for (int mt = 0; mt < MTW; mt++) {
      int m = m0 + mw + mt * 16 + r;
      if (m < M) {
        long orow = (row_base + m) * (long)N;
#pragma unroll
        for (int nt = 0; nt < NTW; nt++) {
          int n = n0 + nw + nt * 16 + gq * 4;
          const v4f v = {acc[nt][mt][0], acc[nt][mt][1], acc[nt][mt][2], acc[nt][mt][3]};
          if (g.out_dtype == 0) {
            *(bf16x4*)((__bf16*)g.out + orow + n) = __builtin_convertvector(v, bf16x4);
          } else {
            *(f16x4*)((_Float16*)g.out + orow + n) = __builtin_convertvector(v, f16x4);
          }
        }
      }
    }
  }
}

// Fused epilogue of an mxfp8 gate_up projection: SwiGLU and the 1x32 E8M0 quantisation of the result, the operand
// format of the down projection: e4m3 bytes [total_rows, I] and scale bytes in the swizzled 512-byte tiles (128 rows x 4
// scale columns) of an operand with K = I, expert base blockscale_offsets[e] * I/32.  The arithmetic and its order are
// those of the unfused sequence (projection rounded to the output type, silu(gate) * up in fp32 rounded to the output
// type, block maximum, power-of-two scale, e4m3), so the bytes are the same.  A wavefront holds NTW/2 * 16 h columns of
// its rows: one whole 1x32 block on tall tiles, half of one on short tiles, where two neighbouring wavefronts exchange
// their maxima through LDS.  Scale bytes of the rows between the expert's last row and the end of its last 128-row
// scale tile are written as 0, as the stand-alone quantisation does.
template <int BM, int MTW, int NTW, int kWavesN, typename Acc>
__device__ __forceinline__ void tile_epilogue_mxq(const GemmArgs& g, Acc& acc, int ebso, int M, int m0, int n0,
                                                  long row_base, int mw, int wn, int lane, uint8_t* lds) {
  constexpr int kHalf = NTW / 2, kRW = NTW * 16;
  constexpr bool kPair = kHalf == 1;
  static_assert(kHalf == 1 || kHalf == 2, "a wavefront holds 16 or 32 h columns");
  const int r = lane & 15, gq = lane >> 4;
  const bool f16 = g.out_dtype != 0;
  const int inter = g.n >> 1;
  constexpr int kCodeOff = 4096, kStageOff = 5120, kStageStride = 144;   // behind s_amax: scale dwords, then the byte rows
  static_assert(kWavesN * BM * 4 <= kCodeOff && BM * 4 <= kStageOff - kCodeOff, "s_amax, the scale dwords and the stage overlap");
  float* s_amax = (float*)lds;   // [kWavesN][BM]; the ring is free: every wavefront has left the K loop
  float h[MTW][kHalf][4], amaxv[MTW];
#pragma unroll
  for (int mt = 0; mt < MTW; mt++) {
    float amax = 0.f;
#pragma unroll
    for (int nt = 0; nt < kHalf; nt++) {
#pragma unroll
      for (int i = 0; i < 4; i++) {
        float gv, uv;
        if (f16) {
          gv = (float)(_Float16)acc[nt][mt][i];
          uv = (float)(_Float16)acc[nt + kHalf][mt][i];
        } else {
          gv = (float)(__bf16)acc[nt][mt][i];
          uv = (float)(__bf16)acc[nt + kHalf][mt][i];
        }
        float hv = swiglu_f32(gv, uv);
        hv = f16 ? (float)(_Float16)hv : (float)(__bf16)hv;
        h[mt][nt][i] = hv;
        amax = __builtin_fmaxf(amax, __builtin_fabsf(hv));
      }
    }
    amax = __builtin_fmaxf(amax, __shfl_xor(amax, 16));
    amax = __builtin_fmaxf(amax, __shfl_xor(amax, 32));
    amaxv[mt] = amax;
    if (kPair && gq == 0) s_amax[wn * BM + mw + mt * 16 + r] = amax;
  }
  if constexpr (kPair) __syncthreads();
  uint8_t* sf_e = g.sf_out + (long)ebso * (inter >> 5);
  const int cblk = (n0 >> 6) + ((wn * (kRW / 2)) >> 5);   // 32-column block of this wavefront's h columns
  const int m_pad = (M + 127) & ~127;
#pragma unroll
  for (int mt = 0; mt < MTW; mt++) {
    const int row = mw + mt * 16 + r;
    const int m = m0 + row;
    float amax = amaxv[mt];
    if constexpr (kPair) amax = __builtin_fmaxf(amax, s_amax[(wn ^ 1) * BM + row]);
    const int code = mx_scale_code(amax);
    const float inv = mx_scale_inverse(amax, code);
    // the row's 128 quantised bytes and its four scale bytes (one dword of the swizzled scale tile) are gathered in LDS
    uint8_t* const qstage = lds + kStageOff + row * kStageStride + wn * (kRW / 2) + gq * 4;
#pragma unroll
    for (int nt = 0; nt < kHalf; nt++) {
      float y[4];
#pragma unroll
      for (int i = 0; i < 4; i++) y[i] = __builtin_amdgcn_fmed3f(h[mt][nt][i] * inv, -448.f, 448.f);
      int w0 = __builtin_amdgcn_cvt_pk_fp8_f32(y[0], y[1], 0, false);
      w0 = __builtin_amdgcn_cvt_pk_fp8_f32(y[2], y[3], w0, true);
      *(int*)(qstage + nt * 16) = w0;
    }
    if (gq == 0 && (!kPair || (wn & 1) == 0)) lds[kCodeOff + row * 4 + (cblk & 3)] = (uint8_t)(m < M ? code : 0);
  }
  __syncthreads();
  store_staged_rows<BM>(lds + kStageOff, kStageStride, (uint8_t*)g.q_out + row_base * (long)inter + (n0 >> 1), inter, M, m0);
  for (int row = threadIdx.x; row < BM; row += kThreads) {
    const int m = m0 + row;
    if (m < m_pad)
      *(uint32_t*)(sf_e + ((long)(m >> 7) * (inter >> 7) + (n0 >> 8)) * 512 + (m & 31) * 16 + ((m & 127) >> 5) * 4) =
          *(const uint32_t*)(lds + kCodeOff + row * 4);
  }
  // rows of the expert's last scale tile that lie below this tile: the tile's four scale columns are one dword
  if (m0 + BM >= M) {
    for (int m = m0 + BM + (int)threadIdx.x; m < m_pad; m += kThreads) {
      *(uint32_t*)(sf_e + ((long)(m >> 7) * (inter >> 7) + (n0 >> 8)) * 512 + (m & 31) * 16 + ((m & 127) >> 5) * 4) = 0u;
    }
  }
  __syncthreads();   // the stages (and s_amax) are ring memory: the next tile's copies must not land before they are read
}

// FUSE: the weights are a gate_up projection [E, 2I, K] (gate rows first) and the tile's 256 weight rows are 128 gate
// rows and the matching 128 up rows, interleaved so that every wavefront holds gate and up of the same columns; the
// epilogue forms silu(gate) * up and quantises it for the down projection (fp8-blockwise: 1x128 blocks with fp32
// scales, tile_epilogue; mxfp8: 1x32 blocks with E8M0 scales, tile_epilogue_mxq) instead of writing the projection.
template <int MT, bool MX, bool FUSE, int BN = kBN>
__device__ __forceinline__ void gemm_tile(const GemmArgs& g, int e, int erow, int ebso, int M, int m0, int n0, uint8_t* lds) {
  static_assert(!(FUSE && BN != kBN), "the fused epilogues need gate and up columns of a whole quantisation block in one tile");
  static_assert(MT == 1 || MT == 2 || MT == 4, "short tiles; 128- and 192-row tiles are gemm_tile_pp / gemm_tile_pp_mx");
  using G = TileGeom<MT, MX, BN>;
  constexpr int MTW = G::MTW, NTW = G::NTW, NBUF = G::kNBuf;
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave / G::kWavesN, wn = wave % G::kWavesN;
  const int r = lane & 15;
  const int gq = lane >> 4;
  const int K = g.k, N = g.n, KB = K >> 7;
  const long row_base = erow;
  const int nw = wn * (NTW * 16);          // first weight row of this wavefront inside the tile
  const int mw = wm * (MTW * 16);          // first token row of this wavefront inside the tile
  const bool wave_active = n0 + nw < N;
  const uint32_t lds0 = (uint32_t)(uintptr_t)lds;
  float* s_sb = (float*)(lds + kRingBytes);  // [2][kMaxKB] weight block scales of the tile's two 128-column blocks
  constexpr int kSaChunkOff = kRingBytes + 2 * kMaxKB * 4;

  // ---- copy plan -------------------------------------------------------------------------
  // A copy instruction moves the 8-row block `blk` of the stage: lane -> (row crow, slot cslot), and
  // the slot holds chunk cslot ^ ((row >> 1) & 7) = cslot ^ (crow >> 1) ^ 4*(blk & 1).  So two
  // per-lane offsets (even / odd block) serve every interior block of both operands; the block's
  // first row goes into the wave-uniform base.  Blocks that cross the end of the expert's rows
  // take a slower path that clamps the row per lane.
  const int crow = lane >> 3, cslot = lane & 7;
  const uint8_t* a_base = (const uint8_t*)g.a + (row_base + m0) * K;
  const uint8_t* w_base = (const uint8_t*)g.b + ((long)e * N + (FUSE ? 0 : n0)) * K;
  const int a_last = M - 1 - m0;   // last valid token row of the tile
  // scales
  const uint8_t* sc_base;
  uint32_t scoff, sclds;
  // fp8-blockwise activation scales sa[row][kb]: when KB is a multiple of 4 they are fetched 4 K blocks
  // at a time (16 bytes per row, one copy per wavefront every 4th K block, double-buffered outside
  // the ring); otherwise one float per row and K block travels with every stage.
  const bool sa4 = !MX && (KB & 3) == 0;
  if constexpr (!MX) {
    int row = (wave & 3) * 64 + lane;                   // wavefronts 4..7 repeat rows 0..255
    if (row > a_last) row = a_last;
    sc_base = (const uint8_t*)(g.sa + (row_base + m0) * KB);
    scoff = (uint32_t)row * (uint32_t)KB * 4;
    sclds = sa4 ? kSaChunkOff + (wave & 3) * 1024 : G::kABytes + G::kWBytes + (wave & 3) * 256;
  } else {
    const int kc = K >> 5;
    int blk;
    if ((wave & 1) == 0) {  // even wavefronts: the two weight scale tiles (FUSE: of the gate rows, of the up rows)
      blk = (n0 >> 7) + (lane >> 5);
      if (blk * 128 >= N) blk = n0 >> 7;
      if constexpr (FUSE) blk = (n0 >> 8) + (lane >> 5) * (N >> 8);
      sc_base = g.sfb + (long)e * N * kc;
    } else {                // odd wavefronts: the token scale tile(s)
      blk = (m0 >> 7) + (lane >> 5);
      if (blk * 128 >= M) blk = m0 >> 7;
      sc_base = g.sfa + (long)ebso * kc;
    }
    scoff = (uint32_t)blk * (uint32_t)KB * 512 + (lane & 31) * 16;
    sclds = G::kABytes + G::kWBytes + (wave & 1) * 1024;
  }

  // scales of K blocks 4c .. 4c+3 into chunk buffer c & 1
  auto issue_sa_chunk = [&](int c) { dma16(sc_base + (long)c * 16, scoff, lds0 + sclds + (c & 1) * 4096); };
  // copies of K block kb into ring slot buf: this wavefront's token blocks (consecutive 8-row blocks
  // wave*kACopies + i; short tiles are copied by several wavefronts), its 4 weight blocks, its share
  // of the scales.  Each copy has a per-lane byte offset from the operand's pointer for the K block: source row
  // (token rows past the expert's last are replaced by the last, weight blocks past the last weight row by valid
  // ones) times K, plus the chunk that belongs in the lane's LDS slot, minus the instruction offset i*1024; kBias
  // keeps the sum non-negative and is taken off the pointers.
  constexpr int kBias = 3072;
  const int ablk0 = (wave * G::kACopies) % G::kABlocks;
  uint32_t va[G::kACopies], vw[G::kWCopies];
#pragma unroll
  for (int i = 0; i < G::kACopies; i++) {
    const int row = (ablk0 + i) * 8 + crow;
    const int grow = row > a_last ? a_last : row;
    va[i] = (uint32_t)grow * (uint32_t)K + (swz(row, cslot) << 4) + kBias - i * 1024;
  }
#pragma unroll
  for (int i = 0; i < G::kWCopies; i++) {
    const int blk = wave * G::kWCopies + i;
    int row;
    if constexpr (FUSE) {
      // LDS rows of wavefront column c (RW rows): RW/2 gate rows of columns n0/2 + c*RW/2 .., then the up rows
      // of the same columns (weight rows I + ...)
      constexpr int kRW = NTW * 16, kBlocks = kRW / 8, kHalfBlocks = kBlocks / 2;
      const int wcol = blk / kBlocks, within = blk % kBlocks;
      row = (within / kHalfBlocks) * (N >> 1) + (n0 >> 1) + wcol * (kRW / 2) + (within % kHalfBlocks) * 8;
    } else {
      row = (n0 + blk * 8 < N ? blk : i) * 8;
    }
    vw[i] = (uint32_t)(row + crow) * (uint32_t)K + (swz(blk * 8 + crow, cslot) << 4) + kBias - i * 1024;
  }
  const uint8_t* a_ptr = a_base - kBias;
  const uint8_t* w_ptr = w_base - kBias;
  auto issue_a = [&](int kb, int buf) {
    const uint32_t sb = lds0 + buf * G::kStageBytes;
    dma16xn<false>(sb + ablk0 * 1024, a_ptr + (long)kb * 128, va);
    if constexpr (!MX) {
      if (!sa4) dma4(sc_base + (long)kb * 4, scoff, sb + sclds);
    } else {
      dma16(sc_base + (long)kb * 512, scoff, sb + sclds);
    }
  };
  const bool w_once = m0 == 0 && M <= G::BM;   // the expert is one tile high: nobody else reads these weight rows
  auto issue_w = [&](int kb, int buf) {
    const uint32_t lw = lds0 + buf * G::kStageBytes + G::kABytes + wave * G::kWCopies * 1024;
    if (w_once) dma16xn<true>(lw, w_ptr + (long)kb * 128, vw);
    else dma16xn<false>(lw, w_ptr + (long)kb * 128, vw);
  };
  auto issue = [&](int kb, int buf) { issue_a(kb, buf); issue_w(kb, buf); };

  // ---- fragment read plan ----------------------------------------------------------------
  // token fragment of row tile mt: LDS row ra = mw + mt*16 + r, chunks gq and gq+4
  // (mw, mt*16 are multiples of 16, so the slot permutation depends on r only)
  // (the high chunk gq+4 sits 4 slots = 64 bytes away in the xor order)
  const int afrag_lo = (mw + r) * 128 + swz(r, gq) * 16;
  const int wfrag_lo = G::kABytes + (nw + r) * 128 + swz(r, gq) * 16;
  constexpr int kScaleOff = G::kABytes + G::kWBytes;
  const float* sb_tab = s_sb + (FUSE ? 0 : (nw >> 7)) * kMaxKB;   // FUSE: table 0 = gate block, table 1 = up block
  // mxfp8: per-lane bases of the scale dwords (weight rows nw + r, token rows mw + r of a tall tile)
  // (FUSE: n-tile 0 = gate rows n0/2 + wn*16 + r in the first tile, n-tile 1 the up rows at the same place in the second)
  const int sfw_lane = FUSE ? kScaleOff + ((wn & 1) * 16 + r) * 16 + (wn >> 1) * 4
                            : kScaleOff + (nw >> 7) * 512 + ((nw & 127) >> 5) * 4 + ((nw & 31) + r) * 16;
  const int sfa_lane = kScaleOff + 1024 + (mw >> 7) * 512 + ((mw & 127) >> 5) * 4 + r * 16;
  const int sa_lane = kScaleOff + (mw + r) * 4;   // fp8-blockwise: float sa of token row mw + r
  const int sa4_lane = kSaChunkOff + (mw + r) * 16;

  v4f acc[NTW][MTW];
#pragma unroll
  for (int nt = 0; nt < NTW; nt++)
#pragma unroll
    for (int mt = 0; mt < MTW; mt++) acc[nt][mt] = v4f{0.f, 0.f, 0.f, 0.f};

  // The work on one K block is split in two phases:
  //   read phase: weight fragments, token fragments and all scales -> registers (every fragment of a short tile fits)
  //   mfma phase: the MFMAs (+ the fp32 promotion for fp8-blockwise) of the K block
  struct Frags {
    v8i wf[NTW];
    v8i af[MTW];
    int sfw[MX ? NTW : 1];
    int sfa[MX ? MTW : 1];
    float sc[MX ? 1 : MTW];   // fp8-blockwise: sa of the row tiles (the product with sb is formed in the mfma phase)
    float sb;
    float sb_up;   // FUSE: scale of the up rows' weight block (sb is the gate rows')
  };

  auto read_scales_fp8 = [&](int kb, int buf, Frags& f) {
    const uint8_t* lb = lds + buf * G::kStageBytes;
    f.sb = sb_tab[kb];
    if constexpr (FUSE) f.sb_up = sb_tab[kMaxKB + kb];
#pragma unroll
    for (int mt = 0; mt < MTW; mt++) {
      f.sc[mt] = sa4 ? *(const float*)(lds + sa4_lane + ((kb >> 2) & 1) * 4096 + (kb & 3) * 4 + mt * 256)
                     : *(const float*)(lb + sa_lane + mt * 64);
    }
  };

  auto read_phase = [&](int kb, int buf, Frags& f) {
    const uint8_t* lb = lds + buf * G::kStageBytes;
#pragma unroll
    for (int nt = 0; nt < NTW; nt++) {
      f.wf[nt] = join(*(const v4i*)(lb + wfrag_lo + nt * 2048), *(const v4i*)(lb + (wfrag_lo ^ 64) + nt * 2048));
    }
#pragma unroll
    for (int mt = 0; mt < MTW; mt++) {
      f.af[mt] = join(*(const v4i*)(lb + afrag_lo + mt * 2048), *(const v4i*)(lb + (afrag_lo ^ 64) + mt * 2048));
    }
    if constexpr (MX) {
      // scale dword of weight row nl = nw + nt*16 + r inside the swizzled 512-byte tiles: nw is a
      // multiple of NTW*16, so the tile / quarter / row parts of nt are compile-time offsets
#pragma unroll
      for (int nt = 0; nt < NTW; nt++) {
        constexpr int kQuarter = NTW == 4 ? 1 : 0;  // NTW = 4: nt/2 selects the 32-row quarter
        uint32_t d = *(const uint32_t*)(lb + sfw_lane + (FUSE ? nt * 512 : (nt & 1) * 256 + (kQuarter ? (nt >> 1) * 4 : 0)));
        f.sfw[nt] = (int)(d >> (gq * 8));
      }
#pragma unroll
      for (int mt = 0; mt < MTW; mt++) {
        // token row inside its 128-row scale tile (a short tile starts on a multiple of 64 rows and never crosses one)
        const int ml = (m0 & 127) + mt * 16 + r;
        const uint32_t d = *(const uint32_t*)(lb + kScaleOff + 1024 + (ml & 31) * 16 + (ml >> 5) * 4);
        f.sfa[mt] = (int)(d >> (gq * 8));
      }
    } else {
      read_scales_fp8(kb, buf, f);
    }
  };

  // fp8-blockwise: MFMAs and promotions form one scheduling region in which the four v_fmac of MFMA j - 3 follow
  // MFMA j, so the vector ALU works in the shadow of the matrix pipe and no promotion waits on the MFMA it has just been
  // issued behind.  mxfp8: the scaled MFMA accumulates in place.
  auto mfma_phase = [&](const Frags& f) {
    if constexpr (!MX) {
      float sc[MTW], sc_up[FUSE ? MTW : 1];
#pragma unroll
      for (int mt = 0; mt < MTW; mt++) {
        sc[mt] = f.sc[mt] * f.sb;
        if constexpr (FUSE) sc_up[mt] = f.sc[mt] * f.sb_up;
      }
      v4f t[MTW][NTW];
#pragma unroll
      for (int mt = 0; mt < MTW; mt++)
#pragma unroll
        for (int nt = 0; nt < NTW; nt++)
          t[mt][nt] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(f.wf[nt], f.af[mt], v4f{0.f, 0.f, 0.f, 0.f}, 0, 0, 0, 0, 0, 0);
#pragma unroll
      for (int mt = 0; mt < MTW; mt++)
#pragma unroll
        for (int nt = 0; nt < NTW; nt++)
#pragma unroll
          for (int i = 0; i < 4; i++)
            acc[nt][mt][i] = __builtin_fmaf(t[mt][nt][i], (FUSE && nt >= NTW / 2) ? sc_up[FUSE ? mt : 0] : sc[mt], acc[nt][mt][i]);
      constexpr int kT = MTW * NTW, kLag = kT < 3 ? kT : 3;
#pragma unroll
      for (int j = 0; j < kLag; j++) __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
#pragma unroll
      for (int j = kLag; j < kT; j++) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x002, 4, 0);
      }
#pragma unroll
      for (int j = 0; j < kLag; j++) __builtin_amdgcn_sched_group_barrier(0x002, 4, 0);
#pragma unroll
      for (int mt = 0; mt < MTW; mt++)
#pragma unroll
        for (int nt = 0; nt < NTW; nt++) asm volatile("" : "+v"(acc[nt][mt]));   // the promotions stay in this phase
    } else {
#pragma unroll
      for (int mt = 0; mt < MTW; mt++) {
#pragma unroll
        for (int nt = 0; nt < NTW; nt++) {
          acc[nt][mt] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(f.wf[nt], f.af[mt], acc[nt][mt], 0, 0, 0, f.sfw[nt], 0, f.sfa[mt]);
        }
        __builtin_amdgcn_sched_barrier(0);
      }
    }
  };

  // ---- pipeline --------------------------------------------------------------------------
  // prologue: the weight block scales of the whole tile ([2 column blocks][KB] floats behind the ring:
  // wavefront w copies K blocks 64*(w & 3) .. +63 of column block w >> 2, lanes past KB repeat the last
  // one), then NBUF-1 K blocks in flight.  The scale copy is asynchronous like the others and older than
  // all of them, so the first wait below covers it and nothing here waits for a whole stage.
  if constexpr (!MX) {
    const int blk = wave >> 2, kb0 = (wave & 3) * 64;
    if (kb0 < KB) {
      int nb = (n0 >> 7) + blk;
      if (nb * 128 >= N) nb = n0 >> 7;
      if constexpr (FUSE) nb = (n0 >> 8) + blk * (N >> 8);   // gate block of these columns, up block I/128 further
      const int kbi = kb0 + lane < KB ? kb0 + lane : KB - 1;
      dma4(g.sb + ((long)e * (N >> 7) + nb) * KB, (uint32_t)kbi * 4, lds0 + kRingBytes + (blk * kMaxKB + kb0) * 4);
    }
  }
  if (sa4 && wave * 64 < G::BM) issue_sa_chunk(0);
#pragma unroll
  for (int s = 0; s < NBUF - 1; s++) {
    if (s < KB) issue(s, s);
  }
  // copies outstanding per in-flight stage (the chunked scale copies are older than any stage that
  // may still be in flight when their data is needed, see the loop)
  if (KB < NBUF - 1) wait_vmcnt<0>();
  else if (sa4) wait_vmcnt<(NBUF - 2) * (G::kCopiesPerStage - 1)>();
  else wait_vmcnt<(NBUF - 2) * G::kCopiesPerStage>();
  block_barrier();

  // All eight wavefronts run in step, one barrier per K block: the stage of K block kb + NBUF - 1 is requested at the
  // top of iteration kb into the slot that iteration kb - 1 read.  (Two groups of wavefronts half an iteration apart, as in
  // the tall tiles, were measured for every short height and both kernels: 0.2-14 % slower; a short tile is bound by its
  // weight stream, not by the overlap of reads and MFMAs.)
  auto wait_stage = [&](bool more, int chunk_young) {
    // all of this wavefront's copies except those of the newest NBUF-2 K blocks have landed
    if (!more) wait_vmcnt<0>();
    else if (!sa4) wait_vmcnt<(NBUF - 2) * G::kCopiesPerStage>();
    else if (chunk_young) wait_vmcnt<(NBUF - 2) * (G::kCopiesPerStage - 1) + 1>();
    else wait_vmcnt<(NBUF - 2) * (G::kCopiesPerStage - 1)>();
  };
  int buf = 0, nbuf = NBUF - 1;  // ring slots of K block kb and of K block kb + NBUF - 1
  int chunk_age = NBUF;          // iterations since this wavefront issued a scale-chunk copy
  Frags f;
  for (int kb = 0; kb < KB; kb++) {
    const bool more = kb + NBUF - 1 < KB;
    // next chunk of activation scales, 4 K blocks before its first use (only the wavefronts whose
    // 64 rows exist in the tile fetch); `chunk_age` counts the iterations since, so that the wait
    // below can leave it in flight with the newest stages
    if (sa4 && (kb & 3) == 0 && kb + 4 < KB && wave * 64 < G::BM) {
      issue_sa_chunk((kb >> 2) + 1);
      chunk_age = 0;
    }
    __builtin_amdgcn_sched_barrier(0);
    if (more) issue(kb + NBUF - 1, nbuf);
    __builtin_amdgcn_sched_barrier(0);
    read_phase(kb, buf, f);
    __builtin_amdgcn_sched_barrier(0);
    mfma_phase(f);
    __builtin_amdgcn_sched_barrier(0);
    wait_stage(more, chunk_age < NBUF - 2);
    chunk_age++;
    block_barrier();
    buf = buf + 1 == NBUF ? 0 : buf + 1;
    nbuf = nbuf + 1 == NBUF ? 0 : nbuf + 1;
  }

  if constexpr (MX && FUSE) tile_epilogue_mxq<G::BM, MTW, NTW, G::kWavesN>(g, acc, ebso, M, m0, n0, row_base, mw, wn, lane, lds);
  else tile_epilogue<G::BM, MTW, NTW, G::kWavesN, FUSE>(g, acc, M, m0, n0, row_base, mw, nw, wn, lane, wave_active, lds);
}

// ---------------------------------------------------------------------------------------------
// Tall fp8-blockwise tiles (MT = 8 or 12, any K): the K block is one hand-scheduled statement
// (pp_phase.h, written by gen_pp_phase.py) and the ring is split by operand.
//
//   LDS   [0, 96 KB)            weight stages, 3 slots of 256 rows x 128 B, shared by the two groups
//         then 4 token regions  group g (wavefronts 4g .. 4g+3, token rows g*GR .. +GR of the tile), 2 slots each:
//                               a group copies, reads and refills only its own rows, so its refill waits for nobody else
//         then 6 scale chunks   sa of the group's rows for 4 K blocks (16 B per row), 3 buffers per group, fetched
//                               two chunks ahead in 16-row pieces, one piece per wavefront and K block
//         then the weight block scales of the tile, [2 column blocks][K blocks]
//
// Timeline in half K blocks h (barrier intervals): group 0 runs the memory phase of K block kb in h = 2kb and its matrix
// phase in 2kb + 1, group 1 one interval later.  Weight stage kb is read in 2kb and 2kb + 1 (memory phases only) and its
// slot is refilled with stage kb + 3 from 2kb + 2 on, three or more intervals before 2kb + 6; a group's token stage
// kb is read in its memory and matrix phase of kb and refilled in its memory phase of kb + 1 with stage kb + 2.
template <int MT, bool FUSE>
__device__ __forceinline__ void gemm_tile_pp(const GemmArgs& g, int e, int erow, int M, int m0, int n0, uint8_t* lds) {
  static_assert(MT == 8 || MT == 12, "hand-scheduled K block: 128- and 192-row tiles");
  constexpr int MTW = MT / 2, NTW = 4, BM = MT * 16, GR = MTW * 16;
  constexpr int kTCopies = MTW / 2;                 // token copies per wavefront and K block (8 rows each)
  constexpr int kWSlot = kBN * 128, kTSlot = GR * 128, kSaBuf = 128 * 16;
  constexpr int kTBase = 3 * kWSlot, kSaBase = kTBase + 4 * kTSlot, kSbBase = kSaBase + 6 * kSaBuf;
  static_assert(kSbBase + 2 * kMaxKB * 4 <= kLdsBytes, "LDS map of the split ring");
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int grp = wave >> 2, wj = wave & 3;
  const int r = lane & 15, gq = lane >> 4;
  // Scale chunk c holds sa of K blocks first_kb(c) .. + 3, first_kb(c) = min(4c, KB - 4) clamped at 0: the last chunk of
  // a K that is no multiple of 512 overlaps the one before instead of reaching past the row.
  const int K = g.k, N = g.n, KB = K >> 7, NCH = (KB + 3) >> 2;
  auto chunk_first_kb = [&](int c) { const int f = 4 * c < KB - 4 ? 4 * c : KB - 4; return f > 0 ? f : 0; };
  const long row_base = erow;
  const int nw = wj * 64, mw = grp * GR;
  const bool wave_active = n0 + nw < N;
  const uint32_t lds0 = (uint32_t)(uintptr_t)lds;

  // ---- copy plan (see gemm_tile for the slot permutation and the instruction offsets) ----------------------
  constexpr int kBias = 3072;
  const int crow = lane >> 3, cslot = lane & 7;
  const int a_last = M - 1 - m0;
  uint32_t va[kTCopies], vw[4], vs[4];
#pragma unroll
  for (int i = 0; i < kTCopies; i++) {
    const int lrow = (wj * kTCopies + i) * 8 + crow;      // row inside the group's token region
    const int trow = mw + lrow;
    const int grow = trow > a_last ? a_last : trow;
    va[i] = (uint32_t)grow * (uint32_t)K + (swz(lrow, cslot) << 4) + kBias - i * 1024;
  }
#pragma unroll
  for (int i = 0; i < 4; i++) {
    const int blk = wave * 4 + i;
    int row;
    if constexpr (FUSE) {
      constexpr int kRW = NTW * 16, kBlocks = kRW / 8, kHalfBlocks = kBlocks / 2;
      const int wcol = blk / kBlocks, within = blk % kBlocks;
      row = (within / kHalfBlocks) * (N >> 1) + (n0 >> 1) + wcol * (kRW / 2) + (within % kHalfBlocks) * 8;
    } else {
      row = (n0 + blk * 8 < N ? blk : i) * 8;
    }
    vw[i] = (uint32_t)(row + crow) * (uint32_t)K + (swz(blk * 8 + crow, cslot) << 4) + kBias - i * 1024;
  }
  // scale pieces: in K block kb (q = kb % 4) wavefront wj fetches rows (wj & 1)*64 + q*16 .. +16 of a chunk, lane ->
  // (row lane / 4, K block lane % 4 of the chunk); wavefronts 2 and 3 repeat what 0 and 1 fetch
#pragma unroll
  for (int q = 0; q < 4; q++) {
    const int trow = mw + (wj & 1) * 64 + q * 16 + (lane >> 2);
    const int grow = trow > a_last ? a_last : trow;
    vs[q] = (uint32_t)grow * (uint32_t)KB * 4 + ((lane & 3) < KB ? (lane & 3) : KB - 1) * 4;
  }
  const uint8_t* a_ptr = (const uint8_t*)g.a + (row_base + m0) * K - kBias;
  const uint8_t* w_ptr = (const uint8_t*)g.b + ((long)e * N + (FUSE ? 0 : n0)) * K - kBias;
  const uint8_t* sa_ptr = (const uint8_t*)(g.sa + (row_base + m0) * KB);
  const uint32_t t_dst = lds0 + kTBase + grp * 2 * kTSlot + wj * kTCopies * 1024;   // + slot * kTSlot
  const uint32_t w_dst = lds0 + wave * 4096;                                        // + slot * kWSlot
  const uint32_t s_dst = lds0 + kSaBase + grp * 3 * kSaBuf + (wj & 1) * 64 * 16;    // + buffer * kSaBuf + q * 256
  auto issue_t = [&](int kb, int slot) { dma16xn<false>(t_dst + slot * kTSlot, a_ptr + (long)kb * 128, va); };
  auto issue_w = [&](int kb, int slot) { dma16xn<false>(w_dst + slot * kWSlot, w_ptr + (long)kb * 128, vw); };

  // ---- fragment and scale read plan --------------------------------------------------------------------------
  const uint32_t wfrag = lds0 + (nw + r) * 128 + swz(r, gq) * 16;                       // + slot * kWSlot, n-tile nt at + nt*2048
  const uint32_t afrag = lds0 + kTBase + grp * 2 * kTSlot + r * 128 + swz(r, gq) * 16;  // + slot * kTSlot, row tile mt at + mt*2048
  const uint32_t sa_rd = lds0 + kSaBase + grp * 3 * kSaBuf + r * 16;                    // + buffer * kSaBuf + q*4, row tile mt at + mt*256
  const uint32_t sb_rd = lds0 + kSbBase + (FUSE ? 0 : (nw >> 7)) * kMaxKB * 4;          // + kb*4 (FUSE: up block at + kMaxKB*4)

  float acc[NTW][MTW][4];
#pragma unroll
  for (int nt = 0; nt < NTW; nt++)
#pragma unroll
    for (int mt = 0; mt < MTW; mt++)
#pragma unroll
      for (int i = 0; i < 4; i++) acc[nt][mt][i] = 0.f;

  // ---- prologue: weight block scales of the tile, scale chunks 0 and 1, token stage 0, weight stages 0 and 1 ----
  {
    const int blk = wave >> 2, kb0 = (wave & 3) * 64;
    if (kb0 < KB) {
      int nb = (n0 >> 7) + blk;
      if (nb * 128 >= N) nb = n0 >> 7;
      if constexpr (FUSE) nb = (n0 >> 8) + blk * (N >> 8);
      const int kbi = kb0 + lane < KB ? kb0 + lane : KB - 1;
      dma4(g.sb + ((long)e * (N >> 7) + nb) * KB, (uint32_t)kbi * 4, lds0 + kSbBase + (blk * kMaxKB + kb0) * 4);
    }
  }
  {
    // scale chunks 0 and 1 in the pieces the loop uses: wavefront wj the four 16-row pieces of rows (wj & 1)*64 .. +64
    // of chunk wj >> 1
    const int ch = (wj >> 1) < NCH ? (wj >> 1) : NCH - 1;
    const uint8_t* src = sa_ptr + (long)chunk_first_kb(ch) * 4;
#pragma unroll
    for (int q = 0; q < 4; q++) dma4(src, vs[q], s_dst + (wj >> 1) * kSaBuf + q * 256);
  }
  issue_t(0, 0);
  issue_w(0, 0);
  issue_w(1 < KB ? 1 : KB - 1, 1);
  wait_vmcnt<4>();
  block_barrier();
  if (grp == 1) block_barrier();

  // Weight rows that no other tile reads (the expert is one tile high) are copied with the non-temporal hint, so
  // that their stream leaves L2 to the operands that are shared.  One loop per form: a statement of each kind on
  // alternative paths of one loop would make the compiler shuffle the accumulators between them.
  const bool w_once = m0 == 0 && M <= BM;
  // The token slot, the weight slot and the copies' source offsets are in/out operands of the statement, which advances
  // them behind its MFMAs (gen_pp_phase.py, bookkeeping); the values below are those of K block 0: token slot 0 is read
  // and slot 1 filled, weight slot 0 is read and slot 2 filled, the copies fetch token stage 1 and weight stage 2.  What
  // goes with the scale chunks stays here.
  uint32_t la = t_dst + kTSlot, td = kTSlot;
  uint32_t lw = w_dst + 2 * kWSlot, woff = 0;
  const uint32_t lwbase = w_dst, lwend = w_dst + 3 * kWSlot;
  uint32_t rem = KB - 1;                       // K blocks after the one at hand
  {
    const int kbt0 = 1 < KB ? 1 : KB - 1, kbw0 = 2 < KB ? 2 : KB - 1;
#pragma unroll
    for (int i = 0; i < kTCopies; i++) va[i] += kbt0 * 128;
#pragma unroll
    for (int i = 0; i < 4; i++) vw[i] += kbw0 * 128;
  }
  uint32_t wl = wfrag, wh = wfrag ^ 64, al = afrag, ah = afrag ^ 64;
  auto k_loop = [&](auto nt_hint) {
    constexpr bool kNt = decltype(nt_hint)::value;
    int sabuf = 0;   // buffer of the scale chunk of K block kb: (kb / 4) % 3
    for (int kb = 0; kb < KB; kb++) {
      const int q = kb & 3;
      const int chw = (kb >> 2) + 2 < NCH ? (kb >> 2) + 2 : NCH - 1;
      const int sanext = sabuf >= 1 ? sabuf - 1 : 2;         // (kb / 4 + 2) % 3
      const uint32_t ls = s_dst + sanext * kSaBuf + q * 256;
      const uint8_t* sp = sa_ptr + (long)chunk_first_kb(chw) * 4;
      const uint32_t sal = sa_rd + sabuf * kSaBuf + (kb - chunk_first_kb(kb >> 2)) * 4;
      const uint32_t sbl = sb_rd + kb * 4;
      const uint32_t vsq = vs[0];
#define ESMOE_PP_STMT(NAME)                                                                                      \
  do {                                                                                                           \
    if constexpr (kNt) asm volatile(NAME##_BODY_NT : NAME##_OUTS : NAME##_INS : NAME##_CLOBBERS);                 \
    else asm volatile(NAME##_BODY : NAME##_OUTS : NAME##_INS : NAME##_CLOBBERS);                                  \
  } while (0)
      if constexpr (MT == 12 && FUSE) ESMOE_PP_STMT(ESMOE_PP12F);
      else if constexpr (MT == 12) ESMOE_PP_STMT(ESMOE_PP12);
      else if constexpr (FUSE) ESMOE_PP_STMT(ESMOE_PP8F);
      else ESMOE_PP_STMT(ESMOE_PP8);
      // the piece offsets rotate with q; the chunk buffer advances every fourth K block
      { const uint32_t t = vs[0]; vs[0] = vs[1]; vs[1] = vs[2]; vs[2] = vs[3]; vs[3] = t; }
      if (q == 3) sabuf = sabuf == 2 ? 0 : sabuf + 1;
    }
  };
  if (w_once) k_loop(std::true_type{}); else k_loop(std::false_type{});
  // the copies past the last K block (they fetched it again) must have landed before anything reuses the ring
  wait_vmcnt<0>();
  if (grp == 0) block_barrier();
  block_barrier();
  tile_epilogue<BM, MTW, NTW, 4, FUSE>(g, acc, M, m0, n0, row_base, mw, nw, wj, lane, wave_active, lds);
}

// ---------------------------------------------------------------------------------------------
// Tall mxfp8 tiles (MT = 8 or 12): the same two-group schedule and split ring as gemm_tile_pp with the scaled MFMA.
//
//   LDS   3 weight slots of 32 KB + 1 KB (the K block's two 512-byte scale tiles of the tile's 256 weight rows)
//         4 token regions (group g, 2 slots) of GR rows x 128 B + 1 KB (the two scale tiles that hold the group's rows)
//         1 KB spare, the target of the scale copies of the wavefronts that have no scale tile to fetch
// A tile may start in the middle of a 128-row scale tile (full tiles are 192 rows): a lane finds the scale dword of
// its row from the row's position inside the two tiles that were fetched for its group.
template <int MT, bool FUSE>
__device__ __forceinline__ void gemm_tile_pp_mx(const GemmArgs& g, int e, int erow, int ebso, int M, int m0, int n0, uint8_t* lds) {
  static_assert(MT == 8 || MT == 12, "hand-scheduled K block: 128- and 192-row tiles");
  constexpr int MTW = MT / 2, NTW = 4, BM = MT * 16, GR = MTW * 16;
  constexpr int kTCopies = MTW / 2;
  constexpr int kWSlot = kBN * 128 + 1024, kTSlot = GR * 128 + 1024;
  constexpr int kTBase = 3 * kWSlot, kSpare = kTBase + 4 * kTSlot;
  static_assert(kSpare + 1024 <= kLdsBytes, "LDS map of the split ring");
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int grp = wave >> 2, wj = wave & 3;
  const int r = lane & 15, gq = lane >> 4;
  const int K = g.k, N = g.n, KB = K >> 7, kc = K >> 5;
  const long row_base = erow;
  const int nw = wj * 64, mw = grp * GR;
  const bool wave_active = n0 + nw < N;
  const uint32_t lds0 = (uint32_t)(uintptr_t)lds;

  // ---- copy plan --------------------------------------------------------------------------------------------
  constexpr int kBias = 3072;
  const int crow = lane >> 3, cslot = lane & 7;
  const int a_last = M - 1 - m0;
  uint32_t va[kTCopies], vw[4];
#pragma unroll
  for (int i = 0; i < kTCopies; i++) {
    const int lrow = (wj * kTCopies + i) * 8 + crow;
    const int trow = mw + lrow;
    const int grow = trow > a_last ? a_last : trow;
    va[i] = (uint32_t)grow * (uint32_t)K + (swz(lrow, cslot) << 4) + kBias - i * 1024;
  }
#pragma unroll
  for (int i = 0; i < 4; i++) {
    const int blk = wave * 4 + i;
    int row;
    if constexpr (FUSE) {   // 32 gate rows, then the matching 32 up rows, per wavefront column (see gemm_tile_pp)
      constexpr int kRW = NTW * 16, kBlocks = kRW / 8, kHalfBlocks = kBlocks / 2;
      const int wcol = blk / kBlocks, within = blk % kBlocks;
      row = (within / kHalfBlocks) * (N >> 1) + (n0 >> 1) + wcol * (kRW / 2) + (within % kHalfBlocks) * 8;
    } else {
      row = (n0 + blk * 8 < N ? blk : i) * 8;
    }
    vw[i] = (uint32_t)(row + crow) * (uint32_t)K + (swz(blk * 8 + crow, cslot) << 4) + kBias - i * 1024;
  }
  const uint8_t* a_ptr = (const uint8_t*)g.a + (row_base + m0) * K - kBias;
  const uint8_t* w_ptr = (const uint8_t*)g.b + ((long)e * N + (FUSE ? 0 : n0)) * K - kBias;
  const uint32_t t_dst = lds0 + kTBase + grp * 2 * kTSlot + wj * kTCopies * 1024;   // + slot * kTSlot
  const uint32_t w_dst = lds0 + wave * 4096;                                        // + slot * kWSlot
  // scale copies, one per wavefront and K block: wavefront 0 the weight scale tiles (with the weight stage),
  // wavefronts 1 and 5 their group's token scale tiles (with the token stage), the others one line into the spare
  const int s_role = wave == 0 ? 0 : (wj == 1 ? 1 : 2);
  const uint8_t* s_ptr;
  uint32_t vs, s_dst;
  const int tblk0 = (m0 + mw) >> 7;          // first 128-row scale tile of the group's rows inside the expert
  if (s_role == 0) {
    int blk = (n0 >> 7) + (lane >> 5);
    if (blk * 128 >= N) blk = n0 >> 7;
    if constexpr (FUSE) blk = (n0 >> 8) + (lane >> 5) * (N >> 8);   // scale tile of the gate rows, of the up rows
    s_ptr = g.sfb + (long)e * N * kc;
    vs = (uint32_t)blk * (uint32_t)KB * 512 + (lane & 31) * 16;
    s_dst = lds0 + kBN * 128;                // + slot * kWSlot
  } else if (s_role == 1) {
    int blk = tblk0 + (lane >> 5);
    if (blk * 128 >= M) blk = tblk0 * 128 < M ? tblk0 : m0 >> 7;
    s_ptr = g.sfa + (long)ebso * kc;
    vs = (uint32_t)blk * (uint32_t)KB * 512 + (lane & 31) * 16;
    s_dst = lds0 + kTBase + grp * 2 * kTSlot + GR * 128;   // + slot * kTSlot
  } else {
    s_ptr = g.sfb + (long)e * N * kc;
    vs = 0;
    s_dst = lds0 + kSpare;
  }
  // (wave-uniform by construction; said again so that they live in scalar registers)
  s_dst = __builtin_amdgcn_readfirstlane(s_dst);
  s_ptr = (const uint8_t*)(((uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane((int)((uint64_t)s_ptr >> 32)) << 32) |
                           (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint64_t)s_ptr));
  auto issue_t = [&](int kb, int slot) { dma16xn<false>(t_dst + slot * kTSlot, a_ptr + (long)kb * 128, va); };
  auto issue_w = [&](int kb, int slot) { dma16xn<false>(w_dst + slot * kWSlot, w_ptr + (long)kb * 128, vw); };
  auto issue_s = [&](int kb, int slot) {
    dma16(s_ptr + (long)kb * 512, vs, s_dst + (s_role == 0 ? slot * kWSlot : s_role == 1 ? slot * kTSlot : 0));
  };

  // ---- fragment and scale read plan -------------------------------------------------------------------------
  const uint32_t wfrag = lds0 + (nw + r) * 128 + swz(r, gq) * 16;                       // + slot * kWSlot
  const uint32_t afrag = lds0 + kTBase + grp * 2 * kTSlot + r * 128 + swz(r, gq) * 16;  // + slot * kTSlot
  // weight scale dword of row nw + nt*16 + r: n-tile nt at + (nt & 1)*256 + (nt >> 1)*4.  FUSE: the wavefront's gate
  // rows are rows wj*32 + nt*16 + r of the first tile (n-tiles 0, 1), its up rows the same rows of the second (2, 3):
  // n-tile nt at + (nt & 1)*256 + (nt >> 1)*512
  // (+ gq: of a row's scale dword a lane reads the byte of its own K sub-block)
  const uint32_t sfw_rd = (FUSE ? lds0 + kBN * 128 + r * 16 + wj * 4
                                : lds0 + kBN * 128 + (nw >> 7) * 512 + ((nw & 127) >> 5) * 4 + ((nw & 31) + r) * 16) + gq;
  uint32_t sfa_rd[MTW];
#pragma unroll
  for (int mt = 0; mt < MTW; mt++) {
    const int ml = ((m0 + mw) & 127) + mt * 16 + r;   // row inside the group's two scale tiles
    sfa_rd[mt] = lds0 + kTBase + grp * 2 * kTSlot + GR * 128 + (ml >> 7) * 512 + (ml & 31) * 16 + ((ml & 127) >> 5) * 4 + gq;
  }

  v4f acc[NTW][MTW];
#pragma unroll
  for (int nt = 0; nt < NTW; nt++)
#pragma unroll
    for (int mt = 0; mt < MTW; mt++) acc[nt][mt] = v4f{0.f, 0.f, 0.f, 0.f};

  // ---- prologue: scale tiles and stages of K blocks 0 (tokens, weights) and 1 (weights) ------------------------
  const int kb1 = 1 < KB ? 1 : KB - 1;
  issue_s(0, 0);
  if (s_role == 0) issue_s(kb1, 1); else issue_s(0, 0);
  issue_t(0, 0);
  issue_w(0, 0);
  issue_w(kb1, 1);
  wait_vmcnt<4>();
  block_barrier();
  if (grp == 1) block_barrier();

  const bool w_once = m0 == 0 && M <= BM;   // nobody else reads these weight rows: non-temporal copies (see gemm_tile_pp)
  // Everything that changes from one K block to the next is an in/out operand of the statement, which advances it
  // behind its MFMAs (gen_pp_phase.py, mx_bookkeeping); the values below are those of K block 0: token slot 0 is
  // read and slot 1 filled, weight slot 0 is read and slot 2 filled, the copies fetch token stage 1 and weight stage 2.
  uint32_t la = t_dst + kTSlot, td = kTSlot;
  uint32_t lw = w_dst + 2 * kWSlot, woff = 0;
  const uint32_t lwbase = w_dst, lwend = w_dst + 3 * kWSlot;
  uint32_t ls = s_dst + (s_role == 0 ? 2 * kWSlot : s_role == 1 ? kTSlot : 0);
  const uint32_t lsinc = s_role == 0 ? kWSlot : s_role == 1 ? kTSlot : 0;
  const uint32_t lsend = s_role == 0 ? s_dst + 3 * kWSlot : s_role == 1 ? s_dst + 2 * kTSlot : 0xffffffffu;
  const uint32_t lswrap = s_role == 0 ? 3 * kWSlot : s_role == 1 ? 2 * kTSlot : 0;
  const uint32_t sthr = s_role == 0 ? 3 : 2;   // the scale copy goes with the weight stage (two K blocks ahead) or the token stage (one)
  uint32_t rem = KB - 1;                       // K blocks after the one at hand
  const int kbt0 = 1 < KB ? 1 : KB - 1, kbw0 = 2 < KB ? 2 : KB - 1;
#pragma unroll
  for (int i = 0; i < kTCopies; i++) va[i] += kbt0 * 128;
#pragma unroll
  for (int i = 0; i < 4; i++) vw[i] += kbw0 * 128;
  vs += (s_role == 0 ? kbw0 : kbt0) * 512;
  uint32_t wl = wfrag, wh = wfrag ^ 64, al = afrag, ah = afrag ^ 64, sfwl = sfw_rd;
  uint32_t sfal[MTW];
#pragma unroll
  for (int mt = 0; mt < MTW; mt++) sfal[mt] = sfa_rd[mt];
  auto k_loop = [&](auto nt_hint) {
    constexpr bool kNt = decltype(nt_hint)::value;
    for (int kb = 0; kb < KB; kb++) {
      if constexpr (MT == 12 && FUSE) ESMOE_PP_STMT(ESMOE_PPX12F);
      else if constexpr (MT == 12) ESMOE_PP_STMT(ESMOE_PPX12);
      else if constexpr (FUSE) ESMOE_PP_STMT(ESMOE_PPX8F);
      else ESMOE_PP_STMT(ESMOE_PPX8);
    }
  };
  if (w_once) k_loop(std::true_type{}); else k_loop(std::false_type{});
  wait_vmcnt<0>();
  if (grp == 0) block_barrier();
  block_barrier();
  if constexpr (FUSE) tile_epilogue_mxq<BM, MTW, NTW, 4>(g, acc, ebso, M, m0, n0, row_base, mw, wj, lane, lds);
  else tile_epilogue<BM, MTW, NTW, 4, false>(g, acc, M, m0, n0, row_base, mw, nw, wj, lane, wave_active, lds);
}

// ---------------------------------------------------------------------------------------------
// Schedule kernel: one workgroup, thread = expert (E <= 1024, as the reference's pre-compute kernel,
// es_fp8_blockwise_launcher.cuh:53,74).  Ranks the experts by rows (most first), prefix-sums the heavy
// experts' tile blocks and the light experts' items over that order, and zeroes the hand-out counters.
__global__ void __launch_bounds__(1024) schedule_kernel(const int* __restrict__ problem_sizes, int num_experts, int n,
                                                        SchedPolicy policy, int* __restrict__ ws) {
  __shared__ int s_m[1024];
  __shared__ int s_blocks[1024];
  __shared__ int s_items[1024];
  __shared__ long s_cost[1024][2];
  const int e = threadIdx.x;
  int m = 0;
  if (e < num_experts) m = problem_sizes[e * 3];
  if (m < 0) m = 0;
  s_m[e] = m;
  __syncthreads();
  int pos = e;
  if (e < num_experts) {
    if (policy.order != 1) {
      pos = 0;
      const int key = sched_order_key(m, policy);
      for (int j = 0; j < num_experts; j++) {
        const int kj = sched_order_key(s_m[j], policy);
        pos += (kj < key) || (kj == key && j < e);
      }
    }
    ws[ws_rec(pos) + kRecExpert] = e;
    ws[ws_rec(pos) + kRecRows] = m;
    s_blocks[pos] = sched_heavy_blocks(m, n, policy);
    s_items[pos] = sched_light_items(m, n, policy);
    s_cost[pos][0] = sched_heavy_cost(m, n, policy);
    s_cost[pos][1] = sched_light_cost(m, n, policy);
  }
  __syncthreads();
  if (e < num_experts) {
    // exclusive prefix sums over schedule positions, one position per thread
    int blocks = 0, items = 0;
    for (int j = 0; j < pos; j++) {
      blocks += s_blocks[j];
      items += s_items[j];
    }
    ws[ws_rec(pos) + kRecBlock] = blocks;
    ws[ws_rec(pos) + kRecItem] = items;
    if (pos == num_experts - 1) {
      blocks += s_blocks[pos];
      items += s_items[pos];
      ws[ws_rec(num_experts) + kRecBlock] = blocks;
      ws[ws_rec(num_experts) + kRecItem] = items;
      ws[ws_rec(num_experts) + kRecExpert] = -1;
      ws[ws_rec(num_experts) + kRecRows] = 0;
      ws[kWsHeavyBlocks] = blocks;
      const int split = sched_light_split(items, policy);
      ws[kWsLightSplit] = split;
      ws[kWsLightTotal] = split + 2 * (items - split);
      ws[kWsLightCounter] = 0;
      ws[kWsExitCounter] = 0;
      long heavy_cost = 0, light_cost = 0;
      for (int j = 0; j < num_experts; j++) {
        heavy_cost += s_cost[j][0];
        light_cost += s_cost[j][1];
      }
      ws[kWsLightShare] = sched_light_share(heavy_cost, light_cost, policy);
    }
    if (pos < kXcds) ws[ws_xcd_counter(pos)] = 0;
  }
  if (num_experts < kXcds && e >= num_experts && e < kXcds) ws[ws_xcd_counter(e)] = 0;
}

// The schedule built by the GEMM kernel itself (one launch per call; schedule.h, kSelfScheduleMaxExperts): every
// workgroup does what schedule_kernel does, one thread per expert, with block-wide scans instead of that kernel's
// per-thread loops (this runs in front of every workgroup's first tile), and writes the records into `ws`, where
// the hand-out loop finds them with scalar loads.  All workgroups write the same values.  The launch constants are
// returned instead of stored.  `lds` is the ring, free before the first tile.
__device__ __forceinline__ void self_schedule(const GemmArgs& g, uint8_t* lds, int& hblocks, int& ltotal, int& lsplit, int& lshare) {
  static_assert(kSelfScheduleMaxExperts <= kThreads, "one thread per expert");
  int* s_m = (int*)lds;                         // rows by expert
  int* s_blocks = s_m + kThreads;               // heavy blocks by schedule position
  int* s_items = s_blocks + kThreads;           // light items by schedule position
  int* s_wave = s_items + kThreads;             // per wavefront: blocks, items
  long* s_cost = (long*)(s_wave + 2 * kWaves);  // per wavefront: heavy cost, light cost
  const int E = g.num_experts, t = threadIdx.x, lane = t & 63, wave = t >> 6;
  const SchedPolicy policy = g.policy;
  int* ws = g.ws;
  int m = 0;
  if (t < E) m = g.problem_sizes[t * 3];
  if (m < 0) m = 0;
  s_m[t] = m;
  s_blocks[t] = 0;
  s_items[t] = 0;
  __syncthreads();
  long hc = 0, lc = 0;
  if (t < E) {
    int pos = t;
    if (policy.order != 1) {
      pos = 0;
      const int key = sched_order_key(m, policy);
      for (int j = 0; j < E; j++) {
        const int kj = sched_order_key(s_m[j], policy);
        pos += (kj < key) || (kj == key && j < t);
      }
    }
    ws[ws_rec(pos) + kRecExpert] = t;
    ws[ws_rec(pos) + kRecRows] = m;
    s_blocks[pos] = sched_heavy_blocks(m, g.n, policy);
    s_items[pos] = sched_light_items(m, g.n, policy);
    hc = sched_heavy_cost(m, g.n, policy);
    lc = sched_light_cost(m, g.n, policy);
  }
  __syncthreads();
  // exclusive prefix sums over the schedule positions (thread = position): inclusive scan inside the wavefront, then
  // the totals of the wavefronts in front
  const int b = s_blocks[t], it = s_items[t];
  int sb = b, si = it;
#pragma unroll
  for (int d = 1; d < 64; d <<= 1) {
    const int ub = __shfl_up(sb, d), ui = __shfl_up(si, d);
    if (lane >= d) {
      sb += ub;
      si += ui;
    }
  }
#pragma unroll
  for (int d = 1; d < 64; d <<= 1) {
    hc += __shfl_xor(hc, d);
    lc += __shfl_xor(lc, d);
  }
  if (lane == 63) {
    s_wave[2 * wave] = sb;
    s_wave[2 * wave + 1] = si;
    s_cost[2 * wave] = hc;
    s_cost[2 * wave + 1] = lc;
  }
  __syncthreads();
  int blocks_before = 0, items_before = 0, blocks = 0, items = 0;
  long heavy_cost = 0, light_cost = 0;
#pragma unroll
  for (int w = 0; w < kWaves; w++) {
    const int wb = s_wave[2 * w], wi = s_wave[2 * w + 1];
    if (w < wave) {
      blocks_before += wb;
      items_before += wi;
    }
    blocks += wb;
    items += wi;
    heavy_cost += s_cost[2 * w];
    light_cost += s_cost[2 * w + 1];
  }
  if (t < E) {
    ws[ws_rec(t) + kRecBlock] = blocks_before + sb - b;
    ws[ws_rec(t) + kRecItem] = items_before + si - it;
  }
  if (t == 0) {
    ws[ws_rec(E) + kRecBlock] = blocks;
    ws[ws_rec(E) + kRecItem] = items;
    ws[ws_rec(E) + kRecExpert] = -1;
    ws[ws_rec(E) + kRecRows] = 0;
  }
  hblocks = __builtin_amdgcn_readfirstlane(blocks);
  lsplit = __builtin_amdgcn_readfirstlane(sched_light_split(items, policy));
  ltotal = __builtin_amdgcn_readfirstlane(lsplit + 2 * (items - lsplit));
  lshare = __builtin_amdgcn_readfirstlane(sched_light_share(heavy_cost, light_cost, policy));
  // the records are read back with scalar loads: every store of this workgroup has to be in L2 first.  (Also a
  // compiler-visible full wait in front of the copy-pipelined K loops, which count their own copies.)
  __builtin_amdgcn_s_waitcnt(0);
  __syncthreads();
}

template <bool MX, bool FUSE>
__global__ void __launch_bounds__(kThreads) grouped_gemm_kernel(GemmArgs g) {
  __shared__ __attribute__((aligned(1024))) uint8_t lds[kLdsBytes];
  __shared__ int s_item;
  __shared__ int s_counters[kXcds + 1];
  int* ws = g.ws;
  int hblocks, ltotal, lsplit, lshare;
  if (g.self_schedule) {
    self_schedule(g, lds, hblocks, ltotal, lsplit, lshare);
  } else {
    hblocks = ws[kWsHeavyBlocks];
    ltotal = ws[kWsLightTotal];
    lsplit = ws[kWsLightSplit];
    lshare = ws[kWsLightShare];
  }
  // Workgroup i runs on XCD i % 8 (HW_REG_XCC_ID = 20, bits [3:0], says so directly).  Of every 32 workgroups
  // of an XCD the last `light_share` start on the light items, the others on the heavy tickets; either kind
  // moves on to the other when its own is exhausted.
  const int xcd = __builtin_amdgcn_s_getreg(20 | (0 << 6) | (3 << 11)) & (kXcds - 1);
  const int per_xcd = (int)gridDim.x / kXcds > 0 ? (int)gridDim.x / kXcds : 1;
  const bool light_first = (int)(blockIdx.x / kXcds) * 32 / per_xcd >= 32 - lshare;
  int phase = 0, q = 0;
  // Queues known to be exhausted (bits 0-7: the XCDs' heavy queues, bit 8: the light items).  When a draw comes back
  // past the end of its queue and the launch has heavy blocks on every XCD, one look at all nine counters marks every
  // queue that has run dry, so that a workgroup leaving its own queue does not spend an atomic round trip (about a
  // microsecond under load) on each empty one.
  int dead = ltotal == 0 ? 256 : 0;
#pragma unroll
  for (int x = 0; x < kXcds; x++)
    if (x >= hblocks) dead |= 1 << x;
  for (;;) {
    const bool light = (phase == 0) == light_first;
    const int xq = (xcd + q) & (kXcds - 1);
    if ((dead >> (light ? 8 : xq)) & 1) {   // nothing (left) in this queue: the next XCD's, then the other kind
      if (light || ++q == kXcds) {
        q = 0;
        if (++phase == 2) break;
      }
      continue;
    }
    if (threadIdx.x == 0) s_item = atomicAdd(light ? &ws[kWsLightCounter] : &ws[ws_xcd_counter(xq)], 1);
    __syncthreads();
    const int ticket = __builtin_amdgcn_readfirstlane(s_item);
    const int kind = light ? kRecItem : kRecBlock;
    const int v = light ? ticket : sched_ticket_block(xq, ticket);
    if (v >= (light ? ltotal : hblocks)) {   // this queue is exhausted: see which others are
      dead |= 1 << (light ? 8 : xq);
      __syncthreads();                        // s_item and s_counters are rewritten next
      // (worth its round trip only when every XCD has a queue to try: the look itself reads the hot counter line)
      if (hblocks <= kXcds) continue;
      if (threadIdx.x < kXcds + 1)
        s_counters[threadIdx.x] = __hip_atomic_load(threadIdx.x < kXcds ? &ws[ws_xcd_counter(threadIdx.x)] : &ws[kWsLightCounter],
                                                    __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      __syncthreads();
#pragma unroll
      for (int x = 0; x < kXcds; x++) {
        // queue x holds the blocks x, x + 8, ...: 32 tickets each
        const int tickets = x < hblocks ? ((hblocks - x + kXcds - 1) / kXcds) * kBlkTiles : 0;
        if (__builtin_amdgcn_readfirstlane(s_counters[x]) >= tickets) dead |= 1 << x;
      }
      if (__builtin_amdgcn_readfirstlane(s_counters[kXcds]) >= ltotal) dead |= 256;
      continue;
    }
    // schedule position of v: the last one whose first block (item) is <= v, found by bisection over the prefix
    // sums with scalar loads.  The records are written by the schedule kernel and only read here, so they stay in
    // the scalar cache, where a step costs a fraction of what a trip to L2 costs while the chip streams weights.
    // (a light ticket past `lsplit` is one half of an item of the narrow tail)
    int half = -1;
    const int idx = light ? sched_light_item_of_ticket(v, lsplit, &half) : v;
    int lo = 0, hi = g.num_experts;
    while (hi - lo > 1) {
      const int mid = (lo + hi) >> 1;
      if (sload(ws, (ws_rec(mid) + kind) * 4) <= idx) lo = mid; else hi = mid;
    }
    // the whole record in one load, then the expert's first row (and first scale row) through the scalar cache as
    // well: a vector load here waits its turn behind the weight streams of the whole chip
    const v4i rec = sload4(ws, ws_rec(lo) * 4);
    const int first = __builtin_amdgcn_readfirstlane(light ? rec[kRecItem] : rec[kRecBlock]);
    const int e = __builtin_amdgcn_readfirstlane(rec[kRecExpert]), M = __builtin_amdgcn_readfirstlane(rec[kRecRows]);
    const int erow = sload(g.expert_offsets, e * 4);
    const int ebso = MX ? sload(g.blockscale_offsets, e * 4) : 0;
    const int local = idx - first;
    TileCoord t;
    if (light) t = sched_decode_light(local, M, g.policy, half);
    else if (!sched_decode_heavy(local, ticket % kBlkTiles, M, g.n, g.policy, &t)) {
      __syncthreads();   // s_item is rewritten next: every wavefront must have read this ticket first
      continue;
    }
    // (wave-uniform by construction; said again so that the copies' base pointers stay in scalar registers)
    t.mt = __builtin_amdgcn_readfirstlane(t.mt);
    t.nt = __builtin_amdgcn_readfirstlane(t.nt);
    t.m0 = __builtin_amdgcn_readfirstlane(t.m0);
    t.n0 = __builtin_amdgcn_readfirstlane(t.n0);
    if (t.n0 >= g.n) {   // second half of a last column tile that is 128 columns wide
      __syncthreads();
      continue;
    }
    // Tile heights (MT * 16 rows): 8 and 12 are the tall tiles with the hand-scheduled K block, 1, 2 and 4 the short
    // ones, also as 128-column halves.  The host refuses a policy that asks for any other height (launch_gemm), so
    // every ticket finds its tile function here.
    if (t.mt == 12) {
      if constexpr (MX) gemm_tile_pp_mx<12, FUSE>(g, e, erow, ebso, M, t.m0, t.n0, lds);
      else gemm_tile_pp<12, FUSE>(g, e, erow, M, t.m0, t.n0, lds);
    } else if (t.mt == 8) {
      if constexpr (MX) gemm_tile_pp_mx<8, FUSE>(g, e, erow, ebso, M, t.m0, t.n0, lds);
      else gemm_tile_pp<8, FUSE>(g, e, erow, M, t.m0, t.n0, lds);
    } else if (!FUSE && t.nt == 2) {
      if constexpr (!FUSE) {
        if (t.mt == 1) gemm_tile<1, MX, false, 128>(g, e, erow, ebso, M, t.m0, t.n0, lds);
        else if (t.mt == 2) gemm_tile<2, MX, false, 128>(g, e, erow, ebso, M, t.m0, t.n0, lds);
        else gemm_tile<4, MX, false, 128>(g, e, erow, ebso, M, t.m0, t.n0, lds);
      }
    } else {
      if (t.mt == 1) gemm_tile<1, MX, FUSE>(g, e, erow, ebso, M, t.m0, t.n0, lds);
      else if (t.mt == 2) gemm_tile<2, MX, FUSE>(g, e, erow, ebso, M, t.m0, t.n0, lds);
      else gemm_tile<4, MX, FUSE>(g, e, erow, ebso, M, t.m0, t.n0, lds);
    }
  }
  // The last workgroup to leave zeroes the hand-out counters (nobody draws any more: every workgroup counts itself
  // out after its last draw), so a workspace that held zero counters before the launch holds them again after it.
  if (threadIdx.x == 0) {
    const int left = atomicAdd(&ws[kWsExitCounter], 1);
    if (left == (int)gridDim.x - 1) {
#pragma unroll
      for (int x = 0; x < kXcds; x++) __hip_atomic_store(&ws[ws_xcd_counter(x)], 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      __hip_atomic_store(&ws[kWsLightCounter], 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      __hip_atomic_store(&ws[kWsExitCounter], 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
  }
}

}  // namespace esmoe

// Schedule workspace owned by the library, for callers that may not allocate (esmoe_fp8_blockwise_grouped_mm_static in
// esmoe.h): room for the records and counters of kStaticScratchExperts experts.  Every GPU the library runs on holds
// its own copy at its own address until the process ends; the name below is only the host-side handle of the
// symbol, never a device address, so host code goes through esmoe_static_scratch().
constexpr int kStaticScratchExperts = 1024;
constexpr int kStaticScratchWords = (esmoe::kWsHeader + (kStaticScratchExperts + 1) * esmoe::kRecWords + 63) / 64 * 64;
static __device__ __align__(256) int32_t scratch[kStaticScratchWords];

// Device address and size of the current device's copy of the static workspace; the address is looked up once
// per device (with that device current) and kept.
extern "C" int esmoe_static_scratch(int32_t** ptr, size_t* bytes, int* max_experts) {
  static int32_t* addr[64];
  static std::mutex mu;
  int dev = 0;
  hipError_t err = hipGetDevice(&dev);
  if (err != hipSuccess) return (int)err;
  if (dev < 0 || dev >= 64) return (int)hipErrorInvalidDevice;
  std::lock_guard<std::mutex> lock(mu);
  if (!addr[dev]) {
    void* p = nullptr;
    err = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (err != hipSuccess) return (int)err;
    if (!p) return (int)hipErrorInvalidSymbol;
    addr[dev] = (int32_t*)p;
  }
  *ptr = addr[dev];
  *bytes = sizeof(int32_t) * kStaticScratchWords;
  *max_experts = kStaticScratchExperts;
  return 0;
}

extern "C" int esmoe_launch_grouped_gemm(const esmoe::GemmArgs* args, int mx, int grid, hipStream_t stream) {
  using namespace esmoe;
  if (args->self_schedule && args->num_experts > kSelfScheduleMaxExperts) return (int)hipErrorInvalidValue;
  if (!args->self_schedule) {
    hipLaunchKernelGGL(schedule_kernel, dim3(1), dim3((args->num_experts + 63) & ~63), 0, stream, args->problem_sizes, args->num_experts,
                       args->n, args->policy, args->ws);
    hipError_t err = hipGetLastError();
    if (err != hipSuccess) return (int)err;
  }
  if (mx && args->q_out)
    hipLaunchKernelGGL((grouped_gemm_kernel<true, true>), dim3(grid), dim3(kThreads), 0, stream, *args);
  else if (mx)
    hipLaunchKernelGGL((grouped_gemm_kernel<true, false>), dim3(grid), dim3(kThreads), 0, stream, *args);
  else if (args->q_out)
    hipLaunchKernelGGL((grouped_gemm_kernel<false, true>), dim3(grid), dim3(kThreads), 0, stream, *args);
  else
    hipLaunchKernelGGL((grouped_gemm_kernel<false, false>), dim3(grid), dim3(kThreads), 0, stream, *args);
  return (int)hipGetLastError();
}
