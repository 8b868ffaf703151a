// Tile schedule of the persistent grouped GEMM: how one expert's M x N output is
// cut into workgroup tiles and how a linear work-item index maps back to a tile.
//
// This takes the place of the reference's three M-bucket problem lists
// (expert_specialization/csrc/cuda/es_fp8_blockwise_functor.cuh:121-256): instead
// of routing whole experts to one of three differently tiled kernels, every
// expert is cut into full "big" row tiles plus one remainder tile whose height is
// the smallest menu entry that covers the leftover rows, and all tiles of all
// experts feed one persistent kernel.
//
// The same functions compile for the device (hipcc) and for the host (plain C++),
// so the index math is unit-tested on the CPU.
#pragma once
#include <stdint.h>

#if defined(__HIPCC__)
#define ESMOE_HD __host__ __device__ __forceinline__
#else
#define ESMOE_HD inline
#endif

namespace esmoe {

// Row-tile heights are MT * 16 rows with MT in {1, 2, 4, 8, 12, 16}; a workgroup tile
// is (MT * 16) rows by 256 columns.
struct SchedPolicy {
  int force_mt;   // 0 = choose per expert; else every tile uses this MT
  int big_mt;     // MT of the full tiles of a many-row expert (8, 12 or 16)
  int order;      // 0: experts sorted by rows, most rows first; 1: expert index order
};

struct TileCoord {
  int mt;  // tile height / 16
  int nt;  // tile width / 64
  int m0;  // first row inside the expert
  int n0;  // first column
};

// Smallest tile height of the menu {1, 2, 4, 8, 12, 16} (x16 rows) that covers `rows`, at most max_mt.
ESMOE_HD int sched_cover_mt(int rows, int max_mt) {
  const int need = (rows + 15) / 16;
  int mt = 1;
  if (need > 1) mt = 2;
  if (need > 2) mt = 4;
  if (need > 4) mt = 8;
  if (need > 8) mt = 12;
  if (need > 12) mt = 16;
  return mt < max_mt ? mt : max_mt;
}

// Every compiled shape is 256 columns wide (NT = 4 units of 64).
ESMOE_HD int sched_nt_for(int, const SchedPolicy&) { return 4; }

ESMOE_HD int sched_ntiles(int n, int nt) { return (n + nt * 64 - 1) / (nt * 64); }

// Number of work items of an expert with `m` rows and `n` columns.
ESMOE_HD int sched_items(int m, int n, const SchedPolicy& p) {
  if (m <= 0) return 0;
  if (p.force_mt) {
    int rows = p.force_mt * 16;
    return ((m + rows - 1) / rows) * sched_ntiles(n, sched_nt_for(p.force_mt, p));
  }
  int big_rows = p.big_mt * 16;
  int full = m / big_rows;
  int rem = m - full * big_rows;
  int items = full * sched_ntiles(n, sched_nt_for(p.big_mt, p));
  if (rem) {
    int rmt = sched_cover_mt(rem, p.big_mt);
    items += sched_ntiles(n, sched_nt_for(rmt, p));
  }
  return items;
}

// Inverse of the enumeration counted by sched_items: column tiles vary fastest,
// full row tiles come first, the remainder tile last.
ESMOE_HD TileCoord sched_decode(int item, int m, int n, const SchedPolicy& p) {
  TileCoord t;
  if (p.force_mt) {
    t.mt = p.force_mt;
    t.nt = sched_nt_for(t.mt, p);
    int ntl = sched_ntiles(n, t.nt);
    t.m0 = (item / ntl) * t.mt * 16;
    t.n0 = (item % ntl) * t.nt * 64;
    return t;
  }
  int big_rows = p.big_mt * 16;
  int full = m / big_rows;
  int nt_big = sched_nt_for(p.big_mt, p);
  int ntl_big = sched_ntiles(n, nt_big);
  int full_items = full * ntl_big;
  if (item < full_items) {
    t.mt = p.big_mt;
    t.nt = nt_big;
    t.m0 = (item / ntl_big) * big_rows;
    t.n0 = (item % ntl_big) * nt_big * 64;
    return t;
  }
  int rem = m - full * big_rows;
  t.mt = sched_cover_mt(rem, p.big_mt);
  t.nt = sched_nt_for(t.mt, p);
  t.m0 = full * big_rows;
  t.n0 = (item - full_items) * t.nt * 64;
  return t;
}

// Workspace layout (int32 words).
constexpr int kWsCounter = 0;   // next work item to hand out
constexpr int kWsTotal = 1;     // number of work items
constexpr int kWsHeader = 8;    // then item_start[E + 1] (by schedule position), then order[E]
ESMOE_HD int ws_item_start(int) { return kWsHeader; }
ESMOE_HD int ws_order(int num_experts) { return kWsHeader + num_experts + 1; }
ESMOE_HD int ws_words(int num_experts) { return kWsHeader + 2 * num_experts + 1; }

}  // namespace esmoe
