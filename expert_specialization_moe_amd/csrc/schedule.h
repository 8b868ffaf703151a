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

// Row-tile heights are MT * 16 rows with MT in {1, 2, 4, 8, 12} (sched_valid_mt); a workgroup tile
// is (MT * 16) rows by 256 columns.
struct SchedPolicy {
  int force_mt;   // 0 = choose per expert; else every tile uses this MT
  int big_mt;     // MT of the full tiles of a many-row expert (8 or 12)
  int order;      // 0: heavy experts by rows ascending, light ones descending (sched_order_key); 1: expert index order;
                  // 2: most rows first for both kinds
  int light_share;  // workgroups (of every 32) that start on the light items; -1 = from the cost estimate
  int narrow_tail;  // the last so many light items are handed out as two 128-column halves each (0: none)
};

struct TileCoord {
  int mt;  // tile height / 16
  int nt;  // tile width / 64
  int m0;  // first row inside the expert
  int n0;  // first column
};

// The tile heights the kernels are compiled for.
ESMOE_HD bool sched_valid_mt(int mt) { return mt == 1 || mt == 2 || mt == 4 || mt == 8 || mt == 12; }

// Smallest tile height of the menu {1, 2, 4, 8, 12} (x16 rows) that covers `rows`, at most max_mt.
ESMOE_HD int sched_cover_mt(int rows, int max_mt) {
  const int need = (rows + 15) / 16;
  int mt = 1;
  if (need > 1) mt = 2;
  if (need > 2) mt = 4;
  if (need > 4) mt = 8;
  if (need > 8) mt = 12;
  return mt < max_mt ? mt : max_mt;
}

// Every compiled shape is 256 columns wide (NT = 4 units of 64).
ESMOE_HD int sched_nt_for(int, const SchedPolicy&) { return 4; }

ESMOE_HD int sched_ntiles(int n, int nt) { return (n + nt * 64 - 1) / (nt * 64); }

// ---- XCD-aware hand-out ------------------------------------------------------------------
// The 256 CUs sit in 8 XCDs with one L2 each, and workgroup i of a launch runs on XCD i % 8.  Tiles
// of one expert that share token rows or weight rows should therefore run at the same time on the
// same XCD: every expert with more than 64 rows ("heavy") has its tile grid cut into blocks of
// up to 32 tiles (one per CU of an XCD, at most kBlkM tiles high), block b of the launch belongs to XCD b % 8, and the
// workgroups of an XCD draw tickets from that XCD's counter: ticket t is tile t % 32 of the XCD's
// (t / 32)-th block.  A dense 6144 x 4096 x 7168 problem fetches 302 MB into L2 this way against
// 557 MB with tiles handed out in plain order.  Tickets that fall outside the grid (edge blocks) are
// skipped.  An XCD that runs out of blocks helps the others.  Experts with at most 64 rows ("light")
// have one short tile per 256 columns that streams its weights once; nothing is shared, and they come
// from one launch-wide counter.  Heavy tiles are bound by the LDS feed of the matrix cores and light
// items by HBM, so the two kinds run side by side: a share of the workgroups (sized by the cost
// estimates below) starts on the light items while the rest start on the heavy tickets, and each
// side moves on to the other kind when its own runs out.
constexpr int kBlkM = 8;
constexpr int kBlkTiles = 32;
constexpr int kXcds = 8;

ESMOE_HD bool sched_is_heavy(int m, const SchedPolicy& p) { return p.force_mt ? m > 0 : m > 64; }

// Sort key of the hand-out order (smallest first, ties by expert index).  The heavy experts and the light ones are
// handed out from separate queues, so only the order inside each kind matters.  Light items: most rows first, the
// longest items first.  Heavy experts: fewest rows first (order 0): the launch then ends on the tiles of the experts with
// the most rows, whose many blocks spread over all eight XCD queues and whose operand panels are shared behind an L2,
// where an expert of one block ends on a single queue and streams its own weights (measured against most rows first,
// order 2: C4 -2.5 %, C3 at 2048 tokens -1.8 %, C1 and C3 at 8192 tokens -0.3 to -0.8 %).
ESMOE_HD int sched_order_key(int m, const SchedPolicy& p) {
  if (p.order == 2 || !sched_is_heavy(m, p)) return (1 << 30) - m;
  return m;
}

// Row tiles of an expert: full big tiles plus one remainder tile.
ESMOE_HD int sched_mtiles(int m, const SchedPolicy& p) {
  const int rows = (p.force_mt ? p.force_mt : p.big_mt) * 16;
  return (m + rows - 1) / rows;
}

// Block shape for an expert with mtl x ntl tiles: at most kBlkM tiles high and kBlkTiles tiles in all, with
// the rows and the columns of the grid split evenly over the blocks (21 x 16 tiles -> blocks of 7 x 4;
// 6 x 16 -> 6 x 4; 1 x 16 -> 1 x 16).  Near-square blocks (in bytes) fetch the least per tile.
ESMOE_HD void sched_block_shape(int mtl, int ntl, int* bm, int* bn) {
  const int rb = (mtl + kBlkM - 1) / kBlkM;
  *bm = (mtl + rb - 1) / rb;
  const int w = kBlkTiles / *bm;
  const int cb = (ntl + w - 1) / w;
  *bn = (ntl + cb - 1) / cb;
}

ESMOE_HD int sched_heavy_blocks(int m, int n, const SchedPolicy& p) {
  if (!sched_is_heavy(m, p)) return 0;
  const int mtl = sched_mtiles(m, p), ntl = sched_ntiles(n, 4);
  int bm, bn;
  sched_block_shape(mtl, ntl, &bm, &bn);
  return ((mtl + bm - 1) / bm) * ((ntl + bn - 1) / bn);
}

ESMOE_HD int sched_light_items(int m, int n, const SchedPolicy& p) {
  return (m > 0 && !sched_is_heavy(m, p)) ? sched_ntiles(n, 4) : 0;
}

// Tile `idx` (0..31) of block `lb` of a heavy expert; false if it falls outside the expert's grid.
ESMOE_HD bool sched_decode_heavy(int lb, int idx, int m, int n, const SchedPolicy& p, TileCoord* t) {
  const int mtl = sched_mtiles(m, p), ntl = sched_ntiles(n, 4);
  int bm, bn;
  sched_block_shape(mtl, ntl, &bm, &bn);
  const int nbc = (ntl + bn - 1) / bn;
  if (idx >= bm * bn) return false;
  const int mi = (lb / nbc) * bm + idx / bn, ni = (lb % nbc) * bn + idx % bn;
  if (mi >= mtl || ni >= ntl) return false;
  const int big = p.force_mt ? p.force_mt : p.big_mt;
  const int m0 = mi * big * 16;
  t->mt = p.force_mt ? p.force_mt : (m - m0 >= big * 16 ? big : sched_cover_mt(m - m0, big));
  t->nt = 4;
  t->m0 = m0;
  t->n0 = ni * 256;
  return true;
}

// Light items are handed out whole (256 columns) except the last `narrow_tail` of the launch, which go out as two
// 128-column halves each: a launch ends on light items (they are the last of the light-first workgroups' queue, and
// what the others turn to when the heavy tickets are gone), fewer of them are left than there are workgroups, and an
// item holds a CU for as long as a tall tile, so halves spread the end of the launch over twice the CUs.
// Tickets [0, split) are the whole items 0 .. split-1, tickets split + 2j and split + 2j + 1 the halves of item split + j.
ESMOE_HD int sched_light_split(int items, const SchedPolicy& p) {
  const int narrow = p.narrow_tail < items ? p.narrow_tail : items;
  return items - (narrow > 0 ? narrow : 0);
}
ESMOE_HD int sched_light_item_of_ticket(int ticket, int split, int* half) {
  if (ticket < split) {
    *half = -1;
    return ticket;
  }
  *half = (ticket - split) & 1;
  return split + ((ticket - split) >> 1);
}

// Item `item` of a light expert; half = -1: the whole 256-column item, 0 / 1: its first / second 128 columns.
ESMOE_HD TileCoord sched_decode_light(int item, int m, const SchedPolicy& p, int half = -1) {
  TileCoord t;
  t.mt = sched_cover_mt(m, p.big_mt);
  t.nt = half < 0 ? 4 : 2;
  t.m0 = 0;
  t.n0 = item * 256 + (half > 0 ? 128 : 0);
  return t;
}

// Cost estimates in units of one tile row streamed through a CU: a heavy tile costs its padded rows; a light
// item is bound by streaming its 256 weight rows (and its few token rows) from HBM at one CU's rate, which
// takes as long as about 75 rows of a heavy tile.
ESMOE_HD long sched_heavy_cost(int m, int n, const SchedPolicy& p) {
  if (!sched_is_heavy(m, p)) return 0;
  const int big = (p.force_mt ? p.force_mt : p.big_mt) * 16;
  const int full = m / big, rem = m - full * big;
  const int rows = full * big + (rem ? (p.force_mt ? big : sched_cover_mt(rem, p.big_mt) * 16) : 0);
  return (long)(rows + 16 * sched_mtiles(m, p)) * sched_ntiles(n, 4);
}
ESMOE_HD long sched_light_cost(int m, int n, const SchedPolicy& p) {
  return (long)sched_light_items(m, n, p) * (75 + m / 3);
}
// Workgroups of every 32 that start on the light items.
ESMOE_HD int sched_light_share(long heavy_cost, long light_cost, const SchedPolicy& p) {
  if (p.light_share >= 0) return p.light_share > 32 ? 32 : p.light_share;
  if (heavy_cost <= 0 || light_cost <= 0) return 0;
  const long total = heavy_cost + light_cost;
  return (int)((32 * light_cost + total / 2) / total);
}

// Heavy ticket `ticket` of XCD `xcd` -> launch-wide block index (the caller compares it with the block total).
ESMOE_HD int sched_ticket_block(int xcd, int ticket) { return (ticket / kBlkTiles) * kXcds + xcd; }

// Workspace layout (int32 words).
constexpr int kWsLightCounter = 32;  // next light ticket to hand out (every counter has a 128-byte line of its own)
constexpr int kWsLightTotal = 1;     // number of light tickets: whole items, then two per item of the narrow tail
constexpr int kWsHeavyBlocks = 2;    // number of heavy blocks
constexpr int kWsLightShare = 3;     // workgroups of every 32 that start on the light items
constexpr int kWsLightSplit = 4;     // first light ticket that is a half item (sched_light_split)
constexpr int kWsExitCounter = 16;   // workgroups of the launch that have left the hand-out loop: the last one zeroes every counter
constexpr int kWsXcdCounter = 64;    // next heavy ticket of XCD x at word kWsXcdCounter + 32 * x (ws_xcd_counter)
constexpr int kWsHeader = 64 + 32 * kXcds;   // then one record of kRecWords per schedule position, E + 1 of them
// Record of schedule position p: first heavy block, first light item, expert index, rows (clamped at 0).
// Record E closes the prefix sums: {heavy blocks, light items, -1, 0}.
constexpr int kRecWords = 4;
constexpr int kRecBlock = 0, kRecItem = 1, kRecExpert = 2, kRecRows = 3;
ESMOE_HD int ws_xcd_counter(int xcd) { return kWsXcdCounter + 32 * xcd; }
ESMOE_HD int ws_rec(int pos) { return kWsHeader + pos * kRecWords; }
ESMOE_HD int ws_words(int num_experts) { return kWsHeader + (num_experts + 1) * kRecWords; }

// One launch per call: when the counters of a workspace are known to be zero (a workspace the library owns: it is
// zeroed when it is allocated, and the last workgroup to leave a launch zeroes the counters again), the GEMM kernel
// needs no schedule kernel in front of it: every workgroup ranks the experts and builds the records itself, one
// thread per expert, and writes them (the same values from every workgroup) for its own scalar loads.
constexpr int kSelfScheduleMaxExperts = 512;

}  // namespace esmoe
