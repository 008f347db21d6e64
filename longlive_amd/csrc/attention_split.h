// How an attention launch is divided between its workgroups: the arithmetic shared by the kernel (device), the
// launcher (host) and the host-side checks of the test suite.  Everything here is integer arithmetic on a few
// launch-wide numbers, identical on both sides.
//
// A launch has T tiles (head x group of queries) of n_iter iterations (128 keys each) and G workgroups.  Workgroup g
// first runs `whole_rounds` whole tiles (tile j * G + g in round j).  The tiles behind those, numbered from 0 as
// "split tiles", are cut into units = split tiles x n_iter; workgroup g works through the units
// [g * units / G, (g + 1) * units / G), cut at tile boundaries into segments and walked from the end backwards.
#pragma once
#include <stdint.h>

#ifndef __HIPCC__
#define LL_SPLIT_FN inline
#else
#define LL_SPLIT_FN __host__ __device__ __forceinline__
#endif

namespace ll {

LL_SPLIT_FN uint32_t first_unit_of(uint32_t g, uint32_t units, uint32_t G) {
  return (uint32_t)((uint64_t)g * units / G);
}

struct Segment {
  uint32_t tile;   // tile number in the launch (whole tiles first, split tiles behind them)
  int begin, end;  // iterations [begin, end) of the tile
};

// Position of a workgroup in its work: whole rounds done, and the end of what is left of its share of the units.
struct WorkCursor {
  uint32_t round;
  uint32_t share_end;
};

LL_SPLIT_FN WorkCursor start_of_work(uint32_t g, uint32_t G, uint32_t units) {
  return WorkCursor{0u, first_unit_of(g + 1, units, G)};
}

// The next segment of workgroup g, or false when its work is done.
LL_SPLIT_FN bool next_segment(WorkCursor& at, uint32_t g, uint32_t G, uint32_t units, uint32_t whole_rounds,
                              uint32_t n_iter, Segment& seg) {
  if (at.round < whole_rounds) {
    seg.tile = at.round * G + g;
    seg.begin = 0;
    seg.end = (int)n_iter;
    ++at.round;
    return true;
  }
  const uint32_t share_begin = first_unit_of(g, units, G);
  if (at.share_end <= share_begin) return false;
  const uint32_t split_tile = (at.share_end - 1) / n_iter;
  const uint32_t tile_first_unit = split_tile * n_iter;
  seg.tile = whole_rounds * G + split_tile;
  seg.begin = share_begin > tile_first_unit ? (int)(share_begin - tile_first_unit) : 0;
  seg.end = (int)(at.share_end - tile_first_unit);
  at.share_end = tile_first_unit + (uint32_t)seg.begin;
  return true;
}

// The workgroups that hold a part of split tile `split_tile`: g_first .. g_last, every one of them (the launcher
// leaves no workgroup without a unit).
LL_SPLIT_FN void parts_of_tile(uint32_t split_tile, uint32_t G, uint32_t units, uint32_t n_iter, uint32_t& g_first,
                               uint32_t& g_last) {
  const uint64_t first = (uint64_t)split_tile * n_iter;
  g_first = (uint32_t)(((first + 1) * G - 1) / units);
  g_last = (uint32_t)(((first + n_iter) * G - 1) / units);
}

// Which of its two records workgroup g uses for its part of `split_tile`: the first one for the first tile it
// touches, the second one otherwise (only the first and the last tile of a share can be partial).
LL_SPLIT_FN uint32_t record_of_part(uint32_t g, uint32_t split_tile, uint32_t G, uint32_t units, uint32_t n_iter) {
  const uint32_t first_tile = first_unit_of(g, units, G) / n_iter;
  return 2 * g + (first_tile == split_tile ? 0u : 1u);
}

// ---- the launcher's choice (host).  Costs are in iterations of the 128-query kernel; whole rounds of workgroups
// count in full.
struct AttentionPlan {
  int mode;               // LL_ATTENTION_NARROW / WIDE / SPLIT
  int n_qtiles;           // query tiles per head
  uint32_t groups;        // workgroups of the launch
  uint32_t whole_rounds;  // whole tiles per workgroup
  uint32_t units;         // units of the split part (0: none)
  int64_t split_tiles;    // tiles of the split part
};

inline AttentionPlan plan_attention(int64_t Lq, int H, int64_t n_keys, int cus, int policy) {
  constexpr double kWideIteration = 1.64;  // an iteration of the 256-query kernel takes this much longer for twice the work
  constexpr double kCombine = 6.0;         // partial results: writing, counting, combining
  const int64_t n_iter = (n_keys + 127) / 128;
  const int64_t tiles_narrow = H * ((Lq + 127) / 128);
  const int64_t tiles_wide = H * ((Lq + 255) / 256);
  // Split: whole rounds first, the tiles behind them in equal shares.  A handful of left-over tiles would be cut
  // into many thin parts each (and combined by a single workgroup): then one whole round joins the split part,
  // whose shares are a little more than one tile.
  int64_t whole_rounds = tiles_wide / cus;
  if (const int64_t left = tiles_wide % cus; left > 0 && left * 4 < cus && whole_rounds > 0) --whole_rounds;
  const int64_t split_tiles = tiles_wide - whole_rounds * cus;
  const double cost_narrow = (double)((tiles_narrow + cus - 1) / cus * n_iter);
  const double cost_wide = kWideIteration * (double)((tiles_wide + cus - 1) / cus * n_iter);
  const double cost_split =
      kWideIteration * (double)(whole_rounds * n_iter + (split_tiles * n_iter + cus - 1) / cus) + kCombine;
  int mode = cost_narrow <= cost_wide && cost_narrow <= cost_split ? 0 : (cost_wide <= cost_split ? 1 : 2);
  if (policy >= 0) mode = policy;
  if (tiles_wide * n_iter >= (1ll << 31)) mode = 0;  // the unit arithmetic is 32-bit
  // Every workgroup needs a unit of the split part when there are whole rounds too (the parts of a tile are
  // counted by shares): otherwise run the tiles whole.
  if (mode == 2 && (split_tiles == 0 || (whole_rounds > 0 && split_tiles * n_iter < cus))) mode = 1;
  AttentionPlan plan{};
  plan.mode = mode;
  plan.whole_rounds = 1;
  if (mode == 0) {
    plan.n_qtiles = (int)((Lq + 127) / 128);
    plan.groups = (uint32_t)tiles_narrow;
  } else {
    plan.n_qtiles = (int)((Lq + 255) / 256);
    plan.groups = (uint32_t)tiles_wide;
    if (mode == 2) {
      plan.whole_rounds = (uint32_t)whole_rounds;
      plan.split_tiles = split_tiles;
      plan.units = (uint32_t)(split_tiles * n_iter);
      // without whole rounds no workgroup may be left without a unit either
      plan.groups = (uint32_t)(whole_rounds == 0 && plan.units < (uint32_t)cus ? plan.units : (uint32_t)cus);
    }
  }
  return plan;
}

}  // namespace ll
