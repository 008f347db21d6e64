// How an attention launch is divided between its workgroups: the arithmetic shared by the kernel (device), the
// launcher (host) and the host-side checks of the test suite.  Everything here is integer arithmetic on a few
// launch-wide numbers, identical on both sides.
//
// A launch has tiles (head x group of queries) of n_iter iterations (128 keys each) and G workgroups.  Tiles whose
// group of queries is full come first in the numbering, the heads' last, partly filled groups behind them: the
// waves of such a tile that have no queries skip the matrix work, so an iteration of it costs less (`light`
// sixteenths of a full one) when the busy waves are few enough to have a SIMD each.  Workgroup g first runs `whole_rounds` whole tiles (tile j * G + g in round j);
// workgroups [0, extra) then run one more whole tile each (tile whole_rounds * G + g) and are done.  The tiles
// behind those, numbered from 0 as "split tiles", are cut into units = split tiles x n_iter, and the workgroups
// [extra, G) divide them into shares of equal cost, each cut at tile boundaries into segments and walked from the
// end backwards.
#pragma once
#include <stdint.h>

#ifndef __HIPCC__
#define LL_SPLIT_FN inline
#else
#define LL_SPLIT_FN __host__ __device__ __forceinline__
#endif

namespace ll {

constexpr uint32_t kFullUnitCost = 16;

struct Division {
  uint32_t G;             // workgroups
  uint32_t whole_rounds;  // whole tiles every workgroup runs first
  uint32_t extra;         // workgroups [0, extra) run one more whole tile and take no share of the split part
  uint32_t n_iter;        // iterations (units) per tile
  uint32_t units;         // units of the split part
  uint32_t full_units;    // of which the first full_units belong to full tiles (cost kFullUnitCost each)
  uint32_t light;         // cost of each unit behind them
};

LL_SPLIT_FN uint64_t cost_before_unit(const Division& d, uint32_t u) {
  return u <= d.full_units ? (uint64_t)kFullUnitCost * u
                           : (uint64_t)kFullUnitCost * d.full_units + (uint64_t)d.light * (u - d.full_units);
}
LL_SPLIT_FN uint64_t split_cost(const Division& d) { return cost_before_unit(d, d.units); }

// First unit of workgroup g's share (g = G: one past the last unit).  Share boundaries sit at equal distances in
// cost and are rounded down to whole units.
LL_SPLIT_FN uint32_t first_unit_of(uint32_t g, const Division& d) {
  if (g <= d.extra) return 0u;
  const uint64_t at = (uint64_t)(g - d.extra) * split_cost(d) / (d.G - d.extra);
  const uint64_t full_cost = (uint64_t)kFullUnitCost * d.full_units;
  return at <= full_cost ? (uint32_t)(at / kFullUnitCost) : d.full_units + (uint32_t)((at - full_cost) / d.light);
}

// The workgroup whose share holds unit u: the g with first_unit_of(g) <= u < first_unit_of(g + 1).
LL_SPLIT_FN uint32_t holder_of_unit(uint32_t u, const Division& d) {
  return d.extra + (uint32_t)((cost_before_unit(d, u + 1) * (d.G - d.extra) - 1) / split_cost(d));
}

struct Segment {
  uint32_t tile;   // tile number in the launch (whole tiles first, split tiles behind them)
  int begin, end;  // iterations [begin, end) of the tile
};

// Position of a workgroup in its work: whole tiles done, and the end of what is left of its share of the units.
struct WorkCursor {
  uint32_t round;
  uint32_t share_end;
};

LL_SPLIT_FN WorkCursor start_of_work(uint32_t g, const Division& d) {
  return WorkCursor{0u, d.units ? first_unit_of(g + 1, d) : 0u};
}

// The next segment of workgroup g, or false when its work is done.
LL_SPLIT_FN bool next_segment(WorkCursor& at, uint32_t g, const Division& d, Segment& seg) {
  if (at.round < d.whole_rounds || (at.round == d.whole_rounds && g < d.extra)) {
    seg.tile = at.round * d.G + g;
    seg.begin = 0;
    seg.end = (int)d.n_iter;
    ++at.round;
    return true;
  }
  if (d.units == 0) return false;
  const uint32_t share_begin = first_unit_of(g, d);
  if (at.share_end <= share_begin) return false;
  const uint32_t split_tile = (at.share_end - 1) / d.n_iter;
  const uint32_t tile_first_unit = split_tile * d.n_iter;
  seg.tile = d.whole_rounds * d.G + d.extra + split_tile;
  seg.begin = share_begin > tile_first_unit ? (int)(share_begin - tile_first_unit) : 0;
  seg.end = (int)(at.share_end - tile_first_unit);
  at.share_end = tile_first_unit + (uint32_t)seg.begin;
  return true;
}

// The workgroups that hold a part of split tile `split_tile`: g_first .. g_last, every one of them (the launcher
// leaves no workgroup of [extra, G) without a unit).
LL_SPLIT_FN void parts_of_tile(uint32_t split_tile, const Division& d, uint32_t& g_first, uint32_t& g_last) {
  g_first = holder_of_unit(split_tile * d.n_iter, d);
  g_last = holder_of_unit(split_tile * d.n_iter + d.n_iter - 1, d);
}

// Which of its two records workgroup g uses for its part of `split_tile`: the first one for the first tile it
// touches, the second one otherwise (only the first and the last tile of a share can be partial).
LL_SPLIT_FN uint32_t record_of_part(uint32_t g, uint32_t split_tile, const Division& d) {
  const uint32_t first_tile = first_unit_of(g, d) / d.n_iter;
  return 2 * g + (first_tile == split_tile ? 0u : 1u);
}

// ---- the launcher's choice (host).  Costs are in iterations of the 128-query kernel; whole rounds of workgroups
// count in full.
struct AttentionPlan {
  int mode;             // LL_ATTENTION_NARROW / WIDE / SPLIT
  int n_qtiles;         // query tiles per head
  int full_qtiles;      // of which this many come first in the tile numbering (all of them unless mode is SPLIT)
  Division d;           // G = workgroups of the launch; units = 0 unless mode is SPLIT
  int64_t split_tiles;  // tiles of the split part
};

// `allow_split` false leaves the split division out of the automatic choice (a launch that may not use the memory
// partial tiles pass through).
inline AttentionPlan plan_attention(int64_t Lq, int H, int64_t n_keys, int cus, int policy, bool allow_split = true) {
  constexpr double kWideIteration = 1.64;  // an iteration of the 256-query kernel takes this much longer for twice the work
  constexpr double kCombine = 6.0;         // partial results when every workgroup shares: writing, counting, combining
  constexpr double kCombineFew = 1.5;      // the same when only the workgroups without a whole extra tile share
  constexpr double kRound = 4.0;           // what a workgroup spends per tile outside the iterations (Q, first K/V
                                           // tile, output); fitted on 256 .. 2640 keys, where it decides
  const int64_t n_iter = (n_keys + 127) / 128;
  const int64_t tiles_narrow = H * ((Lq + 127) / 128);
  const int64_t nq = (Lq + 255) / 256;
  const int64_t tiles_wide = H * nq;
  // The last group of queries of every head holds `rest` of 256 queries.  With at most 128 of them every wave
  // that has queries has its SIMD to itself (waves w and w + 4 share one) and the tile is light: the other waves
  // only help to bring K and V in (measured: 0.68 of the time of a full tile with three of eight waves busy, and
  // 12 sixteenths weighing better than 11 with four).
  // With more, some SIMD carries two busy waves as in a full tile, and the tile counts as full.
  const int64_t rest = Lq - (nq - 1) * 256;
  const int64_t light_tiles = rest <= 128 ? H : 0, full_tiles = tiles_wide - light_tiles;
  const uint32_t light = (uint32_t)(8 + (rest + 31) / 32);  // 9 .. 12 for one to four busy waves

  // Split: `rounds` whole rounds of full tiles, `extra` more whole full tiles on the first workgroups, the rest of
  // the tiles in shares of equal cost for the other workgroups.  Two shapes are weighed against each other:
  //  (a) every left-over full tile runs whole and only the light tiles are shared out, among the workgroups that
  //      have no left-over tile - no tile is combined that need not be;
  //  (b) no extra tiles, all workgroups share everything behind the whole rounds.  A handful of left-over tiles
  //      would be cut into many thin parts each (and combined by a single workgroup): then one whole round joins
  //      the split part, whose shares are a little more than one tile.
  struct Shape { int64_t rounds, extra; double cost; };
  auto weigh = [&](int64_t rounds, int64_t extra) {
    Shape sh{rounds, extra, 1e300};
    const int64_t split_full = full_tiles - rounds * cus - extra, servers = cus - extra;
    if (rounds < 0 || extra < 0 || split_full < 0 || servers < 1) return sh;
    const int64_t cost = n_iter * ((int64_t)kFullUnitCost * split_full + (int64_t)light * light_tiles);
    if (cost == 0) return sh;  // nothing to split
    // every sharing workgroup needs a unit when others run whole tiles too (the parts of a tile are counted by shares)
    if ((rounds > 0 || extra > 0) && cost < (int64_t)kFullUnitCost * servers) return sh;
    const double share = (double)((cost + servers - 1) / servers) / kFullUnitCost;
    sh.cost = kWideIteration * ((double)(rounds * n_iter) + (extra > 0 && share < (double)n_iter ? (double)n_iter : share)) +
              kRound * (double)(rounds + 1) + (extra > 0 ? kCombineFew : kCombine);
    return sh;
  };
  int64_t rounds_b = full_tiles / cus;
  if (const int64_t left = tiles_wide - rounds_b * cus; left > 0 && left * 4 < cus && rounds_b > 0) --rounds_b;
  Shape best = weigh(rounds_b, 0);
  if (light_tiles > 0 && full_tiles % cus > 0) {
    // (a) is taken unless (b) promises more than 4 %: where the two are that close (configs[2]: 107 against 104
    // iterations) they measure the same to half a per cent, and (a) combines 8 tiles instead of 263.
    const Shape a = weigh(full_tiles / cus, full_tiles % cus);
    if (a.cost <= best.cost * 1.04) best = a;
  }
  if (!allow_split) best.cost = 1e300;
  const double cost_narrow = (double)((tiles_narrow + cus - 1) / cus) * ((double)n_iter + kRound);
  const double cost_wide = (double)((tiles_wide + cus - 1) / cus) * (kWideIteration * (double)n_iter + kRound);
  int mode = cost_narrow <= cost_wide && cost_narrow <= best.cost ? 0 : (cost_wide <= best.cost ? 1 : 2);
  if (policy >= 0) mode = policy;
  if (tiles_wide * n_iter >= (1ll << 31)) mode = 0;  // units are counted in 32 bits (costs in 64)
  if (mode == 2 && best.cost >= 1e300) mode = 1;     // nothing that could be split
  AttentionPlan plan{};
  plan.mode = mode;
  plan.d.whole_rounds = 1;
  plan.d.n_iter = (uint32_t)n_iter;
  plan.d.light = kFullUnitCost;
  if (mode == 0) {
    plan.n_qtiles = plan.full_qtiles = (int)((Lq + 127) / 128);
    plan.d.G = (uint32_t)tiles_narrow;
  } else {
    plan.n_qtiles = plan.full_qtiles = (int)nq;
    plan.d.G = (uint32_t)tiles_wide;
    if (mode == 2) {
      const int64_t split_full = full_tiles - best.rounds * cus - best.extra;
      plan.full_qtiles = (int)(light_tiles ? nq - 1 : nq);
      plan.d.whole_rounds = (uint32_t)best.rounds;
      plan.d.extra = (uint32_t)best.extra;
      plan.split_tiles = split_full + light_tiles;
      plan.d.units = (uint32_t)(plan.split_tiles * n_iter);
      plan.d.full_units = (uint32_t)(split_full * n_iter);
      plan.d.light = light_tiles ? light : kFullUnitCost;
      // without whole tiles no workgroup may be left without a unit either
      const uint64_t cost = split_cost(plan.d);
      const uint64_t shares = cost < kFullUnitCost ? 1 : cost / kFullUnitCost;  // a single light unit costs less than 16
      plan.d.G = (uint32_t)(best.rounds == 0 && best.extra == 0 && shares < (uint64_t)cus ? shares : (uint64_t)cus);
    }
  }
  return plan;
}

}  // namespace ll
