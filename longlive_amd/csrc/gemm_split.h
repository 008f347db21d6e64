// How the persistent W4A4 GEMM divides a launch between its workgroups: the arithmetic shared by the kernel (device),
// the launcher (host) and the host-side checks of the test suite.  Integer arithmetic on four launch-wide numbers,
// identical on both sides.
//
// A launch has `tiles` output tiles (128 rows x 512 columns) of `nk` K steps (128 K elements) each and G workgroups.
// Workgroup g first runs `whole_rounds` whole tiles (tile j * G + g in round j): the workgroups of a round start
// together and move through K together, so those that share an XCD find each other's A and B lines in its L2.  The
// tiles behind the whole rounds, numbered from 0 as "split tiles", are cut into units (split tile t, step k is unit
// t * nk + k), and workgroup g takes the units [g * units / G, (g + 1) * units / G): at most the tail of one tile,
// whole tiles, and the head of another, walked from the end backwards one segment (a run of steps of one tile) at a
// time.  A segment that is not a whole tile leaves its fp32 partial tile in a record; the workgroup that arrives
// last at a tile adds the parts up, always in the same order, and writes the output.
#pragma once
#include <stdint.h>

#ifndef __HIPCC__
#define LL_GEMM_SPLIT_FN inline
#else
#define LL_GEMM_SPLIT_FN __host__ __device__ __forceinline__
#endif

namespace ll {

struct GemmDivision {
  uint32_t G;             // workgroups
  uint32_t tiles;         // output tiles
  uint32_t nk;            // K steps per tile
  uint32_t whole_rounds;  // whole tiles every workgroup runs first
};

LL_GEMM_SPLIT_FN uint32_t gemm_split_tiles(const GemmDivision& d) { return d.tiles - d.whole_rounds * d.G; }
LL_GEMM_SPLIT_FN uint64_t gemm_units(const GemmDivision& d) { return (uint64_t)gemm_split_tiles(d) * d.nk; }

// First unit of workgroup g's share (g = G: one past the last unit).
LL_GEMM_SPLIT_FN uint64_t gemm_first_unit(uint32_t g, const GemmDivision& d) { return (uint64_t)g * gemm_units(d) / d.G; }

// The workgroup whose share holds unit u: the g with first_unit(g) <= u < first_unit(g + 1).
LL_GEMM_SPLIT_FN uint32_t gemm_holder_of_unit(uint64_t u, const GemmDivision& d) {
  return (uint32_t)(((u + 1) * d.G - 1) / gemm_units(d));
}

struct GemmSegment {
  uint32_t tile;        // tile number in the launch (whole rounds first, split tiles behind them)
  uint32_t begin, end;  // K steps [begin, end) of the tile
};

// Position of a workgroup in its work: whole tiles done, and the end of what is left of its share of the units.
struct GemmCursor {
  uint32_t round;
  uint64_t share_end;
};

LL_GEMM_SPLIT_FN GemmCursor gemm_start_of_work(uint32_t g, const GemmDivision& d) {
  return GemmCursor{0u, gemm_units(d) ? gemm_first_unit(g + 1, d) : 0u};
}

// The next segment of workgroup g, or false when its work is done.
LL_GEMM_SPLIT_FN bool gemm_next_segment(GemmCursor& at, uint32_t g, const GemmDivision& d, GemmSegment& seg) {
  if (at.round < d.whole_rounds) {
    seg.tile = at.round * d.G + g;
    seg.begin = 0;
    seg.end = d.nk;
    ++at.round;
    return true;
  }
  if (gemm_units(d) == 0) return false;
  const uint64_t share_begin = gemm_first_unit(g, d);
  if (at.share_end <= share_begin) return false;
  const uint64_t split_tile = (at.share_end - 1) / d.nk, first = split_tile * d.nk;
  seg.tile = d.whole_rounds * d.G + (uint32_t)split_tile;
  seg.begin = share_begin > first ? (uint32_t)(share_begin - first) : 0u;
  seg.end = (uint32_t)(at.share_end - first);
  at.share_end = first + seg.begin;
  return true;
}

// The workgroups that hold a part of split tile `split_tile`: g_first .. g_last, every one of them.
LL_GEMM_SPLIT_FN void gemm_parts_of_tile(uint32_t split_tile, const GemmDivision& d, uint32_t& g_first, uint32_t& g_last) {
  g_first = gemm_holder_of_unit((uint64_t)split_tile * d.nk, d);
  g_last = gemm_holder_of_unit((uint64_t)split_tile * d.nk + d.nk - 1, d);
}

// Which of its two records workgroup g uses for its part of `split_tile`: the first one for the first tile its
// share touches, the second one otherwise (only the first and the last tile of a share can be partial).
LL_GEMM_SPLIT_FN uint32_t gemm_record_of_part(uint32_t g, uint32_t split_tile, const GemmDivision& d) {
  return 2 * g + ((uint32_t)(gemm_first_unit(g, d) / d.nk) == split_tile ? 0u : 1u);
}

// ---- the launcher's choice (host)
constexpr int kPTileM = 128, kPTileN = 512;  // rows and columns of an output tile

// Whether a launch runs the persistent kernel, and its division.
struct PersistentPlan {
  bool use;
  GemmDivision d;
  int tiles_m, tiles_n_each;
};
inline PersistentPlan plan_persistent(int64_t M, int64_t N, int64_t Kp, int n_products, int cus, int schedule) {
  PersistentPlan plan{};
  if (schedule == 0 /* LL_GEMM_TILES */ || schedule == 2 /* LL_GEMM_TILES_COMPILED */ || Kp % 128 != 0 || Kp >= (1 << 28) || cus < 1) return plan;
  const int64_t tiles_m = (M + kPTileM - 1) / kPTileM, tiles_n_each = (N + kPTileN - 1) / kPTileN;
  const int64_t tiles = tiles_m * tiles_n_each * n_products, nk = Kp / 128;
  if (tiles >= (1ll << 30) || tiles * nk < cus) return plan;
  // The automatic choice never takes the persistent launch.  One wave per SIMD has nobody to hide a tile's first
  // loads and its epilogue behind, and the tiles behind the whole rounds pay for their partial tiles: inside the DiT
  // block, with bias, GELU or the gated residual in the epilogue, every product measured slower (FFN-down 243 against
  // 221 us, FFN-up 300 against 224 us), and where it used to win alone (long K, at least a whole tile per workgroup:
  // 7040 x 3072 x 14336 in 505 us, 4096 x 4096 x 14336 in 355 us) the hand-scheduled tile kernels have caught up
  // (483 and 359 us).
  if (schedule == -1 /* LL_GEMM_AUTO */) return plan;
  int64_t rounds = tiles / cus;
  // A few left-over tiles would be cut into many thin parts each (or leave workgroups without a single K step, and
  // every workgroup of [first, last] must hold a part of a split tile): then one whole round joins the split part.
  if (const int64_t left = tiles % cus; left > 0 && rounds > 0 && (left * 8 < cus || left * nk < cus)) --rounds;
  plan.use = true;
  plan.d = GemmDivision{(uint32_t)cus, (uint32_t)tiles, (uint32_t)nk, (uint32_t)rounds};
  plan.tiles_m = (int)tiles_m;
  plan.tiles_n_each = (int)tiles_n_each;
  return plan;
}

// ---- which one-workgroup-per-tile kernel a launch takes (host arithmetic; the values are the header's
// LL_GEMM_KERNEL_* codes)
struct TileKernelChoice {
  int kernel;           // 0: 64 x 64, 1: 128 x 128, 2: 128 x 256, 3: 256 x 128 (four waves); 4: 128 x 256, eight waves
  bool hand_scheduled;  // the generated main loop
};
inline TileKernelChoice choose_tile_kernel(int64_t M, int64_t N, int64_t Kp, int n_products, int cus, int schedule) {
  // the generated loops address a row band with 32-bit offsets: 16 rows of Kp / 2 bytes
  const bool generated_ok = Kp % 128 == 0 && Kp < (1 << 28) && schedule != 2 /* LL_GEMM_TILES_COMPILED */;
  // At most one 128 x 256 tile per compute unit, and more than half of the units busy: one workgroup of eight waves
  // per tile, the K range of every step split between its two halves.
  if (generated_ok && Kp >= 512) {
    const int64_t tiles = ((M + 127) / 128) * ((N + 255) / 256) * n_products;
    if (tiles <= cus && 2 * tiles > cus) return {4, true};
  }
  // Small problems: when even 128 x 128 tiles would occupy at most half of the compute units, 64 x 64 tiles (more
  // decode work per MFMA, but four times the workgroups) finish sooner.
  if (((M + 127) / 128) * ((N * n_products + 127) / 128) <= cus / 2) return {0, false};
  // Two workgroups of four waves are resident per compute unit.  The 256 x 128 / 128 x 256 tiles need 6 decode
  // instructions per MFMA, the 128 x 128 tile 8, so the larger tiles win unless they fill the slots much worse.  A last
  // round of at most one workgroup per unit is cheap: alone on its unit a workgroup runs in 0.56 of the time it takes
  // next to another (measured: 252 tiles of 128 x 256 alone, 59 us, against 504 of 128 x 128 in pairs, 55 us).
  const int64_t slots = 2 * (int64_t)cus;
  auto rounds_eff = [&](int bm, int bn) {
    const int64_t tiles = ((M + bm - 1) / bm) * ((N + bn - 1) / bn) * n_products;
    const int64_t whole = tiles / slots, rest = tiles % slots;
    const double time = (double)whole + (rest == 0 ? 0.0 : (rest <= cus ? 0.564 : 1.0));
    return ((double)tiles / (double)slots) / time;
  };
  struct Cfg { int kernel, bm, bn; double bonus; };
  const Cfg cfgs[3] = {{3, 256, 128, 1.00}, {2, 128, 256, 1.00}, {1, 128, 128, 0.90}};
  int best = 3;
  double best_score = -1.0;
  for (const Cfg& c : cfgs) {
    const double sc = rounds_eff(c.bm, c.bn) * c.bonus;
    if (sc > best_score) {
      best_score = sc;
      best = c.kernel;
    }
  }
  return {best, generated_ok && best >= 2};
}

}  // namespace ll
