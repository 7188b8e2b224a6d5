// Work decomposition of the grouped GEMM: which (tile, K range) items a workgroup processes, in which
// order, and which workgroup completes a tile that several workgroups shared along K.  Pure integer
// arithmetic on the problem table.  It runs on the host: fp8gmm_plan_grouped_gemm_launch (plan.cpp) writes the
// schedule out as the work list the kernels read, and the introspection entry points show it to the CPU tests.
#pragma once

#include <stdint.h>

#include "fp8gmm.h"
#include "tiling.h"

#if defined(__HIPCC__)
#define FP8GMM_HD __host__ __device__ inline __attribute__((always_inline))
#else
#define FP8GMM_HD inline
#endif

namespace fp8gmm {

// ---- tail balancing (stream-K over the remainder of an XCD's tile range) ----
// A range of n tiles on W workgroups takes ceil(n / W) rounds; when the last round is mostly empty the
// remainder tiles are cut along K instead: the region's K = 128 steps are dealt out in equal contiguous
// pieces, up to W of them.  A piece that does not cover
// a whole tile leaves its fp32 accumulators in a workspace slot; a second, small kernel adds the pieces
// of such a tile in K order and runs the normal epilogue.  No workgroup ever waits for another one.
constexpr int kSkMinPairs = 4;        // never cut pieces shorter than this many K = 128 steps
constexpr int kSkMaxPieces = 8;       // average pieces per tile the region may be cut into
constexpr int kSkMaxRounds = 24;      // with more full rounds than this the tail cannot cost enough to share it
// The second launch, which completes the shared tiles, costs about kSkFixupLaunch K = 128 steps of time (5 us:
// the gap between two launches) plus kSkFixupPerTile / 100 steps per shared tile of the XCD (four workgroups per
// tile on 256 compute units, a megabyte of partial sums each), three times that when it has the GELU epilogue to
// apply; sharing has to save half as much again.
constexpr int kSkFixupLaunch = 4;
constexpr int kSkFixupPerTile = 75;
constexpr int kPartialBytes = BM * BN * 4;  // one slot: the fp32 accumulators of one tile
constexpr int kTileOverhead = 4;      // fixed cost of a tile (epilogue, switch) in K = 128 steps, measured
constexpr int kSlotsPerWg = 2;        // a piece that starts inside a tile, one that ends inside a tile

struct Sched {
  const fp8gmm_gemm_problem* probs;
  int nprob, total_tiles;
  int wgs;                     // workgroups per XCD
  int range_begin, range_end;  // tiles of this XCD
  int dp_rounds;               // workgroup j takes tile dp_tile(j, i) of rounds i < dp_rounds
  int sk_begin;                // first tile of the stream-K region (== range_end: none)
  int sk_wgs;                  // workgroups that take a piece of the region
  int64_t sk_c0, sk_cost;      // cost before the region, cost of the region (K = 128 steps)
  int64_t total_cost;          // cost of all tiles
  int fixup_weight;            // 1, or 3 when completing a shared tile includes the GELU epilogue
};

FP8GMM_HD int problem_end_tile(const Sched& s, int p) {
  return (p + 1 < s.nprob) ? s.probs[p + 1].tile_begin : s.total_tiles;
}
// last problem whose first tile is <= tile
FP8GMM_HD int problem_of_tile(const Sched& s, int tile) {
  int lo = 0, hi = s.nprob - 1;
  while (lo < hi) {
    const int mid = (lo + hi + 1) >> 1;
    if (s.probs[mid].tile_begin <= tile) lo = mid; else hi = mid - 1;
  }
  return lo;
}
// A tile of problem p costs ceil(k / 128) main-loop steps (1 for k = 0: its epilogue still has to run).
FP8GMM_HD int64_t tile_cost(const Sched& s, int p) {
  const int c = (s.probs[p].k + 127) / 128;
  return (int64_t)(c > 0 ? c : 1);
}
// Work before `tile` (0 <= tile <= total_tiles) when every tile counts its K steps plus `ov` steps of fixed
// overhead; cost_begin is the plan's prefix sum of the K steps alone.  ov = 0 is the unit in which tiles are
// cut along K; ov = kTileOverhead is the weight that balances the XCD ranges.
FP8GMM_HD int64_t work_before(const Sched& s, int tile, int ov) {
  const int p = problem_of_tile(s, tile);
  return (int64_t)s.probs[p].cost_begin + (int64_t)ov * s.probs[p].tile_begin +
         (int64_t)(tile - s.probs[p].tile_begin) * (tile_cost(s, p) + ov);
}
FP8GMM_HD int64_t cost_before(const Sched& s, int tile) { return work_before(s, tile, 0); }
// the tile that holds work offset c: work_before(t) <= c < work_before(t + 1); total_tiles past the end
FP8GMM_HD int tile_holding_work(const Sched& s, int64_t c, int ov) {
  if (c >= s.total_cost + (int64_t)ov * s.total_tiles) return s.total_tiles;
  int lo = 0, hi = s.nprob - 1;  // last problem whose prefix is <= c: it is not empty, as c < the total
  while (lo < hi) {
    const int mid = (lo + hi + 1) >> 1;
    if ((int64_t)s.probs[mid].cost_begin + (int64_t)ov * s.probs[mid].tile_begin <= c) lo = mid; else hi = mid - 1;
  }
  const int64_t before = (int64_t)s.probs[lo].cost_begin + (int64_t)ov * s.probs[lo].tile_begin;
  return s.probs[lo].tile_begin + (int)((c - before) / (tile_cost(s, lo) + ov));
}
FP8GMM_HD int tile_holding_cost(const Sched& s, int64_t c) { return tile_holding_work(s, c, 0); }
// first tile whose preceding work is >= c (total_tiles if there is none)
FP8GMM_HD int first_tile_at_work(const Sched& s, int64_t c, int ov) {
  if (c <= 0) return 0;
  const int t = tile_holding_work(s, c, ov);
  if (t >= s.total_tiles) return s.total_tiles;
  return work_before(s, t, ov) == c ? t : t + 1;
}

// Workgroup i runs on XCD i % 8.  The tile list is cut into 8 contiguous ranges of equal WORK, one per XCD,
// so that workgroups that share an L2 work on neighbouring tiles; the workgroups of an XCD stride through the
// range, and share its remainder along K when that pays.  k differs per problem in the wgrad form, and a
// tile costs its K steps plus a fixed part (epilogue, tile switch) worth about kTileOverhead steps: balancing
// K steps alone left the XCDs that hold the short-K problems 17 % more work than the others.
FP8GMM_HD void sched_init(Sched& s, const fp8gmm_gemm_problem* probs, int nprob, int total_tiles,
                                           int xcd, int wgs_per_xcd, bool sk_enable, int fixup_weight = 1) {
  s.fixup_weight = fixup_weight;
  s.probs = probs;
  s.nprob = nprob;
  s.total_tiles = total_tiles;
  s.wgs = wgs_per_xcd;
  s.total_cost = 0;
  s.total_cost = cost_before(s, total_tiles);
  const int64_t total_work = s.total_cost + (int64_t)kTileOverhead * total_tiles;
  const int64_t lo = (total_work * xcd + kNumXcd - 1) / kNumXcd;
  const int64_t hi = (total_work * (xcd + 1) + kNumXcd - 1) / kNumXcd;
  s.range_begin = first_tile_at_work(s, lo, kTileOverhead);
  s.range_end = first_tile_at_work(s, hi, kTileOverhead);
  const int n_x = s.range_end - s.range_begin;
  const int W = wgs_per_xcd;
  s.dp_rounds = (n_x + W - 1) / W;  // plain striding: the last round may be partial
  s.sk_begin = s.range_end;
  s.sk_wgs = 0;
  s.sk_c0 = 0;
  s.sk_cost = 0;
  const int full = n_x / W, rem = n_x % W;
  if (!sk_enable || rem == 0 || full > kSkMaxRounds) return;
  // striding needs full + 1 rounds, sharing the remainder full + rem / W: take it when that saves a twelfth of the
  // launch by this count.  Measured, sharing returns about half of what the count promises (workgroups do not
  // finish their rounds in step, so part of a last round is hidden anyway), and it costs the second launch and a
  // round trip of the partial sums through memory: config 2's 4.25 rounds (15 % by the count) gain 6.5 %, launches
  // of 14 rounds with a short tail (4 - 6.5 % by the count; the reference's example layer) lost 1 % of their step.
  if ((int64_t)(W - rem) * 12 < (int64_t)W * (full + 1)) return;
  const int n_sk = rem;
  const int rounds = full;
  const int sk_begin = s.range_begin + rounds * W;
  const int64_t c0 = cost_before(s, sk_begin);
  const int64_t cost = cost_before(s, s.range_end) - c0;
  int64_t w = W;
  if (w > cost / kSkMinPairs) w = cost / kSkMinPairs;
  if (w > (int64_t)n_sk * kSkMaxPieces) w = (int64_t)n_sk * kSkMaxPieces;
  if (w <= n_sk) return;  // nothing to gain: at most one piece per tile
  // ... and more time than the launch that completes the shared tiles takes: the last round shrinks from one
  // tile's duration to that of one piece.  (128 experts x 768 outputs x 2048 inputs with the GELU epilogue: 24
  // shared tiles of 16 steps per XCD, the second launch took 75 us to save 10.)
  {
    const int64_t saved_x100 = (cost / n_sk - cost / w) * 100;
    const int64_t fixup_x100 = kSkFixupLaunch * 100 + (int64_t)n_sk * kSkFixupPerTile * s.fixup_weight;
    if (saved_x100 * 2 < fixup_x100 * 3) return;
  }
  s.dp_rounds = rounds;
  s.sk_begin = sk_begin;
  s.sk_wgs = (int)w;
  s.sk_c0 = c0;
  s.sk_cost = cost;
}

// piece boundaries of the stream-K region, relative to sk_c0
FP8GMM_HD int64_t sk_bound(const Sched& s, int j) { return s.sk_cost * j / s.sk_wgs; }

// Tile `local` of a problem with tiles_m x tiles_n tiles -> its row / column block.  The m index runs fastest
// inside groups of kRasterRows m-tiles: 32 consecutive tiles (one round of an XCD's workgroups) then form an
// 8 x 4 block that needs 12 operand slabs, whatever the shape of the problem (a 56 x 16 weight-gradient
// problem walked with m fastest over all 56 rows would need 33).
constexpr int kRasterRows = 8;
FP8GMM_HD void tile_origin(int m, int n, int local, int tile_m, int tile_n, int* m0, int* n0) {
  const int tiles_m = (m + tile_m - 1) / tile_m, tiles_n = (n + tile_n - 1) / tile_n;
  const int group = local / (kRasterRows * tiles_n);
  const int within = local - group * (kRasterRows * tiles_n);
  const int rows = tiles_m - group * kRasterRows < kRasterRows ? tiles_m - group * kRasterRows : kRasterRows;
  *m0 = (group * kRasterRows + within % rows) * tile_m;
  *n0 = (within / rows) * tile_n;
}
FP8GMM_HD void tile_origin(int m, int n, int local, int* m0, int* n0) { tile_origin(m, n, local, BM, BN, m0, n0); }

struct Item {
  int tile, prob, m0, n0;
  int k_begin, nk;  // K = 128 steps: first one, how many (0 for a problem without K)
  int slot;         // workspace slot of a partial piece, -1: the piece is the whole tile
};
struct Cursor {
  int dp_i;     // strided tiles already taken
  int sk_tile;  // next tile of this workgroup's stream-K piece, -1: none left
};

// The tile that workgroup j of the XCD takes in round i of the strided part.  The position inside the round
// rotates from round to round: how fast a workgroup's steps run depends on where its tile sits in the round's
// 8 x 4 block (which operand slabs it shares with its neighbours, which memory channels those fall into - up to
// 6 % between columns of a weight-gradient problem), and a workgroup that kept one position for the whole launch
// would finish that much earlier or later than the others.
constexpr int kRoundRotation = 5;  // coprime to every workgroup count in use (multiples of 8 per XCD: 32, 38, ...)
FP8GMM_HD int dp_tile(const Sched& s, int j, int i) {
  return s.range_begin + s.wgs * i + (j + kRoundRotation * i) % s.wgs;
}

FP8GMM_HD void cursor_init(const Sched& s, int j, Cursor& c) {
  c.dp_i = 0;
  c.sk_tile = -1;
  if (j < s.sk_wgs && sk_bound(s, j) < sk_bound(s, j + 1)) c.sk_tile = tile_holding_cost(s, s.sk_c0 + sk_bound(s, j));
}
FP8GMM_HD bool cursor_valid(const Sched& s, int j, const Cursor& c) {
  return (c.dp_i < s.dp_rounds && dp_tile(s, j, c.dp_i) < s.sk_begin) || c.sk_tile >= 0;
}
// `prob_hint`: a problem at or before the one that holds the cursor's tile (a workgroup's tiles come in
// increasing order, so the previous item's problem will do); negative: search the whole table.
FP8GMM_HD Item cursor_item(const Sched& s, int xcd, int j, const Cursor& c, int prob_hint = -1) {
  const bool dp = c.dp_i < s.dp_rounds && dp_tile(s, j, c.dp_i) < s.sk_begin;
  Item it;
  it.tile = dp ? dp_tile(s, j, c.dp_i) : c.sk_tile;
  if (prob_hint < 0) {
    it.prob = problem_of_tile(s, it.tile);
  } else {
    it.prob = prob_hint;
    while (it.prob + 1 < s.nprob && s.probs[it.prob + 1].tile_begin <= it.tile) ++it.prob;
  }
  tile_origin(s.probs[it.prob].m, s.probs[it.prob].n, it.tile - s.probs[it.prob].tile_begin, &it.m0, &it.n0);
  const int real_nk = (s.probs[it.prob].k + 127) / 128;  // a K tail is zero-filled
  it.k_begin = 0;
  it.nk = real_nk;
  it.slot = -1;
  if (!dp) {
    const int64_t c_t = cost_before(s, it.tile) - s.sk_c0, k_t = tile_cost(s, it.prob);
    const int64_t lo = sk_bound(s, j), hi = sk_bound(s, j + 1);
    const int64_t p_lo = (lo > c_t ? lo : c_t) - c_t;
    const int64_t p_hi = (hi < c_t + k_t ? hi : c_t + k_t) - c_t;
    if (p_hi - p_lo < k_t) {  // only tiles with real K work are ever cut (k_t > 1)
      it.k_begin = (int)p_lo;
      it.nk = (int)(p_hi - p_lo);
      it.slot = kSlotsPerWg * (xcd * s.wgs + j) + (p_lo == 0 ? 1 : 0);
    }
  }
  return it;
}
FP8GMM_HD void cursor_advance(const Sched& s, int j, Cursor& c) {
  if (c.dp_i < s.dp_rounds && dp_tile(s, j, c.dp_i) < s.sk_begin) {
    ++c.dp_i;
    return;
  }
  if (c.sk_tile < 0) return;
  const int p = problem_of_tile(s, c.sk_tile);
  const int64_t t_end_cost = cost_before(s, c.sk_tile) - s.sk_c0 + tile_cost(s, p);
  c.sk_tile = (t_end_cost < sk_bound(s, j + 1) && c.sk_tile + 1 < s.range_end) ? c.sk_tile + 1 : -1;
}



// The tile that the workgroup of piece boundary j (1 <= j < sk_wgs) completes in the fix-up pass, or -1:
// the FIRST boundary strictly inside a tile owns it.  `first_piece_wg` is the workgroup that holds the piece
// from the tile's first K step (slot kSlotsPerWg * wg + 1); the following pieces come from workgroups
// j, j + 1, ... (slot kSlotsPerWg * wg) while their boundary lies inside the tile.
FP8GMM_HD int fixup_tile(const Sched& s, int j, int* n_following) {
  *n_following = 0;
  if (j < 1 || j >= s.sk_wgs) return -1;
  const int64_t b = sk_bound(s, j);
  const int tile = tile_holding_cost(s, s.sk_c0 + b);
  if (tile >= s.range_end) return -1;
  const int64_t c_t = cost_before(s, tile) - s.sk_c0, k_t = tile_cost(s, problem_of_tile(s, tile));
  if (b == c_t) return -1;                    // the boundary coincides with a tile boundary
  if (sk_bound(s, j - 1) > c_t) return -1;    // an earlier boundary inside the same tile owns it
  int n = 0;
  for (int q = j; q < s.sk_wgs && sk_bound(s, q) < c_t + k_t; ++q) ++n;
  *n_following = n;
  return tile;
}

}  // namespace fp8gmm
