// Host-side planning for the single-group tile kernel (gemm_tn_ring.h): which tile, whether to
// split K uniformly, whether to cut the tiles of the last round.  Pure functions of the problem
// size, so that the workspace query and the launch agree.  Counterpart in the reference: the
// compile-time tile choice of DefaultConfig (kernels/gemm_kernels/sm90a/gemm.cuh:420-451) and the
// Scheduler's round structure (gemm.cuh:168-212).
#include "gemm_launch.h"

#include <cstdlib>
#include "ring_common.h"

namespace mi355 {

namespace {

constexpr int64_t kCuSlots = 256;  // one work item per CU of an MI355X; heuristics only, so no device query

int64_t k_steps_of(int64_t K, int elem_bytes) { return (K * elem_bytes + kRowBytes - 1) / kRowBytes; }

int64_t tiles_of(int64_t M, int64_t N, int tile) {
  const int64_t r = ring_tile_rows(tile), c = ring_tile_cols(tile);
  return ((M + r - 1) / r) * ((N + c - 1) / c);
}

// Uniform K split of `tiles` tiles: only when the tiles alone leave more than half of the CUs idle
// (the partial tiles cost S*M*N*8 bytes of extra traffic and a second launch) and every item keeps
// at least 16 k-steps.  One item per CU also for the 128x128 tiles
// (two of which fit a CU): filling both places with K splits measured 7-13 % slower on
// M = 128..256 against N = 14336.
int uniform_splits(int64_t tiles, int64_t steps) {
  int best = 1;
  for (int s = 2; s <= 16; ++s) {
    if (tiles * s > kCuSlots) break;
    if (steps / s < 16) continue;   // the k-steps need not divide: the items' lengths differ by at most one
    best = s;
  }
  return best;
}

// Tail split of `tiles` 256x256 tiles with `steps` k-steps each.  When the tiles fill one or two
// rounds of workgroups plus a last round that is at most half full, the tiles of that round are cut
// along K so that they occupy (almost) all workgroup slots and the round takes 1/S of a tile's
// time; every item keeps at least 16 k-steps.
// Measured at bf16: +5..+10 % for one or two full rounds (4096x6144x4096, 6144^3); with three
// full rounds (4096x14336x4096) the partly filled round, which runs at a higher clock, costs no
// more than the partial tiles' extra traffic and second launch (-1 %), and on 128x128 tiles the
// split loses (-8 % at 4352^2x4096), so only 256x256 tiles are cut.
void tail_plan(int64_t tiles, int64_t steps, int* tail_tiles, int* tail_splits) {
  *tail_tiles = 0;
  *tail_splits = 1;
  const int64_t rest = tiles % kCuSlots;
  if (tiles < kCuSlots || tiles > 3 * kCuSlots || rest == 0) return;
  int best = 1;
  for (int s = 2; s <= 16; ++s) {
    if (rest * s > kCuSlots) break;
    if (steps / s < 16) continue;   // the k-steps need not divide: the items' lengths differ by at most one
    best = s;
  }
  if (best == 1) return;
  *tail_tiles = (int)rest;
  *tail_splits = best;
}

// Estimated duration, in microseconds, of the problem on tile shape `tile`: linear models.  For the two
// large tiles, of which a CU holds one,
//   rounds x k-steps per item x (step + step_busy x occupancy + few_rows / tile rows + few_cols / tile columns)
//   + rounds x fixed + (reduce_mb x MB of partial sums + reduce, if K is split),
// rounds = ceil(items / 256), occupancy = items / (rounds x 256) -- a k-step of a busy chip takes longer
// (lower clock, shared memory system) -- and the two sharing terms for operands that few tiles share and
// that therefore come from HBM rather than from an XCD's L2 (few tile rows: the rows of B; few tile
// columns: the rows of A).  Of the 128 x 128 tiles a CU holds two, which hide each other's waits: a round
// of up to 512 items in which some CU has two costs `pair` per k-step (less `pair_slack` x the unused
// share of the 512 places), a last round of at most 256 items `single + single_busy x occupancy`.
// A k-step is 128 bytes of K per row for every input type and takes the same time for all of them.
// Coefficients: weighted least squares (relative error) over 200 bf16 problems drawn log-uniformly from
// M, N = 256...32768, K = 1024...16384 (1-800 GFLOP), each timed on all three tiles with the rows of B
// rotating through 600 MB so that they come from memory as weights do; residuals 7-9 % rms.  Picking the
// shortest estimate costs 0.4 % of the best tile's time on average over those problems (0.45 % and 0.5 %
// when fitted on one part of them and scored on the other), against 3.6 % for the model this replaces,
// whose constants came from squarer problems and cache-resident operands (its worst choices, 25-45 %
// slower than the best tile, were 256 x 256 tiles on problems with a few tile rows and thousands of
// columns, or the reverse).
struct TileCost {
  double step, step_busy, few_rows, few_cols, fixed, reduce_mb, reduce;
};
constexpr TileCost kCost256x128 = {0.380, 0.449, 0.163, 0.098, 8.02, 0.191, 2.07};
constexpr TileCost kCost256 = {0.580, 0.878, 0.220, 0.0, 15.72, 0.093, 2.64};
struct SmallTileCost {
  double pair, pair_slack, single, single_busy, few_rows, fixed, reduce_mb, reduce;
};
constexpr SmallTileCost kCost128 = {0.990, 0.498, 0.244, 0.352, 0.519, 5.53, 0.101, 1.71};
// Tiles of fewer than 16 k-steps, which none of the problems above had (and which are never split): the k-step part of
// the estimate scaled by k_part, and fixed costs per round and per launch in place of `fixed`.  Weighted least squares
// over 330 bf16 and e4m3 problems of 1...14 k-steps, M, N = 512...16384 (residuals 4-9 % rms).  On 140 further problems
// the shortest estimate costs 0.7 % of the best tile's time on average and more than 5 % on 4 of them, against 1.7 %
// and 16 for the coefficients above with the 10 % preference for larger tiles they needed there.
struct ShortTileCost {
  double k_part, per_round, per_launch;
};
constexpr ShortTileCost kShort256 = {0.889, 5.38, 3.46}, kShort256x128 = {0.775, 3.38, 2.39}, kShort128 = {0.762, 3.36, 0.61};
constexpr int64_t kShortSteps = 16;

// k_loop_factor scales the k-step part of the small tile's estimate (not the fixed and reduction parts): see ring_tile_edge.
double estimate_us(int tile, int64_t M, int64_t N, int64_t K, int elem_bytes, double k_loop_factor = 1.0) {
  const int64_t rows = ring_tile_rows(tile), cols = ring_tile_cols(tile);
  const int64_t tm = (M + rows - 1) / rows, tn = (N + cols - 1) / cols, tiles = tm * tn;
  const int64_t steps = k_steps_of(K, elem_bytes);
  const int s = uniform_splits(tiles, steps);
  const int64_t items = tiles * s;
  const double item_steps = (double)steps / s;
  double partial_mb = s > 1 ? (double)s * (double)M * (double)N * 4.0e-6 : 0.0;
  if (tile != 256 && tile != kRingTile256x128) {
    const SmallTileCost& c = kCost128;
    const int64_t full = items / (2 * kCuSlots), rest = items - full * 2 * kCuSlots;
    const bool pair = rest > kCuSlots, single = rest > 0 && !pair;
    const double pair_rounds = (double)(full + (pair ? 1 : 0));
    const double slack = pair ? 1.0 - (double)rest / (double)(2 * kCuSlots) : 0.0;
    const double rounds = pair_rounds + (single ? 1.0 : 0.0);
    const double step_sum = c.pair * pair_rounds - c.pair_slack * slack +
                            (single ? c.single + c.single_busy * (double)rest / (double)kCuSlots : 0.0) +
                            c.few_rows * rounds / (double)tm;
    if (steps < kShortSteps) return kShort128.k_part * item_steps * step_sum + kShort128.per_round * rounds + kShort128.per_launch;
    return k_loop_factor * item_steps * step_sum + c.fixed * rounds + (partial_mb > 0.0 ? c.reduce_mb * partial_mb + c.reduce : 0.0);
  }
  const TileCost& c = tile == 256 ? kCost256 : kCost256x128;
  double rounds = (double)((items + kCuSlots - 1) / kCuSlots);
  double occupancy = (double)items / (rounds * (double)kCuSlots);
  if (tile == 256 && s == 1) {
    int tail_tiles, tail_splits;
    tail_plan(tiles, steps, &tail_tiles, &tail_splits);
    if (tail_tiles) {   // the last round takes 1/S of a round
      rounds = (double)(tiles / kCuSlots) + 1.0 / tail_splits;
      occupancy = 1.0;
      partial_mb = (double)tail_tiles * tail_splits * 256.0 * 256.0 * 4.0e-6;
    }
  }
  const double step_us = c.step + c.step_busy * occupancy + c.few_rows / (double)tm + c.few_cols / (double)tn;
  if (steps < kShortSteps) {
    const ShortTileCost& k = tile == 256 ? kShort256 : kShort256x128;
    return k.k_part * rounds * item_steps * step_us + k.per_round * rounds + k.per_launch;
  }
  return rounds * (item_steps * step_us + c.fixed) + (partial_mb > 0.0 ? c.reduce_mb * partial_mb + c.reduce : 0.0);
}

}  // namespace

// One row (M <= 128) or one column (N <= 128) of 128 x 128 tiles on the nine-slot ring, K split as
// uniform_splits says: every workgroup streams its own rows of B from HBM, and the ring that keeps
// four k-steps in flight does that faster than the five-slot ring and than the streaming kernel's
// 64-column tiles, which fetch the rows of A twice as often.  Measured, bf16, M = 72...128, weights
// from HBM, against what the planner took before (the streaming kernel up to about 2 MB of A, else
// the tile kernel's estimate): N = 4096...28672 x K = 1024...14336, 75 problems, 66 faster by 5-26 %
// (128 x 8192 x 4096 26.9 -> 22.9 us, 96 x 11008 x 8192 64.9 -> 49.0 us, 80 x 14336 x 4096
// 37.5 -> 30.1 us), 4 slower by 2-8 % (N = 11008 with K = 14336 or 2048); with 16...31 tiles from
// 128 k-steps on 0-11 % faster; with fewer tiles or fewer k-steps than that the streaming kernel's
// finer split wins by 6-23 %, and so it does at M <= 64 (0-21 %).  e4m3, M = 72...128, N = 4096...28672,
// K = 4096...16384: 41 of 45 problems 5-24 % faster, the rest (32 k-steps, 32 tiles) within 3 %.
bool ring_one_row_deep(int64_t M, int64_t N, int64_t K, int elem_bytes) {
  if (M > 128 && N > 128) return false;
  const int64_t tiles = tiles_of(M, N, 128), steps = k_steps_of(K, elem_bytes);
  if (tiles > kCuSlots || tiles * uniform_splits(tiles, steps) < 96) return false;   // under 96 items: no gain, or 1-3 % slower
  // One column of tiles (N <= 128 under many rows: router and adapter projections) is the same picture
  // with the operands' roles exchanged.  bf16, N = 64 and 128, K = 2048...7168 against the estimate's
  // choice (mostly 256 x 128 tiles): M = 8192...32768 19 of 24 problems 3-41 % faster (32768 x 128 x 4096
  // 76 -> 45 us), the rest within 4 %; M = 4096 (32 tiles) from 5 % faster to 10 % slower, so from 64 tiles on;
  // e4m3 on seven such problems 1-31 % faster.
  if (M > 128) return tiles >= 64 && steps >= 16;   // (e4m3 24576 x 128 x 1024, 8 k-steps: 11 % slower)
  return tiles >= 32 || (tiles >= 16 && steps >= 128);
}

// Tile the single-group kernel should use (256, 128, kRingTile256x128 or kRingTile128Deep): the rules for
// one row or column of tiles and for two rows first, then the shortest estimate, a larger tile being
// preferred within 2 % (it moves fewer bytes).
int ring_tile_edge(int64_t M, int64_t N, int64_t K, int elem_bytes, bool block_scaled) {
  // For measurements: MI355_RING_TILE = 256, 128, 384 (256 x 128), 129 (128 x 128 on nine slots, staggered
  // start) or 130 (nine slots, plain) overrides the choice below, so that a profiler can be pointed at a
  // form the planner would not take (the nine-slot forms exist without block scales only).
  if (const char* force = std::getenv("MI355_RING_TILE")) {
    const int t = std::atoi(force);
    if (t == 256 || t == 128 || t == kRingTile256x128 || (!block_scaled && (t == kRingTile128Deep || t == kRingTile128DeepPlain)))
      return t;
  }
  // One or two rows of 128 x 128 tiles that nearly fill the CUs in one round, and a short K: every
  // workgroup streams its own rows of B from HBM, which the nine-slot ring keeps further ahead of the
  // MFMAs than the five-slot one can, and unsplit tiles spare the partial planes of a K split.
  // Instantiated and measured for the 16-bit input types: against the rest of this planner on bf16
  // (256, 11008...14336, 2048...4096) and
  // (192, 14336, 4096): 3-10 % less time; with longer rows of K (from 5120 elements), more tiles than
  // CUs or fewer than two thirds of them it loses by 1-60 %.
  if (!block_scaled && ring_one_row_deep(M, N, K, elem_bytes)) return kRingTile128Deep;   // scales: five-slot ring only
  const int64_t small_tiles = tiles_of(M, N, 128);
  if (elem_bytes == 2 && M <= 256 && small_tiles >= 170 && small_tiles <= kCuSlots && k_steps_of(K, elem_bytes) >= 16 &&
      k_steps_of(K, elem_bytes) <= 64)
    return kRingTile128Deep;
  const double e256 = estimate_us(256, M, N, K, elem_bytes);
  // 128 x 128 tiles that make a single round (at most one per CU) have nobody to hide their waits: there the
  // nine-slot ring, without the staggered start, takes a sixth less time per k-step than the five-slot one (bf16, eleven
  // problems of 2 x 33...22 x 8 tile rows and columns and 29...245 k-steps, weights from memory: 4-27 % less, mean 14 %;
  // with more tiles than CUs, where a CU holds two five-slot workgroups, it takes 3-8 % more).
  // Items of fewer than 16 k-steps stay on five slots: the longer prologue of the deeper ring shows (fp16 512^3, 16 tiles
  // of 8 k-steps: 6.5 us on five slots, 7.2 on nine).
  const int64_t tiles128 = tiles_of(M, N, 128), steps128 = k_steps_of(K, elem_bytes);
  const int splits128 = uniform_splits(tiles128, steps128);
  // (When both operands still sit in the L2 from the previous call -- back-to-back launches of bf16 1024^3,
  // 768^2 x 2048, 2048^2 x 1024, 4-8 MB of operands -- there is nothing to wait for and five slots are 5-8 % faster;
  // with the rows of B coming from memory, as weights do, nine slots win at those sizes too, by 6-16 %.)
  const bool single_round = !block_scaled && tiles128 * splits128 <= kCuSlots && steps128 / splits128 >= 16;
  // The factor on the k-step part of the estimate: 0.82 (on 60 further problems timed on all four forms 0.78...0.80 leave a
  // regret of 0.2 %, 0.82 one of 0.4 %, 0.86 0.8 %, 0.76 0.55 %, no candidate 1.5 %; 0.82 keeps bf16 256 x 6144 x 4096 on
  // 256 x 128 tiles, 28.1 us against 29.5).
  const double e128 = estimate_us(128, M, N, K, elem_bytes, single_round ? 0.82 : 1.0);
  const double e2 = estimate_us(kRingTile256x128, M, N, K, elem_bytes);
  const double margin = 1.02;
  const double best = margin * (e256 < e128 ? (e256 < e2 ? e256 : e2) : (e128 < e2 ? e128 : e2));
  return e256 <= best ? 256 : e2 <= best ? kRingTile256x128 : single_round ? kRingTile128DeepPlain : 128;
}

// Two launches instead of one.  A problem whose 256 x 256 tiles do not fill their last round of workgroups leaves CUs
// idle in it (or pays partial sums for a tail split).  Cut along N (or M) so that the first piece is a whole number of
// rounds, and the rest is a problem of its own, for which the planner may take another tile.  Decided on the estimates
// above: the candidates are the (up to four) largest first pieces that are whole rounds; the best of them is taken
// when it promises at least 2 % over the single launch, the second launch counted with 3 us.  Measured against the
// single launch on 61 problems the estimates would cut (bf16 and e4m3, 1...9 rounds): up to 3.3 rounds all 22 gain,
// 4-21 % (bf16 4096 x 6144 x 1728 72 -> 67 us, 12544 x 4096 x 7104 547 -> 482 us, e4m3 4096 x 6144 x 4096 90 -> 76 us);
// at 3.5 rounds 2-4 % up to 64 k-steps (bf16 4096 x 14336 x 4096 329 -> 321 us) and from 3 % more to 4 % less beyond;
// from 4 rounds on from 5 % less to 5 % more, 1 % on average.  So: at most 3.4 rounds, or 3.6 with at most 64 k-steps.
// Returns the first piece's extent along N (or along M, *along_m set), 0 for a single launch.
int64_t ring_first_piece(int64_t M, int64_t N, int64_t K, int elem_bytes, bool* along_m) {
  *along_m = false;
  if (std::getenv("MI355_ONE_PIECE")) return 0;   // for measurements: never cut
  const int64_t tm = (M + 255) / 256, tn = (N + 255) / 256;
  const int64_t steps = k_steps_of(K, elem_bytes);
  if (tm * tn <= kCuSlots || (tm * tn) % kCuSlots == 0 || steps < kShortSteps) return 0;
  if (10 * tm * tn > 36 * kCuSlots || (10 * tm * tn > 34 * kCuSlots && steps > 64)) return 0;
  const auto best_of = [&](int64_t m, int64_t n) {
    const double a = estimate_us(256, m, n, K, elem_bytes), b = estimate_us(kRingTile256x128, m, n, K, elem_bytes),
                 c = estimate_us(128, m, n, K, elem_bytes);
    return a < b ? (a < c ? a : c) : (b < c ? b : c);
  };
  const double whole = best_of(M, N), second_launch_us = 3.0;
  double best = 0.98 * whole;
  int64_t extent = 0;
  for (int axis = 0; axis < 2; ++axis) {
    const int64_t across = axis == 0 ? tm : tn, along = axis == 0 ? tn : tm;   // axis 0: cut N, axis 1: cut M
    int64_t g = across, h = kCuSlots;                                         // gcd(across, 256)
    while (h) { const int64_t r = g % h; g = h; h = r; }
    const int64_t step = kCuSlots / g;                                        // tile columns (rows) per whole number of rounds
    int64_t c = (along - 1) / step * step;
    for (int tries = 0; tries < 4 && c >= step; ++tries, c -= step) {
      const double e = axis == 0 ? best_of(M, c * 256) + best_of(M, N - c * 256) : best_of(c * 256, N) + best_of(M - c * 256, N);
      if (e + second_launch_us < best) {
        best = e + second_launch_us;
        extent = c * 256;
        *along_m = axis == 1;
      }
    }
  }
  return extent;
}

// K splits for the single-group kernel on the tile ring_tile_edge picks.
int ring_splits(int64_t M, int64_t N, int64_t K, int elem_bytes, bool block_scaled) {
  return uniform_splits(tiles_of(M, N, ring_tile_edge(M, N, K, elem_bytes, block_scaled)), k_steps_of(K, elem_bytes));
}

// The tail split (tail_plan) of this problem, if it runs on 256x256 tiles without a uniform K
// split: returns the workspace bytes of its partial tiles.
size_t ring_tail(int64_t M, int64_t N, int64_t K, int elem_bytes, int* tail_tiles, int* tail_splits, bool block_scaled) {
  *tail_tiles = 0;
  *tail_splits = 1;
  if (M <= 0 || N <= 0 || K <= 0 || ring_tile_edge(M, N, K, elem_bytes, block_scaled) != 256) return 0;
  tail_plan(tiles_of(M, N, 256), k_steps_of(K, elem_bytes), tail_tiles, tail_splits);
  return (size_t)*tail_tiles * (size_t)*tail_splits * 256 * 256 * sizeof(float);
}

int launch_tile_ring(const GemmArgs& g, int in_dtype, int out_dtype, int tile, hipStream_t stream) {
  switch (in_dtype) {
    case 0: return launch_tile_ring_bf16(g, out_dtype, tile, stream);
    case 1: return launch_tile_ring_f16(g, out_dtype, tile, stream);
    case 2: return launch_tile_ring_e4m3(g, out_dtype, tile, stream);
  }
  return -1;
}

}  // namespace mi355
