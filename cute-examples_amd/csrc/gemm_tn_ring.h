// "basic" variant: 256x256 (or 256x128, or 128x128) output tile, ONE wave group of 4 waves (one per
// SIMD), each wave owning a quarter of it (128x128 held in 256 fp32 accumulator registers per lane
// for the 256x256 tile, which the description below uses).  ring_plan.hip picks the tile.
//
// Data path per k-step (128 bytes of K per row: 64 bf16/fp16 or 128 fp8 elements):
//
//   global --buffer_load ... lds (16 B per lane, no VGPR round trip)--> LDS ring
//   LDS --ds_read_b128--> operand fragments in VGPRs --v_mfma--> accumulators in AGPRs
//
// LDS ring.  All 160 KiB of LDS form a ring of five 32 KiB slots; a slot holds the 256 rows x
// 128 B of ONE operand for one k-step.  Operand-steps are queued in the order A0 B0 A1 B1 A2 ...
// so k-step t reads slots (2t)%5 and (2t+1)%5 while three more are in flight.  When the reads of
// k-step t are done, its two slots are refilled with B(t+2) and A(t+3): every k-step therefore
// waits only for ONE operand issued one k-step earlier (the other one has been in flight for two),
// which keeps the per-k-step load latency under the MFMA time of a k-step.  Two full 64 KiB
// stages would leave both operands of a k-step only one k-step of flight time.
//
// Schedule inside a wave (two slices per k-step, fragments double-buffered in registers):
//   slice 0: MFMAs on fragment buffer 0 | ds_reads of slice 1 -> buffer 1
//            then lgkmcnt(0), vmcnt(8), s_barrier   (slots of k-step t free, k-step t+1 landed)
//   slice 1: MFMAs on buffer 1 | ds_reads of slice 0 of k-step t+1 -> buffer 0
//   from the barrier to the end of the k-step: the 16 direct-to-LDS loads of B(t+2), A(t+3),
//            spread evenly between the MFMAs
// One workgroup barrier per k-step and one scalar branch per turn of the ring: a workgroup has one
// wave per SIMD, so every branch is a bubble in its MFMA stream.  The k loop is unrolled over the five
// positions of the ring, which makes every LDS offset an immediate; copies past the end of K re-read the last
// k-step into a slot nobody reads instead of being branched around.  The MFMAs are inline
// assembly with the accumulator tied in place; fragment loads and everything else are compiled
// code pinned between them with scheduling barriers.
//
// Tiles.  The grid is persistent: one workgroup per CU walks (tile, K-split) items blockIdx.x,
// +gridDim.x, ...  After the last k-step of a tile the workgroup first queues the five opening
// copies of its next tile and only then converts and stores the finished accumulators
// (tile_store.h), so the store phase of one tile hides the load latency of the next.
//
// MFMA shape: bf16/fp16 use v_mfma_f32_16x16x32 (8x8 blocks per wave); on random data it sustains
// a higher clock under the board power limit than 32x32x16.  fp8 uses v_mfma_f32_16x16x128_f8f6f4
// (8x8 blocks) for the same reason; one such MFMA spans the whole k-step, so the two slices of a
// k-step are the two halves of the wave's rows of A instead of two halves of K, and the blocks of
// B are reloaded in place, each right after its last use (see the fragment arrays below).
//
// Counterpart in the reference: the cooperative kernel, kernels/gemm_kernels/sm90a/gemm.cuh:246-418
// (TMA producer warpgroup, mbarrier full/empty ring of 3 stages, two consumer warpgroups); here
// every wave is loader and math at once because direct-to-LDS loads need no registers.
//
// This header holds the kernel and its launch templates; gemm_tn_ring_{bf16,f16,e4m3,mx}.hip
// instantiate them per input type, one translation unit each so that they compile in parallel.
#pragma once
#include "gemm_launch.h"
#include "ring_common.h"
#include "tile_map.h"
#include "tile_store.h"

#include <type_traits>
#include <utility>

namespace mi355 {
namespace {

// Waves of a workgroup form a 2 x kWavesN grid over the tile.
constexpr int threads_of(int waves_n) { return 128 * waves_n; }

// MFMA position of copy c when n copies are spread evenly over `span` positions from `first`,
// and the first copy whose position is not before p.
constexpr int copy_position(int c, int first, int span, int n) { return first + c * span / n; }
constexpr int first_copy_at(int p, int first, int span, int n) {
  int c = 0;
  while (c < n && copy_position(c, first, span, n) < p) ++c;
  return c;
}

// Layout of block scales as the kernel reads them ("shuffled", written by mx_scales.hip): one
// 512-byte unit per (group of 128 rows, k-step); lane l of the wave that owns those rows reads the
// 8 bytes at 8*l: byte i is the scale of row 16*i + l%16 of the group for K block 4*kstep + l/16.
// Units are ordered [row group][k-step], and the arrays are padded to whole 256-row tiles.
constexpr uint32_t kMxUnitBytes = 512;

// kRaggedK: K*elem_bytes is not a multiple of the 128-byte k-step.  Kept out of the common
// instantiation because selecting the per-lane offset inside the loop puts a dependent VALU
// chain in front of every copy and costs ~8 % at 8192^3.
// kTileT: rows of A and of B per workgroup, 256 or 128.  The 128 variant (64x64 per wave, 80 KiB
// ring, two workgroups per CU) is for problems with too few 256x256 tiles to occupy the CUs; it
// moves twice the bytes per flop, so it is copy-bound at about two thirds of the MFMA rate.
// kTileNT: rows of B per workgroup when they differ from kTileT: the 256x128 tile (128x64 per wave)
// has three times as many tiles as 256x256 on shapes that leave most CUs without a 256x256 tile,
// and moves 1.5 times the bytes per flop instead of the 128x128 tile's two times.
// kAhead (d): k-steps of copies kept in flight; the ring has 2d + 1 slots.  The ring described
// above is d = 2.  d = 4 (nine 16 KiB slots of the 128-row tile, one workgroup per CU) is for
// problems with one or two tile rows, whose rows of B are read by one or two workgroups only and so
// come from HBM, not from the L2: with d = 2 an operand-step has about one k-step of flight time
// before the barrier that waits for it (a third of a microsecond on the small tile), with d = 4
// about three.
template <class T, class OutT, bool kRaggedK, int kTileT, int kWavesN = 2, int kTileNT = kTileT, int kAhead = 2,
          bool kRotateT = (kAhead > 2)>
__global__ __launch_bounds__(threads_of(kWavesN), (kTileT == 256 || kAhead > 2) ? 1 : 2) void gemm_tn_tile_ring(GemmArgs g) {
  constexpr int kSlots = 2 * kAhead + 1;          // shadows the five of ring_common.h
  constexpr int kTile = kTileT;                   // rows of A per workgroup
  constexpr int kTileN = kTileNT;                 // rows of B per workgroup
  static_assert(kTileN <= kTile, "a slot is sized for the rows of A");
  constexpr int kSlotBytes = kTile * kRowBytes;   // one operand, one k-step (B may use less of it)
  constexpr int kWaveTileM = kTile / 2;           // rows (of A) per wave
  constexpr int kWaveTileN = kTileN / kWavesN;    // columns (rows of B) per wave
  constexpr int kWaves = 2 * kWavesN;
  // One direct-to-LDS instruction moves 16 B per lane: 8 rows of 128 B.  (4 B per lane, 2 rows,
  // costs an MFMA stream nothing per instruction in isolation, but four times as many copies
  // through the texture-address unit made the kernel 11 % slower.)
  constexpr int kCopyRows = 8;
  constexpr int kCopyBytes = kCopyRows * kRowBytes;
  constexpr int kCph = kTile / kWaves / kCopyRows;    // copies of A per k-step per wave
  constexpr int kCphB = kTileN / kWaves / kCopyRows;  // copies of B
  constexpr int kPar = 2;                           // copies j and j+kPar share their per-lane swizzle
  __shared__ __attribute__((aligned(1024))) uint8_t ring[kSlots * kSlotBytes];
  typedef typename RingGeo<T>::type G;
  typedef typename G::Frag Frag;
  typedef typename G::Acc Acc;
  constexpr int kBlk = G::kBlk;
  constexpr int kNbM = kWaveTileM / kBlk, kNbN = kWaveTileN / kBlk;  // blocks per wave
  constexpr int kSliceChunks = G::kGroups * G::kCpl;    // chunks of a row consumed by one MFMA
  constexpr int kAccLen = kBlk * kBlk / 64;
  // A k-step is worked off in two slices: two halves of its 128 bytes of K, or, when one MFMA
  // spans all of them, the two halves of the wave's rows of A.
  constexpr bool kRowSliced = G::kRowSliced;
  constexpr bool kMx = G::kMx;
  static_assert(kSlots * kSlotBytes <= 160 * 1024, "the ring must fit the LDS of a CU");
  static_assert(!kMx || kAhead == 2, "block scales: the scale registers are sized and timed for the five-slot ring");
  static_assert(!kMx || (kRowSliced && !kRaggedK && (kWaveTileM == 128 || kWaveTileM == 64) &&
                         (kWaveTileN == 128 || kWaveTileN == 64)),
                "block scales: whole k-steps, a whole or half 128-row scale group per wave and operand");
  constexpr int kHalfM = kNbM / 2;                       // row blocks of A per slice when kRowSliced
  constexpr int kMfmaPerSlice = kRowSliced ? kHalfM * kNbN : kNbM * kNbN;
  constexpr int kReadsPerSlice = kNbM + kNbN;            // fragment loads per slice (K-sliced case)
  static_assert(8 / kSliceChunks == (kRowSliced ? 1 : 2), "two slices per k-step");

  const uint32_t tid = threadIdx.x;
  const uint32_t lane = tid & 63u;
  const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const uint32_t wm = wave / kWavesN, wn = wave % kWavesN;

  const uint32_t lda_b = (uint32_t)(g.lda * T::kBytes), ldb_b = (uint32_t)(g.ldb * T::kBytes);
  const uint32_t k_bytes = (uint32_t)(g.K * T::kBytes);
  // K need not be a whole number of k-steps: in the last one, chunks past the end of the row are
  // fetched from an out-of-range offset (the hardware returns zeros), see tail_or_oob below.
  const uint32_t k_steps = __builtin_amdgcn_readfirstlane((k_bytes + kRowBytes - 1) / kRowBytes);
  const uint32_t tail_bytes = __builtin_amdgcn_readfirstlane(k_bytes % kRowBytes);
  const uint32_t tiles_m = (uint32_t)g.tiles_m, tiles_n = (uint32_t)g.tiles_n;
  const uint32_t total_tiles = tiles_m * tiles_n;  // the launcher keeps items below 2^31
  // Work items are (tile, split) pairs, split-major, so that workgroups running together read the
  // same range of K.  With a uniform K split every tile has g.splits items; with a tail split only
  // the last g.tail_tiles tiles are cut (g.tail_splits ways) and come after all whole tiles.  Either
  // way a tile is cut into ranges of k-steps that differ by at most one when the k-steps do not divide.
  // steps is the number of k-steps of the current item.
  const uint32_t tail_tiles = (uint32_t)g.tail_tiles, tail_splits = (uint32_t)g.tail_splits;
  const uint32_t whole_tiles = total_tiles - tail_tiles;  // tail_tiles == 0 unless g.splits == 1
  const uint32_t total_items = tail_tiles ? whole_tiles + tail_tiles * tail_splits : total_tiles * (uint32_t)g.splits;
  uint32_t steps = 0;
  // k-steps [sp*k/S, (sp+1)*k/S) of split sp of S: every step once, lengths within one of each other
  auto cut = [&](uint32_t sp, uint32_t of, uint32_t* first_step) __attribute__((always_inline)) {
    const uint32_t begin = __builtin_amdgcn_readfirstlane(sp * k_steps / of);
    const uint32_t end = __builtin_amdgcn_readfirstlane((sp + 1) * k_steps / of);
    *first_step = begin;
    steps = end - begin;
  };
  // item -> (tile number in tile-map order, split, first k-step, whether it writes fp32 partials);
  // sets steps.
  auto decode_item = [&](uint32_t it, uint32_t* tile, uint32_t* split_of, uint32_t* first_step)
      __attribute__((always_inline)) -> bool {
    if (tail_tiles) {
      if (it < whole_tiles) {
        *tile = it;
        *split_of = 0;
        *first_step = 0;
        steps = k_steps;
        return false;
      }
      const uint32_t j = it - whole_tiles;
      const uint32_t sp = j / tail_tiles;
      *tile = whole_tiles + j % tail_tiles;
      *split_of = sp;
      cut(sp, tail_splits, first_step);
      return true;
    }
    *tile = it % total_tiles;
    *split_of = it / total_tiles;
    cut(*split_of, (uint32_t)g.splits, first_step);
    return g.splits > 1;
  };

  // Descriptors of the A and B row panels of a tile; rows past the matrix edge are out of range.
  auto panel_a = [&](int64_t m0) __attribute__((always_inline)) {
    const int64_t rows = g.M - m0 < kTile ? g.M - m0 : kTile;
    return make_raw_buffer((const uint8_t*)g.A + m0 * (int64_t)lda_b, (uint32_t)((rows - 1) * lda_b + k_bytes));
  };
  auto panel_b = [&](int64_t n0) __attribute__((always_inline)) {
    const int64_t rows = g.N - n0 < kTileN ? g.N - n0 : kTileN;
    return make_raw_buffer((const uint8_t*)g.B + n0 * (int64_t)ldb_b, (uint32_t)((rows - 1) * ldb_b + k_bytes));
  };

  // Copy geometry.  Wave w fills a quarter of an operand's rows in a slot, kCopyRows rows per
  // instruction, the LDS side linear in the lane number.  Lane l therefore fills bytes
  // sub..sub+n of LDS chunk lchunk of row lrow of the copy's rows, and fetches them from global
  // chunk lchunk ^ swizzle(row).  swizzle(row) repeats every kPar copies, so kPar per-lane
  // offsets per operand suffice; copy j adds j*kCopyRows rows to them.
  const uint32_t lrow = lane >> 3, lchunk = lane & 7u;
  constexpr uint32_t kOutOfRange = 0x80000000u;  // row panels are smaller than 2 GiB (host check)
  uint32_t voff_a[kPar], voff_b[kPar], tail_a[kRaggedK ? kPar : 1], tail_b[kRaggedK ? kPar : 1];
#pragma unroll
  for (int par = 0; par < kPar; ++par) {
    const uint32_t chunk = lchunk ^ swizzle(par * kCopyRows + lrow);
    voff_a[par] = (wave * (kCph * kCopyRows) + lrow) * lda_b + chunk * 16;
    voff_b[par] = (wave * (kCphB * kCopyRows) + lrow) * ldb_b + chunk * 16;
    if constexpr (kRaggedK) {
      const bool tail_or_oob = tail_bytes != 0 && chunk * 16 >= tail_bytes;
      tail_a[par] = tail_or_oob ? kOutOfRange : voff_a[par];
      tail_b[par] = tail_or_oob ? kOutOfRange : voff_b[par];
    }
  }
  const uint32_t a_step = __builtin_amdgcn_readfirstlane(kCopyRows * lda_b);
  const uint32_t b_step = __builtin_amdgcn_readfirstlane(kCopyRows * ldb_b);
  const uint32_t ring0 = __builtin_amdgcn_readfirstlane(lds_address(ring));
  const uint32_t dma_wave_a = ring0 + wave * (kCph * kCopyBytes);  // this wave's share of a slot
  const uint32_t dma_wave_b = ring0 + wave * (kCphB * kCopyBytes);

  // Copy j of an operand's k-step into slot `slot`; soff is the k-step's byte offset inside a row.
  // The row part of the address stays in the vector offset, the only part the hardware
  // range-checks against the descriptor (rows past the edge of the matrix read zeros); the scalar
  // offset carries the k-step.  Past the end of an item's K range the copies re-read its last
  // k-step, into a slot nobody reads, so the loop body stays branch-free.
  const uint32_t soff_tail = (k_steps - 1) * kRowBytes;  // the k-step that may be ragged
  auto copy_rows = [&](__amdgpu_buffer_rsrc_t rsrc, auto jc, auto slotc, uint32_t soff, const uint32_t* voff,
                       const uint32_t* tail, uint32_t step, uint32_t dma_wave) __attribute__((always_inline)) {
    constexpr int j = decltype(jc)::value;
    constexpr uint32_t slot = decltype(slotc)::value;
    uint32_t v = voff[j % kPar];
    if constexpr (kRaggedK) v = soff == soff_tail ? tail[j % kPar] : v;
    dma_16B_to_lds_at<slot * kSlotBytes + j * kCopyBytes>(dma_wave, v + j * step, rsrc, soff);
  };
  // The same in two steps: the LDS base first, the copy later.
  auto prep_rows = [&](auto jc, auto slotc, uint32_t dma_wave) __attribute__((always_inline)) {
    dma_set_lds_base<decltype(slotc)::value * kSlotBytes + decltype(jc)::value * kCopyBytes>(dma_wave);
  };
  auto fire_rows = [&](__amdgpu_buffer_rsrc_t rsrc, auto jc, uint32_t soff, const uint32_t* voff, const uint32_t* tail,
                       uint32_t step) __attribute__((always_inline)) {
    constexpr int j = decltype(jc)::value;
    uint32_t v = voff[j % kPar];
    if constexpr (kRaggedK) v = soff == soff_tail ? tail[j % kPar] : v;
    dma_16B_to_lds_base_set(v + j * step, rsrc, soff);
  };
  auto copy_a = [&](__amdgpu_buffer_rsrc_t rsrc, auto jc, auto slotc, uint32_t soff) __attribute__((always_inline)) {
    copy_rows(rsrc, jc, slotc, soff, voff_a, tail_a, a_step, dma_wave_a);
  };
  auto copy_b = [&](__amdgpu_buffer_rsrc_t rsrc, auto jc, auto slotc, uint32_t soff) __attribute__((always_inline)) {
    copy_rows(rsrc, jc, slotc, soff, voff_b, tail_b, b_step, dma_wave_b);
  };
  // Byte offset of k-step kt of the item that starts at global k-step step0, clamped to its last.
  // kRotate (the deep ring on problems of one or two tile rows, whose workgroups all read
  // different rows of B): an item walks its k-steps from its own starting point `rot` and wraps
  // around, so that the workgroups running side by side do not all read the same 128-byte column
  // of rows that lie a power of two apart, i.e. the same few memory channels, at the same time.
  // Only the order of the fp32 additions of a tile depends on it, and that order is fixed per item.
  // Where tiles share rows of A and of B through an XCD's L2 (several tile rows and columns) the
  // deep ring runs without it: items at different k-steps would not find each other's panels there
  // (bf16 1184 x 2640 x 7168 on 210 tiles: 79.5 us with, 60.3 us without).
  constexpr bool kRotate = kRotateT;
  uint32_t rot = 0;
  auto soff_of = [&](uint32_t step0, uint32_t kt) __attribute__((always_inline)) -> uint32_t {
    uint32_t at = kt < steps ? kt : steps - 1;
    if constexpr (kRotate) {
      at += rot;
      at = at >= steps ? at - steps : at;
    }
    return __builtin_amdgcn_readfirstlane((step0 + at) * kRowBytes);
  };
  // Opening copies of a tile: A0 B0 A1 B1 A2 into slots 0..4.
  // Block scales (kMx only).  Set ph holds the scales of the k-step worked off in ring phase ph:
  // [0] rows 0..63 and [1] rows 64..127 of the wave's rows of A (sca) and of B (scb), one byte per
  // 16-row block.  A set is loaded two k-steps ahead by load_8B_async; see the waits at its users.
  // A wave with only 64 rows of an operand starts its 8 bytes at the half of the 128-row unit that
  // holds them and uses [0] only ([1] then holds bytes of the next lane, or zeros past the end).
  u32x2 sca[kSlots], scb[kSlots];
  const uint32_t mx_bytes_a = kMx ? (uint32_t)((g.M + 255) / 256) * 2u * k_steps * kMxUnitBytes : 0u;
  const uint32_t mx_bytes_b = kMx ? (uint32_t)((g.N + 255) / 256) * 2u * k_steps * kMxUnitBytes : 0u;
  const __amdgpu_buffer_rsrc_t rsrc_sa = make_raw_buffer(g.mx_a, mx_bytes_a);
  const __amdgpu_buffer_rsrc_t rsrc_sb = make_raw_buffer(g.mx_b, mx_bytes_b);
  uint32_t voff_sa = 0, voff_sb = 0;  // lane's bytes of the current item's first unit
  // Scale offset of k-step kt of the current item, clamped to its last like soff_of.
  auto mx_soff_of = [&](uint32_t kt) __attribute__((always_inline)) -> uint32_t {
    return __builtin_amdgcn_readfirstlane((kt < steps ? kt : steps - 1) * kMxUnitBytes);
  };
  auto mx_open_tile = [&](uint32_t tm, uint32_t tn, uint32_t step0) __attribute__((always_inline)) {
    const uint32_t row_a = tm * kTile + wm * kWaveTileM, row_b = tn * kTileN + wn * kWaveTileN;  // the wave's first rows
    voff_sa = ((row_a / 128) * k_steps + step0) * kMxUnitBytes + lane * 8 + (row_a % 128) / 64 * 4;
    voff_sb = ((row_b / 128) * k_steps + step0) * kMxUnitBytes + lane * 8 + (row_b % 128) / 64 * 4;
    load_8B_async(sca[0], rsrc_sa, voff_sa, mx_soff_of(0));
    load_8B_async(scb[0], rsrc_sb, voff_sb, mx_soff_of(0));
    load_8B_async(sca[1], rsrc_sa, voff_sa, mx_soff_of(1));
    load_8B_async(scb[1], rsrc_sb, voff_sb, mx_soff_of(1));
  };
  auto open_tile = [&](__amdgpu_buffer_rsrc_t ra, __amdgpu_buffer_rsrc_t rb, uint32_t step0) __attribute__((always_inline)) {
    // operand-steps A0 B0 A1 B1 ... A(kAhead) into slots 0 .. 2 kAhead
    static_for<kAhead + 1>([&](auto tc) __attribute__((always_inline)) {
      constexpr int t = decltype(tc)::value;
      const uint32_t st = soff_of(step0, t);
      static_for<kCph>([&](auto j) __attribute__((always_inline)) { copy_a(ra, j, std::integral_constant<uint32_t, 2 * t>{}, st); });
      if constexpr (t < kAhead)
        static_for<kCphB>([&](auto j) __attribute__((always_inline)) { copy_b(rb, j, std::integral_constant<uint32_t, 2 * t + 1>{}, st); });
    });
  };

  // Fragment geometry: lane l supplies row l%kBlk of a block; group l/kBlk picks the chunks.
  const uint32_t rblk = lane & (kBlk - 1), grp = lane / kBlk;
  const uint32_t swz = swizzle(rblk);  // block bases are multiples of 16 rows
  const uint32_t a_lane = (wm * kWaveTileM + rblk) * kRowBytes;
  const uint32_t b_lane = (wn * kWaveTileN + rblk) * kRowBytes;
  // Byte offset inside a row of the e-th chunk this lane reads in slice s.
  // When one MFMA spans the k-step, group g supplies chunks g and 4+g.  With block scales the order
  // of K inside the MFMA demands it; without them any order that is the same for both operands gives
  // the same dot product, and this one is free of LDS bank conflicts: a ds_read_b128 is served 16
  // lanes per cycle, lanes {0-3, 12-15, 20-23, 24-27} first (then {4-11, 16-19, 28-31}, then the same
  // of the upper 32), i.e. rows from two neighbouring groups together, and the chunks 2g, 2g+1 of
  // neighbouring groups differ in bit 1, which the row swizzle maps onto the same banks (counted:
  // one conflict cycle per access cycle), while g and g+1 differ in bit 0 and do not collide.
  auto chunk_off = [&](int s, int e) __attribute__((always_inline)) -> uint32_t {
    if constexpr (kRowSliced) return ((uint32_t)(grp + 4 * e) ^ swz) << 4;
    else return ((uint32_t)(s * kSliceChunks + grp * G::kCpl + e) ^ swz) << 4;
  };
  auto load_frag = [&](const uint8_t* slot_rows, int blk, int s) __attribute__((always_inline)) -> Frag {
    const uint8_t* p = slot_rows + blk * kBlk * kRowBytes;
    if constexpr (G::kCpl == 1) {
      return *(const i32x4*)(p + chunk_off(s, 0));
    } else {
      i32x4 lo = *(const i32x4*)(p + chunk_off(s, 0));
      i32x4 hi = *(const i32x4*)(p + chunk_off(s, 1));
      return (i32x8){lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
    }
  };

  Acc acc[kNbM][kNbN];
  // Fragments, [buffer][block].  K-sliced: slice s computes from buffer s while the other buffer is
  // loaded for the next slice.  Row-sliced: slice s uses rows fa[s][0..kHalfM) of A and all of
  // fb[0]; fa[s^1] is loaded meanwhile, and in slice 1 each block of B is reloaded for the next
  // k-step as soon as its last MFMA has been issued (the MFMAs run B-block by B-block there).
  Frag fa[2][kRowSliced ? kHalfM : kNbM], fb[kRowSliced ? 1 : 2][kNbN];

  // Load number q (0..kReadsPerSlice-1) of a slice: B blocks first (every MFMA row needs them all).
  auto read_q = [&](int buf, int q, const uint8_t* a_rows, const uint8_t* b_rows, int s)
      __attribute__((always_inline)) {
    if (q < kNbN) fb[buf][q] = load_frag(b_rows, q, s);
    else fa[buf][q - kNbN] = load_frag(a_rows, q - kNbN, s);
  };
  auto mfma_u = [&](int buf, int u) __attribute__((always_inline)) {
    const int i = u / kNbN, j = u % kNbN;
    // B supplies the MFMA "rows" so each lane ends up with consecutive n of one m.
    // In the 256-wide tile all 256 accumulator registers are live; the in-place form keeps the
    // compiler from rotating them through copies when it allocates the MFMA's result.
    if constexpr (kTile == 256) G::mfma_inplace(fb[buf][j], fa[buf][i], acc[i][j]);
    else acc[i][j] = G::mfma(fb[buf][j], fa[buf][i], acc[i][j]);
  };
  // Row-sliced order: B-block j outermost, the slice's kHalfM row blocks of A inside.
  auto mfma_rows = [&](auto phc, auto sc, auto uc) __attribute__((always_inline)) {
    constexpr int ph = decltype(phc)::value, s = decltype(sc)::value, u = decltype(uc)::value;
    constexpr int j = u / kHalfM, r = u % kHalfM, i = s * kHalfM + r;
    if constexpr (kMx) {
      G::template mfma_scaled_inplace<j % 4, i % 4>(fb[0][j], fa[s][r], acc[i][j], scb[ph][j / 4], sca[ph][i / 4]);
    } else {
      (void)ph;
      if constexpr (kTile == 256) G::mfma_inplace(fb[0][j], fa[s][r], acc[i][j]);
      else acc[i][j] = G::mfma(fb[0][j], fa[s][r], acc[i][j]);
    }
  };

  // Stores of the tile at (m0, n0): converted output, or fp32 partials for a split-K item.
  const float scale = output_scale(g);
  constexpr bool kAsmMfma = kTile == 256 || kMx;  // see mfma_u; the scaled MFMA is always inline assembly
  auto epilogue = [&](int64_t m0, int64_t n0) __attribute__((always_inline)) {
    store_output_tile<G, OutT, kNbM, kNbN, kAsmMfma>(acc, g, m0, n0, kTile, kTileN, wm * kWaveTileM, wn * kWaveTileN, lane, scale);
  };
  auto store_partial = [&](int64_t m0, int64_t n0, uint32_t split, uint32_t tile_no) __attribute__((always_inline)) {
    if (tail_tiles) {
      // a whole tile of the compact tail workspace (rows past M hold zeros: their operands read as 0)
      float* base = g.partial + ((int64_t)split * tail_tiles + (tile_no - whole_tiles)) * (kTile * kTileN);
      store_partial_tile<G, kNbM, kNbN, kAsmMfma>(acc, base, kTileN, kTile, kTileN, wm * kWaveTileM, wn * kWaveTileN, lane);
    } else {
      // plane `split` of M x N floats, clipped at the matrix edge
      const int64_t rows = g.M - m0 < kTile ? g.M - m0 : kTile;
      const uint32_t cols = (uint32_t)(g.N - n0 < kTileN ? g.N - n0 : kTileN);
      float* base = g.partial + ((int64_t)split * g.M + m0) * g.N + n0;
      store_partial_tile<G, kNbM, kNbN, kAsmMfma>(acc, base, (uint32_t)g.N, rows, cols, wm * kWaveTileM, wn * kWaveTileN, lane);
    }
  };

  uint32_t item = blockIdx.x;
  uint32_t tile_m, tile_n, tile_no, split;
  uint32_t step0;  // first k-step of the current item
  bool partial_item = decode_item(item, &tile_no, &split, &step0);
  // spread the starting points of the items evenly over their k-steps
  auto rot_of = [&](uint32_t it) __attribute__((always_inline)) -> uint32_t {
    // 32-bit arithmetic: a row panel is below 2 GiB (host check), so an item has fewer than 2^16 k-steps
    return kRotate ? __builtin_amdgcn_readfirstlane((it & 0xffffu) * steps / total_items % steps) : 0u;
  };
  rot = rot_of(item);
  tile_coord_t<uint32_t>(tile_no, tiles_m, tiles_n, &tile_m, &tile_n);
  __amdgpu_buffer_rsrc_t rsrc_a = panel_a((int64_t)tile_m * kTile), rsrc_b = panel_b((int64_t)tile_n * kTileN);
  if constexpr (kMx) mx_open_tile(tile_m, tile_n, step0);  // before the copies: see the waits
  open_tile(rsrc_a, rsrc_b, step0);

  for (;;) {
#pragma unroll
    for (int i = 0; i < kNbM; ++i)
#pragma unroll
      for (int j = 0; j < kNbN; ++j)
#pragma unroll
        for (int r = 0; r < kAccLen; ++r) acc[i][j][r] = 0.f;

    // A0 and B0 have landed; A1, B1, ... A(kAhead) may be in flight (the counter saturates at 63).
    constexpr int kOpenInFlight = kAhead * kCph + (kAhead - 1) * kCphB;
    wait_vmcnt<(kOpenInFlight < 63 ? kOpenInFlight : 63)>();
    __builtin_amdgcn_s_barrier();
    if constexpr (kRowSliced) {
#pragma unroll
      for (int j = 0; j < kNbN; ++j) fb[0][j] = load_frag(ring + kSlotBytes + b_lane, j, 0);
#pragma unroll
      for (int r = 0; r < kHalfM; ++r) fa[0][r] = load_frag(ring + a_lane, r, 0);
    } else {
#pragma unroll
      for (int q = 0; q < kReadsPerSlice; ++q) read_q(0, q, ring + a_lane, ring + kSlotBytes + b_lane, 0);
    }

    // The slot of A(t) walks 0, 2, 4, 1, 3 and repeats, so the loop is unrolled over five phases in
    // which every slot number, and with it every LDS offset, is a compile-time constant.
    // Row offsets of the operand k-steps the loop copies next, B(t+kAhead) and A(t+kAhead+1).
    const uint32_t soff_last = soff_of(step0, steps - 1);
    uint32_t soff_b = soff_of(step0, kAhead), soff_a = soff_of(step0, kAhead + 1);
    uint32_t kt_b = kAhead, kt_a = kAhead + 1;   // kRotate: k-steps (of the item) the loop copies next
    // Offset of the scales the loop loads next (those of k-step t+2).
    const uint32_t mx_soff_last = mx_soff_of(steps - 1);
    uint32_t mx_soff = mx_soff_of(2);
    uint32_t kt = 0;
    bool last = false;
    auto k_step = [&](auto phase) __attribute__((always_inline)) {
      constexpr uint32_t slot_a = (2 * decltype(phase)::value) % kSlots;
      constexpr uint32_t slot_b = (slot_a + 1) % kSlots, slot_a1 = (slot_a + 2) % kSlots, slot_b1 = (slot_a + 3) % kSlots;
      const uint8_t* a_rows = ring + slot_a * kSlotBytes + a_lane;
      const uint8_t* b_rows = ring + slot_b * kSlotBytes + b_lane;
      const uint8_t* a1_rows = ring + slot_a1 * kSlotBytes + a_lane;
      const uint8_t* b1_rows = ring + slot_b1 * kSlotBytes + b_lane;

      // Event schedule of one k-step, in MFMA positions p = slice * kMfmaPerSlice + u:
      //   reads    one fragment load per MFMA at the start of each slice (for the following slice)
      //   barrier  in slice 0, a few MFMAs after the last read so its data is back
      //   copies   spread evenly over the MFMAs after the barrier, B(t+2) first.  They must not be
      //            issued faster than the texture-address unit retires them (one 1 KiB copy takes
      //            it ~23 cycles and it serves all four waves): a wave whose copy finds the unit's
      //            queue full stalls at issue and its MFMA stream stops with it.
      // Row-sliced read schedule (position u of a slice, before MFMA u is issued):
      //   slice 0  u = 1: B block kNbN-1 of THIS k-step (its last MFMA of the previous k-step was the
      //            last one of that k-step); u = 2 .. kHalfM+1: the second half of A's rows
      //   slice 1  u = 0 .. kHalfM-1: the first half of A's rows of the next k-step;
      //            u = kHalfM*(j+1)+1: B block j of the next k-step, one MFMA after its last use
      constexpr int kLastOwnRead = kRowSliced ? kHalfM + 1 : kReadsPerSlice - 1;
      constexpr int kBarrierWant = kLastOwnRead + 1 + kMfmaPerSlice / 8;
      constexpr int kBarrierAt = kBarrierWant < kMfmaPerSlice ? kBarrierWant : kMfmaPerSlice - 1;
      constexpr int kFirstCopy = kBarrierAt + 1;
      constexpr int kCopies = kCphB + kCph;                              // B(t+2) then A(t+3)
      constexpr int kCopySpan = 2 * kMfmaPerSlice - kFirstCopy;          // positions left in the k-step
      static_assert(kCopySpan > 0, "no room for the copies");
      // copy c is issued at position kFirstCopy + c * kCopySpan / kCopies (evenly spread)
      constexpr int kMaxCopiesPerGap = (kCopies + kCopySpan - 1) / kCopySpan + 1;
      constexpr int ph = decltype(phase)::value;
      if constexpr (kMx) {
        // The scales of this k-step were requested two k-steps ago (or with the opening copies of
        // the tile, ahead of them).  Vector-memory instructions issued since: that k-step's copies,
        // the next request, the copies of the k-step after it.  Loads return in order.
        wait_vmcnt_for<2 * kCopies + 2>(sca[ph], scb[ph]);
        load_8B_async(sca[(ph + 2) % kSlots], rsrc_sa, voff_sa, mx_soff);
        load_8B_async(scb[(ph + 2) % kSlots], rsrc_sb, voff_sb, mx_soff);
      }
      static_for<2 * kMfmaPerSlice>([&](auto pc) __attribute__((always_inline)) {
        constexpr int p = decltype(pc)::value;
        constexpr int s = p / kMfmaPerSlice, u = p % kMfmaPerSlice;
        if constexpr (kRowSliced) {
          if constexpr (s == 0) {
            if constexpr (u == 1) fb[0][kNbN - 1] = load_frag(b_rows, kNbN - 1, 0);
            if constexpr (u >= 2 && u < 2 + kHalfM) fa[1][u - 2] = load_frag(a_rows, kHalfM + u - 2, 0);
          } else {
            if constexpr (u < kHalfM) fa[0][u] = load_frag(a1_rows, u, 0);
            if constexpr (u > kHalfM && (u - 1) % kHalfM == 0 && (u - 1) / kHalfM - 1 < kNbN - 1)
              fb[0][(u - 1) / kHalfM - 1] = load_frag(b1_rows, (u - 1) / kHalfM - 1, 0);
          }
        } else if constexpr (u < kReadsPerSlice) {
          if constexpr (s == 0) read_q(1, u, a_rows, b_rows, 1);       // slice 1 of this k-step
          else read_q(0, u, a1_rows, b1_rows, 0);                      // slice 0 of the next k-step
        }
        if constexpr (s == 0 && u == kBarrierAt) {
          // My reads of this k-step's slots are back; B(t+1) (and A(t+1) before it) have
          // landed; only this wave's copies of A(t+2) [... B(t+kAhead-1), A(t+kAhead)] may still be
          // in flight.
          wait_lgkmcnt0();
          constexpr int kLoopInFlight = (kAhead - 1) * kCph + (kAhead - 2) * kCphB;
          static_assert(kLoopInFlight + 2 < 64, "vmcnt is a 6-bit counter");
          wait_vmcnt<kLoopInFlight + (kMx ? 2 : 0)>();  // the two scale requests of this k-step are younger still
          __builtin_amdgcn_s_barrier();
        }
        // Copy c is "prepared" (its LDS base written to M0) one MFMA before it is issued when it
        // is alone at its position; otherwise M0 is written right in front of it.
        if constexpr (p >= kFirstCopy) {
          constexpr int c0 = first_copy_at(p, kFirstCopy, kCopySpan, kCopies);
          static_for<kMaxCopiesPerGap>([&](auto ic) __attribute__((always_inline)) {
            constexpr int c = c0 + decltype(ic)::value;
            if constexpr (c < kCopies && copy_position(c, kFirstCopy, kCopySpan, kCopies) == p) {
              constexpr bool prepared = c > 0 && copy_position(c - 1, kFirstCopy, kCopySpan, kCopies) < p - 1 &&
                                        (c + 1 >= kCopies || copy_position(c + 1, kFirstCopy, kCopySpan, kCopies) > p);
              if constexpr (c < kCphB) {
                if constexpr (!prepared) prep_rows(std::integral_constant<int, c>{}, std::integral_constant<uint32_t, slot_a>{}, dma_wave_b);
                fire_rows(rsrc_b, std::integral_constant<int, c>{}, soff_b, voff_b, tail_b, b_step);
              } else {
                if constexpr (!prepared) prep_rows(std::integral_constant<int, c - kCphB>{}, std::integral_constant<uint32_t, slot_b>{}, dma_wave_a);
                fire_rows(rsrc_a, std::integral_constant<int, c - kCphB>{}, soff_a, voff_a, tail_a, a_step);
              }
            }
          });
        }
        if constexpr (p + 1 >= kFirstCopy && p + 1 < 2 * kMfmaPerSlice) {
          constexpr int c = first_copy_at(p + 1, kFirstCopy, kCopySpan, kCopies);
          if constexpr (c > 0 && c < kCopies && copy_position(c, kFirstCopy, kCopySpan, kCopies) == p + 1 &&
                        copy_position(c - 1, kFirstCopy, kCopySpan, kCopies) < p &&
                        (c + 1 >= kCopies || copy_position(c + 1, kFirstCopy, kCopySpan, kCopies) > p + 1)) {
            if constexpr (c < kCphB) prep_rows(std::integral_constant<int, c>{}, std::integral_constant<uint32_t, slot_a>{}, dma_wave_b);
            else prep_rows(std::integral_constant<int, c - kCphB>{}, std::integral_constant<uint32_t, slot_b>{}, dma_wave_a);
          }
        }
        if constexpr (kRowSliced)
          mfma_rows(phase, std::integral_constant<int, s>{}, std::integral_constant<int, u>{});
        else mfma_u(s, u);
        MI355_FENCE();
      });
      if constexpr (kRotate) {
        soff_b = soff_of(step0, ++kt_b);
        soff_a = soff_of(step0, ++kt_a);
      } else {
        soff_b = soff_b + kRowBytes < soff_last ? soff_b + kRowBytes : soff_last;
        soff_a = soff_a + kRowBytes < soff_last ? soff_a + kRowBytes : soff_last;
      }
      if constexpr (kMx) mx_soff = mx_soff + kMxUnitBytes < mx_soff_last ? mx_soff + kMxUnitBytes : mx_soff_last;
      ++kt;
      last = kt == steps;
    };
    // Whole turns of the ring run without a test between their k-steps (a workgroup has one wave per SIMD,
    // so every scalar branch, taken or not, is a bubble in its MFMA stream: one branch per five k-steps
    // instead of one per k-step is worth 0.4-0.8 % on long K); the remaining k-steps go one by one.  The
    // row-sliced kernels keep one test per k-step: with two loops around their 256 accumulator registers
    // the register allocator carries one accumulator block through vector registers.
    if constexpr (!kRowSliced)
      for (uint32_t turns = steps / kSlots; turns > 0; --turns) static_for<kSlots>(k_step);
    while (!last) static_for<kSlots>([&](auto phase) __attribute__((always_inline)) {
      if (last) return;
      k_step(phase);
    });
    // The tail copies (past the end of K) must have landed, and every wave must be past its last
    // LDS read, before the ring is refilled for the next tile.
    wait_vmcnt<0>();
    wait_lgkmcnt0();
    __builtin_amdgcn_s_barrier();

    const int64_t done_m0 = (int64_t)tile_m * kTile, done_n0 = (int64_t)tile_n * kTileN;
    const uint32_t done_split = split, done_tile = tile_no;
    const bool done_partial = partial_item;
    item += gridDim.x;
    const bool more = item < total_items;
    if (more) {
      partial_item = decode_item(item, &tile_no, &split, &step0);
      rot = rot_of(item);
      tile_coord_t<uint32_t>(tile_no, tiles_m, tiles_n, &tile_m, &tile_n);
      rsrc_a = panel_a((int64_t)tile_m * kTile);
      rsrc_b = panel_b((int64_t)tile_n * kTileN);
      if constexpr (kMx) mx_open_tile(tile_m, tile_n, step0);
      open_tile(rsrc_a, rsrc_b, step0);  // in flight while the finished tile is stored
    }
    if (done_partial) store_partial(done_m0, done_n0, done_split, done_tile);
    else epilogue(done_m0, done_n0);
    if (!more) break;
  }
}

// C tiles of a tail split: rne(scale * (partial[0] + ... + partial[S-1])) in that order, for the
// last g.tail_tiles tiles in tile-map order; one thread per 4 consecutive columns.
template <class OutT, int kTileT, int kTileNT>
__global__ __launch_bounds__(256) void tail_reduce(GemmArgs g) {
  constexpr uint32_t kQuadsPerTile = kTileT * kTileNT / 4;
  const uint32_t q = blockIdx.x * 256u + threadIdx.x;
  const uint32_t t = q / kQuadsPerTile, in_tile = q % kQuadsPerTile;
  if (t >= (uint32_t)g.tail_tiles) return;
  const uint32_t r = in_tile / (kTileNT / 4), c = (in_tile % (kTileNT / 4)) * 4;
  uint32_t tile_m, tile_n;
  tile_coord_t<uint32_t>((uint32_t)(g.tiles_m * g.tiles_n) - (uint32_t)g.tail_tiles + t, (uint32_t)g.tiles_m,
                         (uint32_t)g.tiles_n, &tile_m, &tile_n);
  const int64_t m = (int64_t)tile_m * kTileT + r, n = (int64_t)tile_n * kTileNT + c;
  if (m >= g.M || n >= g.N) return;  // N % 4 == 0: a quad is in or out as a whole
  const float* p = g.partial + (int64_t)t * (kTileT * kTileNT) + r * kTileNT + c;
  const int64_t split_stride = (int64_t)g.tail_tiles * (kTileT * kTileNT);
  f32x4 sum = *(const f32x4*)p;
  for (int s = 1; s < g.tail_splits; ++s) sum += *(const f32x4*)(p + s * split_stride);
  const float scale = output_scale(g);
  *(u32x2*)((uint16_t*)g.C + m * g.ldc + n) = Pack4<OutT>::run(sum[0] * scale, sum[1] * scale, sum[2] * scale, sum[3] * scale);
}

template <class T, class OutT, int kTileT, int kTileNT = kTileT, int kAhead = 2, int kWavesN = 2, bool kRotateT = (kAhead > 2)>
int launch_tile(const GemmArgs& g, hipStream_t stream) {
  const int64_t items = g.tail_tiles ? g.tiles_m * g.tiles_n + (int64_t)g.tail_tiles * (g.tail_splits - 1)
                                     : g.tiles_m * g.tiles_n * g.splits;
  if (items >= ((int64_t)1 << 31)) return -1;  // the kernel counts items in 32 bits
  const int64_t slots = (int64_t)compute_units() * ((kTileT == 256 || kAhead > 2) ? 1 : 2);  // resident workgroups (LDS-bound)
  const int64_t blocks = items < slots ? items : slots;
  if ((g.K * T::kBytes) % kRowBytes == 0) {
    hipLaunchKernelGGL((gemm_tn_tile_ring<T, OutT, false, kTileT, kWavesN, kTileNT, kAhead, kRotateT>), dim3((unsigned)blocks), dim3(threads_of(kWavesN)), 0, stream, g);
  } else {
    if constexpr (std::is_same<T, MxE4M3>::value) return -1;  // block scales need whole k-steps (host check)
    else hipLaunchKernelGGL((gemm_tn_tile_ring<T, OutT, true, kTileT, kWavesN, kTileNT, kAhead, kRotateT>), dim3((unsigned)blocks), dim3(threads_of(kWavesN)), 0, stream, g);
  }
  if (hipGetLastError() != hipSuccess) return -1;
  if (g.splits > 1)
    return launch_splitk_reduce(g.partial, g, std::is_same<OutT, BF16>::value ? 0 : 1, stream);
  if (g.tail_tiles) {
    const int64_t quads = (int64_t)g.tail_tiles * (kTileT * kTileNT / 4);
    hipLaunchKernelGGL((tail_reduce<OutT, kTileT, kTileNT>), dim3((unsigned)((quads + 255) / 256)), dim3(256), 0, stream, g);
    if (hipGetLastError() != hipSuccess) return -1;
  }
  return 0;
}

template <class T, class OutT>
int launch(const GemmArgs& g, int tile, hipStream_t stream) {
  if (tile == kRingTile256x128) return launch_tile<T, OutT, 256, 128>(g, stream);
  if (tile == kRingTile128Deep || tile == kRingTile128DeepPlain) {
    // the planner does not pick these with block scales (their registers are timed for five slots)
    if constexpr (std::is_same<T, MxE4M3>::value) return -1;
    else if (tile == kRingTile128Deep) return launch_tile<T, OutT, 128, 128, 4>(g, stream);
    else return launch_tile<T, OutT, 128, 128, 4, 2, false>(g, stream);
  }
  return tile == 128 ? launch_tile<T, OutT, 128>(g, stream) : launch_tile<T, OutT, 256>(g, stream);
}

}  // namespace

}  // namespace mi355
