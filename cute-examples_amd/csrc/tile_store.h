// Writing a finished tile: accumulators -> bf16/fp16 rows of C, or -> fp32 rows of a split-K plane.
// Shared by the ring-buffered tile kernels; each wave stores the kNbM x kNbN MFMA blocks it owns.
//
// Register-to-element map (MFMA with B as the "row" operand): accumulator register 4q+e of block
// (i, j) in lane l is the output element
//   m = wave_row + i*kBlk + l%kBlk,   n = wave_col + j*kBlk + q*4*kGroups + 4*(l/kBlk) + e.
//
// All stores go through a buffer descriptor of the tile itself: offsets are 32 bits, the
// descriptor's size cuts off rows past M, and a lane whose columns lie past N gets an
// out-of-range offset, so the hardware drops what must not be written and the code has no
// per-store branch or 64-bit address arithmetic.  Row block i goes into the scalar offset, the
// column into the instruction's immediate.  Few live registers matter here as much as few
// instructions: a spill reload between two stores waits on the memory counter, i.e. for every
// store issued before it, and that serialisation once made this phase four times longer.
#pragma once
#include "gemm_launch.h"
#include "ring_common.h"

namespace mi355 {

constexpr uint32_t kStoreOutOfRange = 0x80000000u;  // tiles of C span less than 2 GiB (host check)

// Called on an accumulator block right before it is read element by element.  kPinned: the kernel's
// MFMAs are inline assembly on accumulation registers; the empty statement here keeps the block in
// those registers up to this point of the program, so the register allocator moves it to VGPRs
// here, block by block, and not all 256 registers at once when the k loop ends (which would
// spill).  The reads themselves stay ordinary compiler-generated moves: the compiler then also keeps
// them clear of the data registers of stores still being issued, which hand-placed reads once
// overwrote.
template <bool kPinned, class Acc>
__device__ __forceinline__ void pin_acc_block(Acc& a) {
  if constexpr (kPinned) asm volatile("" : "+a"(a));
}

// The wave's part of the output tile at (m0, n0), tile_rows x tile_cols at most.
// wave_row / wave_col: first row / column of the wave inside the tile.
template <class G, class OutT, int kNbM, int kNbN, bool kAsmRead>
__device__ __forceinline__ void store_output_tile(typename G::Acc (&acc)[kNbM][kNbN], const GemmArgs& g,
                                                  int64_t m0, int64_t n0, int tile_rows, int tile_cols,
                                                  uint32_t wave_row, uint32_t wave_col, uint32_t lane, float scale) {
  typedef typename G::Acc Acc;
  constexpr int kBlk = G::kBlk;
  // Cache policy of the stores.  Write-through (sc1) always: C is written once and read by nobody here.  Non-temporal
  // on top of that (nt + sc1) when the host finds the output too large to pass through the Infinity Cache beside the
  // operands (g.c_streams): then it would push operand panels out (16384^2 x 4096: 2-6 % faster with nt), while a
  // smaller C is written faster without nt (8192^2 x 1024..2048: 6 %, fp8 8192^3: 2-3 %).  Either only pays when a
  // store instruction covers at least 64 contiguous bytes per row, which the 16-wide blocks do (two blocks side by
  // side) and the 32-wide blocks do not (32 bytes: measured 3 % slower with sc1, 25 % with nt + sc1).
  const uint32_t rblk = lane & (kBlk - 1), grp = lane / kBlk;
  const int64_t rows = g.M - m0 < tile_rows ? g.M - m0 : tile_rows;
  const uint32_t cols = (uint32_t)(g.N - n0 < tile_cols ? g.N - n0 : tile_cols);
  const uint32_t ldc_b = (uint32_t)g.ldc * 2;
  const __amdgpu_buffer_rsrc_t rc =
      make_raw_buffer((const uint16_t*)g.C + m0 * g.ldc + n0, (uint32_t)(((rows - 1) * g.ldc + cols) * 2));
  // After the lane-group swaps below every lane holds 8 consecutive columns, starting here.
  const uint32_t lane_col = kBlk == 16 ? (grp & 1) * 16 + (grp >> 1) * 8 : grp * 8;
  const uint32_t col0 = wave_col + lane_col;
  const uint32_t v0 = (wave_row + rblk) * ldc_b + col0 * 2;
  const uint32_t block_step = __builtin_amdgcn_readfirstlane(kBlk * ldc_b);

  float factor = scale;
  auto pack_quad = [&](const Acc& a, int q) __attribute__((always_inline)) -> u32x2 {
    return Pack4<OutT>::run(a[4 * q] * factor, a[4 * q + 1] * factor, a[4 * q + 2] * factor, a[4 * q + 3] * factor);
  };
  // emit(i, col, x, y): x = the lane's first four outputs, y = the last four, `col` columns right of
  // col0 in row block i (both compile-time values).
  auto convert = [&](auto&& emit) __attribute__((always_inline)) {
    static_for<kNbM>([&](auto ic) __attribute__((always_inline)) {
      constexpr int i = decltype(ic)::value;
      if constexpr (kBlk == 16) {
        // Lane group g = l/16 holds columns 4g..4g+3 of every 16-wide block.  After swapping the
        // odd groups of block j with the even groups of block j+1, groups 0,2 hold columns
        // 0..7 / 8..15 of block j and groups 1,3 the same of block j+1.
        static_for<kNbN / 2>([&](auto jc) __attribute__((always_inline)) {
          constexpr int j = 2 * decltype(jc)::value;
          pin_acc_block<kAsmRead>(acc[i][j]);
          pin_acc_block<kAsmRead>(acc[i][j + 1]);
          u32x2 x = pack_quad(acc[i][j], 0), y = pack_quad(acc[i][j + 1], 0);
          u32x2 lo = __builtin_amdgcn_permlane16_swap(x[0], y[0], false, false);
          u32x2 hi = __builtin_amdgcn_permlane16_swap(x[1], y[1], false, false);
          emit(ic, std::integral_constant<int, j * 16>{}, (u32x2){lo[0], hi[0]}, (u32x2){lo[1], hi[1]});
        });
      } else {
        // Lane group g = l/32 holds columns 8q+4g..8q+4g+3 (q = 0..3) of every 32-wide block.
        // After swapping the upper half of quad q with the lower half of quad q+1, group 0 holds
        // columns 16(q/2)..+7 and group 1 columns 16(q/2)+8..+15.
        static_for<kNbN * 2>([&](auto jq) __attribute__((always_inline)) {
          constexpr int j = decltype(jq)::value / 2, q = 2 * (decltype(jq)::value % 2);
          if constexpr (q == 0) pin_acc_block<kAsmRead>(acc[i][j]);
          u32x2 x = pack_quad(acc[i][j], q), y = pack_quad(acc[i][j], q + 1);
          u32x2 lo = __builtin_amdgcn_permlane32_swap(x[0], y[0], false, false);
          u32x2 hi = __builtin_amdgcn_permlane32_swap(x[1], y[1], false, false);
          emit(ic, std::integral_constant<int, j * 32 + (q >> 1) * 16>{}, (u32x2){lo[0], hi[0]},
               (u32x2){lo[1], hi[1]});
        });
      }
    });
  };
  if (cols == (uint32_t)tile_cols) {
    auto whole_rows = [&](auto auxc) __attribute__((always_inline)) {
      // The two forms of this phase differ in one bit of their stores.  Each takes the scale through a statement of
      // its own, so that the compiler cannot lift the first conversions, which would otherwise be the same in both,
      // in front of the choice between them: the distance between a store and the next write of its data registers
      // rests on every conversion standing between the stores of its own form.
      if constexpr (decltype(auxc)::value == 18) asm volatile("; C streamed" : "+v"(factor));
      else asm volatile("; C kept" : "+v"(factor));
      u32x4 previous = {0u, 0u, 0u, 0u}, before = {0u, 0u, 0u, 0u};
      convert([&](auto ic, auto colc, u32x2 x, u32x2 y) __attribute__((always_inline)) {
        constexpr int i = decltype(ic)::value, col = decltype(colc)::value;
        u32x4 data = {x[0], x[1], y[0], y[1]};
        hold_previous(data, previous, before);
        __builtin_amdgcn_raw_buffer_store_b128(data, rc, v0 + col * 2, i * block_step, decltype(auxc)::value);
        MI355_FENCE();   // the next block's conversion stays behind this store
        before = previous;
        previous = data;
      });
      hold_last(previous);
    };
    if constexpr (kBlk != 16) whole_rows(std::integral_constant<int, 0>{});
    else if (g.c_streams) whole_rows(std::integral_constant<int, 18>{});
    else whole_rows(std::integral_constant<int, 16>{});
  } else {
    // N is a multiple of 4 (host check), so each half of the 8 columns is in or out as a whole.
    u32x4 previous = {0u, 0u, 0u, 0u}, before = {0u, 0u, 0u, 0u};
    convert([&](auto ic, auto colc, u32x2 x, u32x2 y) __attribute__((always_inline)) {
      constexpr int i = decltype(ic)::value, col = decltype(colc)::value;
      const uint32_t vx = col0 + col + 4 <= cols ? v0 + col * 2 : kStoreOutOfRange;
      const uint32_t vy = col0 + col + 8 <= cols ? v0 + col * 2 + 8 : kStoreOutOfRange;
      u32x4 data = {x[0], x[1], y[0], y[1]};
      hold_previous(data, previous, before);
      __builtin_amdgcn_raw_buffer_store_b64((u32x2){data[0], data[1]}, rc, vx, i * block_step, 0);
      __builtin_amdgcn_raw_buffer_store_b64((u32x2){data[2], data[3]}, rc, vy, i * block_step, 0);
      MI355_FENCE();
      before = previous;
      previous = data;
    });
    hold_last(previous);
  }
}

// The same part of the tile as raw fp32 accumulators into the split-K workspace: `rows` x `cols`
// floats at `base` with row stride `ld` floats; 4 consecutive columns per register quad, no lane
// exchange.
template <class G, int kNbM, int kNbN, bool kAsmRead>
__device__ __forceinline__ void store_partial_tile(typename G::Acc (&acc)[kNbM][kNbN], float* base, uint32_t ld,
                                                   int64_t rows, uint32_t cols, uint32_t wave_row,
                                                   uint32_t wave_col, uint32_t lane) {
  constexpr int kBlk = G::kBlk;
  constexpr int kQuads = kBlk * kBlk / 64 / 4;
  const uint32_t rblk = lane & (kBlk - 1), grp = lane / kBlk;
  const uint32_t ldp_b = ld * 4;
  const __amdgpu_buffer_rsrc_t rp = make_raw_buffer(base, (uint32_t)(((rows - 1) * ld + cols) * 4));
  const uint32_t col0 = wave_col + grp * 4;
  const uint32_t v0 = (wave_row + rblk) * ldp_b + col0 * 4;
  const uint32_t block_step = __builtin_amdgcn_readfirstlane(kBlk * ldp_b);
  static_for<kNbM>([&](auto ic) __attribute__((always_inline)) {
    constexpr int i = decltype(ic)::value;
    static_for<kNbN * kQuads>([&](auto jq) __attribute__((always_inline)) {
      constexpr int j = decltype(jq)::value / kQuads, q = decltype(jq)::value % kQuads;
      constexpr int col = j * kBlk + q * 4 * G::kGroups;
      const uint32_t v = col0 + col + 4 <= cols ? v0 + col * 4 : kStoreOutOfRange;
      if constexpr (q == 0) pin_acc_block<kAsmRead>(acc[i][j]);
      const typename G::Acc& c = acc[i][j];
      const f32x4 quad = {c[4 * q], c[4 * q + 1], c[4 * q + 2], c[4 * q + 3]};
      u32x4 data = __builtin_bit_cast(u32x4, quad);
      asm volatile("" : "+v"(data));   // the store reads these registers, the ones hold_last then holds
      // write-through: the partials are read back by another kernel, not by this one (+8 % measured)
      __builtin_amdgcn_raw_buffer_store_b128(data, rp, v, i * block_step, 16);
      hold_last(data);   // 12 idle cycles per store: this path runs once per split item, not per k-step
    });
  });
}

}  // namespace mi355
