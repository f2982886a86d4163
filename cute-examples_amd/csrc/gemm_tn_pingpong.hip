// "pingpong" variant: 256x256 output tile, TWO wave groups of 4 waves (8 waves, two per SIMD, one
// of each group).  Group g owns the 128 output columns [128g, 128g+128); inside a group the four
// waves own 128x64 sub-tiles (128 fp32 accumulator registers per lane).
//
// The two groups run the same program one phase apart, so that on every SIMD one wave is in an
// MFMA phase while the other is in a load phase, and they swap at every workgroup barrier:
//
//   phase  group 0                              group 1
//   4t+0   M0: MFMAs of slice 0, k-step t       L1: LDS reads of slice 0 of t   + copies
//   4t+1   L0: LDS reads of slice 1 of t        M0: MFMAs of slice 0 of t
//   4t+2   M1: MFMAs of slice 1 of t            L0: LDS reads of slice 1 of t
//   4t+3   L1: LDS reads of slice 0 of t+1      M1: MFMAs of slice 1 of t
//          + copies of B(t+2), A(t+3)
//
// A wave's MFMA and load phases never overlap, so its operand fragments are single-buffered: a
// load phase refills the registers the preceding MFMA phase has just finished with, and the other
// group's MFMA phase (512 MFMA cycles) hides the LDS latency.  MFMA phases run at raised wave
// priority.  For the 16-bit types the two slices of a k-step are the two halves of its 128 bytes
// of K (v_mfma_f32_16x16x32, 32 MFMAs per phase); for fp8 one v_mfma_f32_16x16x128_f8f6f4 spans the
// k-step, so the slices are the two halves of the wave's rows of A (16 MFMAs per phase) and the
// fragments of B are loaded once per k-step, in L1.
//
// Everything else is the single-group kernel's (gemm_tn_ring.h): the five-slot LDS ring with
// operand-steps queued as A0 B0 A1 B1 A2 ..., the row swizzle, the copy geometry, the k loop
// unrolled over the five positions of the ring so that every LDS offset is an immediate, MFMAs as
// inline assembly with the accumulator tied in place, the copies of a k-step spread between the
// LDS reads of their phase, the next tile's opening copies in flight while the finished tile is
// stored (tile_store.h).  The two slots of k-step t are refilled with B(t+2), A(t+3) once both groups
// have read them (end of phase 4t+2).
//
// Counterpart in the reference: kernels/gemm_kernels/sm90a/gemm_pingpong.cuh:121-349, where two
// consumer warpgroups alternate whole output tiles under an ordering barrier (:244-286) so that
// one's epilogue overlaps the other's MMA.  gfx950 has no asynchronous MMA to overlap with, so
// here the alternation is between the MFMA and the LDS/global load phases inside the k-loop.
#include "gemm_launch.h"
#include "ring_common.h"
#include "tile_map.h"
#include "tile_store.h"

namespace mi355 {
namespace {

constexpr int kThreads = 512;
constexpr int kSlotBytes = kTile * kRowBytes;  // 32 KiB: one operand, one k-step

// kRaggedK: K*elem_bytes is not a multiple of the 128-byte k-step.  Kept out of the common
// instantiation because selecting the per-lane offset inside the loop puts a dependent VALU
// chain in front of every copy.
template <class T, class OutT, bool kRaggedK>
__global__ __launch_bounds__(kThreads, 1) void gemm_tn_tile256_pingpong(GemmArgs g) {
  __shared__ __attribute__((aligned(1024))) uint8_t ring[kSlots * kSlotBytes];
  typedef typename RingGeo<T>::type G;
  typedef typename G::Frag Frag;
  typedef typename G::Acc Acc;
  static_assert(G::kBlk == 16 && !G::kMx, "16 x 16 blocks, no block scales");
  constexpr bool kRowSliced = G::kRowSliced;            // fp8: one MFMA spans the k-step
  constexpr int kNbA = 8;                               // 16-row blocks of A per wave (128 rows)
  constexpr int kNbB = 4;                               // 16-row blocks of B per wave (64 columns)
  constexpr int kHalfA = kNbA / 2;
  constexpr int kSliceChunks = G::kGroups * G::kCpl;

  const uint32_t tid = threadIdx.x;
  const uint32_t lane = tid & 63u;
  const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const uint32_t group = wave >> 2;            // waves 0-3 and 4-7 land on SIMDs 0-3 each
  const uint32_t wm = (wave >> 1) & 1u;        // which 128 rows
  const uint32_t wn = group * 2 + (wave & 1u); // which 64 columns

  const uint32_t lda_b = (uint32_t)(g.lda * T::kBytes), ldb_b = (uint32_t)(g.ldb * T::kBytes);
  const uint32_t k_bytes = (uint32_t)(g.K * T::kBytes);
  // K need not be a whole number of k-steps: in the last one, chunks past the end of the row are
  // fetched from an out-of-range offset (the hardware returns zeros), see tail_or_oob below.
  const uint32_t k_steps = __builtin_amdgcn_readfirstlane((k_bytes + kRowBytes - 1) / kRowBytes);
  const uint32_t tail_bytes = __builtin_amdgcn_readfirstlane(k_bytes % kRowBytes);
  const uint32_t total_tiles = (uint32_t)(g.tiles_m * g.tiles_n);

  auto panel_a = [&](int64_t m0) __attribute__((always_inline)) {
    const int64_t rows = g.M - m0 < kTile ? g.M - m0 : kTile;
    return make_raw_buffer((const uint8_t*)g.A + m0 * (int64_t)lda_b, (uint32_t)((rows - 1) * lda_b + k_bytes));
  };
  auto panel_b = [&](int64_t n0) __attribute__((always_inline)) {
    const int64_t rows = g.N - n0 < kTile ? g.N - n0 : kTile;
    return make_raw_buffer((const uint8_t*)g.B + n0 * (int64_t)ldb_b, (uint32_t)((rows - 1) * ldb_b + k_bytes));
  };

  // Copy geometry as in the single-group kernel, but each of the 8 waves moves 32 rows of an
  // operand per k-step: copies 4w..4w+3 of 8 rows x 128 B.
  constexpr int kCph = 4;
  const uint32_t r8 = lane >> 3, c8 = lane & 7u;
  constexpr uint32_t kOutOfRange = 0x80000000u;  // row panels are smaller than 2 GiB (host check)
  uint32_t voff_a[2], voff_b[2], tail_a[kRaggedK ? 2 : 1], tail_b[kRaggedK ? 2 : 1];
#pragma unroll
  for (int par = 0; par < 2; ++par) {
    const uint32_t chunk = c8 ^ swizzle(par * 8 + r8);
    voff_a[par] = (wave * 32 + r8) * lda_b + chunk * 16;
    voff_b[par] = (wave * 32 + r8) * ldb_b + chunk * 16;
    if constexpr (kRaggedK) {
      const bool tail_or_oob = tail_bytes != 0 && chunk * 16 >= tail_bytes;
      tail_a[par] = tail_or_oob ? kOutOfRange : voff_a[par];
      tail_b[par] = tail_or_oob ? kOutOfRange : voff_b[par];
    }
  }
  const uint32_t a_step = __builtin_amdgcn_readfirstlane(8 * lda_b);
  const uint32_t b_step = __builtin_amdgcn_readfirstlane(8 * ldb_b);
  const uint32_t ring0 = __builtin_amdgcn_readfirstlane(lds_address(ring));
  const uint32_t dma_wave = ring0 + wave * (kCph * 1024);  // this wave's share of a slot
  const uint32_t soff_tail = (k_steps - 1) * kRowBytes;     // the k-step that may be ragged

  // Copy j of an operand's k-step into slot `slot` (a compile-time number); soff is the k-step's
  // byte offset inside a row.
  auto copy_rows = [&](__amdgpu_buffer_rsrc_t rsrc, auto jc, auto slotc, uint32_t soff, const uint32_t* voff,
                       const uint32_t* tail, uint32_t step) __attribute__((always_inline)) {
    constexpr int j = decltype(jc)::value;
    constexpr uint32_t slot = decltype(slotc)::value;
    uint32_t v = voff[j & 1];
    if constexpr (kRaggedK) v = soff == soff_tail ? tail[j & 1] : v;
    dma_16B_to_lds_at<slot * kSlotBytes + j * 1024>(dma_wave, v + j * step, rsrc, soff);
  };
  // Byte offset of k-step kt, clamped to the last: copies past the end of K re-read it into a slot
  // nobody reads, so the loop body stays branch-free.
  auto soff_of = [&](uint32_t kt) __attribute__((always_inline)) -> uint32_t {
    return __builtin_amdgcn_readfirstlane((kt < k_steps ? kt : k_steps - 1) * kRowBytes);
  };
  auto open_tile = [&](__amdgpu_buffer_rsrc_t ra, __amdgpu_buffer_rsrc_t rb) __attribute__((always_inline)) {
    const uint32_t s0 = soff_of(0), s1 = soff_of(1), s2 = soff_of(2);
    static_for<kCph>([&](auto j) __attribute__((always_inline)) { copy_rows(ra, j, std::integral_constant<uint32_t, 0>{}, s0, voff_a, tail_a, a_step); });
    static_for<kCph>([&](auto j) __attribute__((always_inline)) { copy_rows(rb, j, std::integral_constant<uint32_t, 1>{}, s0, voff_b, tail_b, b_step); });
    static_for<kCph>([&](auto j) __attribute__((always_inline)) { copy_rows(ra, j, std::integral_constant<uint32_t, 2>{}, s1, voff_a, tail_a, a_step); });
    static_for<kCph>([&](auto j) __attribute__((always_inline)) { copy_rows(rb, j, std::integral_constant<uint32_t, 3>{}, s1, voff_b, tail_b, b_step); });
    static_for<kCph>([&](auto j) __attribute__((always_inline)) { copy_rows(ra, j, std::integral_constant<uint32_t, 4>{}, s2, voff_a, tail_a, a_step); });
  };

  // Fragment geometry: lane l supplies row l%16 of a block; group l/16 picks the chunks.
  const uint32_t rblk = lane & 15u, grp = lane >> 4;
  const uint32_t swz = swizzle(rblk);
  const uint32_t a_lane = (wm * 128 + rblk) * kRowBytes;
  const uint32_t b_lane = (wn * 64 + rblk) * kRowBytes;
  // Byte offset inside a row of the e-th chunk this lane reads in slice s (row-sliced: chunks g
  // and 4+g, the conflict-free order, see chunk_off in gemm_tn_ring.h).
  auto chunk_off = [&](int s, int e) __attribute__((always_inline)) -> uint32_t {
    if constexpr (kRowSliced) return ((uint32_t)(grp + 4 * e) ^ swz) << 4;
    else return ((uint32_t)(s * kSliceChunks + grp * G::kCpl + e) ^ swz) << 4;
  };
  auto load_frag = [&](const uint8_t* slot_rows, int blk, int s) __attribute__((always_inline)) -> Frag {
    const uint8_t* p = slot_rows + blk * 16 * kRowBytes;
    if constexpr (G::kCpl == 1) {
      return *(const i32x4*)(p + chunk_off(s, 0));
    } else {
      i32x4 lo = *(const i32x4*)(p + chunk_off(s, 0));
      i32x4 hi = *(const i32x4*)(p + chunk_off(s, 1));
      return (i32x8){lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
    }
  };

  Acc acc[kNbA][kNbB];
  // K-sliced: all blocks of A and of B, one slice of K at a time.  Row-sliced: all of B for the
  // k-step and half of the wave's rows of A at a time.
  Frag fa[kRowSliced ? kHalfA : kNbA], fb[kNbB];

  // Load number q of the load phase in front of slice s (a_rows / b_rows: the slot rows of the k-step
  // that slice belongs to); returns the number of loads of that phase through kReads.
  constexpr int kReads0 = kRowSliced ? kNbB + kHalfA : kNbB + kNbA;   // in front of slice 0 (phase L1)
  constexpr int kReads1 = kRowSliced ? kHalfA : kNbB + kNbA;          // in front of slice 1 (phase L0)
  auto read_q = [&](auto sc, auto qc, const uint8_t* a_rows, const uint8_t* b_rows) __attribute__((always_inline)) {
    constexpr int s = decltype(sc)::value, q = decltype(qc)::value;
    if constexpr (kRowSliced) {
      if constexpr (s == 0) {
        if constexpr (q < kNbB) fb[q] = load_frag(b_rows, q, 0);
        else fa[q - kNbB] = load_frag(a_rows, q - kNbB, 0);
      } else {
        fa[q] = load_frag(a_rows, kHalfA + q, 0);
      }
    } else {
      if constexpr (q < kNbB) fb[q] = load_frag(b_rows, q, s);
      else fa[q - kNbB] = load_frag(a_rows, q - kNbB, s);
    }
  };
  auto mfma_phase = [&](auto sc) __attribute__((always_inline)) {
    constexpr int s = decltype(sc)::value;
    __builtin_amdgcn_s_setprio(1);
    if constexpr (kRowSliced) {
      static_for<kHalfA * kNbB>([&](auto uc) __attribute__((always_inline)) {
        constexpr int r = decltype(uc)::value / kNbB, j = decltype(uc)::value % kNbB;
        G::mfma_inplace(fb[j], fa[r], acc[s * kHalfA + r][j]);
      });
    } else {
      static_for<kNbA * kNbB>([&](auto uc) __attribute__((always_inline)) {
        constexpr int i = decltype(uc)::value / kNbB, j = decltype(uc)::value % kNbB;
        G::mfma_inplace(fb[j], fa[i], acc[i][j]);
      });
    }
    __builtin_amdgcn_s_setprio(0);
  };
  // Phase boundary: nothing may move across it.
  auto phase_barrier = [&]() __attribute__((always_inline)) {
    MI355_FENCE();
    __builtin_amdgcn_s_barrier();
    MI355_FENCE();
  };

  const float scale = output_scale(g);
  auto epilogue = [&](int64_t m0, int64_t n0) __attribute__((always_inline)) {
    store_output_tile<G, OutT, kNbA, kNbB, true>(acc, g, m0, n0, kTile, kTile, wm * 128, wn * 64, lane, scale);
  };

  const uint32_t tiles_m = (uint32_t)g.tiles_m, tiles_n = (uint32_t)g.tiles_n;  // below 2^31 tiles (launcher)
  uint32_t tile = blockIdx.x;
  uint32_t tile_m, tile_n;
  tile_coord_t<uint32_t>(tile, tiles_m, tiles_n, &tile_m, &tile_n);
  __amdgpu_buffer_rsrc_t rsrc_a = panel_a((int64_t)tile_m * kTile), rsrc_b = panel_b((int64_t)tile_n * kTile);
  open_tile(rsrc_a, rsrc_b);

  for (;;) {
#pragma unroll
    for (int i = 0; i < kNbA; ++i)
#pragma unroll
      for (int j = 0; j < kNbB; ++j)
#pragma unroll
        for (int r = 0; r < 4; ++r) acc[i][j][r] = 0.f;

    wait_vmcnt<3 * kCph>();  // A0 and B0 have landed (A1, B1, A2 may be in flight)
    phase_barrier();
    static_for<kReads0>([&](auto q) __attribute__((always_inline)) {
      read_q(std::integral_constant<int, 0>{}, q, ring + a_lane, ring + kSlotBytes + b_lane);
    });
    wait_lgkmcnt0();
    if (group == 1) phase_barrier();  // group 1 runs one phase behind group 0

    // Row offsets of the operand k-steps the loop copies next, B(t+2) and A(t+3).
    const uint32_t soff_last = soff_of(k_steps - 1);
    uint32_t soff_b = soff_of(2), soff_a = soff_of(3);
    uint32_t kt = 0;
    bool last = false;
    for (;;) {
      // The slot of A(t) walks 0, 2, 4, 1, 3: unrolled over the five positions, every slot number and
      // with it every LDS offset is a compile-time constant.
      static_for<kSlots>([&](auto phase) __attribute__((always_inline)) {
        if (last) return;
        constexpr uint32_t slot_a = (2 * decltype(phase)::value) % kSlots;
        constexpr uint32_t slot_b = (slot_a + 1) % kSlots, slot_a1 = (slot_a + 2) % kSlots, slot_b1 = (slot_a + 3) % kSlots;
        const uint8_t* a_rows = ring + slot_a * kSlotBytes + a_lane;
        const uint8_t* b_rows = ring + slot_b * kSlotBytes + b_lane;
        const uint8_t* a1_rows = ring + slot_a1 * kSlotBytes + a_lane;
        const uint8_t* b1_rows = ring + slot_b1 * kSlotBytes + b_lane;

        // M0: slice 0 of this k-step.
        mfma_phase(std::integral_constant<int, 0>{});
        phase_barrier();
        // L0: slice 1 of this k-step.  For group 1 this phase ends at global phase 4t+2, the point
        // by which B(t+1) must have landed everywhere (only the copies of A(t+2) may be in flight).
        static_for<kReads1>([&](auto q) __attribute__((always_inline)) {
          read_q(std::integral_constant<int, 1>{}, q, a_rows, b_rows);
        });
        wait_lgkmcnt0();
        if (group == 1) wait_vmcnt<kCph>();
        phase_barrier();
        // M1: slice 1.  For group 0 this phase ends at global phase 4t+2.
        mfma_phase(std::integral_constant<int, 1>{});
        if (group == 0) wait_vmcnt<kCph>();
        phase_barrier();
        // L1: slice 0 of the next k-step, and this wave's share of the refill, one copy after
        // every second read so that the copies do not queue up behind each other in the
        // texture-address unit.  Both groups have finished reading the slots of k-step t by now
        // (group 1 did so in its L0, one phase ago from group 0's point of view, three phases ago
        // from its own).
        static_for<kReads0>([&](auto qc) __attribute__((always_inline)) {
          constexpr int q = decltype(qc)::value;
          read_q(std::integral_constant<int, 0>{}, qc, a1_rows, b1_rows);
          constexpr int kCopies = 2 * kCph;
          // copy c goes after read number (c + 1) * kReads0 / kCopies - 1
          static_for<kCopies>([&](auto cc) __attribute__((always_inline)) {
            constexpr int c = decltype(cc)::value;
            if constexpr ((c + 1) * kReads0 / kCopies - 1 == q) {
              if constexpr (c < kCph)
                copy_rows(rsrc_b, std::integral_constant<int, c>{}, std::integral_constant<uint32_t, slot_a>{}, soff_b, voff_b, tail_b, b_step);
              else
                copy_rows(rsrc_a, std::integral_constant<int, c - kCph>{}, std::integral_constant<uint32_t, slot_b>{}, soff_a, voff_a, tail_a, a_step);
            }
          });
        });
        wait_lgkmcnt0();
        phase_barrier();
        soff_b = soff_b + kRowBytes < soff_last ? soff_b + kRowBytes : soff_last;
        soff_a = soff_a + kRowBytes < soff_last ? soff_a + kRowBytes : soff_last;
        ++kt;
        last = kt == k_steps;
      });
      if (last) break;
    }
    if (group == 0) phase_barrier();  // let group 1 finish its last phase; barrier counts now match
    wait_vmcnt<0>();
    phase_barrier();

    const int64_t done_m0 = (int64_t)tile_m * kTile, done_n0 = (int64_t)tile_n * kTile;
    tile += gridDim.x;
    const bool more = tile < total_tiles;
    if (more) {
      tile_coord_t<uint32_t>(tile, tiles_m, tiles_n, &tile_m, &tile_n);
      rsrc_a = panel_a((int64_t)tile_m * kTile);
      rsrc_b = panel_b((int64_t)tile_n * kTile);
      open_tile(rsrc_a, rsrc_b);
    }
    epilogue(done_m0, done_n0);
    if (!more) break;
  }
}

template <class T, class OutT>
int launch(const GemmArgs& g, hipStream_t stream) {
  const int64_t tiles = g.tiles_m * g.tiles_n;
  if (tiles >= ((int64_t)1 << 31)) return -1;  // the kernel counts tiles in 32 bits
  const int64_t cus = compute_units();
  const int64_t blocks = tiles < cus ? tiles : cus;
  if ((g.K * T::kBytes) % kRowBytes == 0)
    hipLaunchKernelGGL((gemm_tn_tile256_pingpong<T, OutT, false>), dim3((unsigned)blocks), dim3(kThreads), 0, stream, g);
  else
    hipLaunchKernelGGL((gemm_tn_tile256_pingpong<T, OutT, true>), dim3((unsigned)blocks), dim3(kThreads), 0, stream, g);
  return hipGetLastError() == hipSuccess ? 0 : -1;
}

}  // namespace

int launch_tile256_pingpong(const GemmArgs& g, int in_dtype, int out_dtype, hipStream_t stream) {
  const bool out_bf16 = out_dtype == 0;
  switch (in_dtype) {
    case 0: return out_bf16 ? launch<BF16, BF16>(g, stream) : launch<BF16, F16>(g, stream);
    case 1: return out_bf16 ? launch<F16, BF16>(g, stream) : launch<F16, F16>(g, stream);
    case 2: return out_bf16 ? launch<E4M3, BF16>(g, stream) : launch<E4M3, F16>(g, stream);
  }
  return -1;
}

}  // namespace mi355
