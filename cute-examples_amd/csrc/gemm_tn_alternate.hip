// "alternate" variant: TWO workgroups of 4 waves per compute unit, each on its OWN stream of 256x128
// output tiles with its own half of the LDS, so that one workgroup's epilogue (conversion, stores,
// the opening copies of its next tile) runs under the other workgroup's MFMAs.
//
// Counterpart in the reference: the ping-pong kernel, kernels/gemm_kernels/sm90a/gemm_pingpong.cuh:
// 121-349 -- two consumer warpgroups on different output tiles (64x256 each, :351-384), an ordering
// barrier that makes them take turns on the tensor cores (:244-257, :281-286), so that the stores of
// one tile (:287-319) overlap the other tile's MMAs.  On gfx950 the two "groups" are two independent
// workgroups resident on one CU: a SIMD holds one wave of each, its MFMA pipe goes to whichever wave
// has an MFMA ready, and the turn-taking that the reference enforces with a barrier falls out of the
// hardware's arbitration -- a wave that waits (for its LDS reads, for a copy, at its workgroup's
// barrier, in its epilogue) simply leaves the pipe to the other one.  Workgroup barriers stay
// private to a group because the groups are separate workgroups.
//
// What the halves cost.  A wave has 256 registers instead of 512, i.e. 128 accumulators: a 256x128
// tile per workgroup, 128x64 per wave.  Per flop that is 1.5 times the bytes copied into LDS and 1.5
// times the fragment bytes read from it, compared with the 256x256 tile of gemm_tn_ring.h.
//
// LDS of a workgroup: 80 KiB = two 32 KiB slots of A (256 rows x 128 B, one k-step each) and ONE
// 16 KiB slot of B (128 rows).  k-step t computes from A slot t%2 and the B slot while A(t+1) sits in
// (or is on its way into) the other A slot.  The one B slot is refilled early in the k-step, as soon
// as every wave holds both K-halves of B(t) in registers, and must be back by the middle of it: B is
// the operand with the short flight time (about half a k-step of the workgroup's own MFMAs, twice
// that on the clock while the other workgroup takes its turns).
//
// Schedule of a k-step inside a wave (two slices = the two 64-byte halves of K; 32 MFMAs per slice,
// A-major: row block i of A against the four blocks of B):
//   slice 0   MFMAs on fa[0..7] (A(t) slice 0) and fb[0][..] (B(t) slice 0)
//             reads: fb[1][..] <- B(t) slice 1 at the start; fa[i] <- A(t) slice 1, in place, one MFMA
//             after the last MFMA of row i (a row is next used 32 MFMAs later)
//             after row 1: lgkmcnt(0), s_barrier -- the B slot is free; copies B(t+1) -> B slot
//   slice 1   MFMAs on fa (now slice 1) and fb[1]
//             after row 1: lgkmcnt(0), vmcnt(0), s_barrier -- every wave has read the slot of A(t);
//             A(t+1) and B(t+1) have landed; then the copies A(t+2) -> the slot of A(t), spread over
//             the rest of the slice
//             reads: fb[0][..] <- B(t+1) slice 0 right after the barrier; fa[i] <- A(t+1) slice 0, in
//             place, two rows behind the MFMAs
// Two workgroup barriers per k-step; every wait in this list is time the other workgroup computes in.
// (A first form refilled the B slot together with A's, after the second barrier, and waited for it
// with a third barrier at the end of the k-step: 3-4 % slower from 16 k-steps on.)
//
// 16-bit input types only.
#include "gemm_launch.h"
#include "ring_common.h"
#include "tile_map.h"
#include "tile_store.h"

namespace mi355 {
namespace {

constexpr int kAltTileM = 256, kAltTileN = 128;
constexpr int kAltSlotA = kAltTileM * kRowBytes;        // 32 KiB
constexpr int kAltSlotB = kAltTileN * kRowBytes;        // 16 KiB
constexpr int kAltLdsBytes = 2 * kAltSlotA + kAltSlotB;  // 80 KiB: two workgroups per CU
constexpr int kAltOffB = 2 * kAltSlotA;

template <class T, class OutT, bool kRaggedK>
__global__ __launch_bounds__(256, 2) void gemm_tn_tile_alternate(GemmArgs g) {
  __shared__ __attribute__((aligned(1024))) uint8_t lds[kAltLdsBytes];
  static_assert(2 * kAltLdsBytes <= 160 * 1024, "two workgroups share the LDS of a CU");
  typedef typename RingGeo<T>::type G;
  typedef typename G::Frag Frag;
  typedef typename G::Acc Acc;
  static_assert(G::kBlk == 16 && !G::kMx && !G::kRowSliced, "16 x 16 blocks, two K slices per k-step, no block scales");
  constexpr int kNbA = 8, kNbB = 4;              // 16-row blocks per wave: 128 rows of A, 64 of B
  constexpr int kSliceChunks = G::kGroups * G::kCpl;
  constexpr int kCphA = 8, kCphB = 4;            // copies (8 rows x 128 B) per wave and k-step

  const uint32_t tid = threadIdx.x;
  const uint32_t lane = tid & 63u;
  const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const uint32_t wm = wave >> 1, wn = wave & 1u;

  const uint32_t lda_b = (uint32_t)(g.lda * T::kBytes), ldb_b = (uint32_t)(g.ldb * T::kBytes);
  const uint32_t k_bytes = (uint32_t)(g.K * T::kBytes);
  const uint32_t k_steps = __builtin_amdgcn_readfirstlane((k_bytes + kRowBytes - 1) / kRowBytes);
  const uint32_t tail_bytes = __builtin_amdgcn_readfirstlane(k_bytes % kRowBytes);
  const uint32_t tiles_m = (uint32_t)g.tiles_m, tiles_n = (uint32_t)g.tiles_n;
  const uint32_t total_tiles = tiles_m * tiles_n;   // the launcher keeps this below 2^31

  auto panel_a = [&](int64_t m0) __attribute__((always_inline)) {
    const int64_t rows = g.M - m0 < kAltTileM ? g.M - m0 : kAltTileM;
    return make_raw_buffer((const uint8_t*)g.A + m0 * (int64_t)lda_b, (uint32_t)((rows - 1) * lda_b + k_bytes));
  };
  auto panel_b = [&](int64_t n0) __attribute__((always_inline)) {
    const int64_t rows = g.N - n0 < kAltTileN ? g.N - n0 : kAltTileN;
    return make_raw_buffer((const uint8_t*)g.B + n0 * (int64_t)ldb_b, (uint32_t)((rows - 1) * ldb_b + k_bytes));
  };

  // Copy geometry as in gemm_tn_ring.h: wave w moves rows [64w, 64w+64) of A and [32w, 32w+32) of B,
  // 8 rows per instruction, the LDS side linear in the lane number and the row swizzle applied on
  // the global side.
  const uint32_t lrow = lane >> 3, lchunk = lane & 7u;
  constexpr uint32_t kOutOfRange = 0x80000000u;
  uint32_t voff_a[2], voff_b[2], tail_a[kRaggedK ? 2 : 1], tail_b[kRaggedK ? 2 : 1];
#pragma unroll
  for (int par = 0; par < 2; ++par) {
    const uint32_t chunk = lchunk ^ swizzle(par * 8 + lrow);
    voff_a[par] = (wave * (kCphA * 8) + lrow) * lda_b + chunk * 16;
    voff_b[par] = (wave * (kCphB * 8) + lrow) * ldb_b + chunk * 16;
    if constexpr (kRaggedK) {
      const bool tail_or_oob = tail_bytes != 0 && chunk * 16 >= tail_bytes;
      tail_a[par] = tail_or_oob ? kOutOfRange : voff_a[par];
      tail_b[par] = tail_or_oob ? kOutOfRange : voff_b[par];
    }
  }
  const uint32_t a_step = __builtin_amdgcn_readfirstlane(8 * lda_b);
  const uint32_t b_step = __builtin_amdgcn_readfirstlane(8 * ldb_b);
  const uint32_t lds0 = __builtin_amdgcn_readfirstlane(lds_address(lds));
  const uint32_t dma_a = lds0 + wave * (kCphA * 1024);            // + slot * kAltSlotA + j * 1024
  const uint32_t dma_b = lds0 + kAltOffB + wave * (kCphB * 1024);
  const uint32_t soff_tail = (k_steps - 1) * kRowBytes;             // the k-step that may be ragged

  auto copy_a = [&](__amdgpu_buffer_rsrc_t rsrc, auto jc, auto slotc, uint32_t soff) __attribute__((always_inline)) {
    constexpr int j = decltype(jc)::value;
    uint32_t v = voff_a[j & 1];
    if constexpr (kRaggedK) v = soff == soff_tail ? tail_a[j & 1] : v;
    dma_16B_to_lds_at<decltype(slotc)::value * kAltSlotA + j * 1024>(dma_a, v + j * a_step, rsrc, soff);
  };
  auto copy_b = [&](__amdgpu_buffer_rsrc_t rsrc, auto jc, uint32_t soff) __attribute__((always_inline)) {
    constexpr int j = decltype(jc)::value;
    uint32_t v = voff_b[j & 1];
    if constexpr (kRaggedK) v = soff == soff_tail ? tail_b[j & 1] : v;
    dma_16B_to_lds_at<j * 1024>(dma_b, v + j * b_step, rsrc, soff);
  };
  // Byte offset of k-step kt, clamped to the last: copies past the end of K re-read it into a slot
  // nobody reads any more, so the loop body stays branch-free.
  auto soff_of = [&](uint32_t kt) __attribute__((always_inline)) -> uint32_t {
    return __builtin_amdgcn_readfirstlane((kt < k_steps ? kt : k_steps - 1) * kRowBytes);
  };
  auto open_tile = [&](__amdgpu_buffer_rsrc_t ra, __amdgpu_buffer_rsrc_t rb) __attribute__((always_inline)) {
    const uint32_t s0 = soff_of(0), s1 = soff_of(1);
    static_for<kCphA>([&](auto j) __attribute__((always_inline)) { copy_a(ra, j, std::integral_constant<int, 0>{}, s0); });
    static_for<kCphB>([&](auto j) __attribute__((always_inline)) { copy_b(rb, j, s0); });
    static_for<kCphA>([&](auto j) __attribute__((always_inline)) { copy_a(ra, j, std::integral_constant<int, 1>{}, s1); });
  };

  // Fragment geometry: lane l supplies row l%16 of a block; group l/16 picks the chunks.
  const uint32_t rblk = lane & 15u, grp = lane >> 4;
  const uint32_t swz = swizzle(rblk);
  const uint32_t a_lane = (wm * 128 + rblk) * kRowBytes;
  const uint32_t b_lane = kAltOffB + (wn * 64 + rblk) * kRowBytes;
  auto chunk_off = [&](int s, int e) __attribute__((always_inline)) -> uint32_t {
    return ((uint32_t)(s * kSliceChunks + grp * G::kCpl + e) ^ swz) << 4;
  };
  auto load_frag = [&](const uint8_t* rows, int blk, int s) __attribute__((always_inline)) -> Frag {
    const uint8_t* p = rows + blk * 16 * kRowBytes;
    if constexpr (G::kCpl == 1) {
      return *(const i32x4*)(p + chunk_off(s, 0));
    } else {
      i32x4 lo = *(const i32x4*)(p + chunk_off(s, 0));
      i32x4 hi = *(const i32x4*)(p + chunk_off(s, 1));
      return (i32x8){lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
    }
  };

  Acc acc[kNbA][kNbB];
  // fa holds one slice of all 8 row blocks of A (reloaded in place), fb both slices of B.
  Frag fa[kNbA], fb[2][kNbB];

  const float scale = output_scale(g);
  auto epilogue = [&](int64_t m0, int64_t n0) __attribute__((always_inline)) {
    store_output_tile<G, OutT, kNbA, kNbB, true>(acc, g, m0, n0, kAltTileM, kAltTileN, wm * 128, wn * 64, lane, scale);
  };

  // Half a tile apart.  Two workgroups that start together on a CU stay in step: they wait for their
  // first copies together, reach their barriers together and store together, and nothing overlaps.
  // So every second workgroup of an XCD (consecutive block numbers go to the XCDs round-robin) begins
  // half a tile's time late -- about 1200 cycles per k-step of a tile when two workgroups share the
  // matrix cores -- and from then on each one's epilogue and tile start-up falls into the middle of
  // the other one's k loop.  Measured at bf16 8192 x 8192 x K against no delay: K = 256 55.6 -> 53.4 us,
  // K = 512 78.9 -> 74.5 us, K = 1024 127.7 -> 124.3 us; but K = 2048 223.7 -> 232.8 us and K = 8192
  // 790 -> 849 us: workgroups that are many k-steps apart no longer find each other's operand panels
  // in their XCD's L2, so only tiles whose whole K range stays in the L2 (16 k-steps) are staggered.
  // (Delaying the upper half of the grid instead gained nothing: 59.9 us at K = 256.)
  constexpr uint32_t kStaggerMaxSteps = 16;
  if (k_steps <= kStaggerMaxSteps && total_tiles > gridDim.x / 2 && (blockIdx.x / kNumXcd) % 2 == 1)
    for (uint32_t i = 0; i < k_steps; ++i) __builtin_amdgcn_s_sleep(19);   // 19 x 64 cycles per k-step
  uint32_t tile = blockIdx.x;
  uint32_t tile_m, tile_n;
  tile_coord_t<uint32_t>(tile, tiles_m, tiles_n, &tile_m, &tile_n);
  __amdgpu_buffer_rsrc_t rsrc_a = panel_a((int64_t)tile_m * kAltTileM), rsrc_b = panel_b((int64_t)tile_n * kAltTileN);
  open_tile(rsrc_a, rsrc_b);

  for (;;) {
#pragma unroll
    for (int i = 0; i < kNbA; ++i)
#pragma unroll
      for (int j = 0; j < kNbB; ++j)
#pragma unroll
        for (int r = 0; r < 4; ++r) acc[i][j][r] = 0.f;

    wait_vmcnt<kCphA>();   // A0 and B0 have landed; A1 may be in flight
    __builtin_amdgcn_s_barrier();
#pragma unroll
    for (int j = 0; j < kNbB; ++j) fb[0][j] = load_frag(lds + b_lane, j, 0);
#pragma unroll
    for (int i = 0; i < kNbA; ++i) fa[i] = load_frag(lds + a_lane, i, 0);

    const uint32_t soff_last = soff_of(k_steps - 1);
    uint32_t soff_b = soff_of(1), soff_a = soff_of(2);   // B(t+1) and A(t+2), the copies of k-step t
    uint32_t kt = 0;
    bool last = false;
    for (;;) {
      static_for<2>([&](auto phase) __attribute__((always_inline)) {
        if (last) return;
        constexpr int slot = decltype(phase)::value;
        const uint8_t* a_rows = lds + slot * kAltSlotA + a_lane;          // A(t)
        const uint8_t* a1_rows = lds + (slot ^ 1) * kAltSlotA + a_lane;   // A(t+1)
        const uint8_t* b_rows = lds + b_lane;
        // Second sync point of the k-step: every wave has read the slot of A(t); A(t+1) and B(t+1) have landed.
        auto slots_free = [&]() __attribute__((always_inline)) {
          wait_lgkmcnt0();
          wait_vmcnt<0>();
          __builtin_amdgcn_s_barrier();
        };
        {
          constexpr int kPerSlice = kNbA * kNbB;   // 32
          // ---- slice 0
          constexpr int kSyncB = 2 * kNbB;                    // after row 1: the B slot is free
          static_for<kPerSlice>([&](auto uc) __attribute__((always_inline)) {
            constexpr int u = decltype(uc)::value, i = u / kNbB, j = u % kNbB;
            if constexpr (u < kNbB) fb[1][u] = load_frag(b_rows, u, 1);
            if constexpr (u >= kNbB && j == 1) fa[i - 1] = load_frag(a_rows, i - 1, 1);   // one MFMA after the row's last use
            if constexpr (u == kSyncB) {
              // Every wave holds both slices of B(t) in registers: fb[0] since the previous k-step, fb[1]
              // from the loads above (issued at least four MFMAs ago; the wait also covers the first
              // reload of A, three MFMAs old, so that no LDS wait in this kernel is counted by hand).
              wait_lgkmcnt0();
              __builtin_amdgcn_s_barrier();
            }
            if constexpr (u >= kSyncB && (u - kSyncB) % 2 == 0 && (u - kSyncB) / 2 < kCphB)
              copy_b(rsrc_b, std::integral_constant<int, (u - kSyncB) / 2>{}, soff_b);           // B(t+1)
            G::mfma_inplace(fb[0][j], fa[i], acc[i][j]);
            MI355_FENCE();
          });
          // ---- slice 1 (the last row of A's slice 1 is loaded behind its first MFMA)
          constexpr int kSync = 2 * kNbB;                   // after row 1: the slot of A(t) is free (its last read is 7 MFMAs old)
          static_assert(kSync <= 2 * kNbB, "the first read of A(t+1) follows the sync");
          constexpr int kFirstCopy = kSync + 1, kSpan = kPerSlice - kFirstCopy;
          static_for<kPerSlice>([&](auto uc) __attribute__((always_inline)) {
            constexpr int u = decltype(uc)::value, i = u / kNbB, j = u % kNbB;
            if constexpr (u == 1) fa[kNbA - 1] = load_frag(a_rows, kNbA - 1, 1);
            if constexpr (u == kSync) slots_free();           // ... and A(t+1), B(t+1) have landed
            if constexpr (u > kSync && u <= kSync + kNbB) fb[0][u - kSync - 1] = load_frag(b_rows, u - kSync - 1, 0);   // B(t+1)
            if constexpr (u >= 2 * kNbB && j == 0) fa[i - 2] = load_frag(a1_rows, i - 2, 0);
            static_for<kCphA>([&](auto cc) __attribute__((always_inline)) {
              if constexpr (kFirstCopy + decltype(cc)::value * kSpan / kCphA == u)
                copy_a(rsrc_a, cc, std::integral_constant<int, slot>{}, soff_a);                 // A(t+2)
            });
            G::mfma_inplace(fb[1][j], fa[i], acc[i][j]);
            MI355_FENCE();
          });
          fa[kNbA - 2] = load_frag(a1_rows, kNbA - 2, 0);
          fa[kNbA - 1] = load_frag(a1_rows, kNbA - 1, 0);
          MI355_FENCE();
        }
        soff_b = soff_b + kRowBytes < soff_last ? soff_b + kRowBytes : soff_last;
        soff_a = soff_a + kRowBytes < soff_last ? soff_a + kRowBytes : soff_last;
        ++kt;
        last = kt == k_steps;
      });
      if (last) break;
    }
    // The clamped copies of the last k-steps must have landed, and every wave must be past its last
    // LDS read, before the slots are refilled for the next tile.
    wait_vmcnt<0>();
    wait_lgkmcnt0();
    __builtin_amdgcn_s_barrier();

    const int64_t done_m0 = (int64_t)tile_m * kAltTileM, done_n0 = (int64_t)tile_n * kAltTileN;
    tile += gridDim.x;
    const bool more = tile < total_tiles;
    if (more) {
      tile_coord_t<uint32_t>(tile, tiles_m, tiles_n, &tile_m, &tile_n);
      rsrc_a = panel_a((int64_t)tile_m * kAltTileM);
      rsrc_b = panel_b((int64_t)tile_n * kAltTileN);
      open_tile(rsrc_a, rsrc_b);   // in flight while the finished tile is stored
    }
    epilogue(done_m0, done_n0);
    if (!more) break;
  }
}

template <class T, class OutT>
int launch(const GemmArgs& g, hipStream_t stream) {
  const int64_t tiles = g.tiles_m * g.tiles_n;
  if (tiles >= ((int64_t)1 << 31)) return -1;   // the kernel counts tiles in 32 bits
  const int64_t slots = 2 * (int64_t)compute_units();
  const int64_t blocks = tiles < slots ? tiles : slots;
  if ((g.K * T::kBytes) % kRowBytes == 0)
    hipLaunchKernelGGL((gemm_tn_tile_alternate<T, OutT, false>), dim3((unsigned)blocks), dim3(256), 0, stream, g);
  else
    hipLaunchKernelGGL((gemm_tn_tile_alternate<T, OutT, true>), dim3((unsigned)blocks), dim3(256), 0, stream, g);
  return hipGetLastError() == hipSuccess ? 0 : -1;
}

}  // namespace

int launch_tile_alternate(const GemmArgs& g, int in_dtype, int out_dtype, hipStream_t stream) {
  const bool out_bf16 = out_dtype == 0;
  switch (in_dtype) {
    case 0: return out_bf16 ? launch<BF16, BF16>(g, stream) : launch<BF16, F16>(g, stream);
    case 1: return out_bf16 ? launch<F16, BF16>(g, stream) : launch<F16, F16>(g, stream);
  }
  return -1;
}

}  // namespace mi355
