// "basic" variant: 256x256 output tile, ONE wave group of 4 waves (one per SIMD), each wave owning
// a 128x128 sub-tile held in 256 fp32 accumulator registers per lane.
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
// One workgroup barrier per k-step; the loop body is branch-free (loads past the end of K re-read the
// last k-step into a slot nobody reads).
//
// MFMA shape: bf16/fp16 use v_mfma_f32_16x16x32 (8x8 blocks per wave); on random data it sustains
// a higher clock under the board power limit than 32x32x16.  fp8 uses v_mfma_f32_32x32x64_f8f6f4
// (4x4 blocks), which keeps the fragment registers within budget.
//
// Counterpart in the reference: the cooperative kernel, kernels/gemm_kernels/sm90a/gemm.cuh:246-418
// (TMA producer warpgroup, mbarrier full/empty ring of 3 stages, two consumer warpgroups); here
// every wave is loader and math at once because direct-to-LDS loads need no registers.
#include "cdna4_primitives.h"
#include "gemm_launch.h"
#include "tile_map.h"

namespace mi355 {
namespace {

constexpr int kTile = 256;
constexpr int kRowBytes = 128;
constexpr int kSlotBytes = kTile * kRowBytes;  // 32 KiB: one operand, one k-step
constexpr int kSlots = 5;
constexpr int kThreads = 256;

__device__ __forceinline__ uint32_t swizzle(uint32_t row) { return (row >> 1) & 7u; }

#define MI355_FENCE() __builtin_amdgcn_sched_barrier(0)
#ifndef MI355_DEBUG_MODE
// Timing experiments only (results are wrong when non-zero):
//   1 no MFMA, 2 no copies in the main loop, 3 = 2 + no barrier, 4 = 3 + no LDS reads, 5 no LDS reads only
#define MI355_DEBUG_MODE 0
#endif

// Per-dtype MFMA geometry.
//   kBlk      rows (and columns) of one MFMA block
//   kGroups   lane groups of kBlk lanes; group g feeds k-chunks g*kCpl .. g*kCpl+kCpl-1 of a slice
//   kCpl      16-byte chunks per lane per MFMA
template <class T> struct Geo;
template <> struct Geo<BF16> {
  static constexpr int kBlk = 16, kGroups = 4, kCpl = 1;
  typedef i32x4 Frag;
  typedef f32x4 Acc;
  static __device__ __forceinline__ Acc mfma(Frag x, Frag y, Acc c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, x),
                                                   __builtin_bit_cast(bf16x8, y), c, 0, 0, 0);
  }
};
template <> struct Geo<F16> {
  static constexpr int kBlk = 16, kGroups = 4, kCpl = 1;
  typedef i32x4 Frag;
  typedef f32x4 Acc;
  static __device__ __forceinline__ Acc mfma(Frag x, Frag y, Acc c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, x),
                                                  __builtin_bit_cast(f16x8, y), c, 0, 0, 0);
  }
};
template <> struct Geo<E4M3> {
  static constexpr int kBlk = 32, kGroups = 2, kCpl = 2;
  typedef i32x8 Frag;
  typedef f32x16 Acc;
  static __device__ __forceinline__ Acc mfma(Frag x, Frag y, Acc c) {
    return __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(x, y, c, 0, 0, 0, 0, 0, 0);
  }
};

template <class T, class OutT>
__global__ __launch_bounds__(kThreads, 1) void gemm_tn_tile256_ring(GemmArgs g) {
  __shared__ __attribute__((aligned(1024))) uint8_t ring[kSlots * kSlotBytes];
  typedef Geo<T> G;
  typedef typename G::Frag Frag;
  typedef typename G::Acc Acc;
  constexpr int kBlk = G::kBlk;
  constexpr int kNb = 128 / kBlk;                       // blocks per wave per dimension
  constexpr int kSliceChunks = G::kGroups * G::kCpl;    // chunks of a row consumed per slice
  constexpr int kSlices = 8 / kSliceChunks;
  constexpr int kAccLen = kBlk * kBlk / 64;
  constexpr int kMfmaPerSlice = kNb * kNb;
  constexpr int kReadsPerSlice = 2 * kNb;               // fragment loads (each kCpl ds_read_b128)
  static_assert(kSlices == 2, "the schedule below assumes two slices per k-step");

  const uint32_t tid = threadIdx.x;
  const uint32_t lane = tid & 63u;
  const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const uint32_t wm = wave >> 1, wn = wave & 1u;

  int64_t tile_m, tile_n;
  tile_coord(blockIdx.x, g.tiles_m, g.tiles_n, &tile_m, &tile_n);
  const int64_t m0 = tile_m * kTile, n0 = tile_n * kTile;

  const uint32_t lda_b = (uint32_t)(g.lda * T::kBytes), ldb_b = (uint32_t)(g.ldb * T::kBytes);
  const uint32_t k_bytes = (uint32_t)(g.K * T::kBytes);
  const int64_t rows_a = g.M - m0 < kTile ? g.M - m0 : kTile;
  const int64_t rows_b = g.N - n0 < kTile ? g.N - n0 : kTile;
  const __amdgpu_buffer_rsrc_t rsrc_a = make_raw_buffer(
      (const uint8_t*)g.A + m0 * (int64_t)lda_b, (uint32_t)((rows_a - 1) * lda_b + k_bytes));
  const __amdgpu_buffer_rsrc_t rsrc_b = make_raw_buffer(
      (const uint8_t*)g.B + n0 * (int64_t)ldb_b, (uint32_t)((rows_b - 1) * ldb_b + k_bytes));
  const uint32_t k_steps = __builtin_amdgcn_readfirstlane(k_bytes / kRowBytes);

  // Copy geometry: one wave instruction moves 8 rows x 128 B.  Wave w issues copies 8w..8w+7 of
  // an operand (rows 64w .. 64w+63).  Lane l fills LDS chunk l%8 of row l/8 with the global
  // chunk (l%8) ^ swizzle(row); swizzle(row) depends only on the copy's parity and l/16, so two
  // per-lane offsets per operand suffice; copy j adds j*8 rows to them.
  const uint32_t r8 = lane >> 3, c8 = lane & 7u;
  uint32_t voff_a[2], voff_b[2];
#pragma unroll
  for (int par = 0; par < 2; ++par) {
    const uint32_t chunk = c8 ^ swizzle(par * 8 + r8);
    voff_a[par] = (wave * 64 + r8) * lda_b + chunk * 16;
    voff_b[par] = (wave * 64 + r8) * ldb_b + chunk * 16;
  }
  const uint32_t a_step = __builtin_amdgcn_readfirstlane(8 * lda_b);
  const uint32_t b_step = __builtin_amdgcn_readfirstlane(8 * ldb_b);
  const uint32_t ring0 = __builtin_amdgcn_readfirstlane(lds_address(ring));
  const uint32_t dma_wave = ring0 + wave * 8192;  // this wave's 8 KiB inside a slot

  // Copy j (0..7) of an operand's k-step kt into slot `slot`.  The row part of the address stays
  // in the vector offset, the only part the hardware range-checks against the descriptor (rows
  // past the edge of the matrix read zeros); the scalar offset carries the k-step and is kept
  // inside the row by re-reading the last k-step for kt past the end (the slot is never used).
  auto copy_a = [&](int j, uint32_t slot, uint32_t kt) __attribute__((always_inline)) {
    const uint32_t soff = (kt < k_steps ? kt : k_steps - 1) * kRowBytes;
    dma_16B_to_lds(dma_wave + slot * kSlotBytes + j * 1024, voff_a[j & 1] + j * a_step, rsrc_a, soff);
  };
  auto copy_b = [&](int j, uint32_t slot, uint32_t kt) __attribute__((always_inline)) {
    const uint32_t soff = (kt < k_steps ? kt : k_steps - 1) * kRowBytes;
    dma_16B_to_lds(dma_wave + slot * kSlotBytes + j * 1024, voff_b[j & 1] + j * b_step, rsrc_b, soff);
  };

  // Fragment geometry: lane l supplies row l%kBlk of a block; group l/kBlk picks the chunks.
  const uint32_t rblk = lane & (kBlk - 1), grp = lane / kBlk;
  const uint32_t swz = swizzle(rblk);  // block bases are multiples of 16 rows
  const uint32_t a_lane = (wm * 128 + rblk) * kRowBytes;
  const uint32_t b_lane = (wn * 128 + rblk) * kRowBytes;
  // Byte offset inside a row of the e-th chunk this lane reads in slice s.
  auto chunk_off = [&](int s, int e) __attribute__((always_inline)) -> uint32_t {
    return ((uint32_t)(s * kSliceChunks + grp * G::kCpl + e) ^ swz) << 4;
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

#ifdef MI355_CLOCK_PROBE
  const uint64_t probe_c0 = __builtin_readcyclecounter(), probe_r0 = __builtin_amdgcn_s_memrealtime();
  uint64_t probe_r_loop = 0;
#endif
  Acc acc[kNb][kNb];
#pragma unroll
  for (int i = 0; i < kNb; ++i)
#pragma unroll
    for (int j = 0; j < kNb; ++j)
#pragma unroll
      for (int r = 0; r < kAccLen; ++r) acc[i][j][r] = 0.f;

  Frag fa[2][kNb], fb[2][kNb];  // [fragment buffer][block]

  // Load number q (0..kReadsPerSlice-1) of a slice: B blocks first (every MFMA row needs them all).
  auto read_q = [&](int buf, int q, const uint8_t* a_rows, const uint8_t* b_rows, int s)
      __attribute__((always_inline)) {
    if (MI355_DEBUG_MODE >= 4) return;
    if (q < kNb) fb[buf][q] = load_frag(b_rows, q, s);
    else fa[buf][q - kNb] = load_frag(a_rows, q - kNb, s);
  };
  auto mfma_u = [&](int buf, int u) __attribute__((always_inline)) {
    const int i = u / kNb, j = u % kNb;
    // B supplies the MFMA "rows" so each lane ends up with consecutive n of one m.
#if MI355_DEBUG_MODE == 1
    acc[i][j][0] += __builtin_bit_cast(float, fb[buf][j][0] ^ fa[buf][i][0]);
#else
    acc[i][j] = G::mfma(fb[buf][j], fa[buf][i], acc[i][j]);
#endif
  };

  // Prologue: A0 B0 A1 B1 A2 into slots 0..4.
#pragma unroll
  for (int j = 0; j < 8; ++j) copy_a(j, 0, 0);
#pragma unroll
  for (int j = 0; j < 8; ++j) copy_b(j, 1, 0);
#pragma unroll
  for (int j = 0; j < 8; ++j) copy_a(j, 2, 1);
#pragma unroll
  for (int j = 0; j < 8; ++j) copy_b(j, 3, 1);
#pragma unroll
  for (int j = 0; j < 8; ++j) copy_a(j, 4, 2);
  wait_vmcnt<24>();  // A0 and B0 have landed
  __builtin_amdgcn_s_barrier();
#pragma unroll
  for (int q = 0; q < kReadsPerSlice; ++q)
    read_q(0, q, ring + a_lane, ring + kSlotBytes + b_lane, 0);

#ifdef MI355_CLOCK_PROBE
  probe_r_loop = __builtin_amdgcn_s_memrealtime();
#endif
  uint32_t slot_a = 0;  // slot of A(t); B(t) is in slot_a+1, A(t+1) in slot_a+2, B(t+1) in slot_a+3 (mod 5)
  for (uint32_t kt = 0; kt < k_steps; ++kt) {
    const uint32_t slot_b = slot_a + 1 >= kSlots ? slot_a + 1 - kSlots : slot_a + 1;
    const uint32_t slot_a1 = slot_a + 2 >= kSlots ? slot_a + 2 - kSlots : slot_a + 2;
    const uint32_t slot_b1 = slot_a + 3 >= kSlots ? slot_a + 3 - kSlots : slot_a + 3;
    const uint8_t* a_rows = ring + slot_a * kSlotBytes + a_lane;
    const uint8_t* b_rows = ring + slot_b * kSlotBytes + b_lane;
    const uint8_t* a1_rows = ring + slot_a1 * kSlotBytes + a_lane;
    const uint8_t* b1_rows = ring + slot_b1 * kSlotBytes + b_lane;

    // Event schedule of one k-step, in MFMA positions p = slice * kMfmaPerSlice + u:
    //   reads    one fragment load per MFMA at the start of each slice (for the following slice)
    //   barrier  in slice 0, a few MFMAs after the last read so its data is back
    //   copies   one every kCopyEvery MFMAs after the barrier, B(t+2) first.  They must not be
    //            issued faster than the texture-address unit retires them (one 1 KiB copy takes
    //            it ~23 cycles and it serves all four waves): a wave whose copy finds the unit's
    //            queue full stalls at issue and its MFMA stream stops with it.
    constexpr int kBarrierAt = kReadsPerSlice + kMfmaPerSlice / 8;
    constexpr int kFirstCopy = kBarrierAt + 1;
    constexpr int kCopyEvery = (2 * kMfmaPerSlice - kFirstCopy) / 16 > 0 ? (2 * kMfmaPerSlice - kFirstCopy) / 16 : 1;
    static_assert(kFirstCopy + 15 * kCopyEvery < 2 * kMfmaPerSlice, "copies must fit in the k-step");
#pragma unroll
    for (int s = 0; s < 2; ++s) {
#pragma unroll
      for (int u = 0; u < kMfmaPerSlice; ++u) {
        const int p = s * kMfmaPerSlice + u;
        if (u < kReadsPerSlice) {
          if (s == 0) read_q(1, u, a_rows, b_rows, 1);        // slice 1 of this k-step
          else read_q(0, u, a1_rows, b1_rows, 0);            // slice 0 of the next k-step
        }
        if (s == 0 && u == kBarrierAt) {
          // My reads of this k-step's slots are back; B(t+1) (and A(t+1) before it) have landed;
          // only the 8 copies of A(t+2) may still be in flight.
          wait_lgkmcnt0();
          wait_vmcnt<8>();
          if (MI355_DEBUG_MODE != 3 && MI355_DEBUG_MODE != 4) __builtin_amdgcn_s_barrier();
        }
        if (p >= kFirstCopy && (p - kFirstCopy) % kCopyEvery == 0 && (p - kFirstCopy) / kCopyEvery < 16 &&
            (MI355_DEBUG_MODE < 2 || MI355_DEBUG_MODE == 5)) {
          const int c = (p - kFirstCopy) / kCopyEvery;
          if (c < 8) copy_b(c, slot_a, kt + 2);
          else copy_a(c - 8, slot_b, kt + 3);
        }
        mfma_u(s, u);
        MI355_FENCE();
      }
    }
    slot_a = slot_a1;
  }
  wait_vmcnt<0>();  // drain the unused tail copies before the wave ends
#ifdef MI355_CLOCK_PROBE
  const uint64_t probe_c1 = __builtin_readcyclecounter(), probe_r1 = __builtin_amdgcn_s_memrealtime();
#endif

  // Epilogue.  Accumulator register 4q+e of block (i,j) in lane l is C[m][n] with
  //   m = m0 + wm*128 + i*kBlk + l%kBlk,   n = n0 + wn*128 + j*kBlk + q*4*kGroups + 4*(l/kBlk) + e.
  const float scale = g.scale;
  const int64_t ldc = g.ldc;
  uint16_t* C = (uint16_t*)g.C;
#pragma unroll
  for (int i = 0; i < kNb; ++i) {
    const int64_t m = m0 + wm * 128 + i * kBlk + rblk;
    if (m >= g.M) continue;
#pragma unroll
    for (int j = 0; j < kNb; ++j) {
#pragma unroll
      for (int q = 0; q < kAccLen / 4; ++q) {
        const int64_t n = n0 + wn * 128 + j * kBlk + q * 4 * G::kGroups + grp * 4;
        if (n < g.N) {
          u32x2 v = Pack4<OutT>::run(acc[i][j][4 * q] * scale, acc[i][j][4 * q + 1] * scale,
                                     acc[i][j][4 * q + 2] * scale, acc[i][j][4 * q + 3] * scale);
          *(u32x2*)(C + m * ldc + n) = v;
        }
      }
    }
  }
#ifdef MI355_CLOCK_PROBE
  // Timing experiments only: every block overwrites 64 bytes of C with time stamps.
  __builtin_amdgcn_s_barrier();
  if (tid == 0) {
    uint64_t* rec = (uint64_t*)g.C + 8 * (uint64_t)blockIdx.x;
    rec[0] = probe_c1 - probe_c0;
    rec[1] = probe_r1 - probe_r0;
    rec[2] = probe_r0;
    rec[3] = probe_r_loop;
    rec[4] = probe_r1;
    rec[5] = __builtin_amdgcn_s_memrealtime();
    rec[6] = __builtin_amdgcn_s_getreg((4 << 0) | (0 << 6) | (31 << 11));   // HW_ID
    rec[7] = __builtin_amdgcn_s_getreg((20 << 0) | (0 << 6) | (31 << 11));  // XCC_ID
  }
#endif
}

template <class T, class OutT>
int launch(const GemmArgs& g, hipStream_t stream) {
  const int64_t blocks = g.tiles_m * g.tiles_n;
  hipLaunchKernelGGL((gemm_tn_tile256_ring<T, OutT>), dim3((unsigned)blocks), dim3(kThreads), 0, stream, g);
  return hipGetLastError() == hipSuccess ? 0 : -1;
}

}  // namespace

int launch_tile256_ring(const GemmArgs& g, int in_dtype, int out_dtype, hipStream_t stream) {
  const bool out_bf16 = out_dtype == 0;
  switch (in_dtype) {
    case 0: return out_bf16 ? launch<BF16, BF16>(g, stream) : launch<BF16, F16>(g, stream);
    case 1: return out_bf16 ? launch<F16, BF16>(g, stream) : launch<F16, F16>(g, stream);
    case 2: return out_bf16 ? launch<E4M3, BF16>(g, stream) : launch<E4M3, F16>(g, stream);
  }
  return -1;
}

}  // namespace mi355
