// "basic" variant: 256x256 output tile, ONE wave group of 4 waves (one per SIMD), each wave owning
// a 128x128 sub-tile (4x4 blocks of 32x32, 256 fp32 accumulator registers per lane).
//
// Two 64 KiB LDS stages; a k-step is 128 bytes of K per row (4 MFMA slices for 16-bit types,
// 2 for fp8).  Everything is software-pipelined inside the wave:
//
//   slice s of k-step t   : MFMAs on register fragments F[s%2], interleaved one-for-two with the
//                           ds_read_b128 of slice s+1 into F[(s+1)%2]
//   before the last slice : lgkmcnt(0) (all my reads of this stage are back), vmcnt(0) (my part
//                           of stage t+1 has landed), s_barrier
//   during the last slice : direct-to-LDS loads of k-step t+2 into the stage just drained, and
//                           the reads of slice 0 of k-step t+1
//
// so there is one workgroup barrier per k-step and the MFMA pipe only idles while that barrier
// resolves.  Counterpart in the reference: the cooperative kernel, kernels/gemm_kernels/sm90a/
// gemm.cuh:246-418 (TMA producer warpgroup + two consumer warpgroups sharing one accumulator
// tile); here every wave is loader and math at once because direct-to-LDS loads need no registers.
#include "cdna4_primitives.h"
#include "gemm_launch.h"
#include "tile_map.h"

namespace mi355 {
namespace {

constexpr int kTile = 256;
constexpr int kRowBytes = 128;
constexpr int kOperandBytes = kTile * kRowBytes;  // 32 KiB
constexpr int kStageBytes = 2 * kOperandBytes;    // A then B
constexpr int kThreads = 256;

__device__ __forceinline__ uint32_t swizzle(uint32_t row) { return (row >> 1) & 7u; }

#define MI355_FENCE() __builtin_amdgcn_sched_barrier(0)
#ifndef MI355_DEBUG_MODE
#define MI355_DEBUG_MODE 0   // 1: no MFMA, 2: no global->LDS copies in the main loop (timing experiments only)
#endif

template <class T, class OutT>
__global__ __launch_bounds__(kThreads, 1) void gemm_tn_tile256_w4(GemmArgs g) {
  // Two separate LDS objects so the compiler can tell copies into one stage from reads of the other.
  __shared__ __attribute__((aligned(1024))) uint8_t stage0[kStageBytes];
  __shared__ __attribute__((aligned(1024))) uint8_t stage1[kStageBytes];
  typedef typename Mfma32<T>::Frag Frag;
  constexpr int kChunksPerSlice = 2 * T::kSliceChunks;  // both lane halves
  constexpr int kSlices = 8 / kChunksPerSlice;

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

  // Copy geometry: one wave instruction moves 8 rows x 128 B.  Wave w issues copies 8w..8w+7 of
  // each operand (rows 64w .. 64w+63).  Lane l fills LDS chunk l%8 of row l/8 with the global
  // chunk (l%8) ^ swizzle(row).  swizzle(row) only depends on the copy's parity and l/16, so two
  // per-lane offsets per operand suffice; the row block advances through the scalar offset.
  const uint32_t r8 = lane >> 3, c8 = lane & 7u;
  uint32_t voff_a[2], voff_b[2];
#pragma unroll
  for (int par = 0; par < 2; ++par) {
    const uint32_t chunk = c8 ^ swizzle(par * 8 + r8);
    voff_a[par] = (wave * 64 + r8) * lda_b + chunk * 16;
    voff_b[par] = (wave * 64 + r8) * ldb_b + chunk * 16;
  }
  const uint32_t a_step = 8 * lda_b, b_step = 8 * ldb_b;

  auto issue_copies = [&](uint8_t* stage, uint32_t kt) __attribute__((always_inline)) {
    const uint32_t koff = kt * kRowBytes;
    uint8_t* dst_a = stage + wave * 8192;
    uint8_t* dst_b = stage + kOperandBytes + wave * 8192;
#pragma unroll
    for (int j = 0; j < 8; ++j)
      dma_16B_to_lds_tracked(dst_a + j * 1024, voff_a[j & 1], rsrc_a, koff + j * a_step);
#pragma unroll
    for (int j = 0; j < 8; ++j)
      dma_16B_to_lds_tracked(dst_b + j * 1024, voff_b[j & 1], rsrc_b, koff + j * b_step);
  };

  const uint32_t r32 = lane & 31u, half = lane >> 5;
  const uint32_t swz = swizzle(r32);
  const uint32_t a_row = (wm * 128 + r32) * kRowBytes;
  const uint32_t b_row = kOperandBytes + (wn * 128 + r32) * kRowBytes;

  // Fragment of 32-row block `blk` of operand rows starting at row_off, slice s.
  auto load_frag = [&](const uint8_t* stage, uint32_t row_off, int blk, int s) __attribute__((always_inline)) -> Frag {
    const uint8_t* p = stage + row_off + blk * 32 * kRowBytes;
    if constexpr (T::kSliceChunks == 1) {
      return *(const i32x4*)(p + (((2u * s + half) ^ swz) << 4));
    } else {
      const uint32_t c = 4u * s + 2u * half;
      i32x4 lo = *(const i32x4*)(p + ((c ^ swz) << 4));
      i32x4 hi = *(const i32x4*)(p + (((c + 1u) ^ swz) << 4));
      return (i32x8){lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
    }
  };

#ifdef MI355_CLOCK_PROBE
  const uint64_t probe_c0 = __builtin_readcyclecounter(), probe_r0 = __builtin_amdgcn_s_memrealtime();
#endif
  f32x16 acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  Frag fa[2][4], fb[2][4];  // double-buffered fragments: [buffer][block]

  // MFMAs of one slice from buffer `cur`, interleaved with loading slice `ns` of `nstage` into the
  // other buffer (8 fragment loads spread over 16 MFMAs).
  auto slice = [&](int cur, const uint8_t* nstage, int ns, bool load_next) __attribute__((always_inline)) {
    const int nxt = cur ^ 1;
#pragma unroll
    for (int q = 0; q < 8; ++q) {
      if (load_next && MI355_DEBUG_MODE < 4) {
        if (q < 4) fb[nxt][q] = load_frag(nstage, b_row, q, ns);
        else fa[nxt][q - 4] = load_frag(nstage, a_row, q - 4, ns);
      }
      // two MFMAs per step: blocks (i, j) in an order that touches each accumulator once
      const int i = q >> 1, j0 = (q & 1) * 2;
#if MI355_DEBUG_MODE == 1
      acc[i][j0][0] += __builtin_bit_cast(float, fb[cur][j0][0] ^ fa[cur][i][0]);
      acc[i][j0 + 1][0] += __builtin_bit_cast(float, fb[cur][j0 + 1][1] ^ fa[cur][i][1]);
#else
      acc[i][j0] = Mfma32<T>::run(fb[cur][j0], fa[cur][i], acc[i][j0]);
      acc[i][j0 + 1] = Mfma32<T>::run(fb[cur][j0 + 1], fa[cur][i], acc[i][j0 + 1]);
#endif
      MI355_FENCE();
    }
  };

  const uint32_t k_steps = k_bytes / kRowBytes;

  // One k-step on stage `cur_stage`; fragments of its slice 0 are already in buffer 0.
  auto kstep = [&](uint8_t* cur_stage, uint8_t* other_stage, uint32_t kt, bool copy_next2, bool read_next) __attribute__((always_inline)) {
#pragma unroll
    for (int s = 0; s < kSlices - 1; ++s) slice(s & 1, cur_stage, s + 1, true);
    // All my reads of cur_stage are issued; they must be back, and my copies into other_stage
    // landed, before anyone overwrites cur_stage or reads other_stage.
    wait_lgkmcnt0();
    if (read_next) {
      wait_vmcnt<0>();
#if MI355_DEBUG_MODE < 3
      __builtin_amdgcn_s_barrier();
#endif
    }
    MI355_FENCE();
#if MI355_DEBUG_MODE < 2
    if (copy_next2) issue_copies(cur_stage, kt + 2);
#endif
    MI355_FENCE();
    slice((kSlices - 1) & 1, other_stage, 0, read_next);
  };

  if (k_steps > 0) {
    issue_copies(stage0, 0);
    if (k_steps > 1) {
      issue_copies(stage1, 1);
      wait_vmcnt<16>();
    } else {
      wait_vmcnt<0>();
    }
    __builtin_amdgcn_s_barrier();
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      fb[0][q] = load_frag(stage0, b_row, q, 0);
      fa[0][q] = load_frag(stage0, a_row, q, 0);
    }
    static_assert(kSlices % 2 == 0, "slice 0 of the next k-step must land in fragment buffer 0");
    uint32_t kt = 0;
    for (; kt + 3 < k_steps; kt += 2) {
      kstep(stage0, stage1, kt, true, true);
      kstep(stage1, stage0, kt + 1, true, true);
    }
    const uint32_t rem = k_steps - kt;
    if (rem == 3) {
      kstep(stage0, stage1, kt, true, true);
      kstep(stage1, stage0, kt + 1, false, true);
      kstep(stage0, stage1, kt + 2, false, false);
    } else if (rem == 2) {
      kstep(stage0, stage1, kt, false, true);
      kstep(stage1, stage0, kt + 1, false, false);
    } else {
      kstep(stage0, stage1, kt, false, false);
    }
  }

#ifdef MI355_CLOCK_PROBE
  const uint64_t probe_c1 = __builtin_readcyclecounter(), probe_r1 = __builtin_amdgcn_s_memrealtime();
#endif
  // Epilogue: acc[i][j][4q+e] of lane l is C[m][n], m = m0 + wm*128 + i*32 + l%32,
  // n = n0 + wn*128 + j*32 + 8q + 4*(l/32) + e.
  const float scale = g.scale;
  const int64_t ldc = g.ldc;
  uint16_t* C = (uint16_t*)g.C;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int64_t m = m0 + wm * 128 + i * 32 + r32;
    if (m >= g.M) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int64_t n = n0 + wn * 128 + j * 32 + q * 8 + half * 4;
        if (n < g.N) {
          u32x2 v = Pack4<OutT>::run(acc[i][j][4 * q] * scale, acc[i][j][4 * q + 1] * scale,
                                     acc[i][j][4 * q + 2] * scale, acc[i][j][4 * q + 3] * scale);
          *(u32x2*)(C + m * ldc + n) = v;
        }
      }
    }
  }
#ifdef MI355_CLOCK_PROBE
  // Timing experiments only: the last block overwrites the start of C with cycle counts.
  __builtin_amdgcn_s_barrier();
  if (blockIdx.x == gridDim.x - 1 && tid == 0) {
    ((uint64_t*)g.C)[0] = probe_c1 - probe_c0;
    ((uint64_t*)g.C)[1] = probe_r1 - probe_r0;
  }
#endif
}

template <class T, class OutT>
int launch(const GemmArgs& g, hipStream_t stream) {
  const int64_t blocks = g.tiles_m * g.tiles_n;
  hipLaunchKernelGGL((gemm_tn_tile256_w4<T, OutT>), dim3((unsigned)blocks), dim3(kThreads), 0, stream, g);
  return hipGetLastError() == hipSuccess ? 0 : -1;
}

}  // namespace

int launch_tile256_w4(const GemmArgs& g, int in_dtype, int out_dtype, hipStream_t stream) {
  const bool out_bf16 = out_dtype == 0;
  switch (in_dtype) {
    case 0: return out_bf16 ? launch<BF16, BF16>(g, stream) : launch<BF16, F16>(g, stream);
    case 1: return out_bf16 ? launch<F16, BF16>(g, stream) : launch<F16, F16>(g, stream);
    case 2: return out_bf16 ? launch<E4M3, BF16>(g, stream) : launch<E4M3, F16>(g, stream);
  }
  return -1;
}

}  // namespace mi355
