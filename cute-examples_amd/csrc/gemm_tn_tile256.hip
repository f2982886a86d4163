// 256x256 output tile GEMM for gfx950: C = scale * A · B^T, A (M,K) and B (N,K) K-contiguous.
//
// One workgroup of 8 waves owns one 256x256 tile of C.  Per k-step it consumes 128 bytes of K
// from each of the 256 A rows and 256 B rows (64 bf16/fp16 elements or 128 fp8 elements):
//
//   global --(buffer_load ... lds, 16 B per lane, no VGPR round trip)--> LDS stage (64 KiB)
//   LDS --(ds_read_b128)--> MFMA operand registers --(v_mfma_f32_32x32x*)--> fp32 accumulators
//
// LDS holds two stages; the loads of k-step t+1 are in flight while k-step t is multiplied.
// Wave w computes the 128x64 sub-tile (w/4, w%4) as 4x2 blocks of 32x32.
//
// Role in the reference: this file is the counterpart of the device kernels
// kernels/gemm_kernels/sm90a/gemm.cuh:246-418 (cooperative mainloop + epilogue) and
// gemm_pingpong.cuh:121-349 (ping-pong), with TMA + mbarrier pipelines replaced by
// direct-to-LDS loads ordered with vmcnt waits and workgroup barriers.
#include "cdna4_primitives.h"
#include "gemm_launch.h"
#include "tile_map.h"

namespace mi355 {

namespace {

constexpr int kTile = 256;                          // rows of A and of B per workgroup
constexpr int kRowBytes = 128;                      // bytes of K per row per k-step
constexpr int kOperandBytes = kTile * kRowBytes;    // 32 KiB
constexpr int kStageBytes = 2 * kOperandBytes;      // A then B
constexpr int kStages = 2;
constexpr int kThreads = 512;

// 16-byte chunk c of LDS row r is stored at chunk position c ^ swizzle(r).  With 128-byte rows
// two consecutive rows span all 64 banks, so (r >> 1) & 7 makes any 16 consecutive rows read at
// one logical chunk hit 16 different 16-byte bank groups.
__device__ __forceinline__ uint32_t swizzle(uint32_t row) { return (row >> 1) & 7u; }

template <class T>
struct FragLoader {
  typedef typename Mfma32<T>::Frag Frag;
  // Slices per k-step: 4 for 16-bit elements (2 chunks per slice), 2 for fp8 (4 chunks).
  static constexpr int kSlices = 8 / (2 * T::kSliceChunks);
  // Logical chunk(s) lane-half h feeds into slice s.
  static __device__ __forceinline__ Frag load(const uint8_t* row_ptr, uint32_t swz, int s, uint32_t h) {
    if constexpr (T::kSliceChunks == 1) {
      const uint32_t c = 2u * s + h;
      return *(const i32x4*)(row_ptr + ((c ^ swz) << 4));
    } else {
      const uint32_t c = 4u * s + 2u * h;
      i32x4 lo = *(const i32x4*)(row_ptr + ((c ^ swz) << 4));
      i32x4 hi = *(const i32x4*)(row_ptr + (((c + 1u) ^ swz) << 4));
      return (i32x8){lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
    }
  }
};

template <class T, class OutT>
__global__ __launch_bounds__(kThreads, 1) void gemm_tn_tile256_basic(GemmArgs g) {
  __shared__ __attribute__((aligned(1024))) uint8_t lds[kStages * kStageBytes];
  typedef typename Mfma32<T>::Frag Frag;
  constexpr int kSlices = FragLoader<T>::kSlices;

  const uint32_t tid = threadIdx.x;
  const uint32_t lane = tid & 63u;
  const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const uint32_t wm = wave >> 2, wn = wave & 3u;

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

  // Global->LDS copy geometry: one wave instruction moves 8 rows x 128 B; wave w issues copies
  // 4w..4w+3 of each operand per k-step.  Lane l fills LDS chunk l%8 of row l/8, which must hold
  // logical chunk (l%8) ^ swizzle(row), so that is the global chunk it fetches.
  const uint32_t r8 = lane >> 3, c8 = lane & 7u;
  uint32_t voff_a[4], voff_b[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const uint32_t row = (wave * 4 + j) * 8 + r8;
    const uint32_t chunk = c8 ^ swizzle(row);
    voff_a[j] = row * lda_b + chunk * 16;
    voff_b[j] = row * ldb_b + chunk * 16;
  }
  const uint32_t lds0 = lds_address(lds);
  const uint32_t dma_dst = lds0 + wave * 4096;  // 4 copies x 1 KiB per wave per operand

  auto issue_loads = [&](int stage, uint32_t kt) {
    const uint32_t soff = kt * kRowBytes;
    const uint32_t dst = dma_dst + stage * kStageBytes;
#pragma unroll
    for (int j = 0; j < 4; ++j) dma_16B_to_lds(dst + j * 1024, voff_a[j], rsrc_a, soff);
#pragma unroll
    for (int j = 0; j < 4; ++j) dma_16B_to_lds(dst + kOperandBytes + j * 1024, voff_b[j], rsrc_b, soff);
  };

  // MFMA operand geometry: lane l supplies row l%32 of a 32-row block; lane half l/32 selects
  // which chunks of the slice.
  const uint32_t r32 = lane & 31u, half = lane >> 5;
  const uint32_t swz = swizzle(r32);  // block bases are multiples of 32, so only r32 matters
  const uint8_t* a_rows = lds + (wm * 128 + r32) * kRowBytes;
  const uint8_t* b_rows = lds + kOperandBytes + (wn * 64 + r32) * kRowBytes;

  f32x16 acc[4][2];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  const uint32_t k_steps = (k_bytes + kRowBytes - 1) / kRowBytes;

  auto multiply_stage = [&](int stage) {
    const uint8_t* a_st = a_rows + stage * kStageBytes;
    const uint8_t* b_st = b_rows + stage * kStageBytes;
#pragma unroll
    for (int s = 0; s < kSlices; ++s) {
      Frag af[4], bf[2];
#pragma unroll
      for (int i = 0; i < 4; ++i) af[i] = FragLoader<T>::load(a_st + i * 32 * kRowBytes, swz, s, half);
#pragma unroll
      for (int j = 0; j < 2; ++j) bf[j] = FragLoader<T>::load(b_st + j * 32 * kRowBytes, swz, s, half);
      // B supplies the MFMA "rows" so that each lane ends up with 4 consecutive n of one m.
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) acc[i][j] = Mfma32<T>::run(bf[j], af[i], acc[i][j]);
    }
  };

  issue_loads(0, 0);
  for (uint32_t kt = 0; kt < k_steps; kt += 2) {
    wait_vmcnt<0>();
    __builtin_amdgcn_s_barrier();
    if (kt + 1 < k_steps) issue_loads(1, kt + 1);
    multiply_stage(0);
    if (kt + 1 < k_steps) {
      wait_vmcnt<0>();
      __builtin_amdgcn_s_barrier();
      if (kt + 2 < k_steps) issue_loads(0, kt + 2);
      multiply_stage(1);
    }
  }

  // Epilogue.  acc[i][j][4q+e] of lane l is C[m][n] with m = m0 + wm*128 + i*32 + l%32 and
  // n = n0 + wn*64 + j*32 + 8q + 4*(l/32) + e: four consecutive n per lane -> one 8-byte store.
  const float scale = g.scale;
  const int64_t ldc = g.ldc;
  uint16_t* C = (uint16_t*)g.C;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int64_t m = m0 + wm * 128 + i * 32 + r32;
    if (m >= g.M) continue;
#pragma unroll
    for (int j = 0; j < 2; ++j) {
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int64_t n = n0 + wn * 64 + j * 32 + q * 8 + half * 4;
        if (n < g.N) {
          u32x2 v = Pack4<OutT>::run(acc[i][j][4 * q] * scale, acc[i][j][4 * q + 1] * scale,
                                     acc[i][j][4 * q + 2] * scale, acc[i][j][4 * q + 3] * scale);
          *(u32x2*)(C + m * ldc + n) = v;
        }
      }
    }
  }
}

template <class T, class OutT>
int launch_basic(const GemmArgs& g, hipStream_t stream) {
  const int64_t blocks = g.tiles_m * g.tiles_n;
  hipLaunchKernelGGL((gemm_tn_tile256_basic<T, OutT>), dim3((unsigned)blocks), dim3(kThreads), 0,
                     stream, g);
  return hipGetLastError() == hipSuccess ? 0 : -1;
}

}  // namespace

int launch_tile256(const GemmArgs& g, int in_dtype, int out_dtype, bool pingpong, hipStream_t stream) {
  (void)pingpong;
  const bool out_bf16 = out_dtype == 0;
  switch (in_dtype) {
    case 0: return out_bf16 ? launch_basic<BF16, BF16>(g, stream) : launch_basic<BF16, F16>(g, stream);
    case 1: return out_bf16 ? launch_basic<F16, BF16>(g, stream) : launch_basic<F16, F16>(g, stream);
    case 2: return out_bf16 ? launch_basic<E4M3, BF16>(g, stream) : launch_basic<E4M3, F16>(g, stream);
  }
  return -1;
}

}  // namespace mi355
