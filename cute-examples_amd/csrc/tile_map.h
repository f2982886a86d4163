// Workgroup id -> output tile, shared by host (tests, C ABI) and device code.
//
// The reference walks tiles in groups of 16 M-blocks so that co-resident CTAs reuse operand
// panels in L2 (Scheduler::get_swizzled_block_idx, kernels/gemm_kernels/sm90a/gemm.cuh:184-197).
// MI355X has 8 XCDs, each with a private L2, and hands consecutive workgroup ids to the XCDs
// round-robin.  The map below first undoes that round-robin, so every XCD owns one contiguous
// range of logical tile ids, and then walks each range in bands of kGroupM tile rows, M fastest,
// so the ~32 workgroups resident on an XCD cover a compact kGroupM x 4 patch of C and share
// A/B panels through that XCD's L2.  It is a bijection from [0, tiles_m*tiles_n) onto the grid.
#pragma once
#include <stdint.h>

#if defined(__HIPCC__)
#define MI355_HD __host__ __device__ __forceinline__
#else
#define MI355_HD inline
#endif

namespace mi355 {

constexpr int kNumXcd = 8;
constexpr int kGroupM = 8;

MI355_HD int64_t xcd_contiguous_id(int64_t block, int64_t total) {
  // XCD x receives blocks x, x+8, x+16, ...: the first (total % 8) XCDs get one more block.
  const int64_t per = (total + kNumXcd - 1) / kNumXcd;
  const int64_t tall = total % kNumXcd == 0 ? kNumXcd : total % kNumXcd;
  const int64_t xcd = block % kNumXcd;
  const int64_t local = block / kNumXcd;
  if (xcd < tall) return xcd * per + local;
  return tall * per + (xcd - tall) * (per - 1) + local;
}

MI355_HD void tile_coord(int64_t block, int64_t tiles_m, int64_t tiles_n,
                         int64_t* tile_m, int64_t* tile_n) {
  const int64_t p = xcd_contiguous_id(block, tiles_m * tiles_n);
  const int64_t band_size = (int64_t)kGroupM * tiles_n;
  const int64_t band = p / band_size;
  const int64_t in_band = p % band_size;
  const int64_t first_m = band * kGroupM;
  const int64_t rows = tiles_m - first_m < kGroupM ? tiles_m - first_m : kGroupM;
  *tile_m = first_m + in_band % rows;
  *tile_n = in_band / rows;
}

}  // namespace mi355
