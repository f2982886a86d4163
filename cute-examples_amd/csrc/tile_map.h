// Workgroup id -> output tile, shared by host (tests, C ABI) and device code.
//
// The reference walks tiles in groups of 16 M-blocks so that co-resident CTAs reuse operand
// panels in L2 (Scheduler::get_swizzled_block_idx, kernels/gemm_kernels/sm90a/gemm.cuh:184-197).
// MI355X has 8 XCDs, each with a private L2, and hands consecutive workgroup ids to the XCDs
// round-robin.  The map below first undoes that round-robin, so every XCD owns one contiguous
// range of logical tile ids, and then walks each range in bands of kGroupM tile rows, M fastest,
// so the ~32 workgroups resident on an XCD cover a compact kGroupM x 8 patch of C and share
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
// Patch of an XCD's 32 resident workgroups: kGroupM tile rows by 32 / kGroupM tile columns.  4 x 8 and
// 8 x 4 touch the same number of operand panels (12), yet 4 rows measured 7 % fewer bytes fetched by
// the L2s (FETCH_SIZE at bf16 8192^3: 787 against 844 GiB/1024 per launch) and 0.3-2.6 % less time on
// nine of ten large bf16 shapes (4096^3: 1496 against 1458 TFLOP/s); 16 rows fetched 67 % more.  A
// map that also packs the eight XCDs' patches into one 16 x 16 square of tiles per round measured
// the same as 4 rows.
constexpr int kGroupM = 4;

// I is int64_t on the host and uint32_t in kernels (the launchers refuse grids of 2^31 tiles or
// more), where 64-bit division would cost thousands of cycles per tile.
template <class I>
MI355_HD I xcd_contiguous_id_t(I block, I total) {
  // XCD x receives blocks x, x+8, x+16, ...: the first (total % 8) XCDs get one more block.
  const I per = (total + kNumXcd - 1) / kNumXcd;
  const I tall = total % kNumXcd == 0 ? (I)kNumXcd : total % kNumXcd;
  const I xcd = block % kNumXcd;
  const I local = block / kNumXcd;
  if (xcd < tall) return xcd * per + local;
  return tall * per + (xcd - tall) * (per - 1) + local;
}

template <class I>
MI355_HD void tile_coord_t(I block, I tiles_m, I tiles_n, I* tile_m, I* tile_n) {
  const I p = xcd_contiguous_id_t<I>(block, tiles_m * tiles_n);
  const I band_size = (I)kGroupM * tiles_n;
  const I band = p / band_size;
  const I in_band = p % band_size;
  const I first_m = band * kGroupM;
  const I rows = tiles_m - first_m < (I)kGroupM ? tiles_m - first_m : (I)kGroupM;
  *tile_m = first_m + in_band % rows;
  *tile_n = in_band / rows;
}

MI355_HD int64_t xcd_contiguous_id(int64_t block, int64_t total) {
  return xcd_contiguous_id_t<int64_t>(block, total);
}

MI355_HD void tile_coord(int64_t block, int64_t tiles_m, int64_t tiles_n,
                         int64_t* tile_m, int64_t* tile_n) {
  tile_coord_t<int64_t>(block, tiles_m, tiles_n, tile_m, tile_n);
}

}  // namespace mi355
