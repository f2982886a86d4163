// Pieces shared by the ring-buffered 256x256-tile kernels (single wave group and ping-pong):
// LDS ring geometry, the bank-conflict-free chunk swizzle, and the per-dtype MFMA geometry.
#pragma once
#include "cdna4_primitives.h"

#include <atomic>
#include <type_traits>
#include <utility>

namespace mi355 {

constexpr int kTile = 256;
constexpr int kRowBytes = 128;
constexpr int kSlots = 5;

__device__ __forceinline__ uint32_t swizzle(uint32_t row) { return (row >> 1) & 7u; }

#define MI355_FENCE() __builtin_amdgcn_sched_barrier(0)

// f(integral_constant<int, 0>) ... f(integral_constant<int, kN - 1>), unrolled at compile time.
template <int kN, class F, int... kI>
__device__ __forceinline__ void static_for_impl(F&& f, std::integer_sequence<int, kI...>) {
  (f(std::integral_constant<int, kI>{}), ...);
}
template <int kN, class F>
__device__ __forceinline__ void static_for(F&& f) {
  static_for_impl<kN>(f, std::make_integer_sequence<int, kN>{});
}


// Per-dtype MFMA geometry.
//   kBlk      rows (and columns) of one MFMA block
//   kGroups   lane groups of kBlk lanes; group g feeds k-chunks g*kCpl .. g*kCpl+kCpl-1 of a slice
//   kCpl      16-byte chunks per lane per MFMA
template <class T> struct Geo;
template <> struct Geo<BF16> {
  static constexpr int kBlk = 16, kGroups = 4, kCpl = 1;
  static constexpr bool kRowSliced = false, kMx = false;
  typedef i32x4 Frag;
  typedef f32x4 Acc;
  static __device__ __forceinline__ Acc mfma(Frag x, Frag y, Acc c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, x),
                                                   __builtin_bit_cast(bf16x8, y), c, 0, 0, 0);
  }
  // The same instruction with the accumulator tied in place in an accumulation register.  The
  // single-group 256x256 kernel uses it: with 256 accumulator registers live across a loop
  // nest the register allocator otherwise rotates a few accumulator tiles through VGPR copies
  // every k-step.  The callers keep dependent uses of c far apart (64 MFMAs, or a barrier and
  // the whole tile set-up before the epilogue), beyond any MFMA result hazard.
  static __device__ __forceinline__ void mfma_inplace(Frag x, Frag y, Acc& c) {
    asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(c) : "v"(x), "v"(y));
  }
};
template <> struct Geo<F16> {
  static constexpr int kBlk = 16, kGroups = 4, kCpl = 1;
  static constexpr bool kRowSliced = false, kMx = false;
  typedef i32x4 Frag;
  typedef f32x4 Acc;
  static __device__ __forceinline__ Acc mfma(Frag x, Frag y, Acc c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, x),
                                                  __builtin_bit_cast(f16x8, y), c, 0, 0, 0);
  }
  static __device__ __forceinline__ void mfma_inplace(Frag x, Frag y, Acc& c) {
    asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+a"(c) : "v"(x), "v"(y));
  }
};
template <> struct Geo<E4M3> {
  static constexpr int kBlk = 32, kGroups = 2, kCpl = 2;
  static constexpr bool kRowSliced = false, kMx = false;
  typedef i32x8 Frag;
  typedef f32x16 Acc;
  static __device__ __forceinline__ Acc mfma(Frag x, Frag y, Acc c) {
    return __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(x, y, c, 0, 0, 0, 0, 0, 0);
  }
  // Both operand formats default to e4m3 (cbsz = blgp = 0), as the builtin call above passes.
  static __device__ __forceinline__ void mfma_inplace(Frag x, Frag y, Acc& c) {
    asm volatile("v_mfma_f32_32x32x64_f8f6f4 %0, %1, %2, %0" : "+a"(c) : "v"(x), "v"(y));
  }
};


// fp8 on the 16x16x128 shape: one MFMA consumes a whole k-step (8 chunks) of a 16-row block, so a
// k-step cannot be cut in two along K.  Kernels that use this geometry cut it along the rows of A
// instead (kRowSliced).  On random data the shape sustains a ~9 % higher MFMA rate under the board
// power limit than 32x32x64, and its 16-wide blocks store 64-byte runs like the 16-bit types.
struct GeoE4M3Rows {
  static constexpr int kBlk = 16, kGroups = 4, kCpl = 2;
  static constexpr bool kRowSliced = true, kMx = false;
  typedef i32x8 Frag;
  typedef f32x4 Acc;
  static __device__ __forceinline__ Acc mfma(Frag x, Frag y, Acc c) {
    return __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(x, y, c, 0, 0, 0, 0, 0, 0);
  }
  static __device__ __forceinline__ void mfma_inplace(Frag x, Frag y, Acc& c) {
    asm volatile("v_mfma_f32_16x16x128_f8f6f4 %0, %1, %2, %0" : "+a"(c) : "v"(x), "v"(y));
  }
};

// The same shape with OCP MX block scaling: every lane passes, with its fragment, a register that
// holds the E8M0 scale of its row for one 32-element block of K in the byte picked by kByteX /
// kByteY (0..3), and the hardware multiplies each block's partial dot product by both scales.
// Which block a lane's scale applies to fixes the order of K inside the MFMA (measured): the lanes
// of group g = lane/16 supply bytes [16g, 16g+16) and [64+16g, 64+16g+16) of the 128-byte k-step,
// and the scale of the lanes of group g applies to bytes [32g, 32g+32), whoever supplied them.
struct GeoMxE4M3Rows : GeoE4M3Rows {
  static constexpr bool kMx = true;
  template <int kByteX, int kByteY>
  static __device__ __forceinline__ void mfma_scaled_inplace(Frag x, Frag y, Acc& c, uint32_t sx, uint32_t sy) {
    asm volatile("v_mfma_scale_f32_16x16x128_f8f6f4 %0, %1, %2, %0, %3, %4 op_sel:[%5,%6,0] op_sel_hi:[%7,%8,0]"
                 : "+a"(c)
                 : "v"(x), "v"(y), "v"(sx), "v"(sy), "n"(kByteX & 1), "n"(kByteY & 1), "n"(kByteX >> 1),
                   "n"(kByteY >> 1));
  }
};

// Geometry the ring-buffered tile kernels use for an input type: fp8 runs on the 16x16x128 shape.
template <class T> struct RingGeo { typedef Geo<T> type; };
template <> struct RingGeo<E4M3> { typedef GeoE4M3Rows type; };
template <> struct RingGeo<MxE4M3> { typedef GeoMxE4M3Rows type; };

// Compute units of the current device (256 on MI355X); queried once per device.
inline int compute_units() {
  static std::atomic<int> cached[64];
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) dev = 0;
  int n = cached[dev].load(std::memory_order_relaxed);
  if (n == 0) {
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
    cached[dev].store(n, std::memory_order_relaxed);
  }
  return n;
}

}  // namespace mi355
