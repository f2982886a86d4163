// Measured ceilings of one GPU, for the benchmark's roofline line: what the matrix cores sustain
// with nothing else going on, and what a plain read of HBM reaches.  The published peaks assume the
// nominal clock; under the board power limit the sustained figures are lower and depend on the data
// (all-zero operands draw far less power than random ones), so both kernels work on the caller's
// own operands.
//
//   mfma_ceiling   every wave holds 8 + 8 operand fragments in registers (loaded once from the
//                  caller's A and B) and runs the tile kernel's MFMA pattern on them -- 64
//                  accumulator blocks, acc[i][j] += a[i] * b[j], the same instruction and the same
//                  dependency distance as a k-step of gemm_tn_tile_ring -- with no LDS traffic, no
//                  copies, no barriers.  One workgroup of four waves per CU.  The same loop also
//                  exists on the 32-wide MFMA shapes the kernels do not use (4 + 4 fragments, 16
//                  blocks: the same 128 x 128 outputs per wave), so that a benchmark can show what
//                  the choice of shape is worth on the GPU and the data at hand.
//   read_ceiling   16-byte loads, grid-stride over the buffer, xor-reduced so nothing is elided.
//   clock_probe    single-wave workgroups that sleep and, every so often, read the shader-cycle counter
//                  and the constant 100 MHz counter: launched on a second stream beside other work
//                  (a wave of it needs 8 registers and no LDS, so it fits beside a workgroup of the
//                  tile kernels), it tells the shader clock that work runs at without a profiler.
//
// Counterpart in the reference: none (its benchmark takes the peak from a table,
// kernels/tests/gemm_bench.py:592-599).
#include "../../include/mi355_gemm.h"

#include "ring_common.h"

namespace mi355 {
namespace {

// v_mfma_f32_32x32x16 for the 16-bit types: the shape the tile kernels do NOT run on (measured
// here so that the choice is visible); fp8 on 32x32x64 is Geo<E4M3> of ring_common.h.
template <class T> struct Geo32;
template <> struct Geo32<BF16> {
  static constexpr int kBlk = 32;
  typedef i32x4 Frag;
  typedef f32x16 Acc;
  static __device__ __forceinline__ void mfma_inplace(Frag x, Frag y, Acc& c) {
    asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+a"(c) : "v"(x), "v"(y));
  }
};
template <> struct Geo32<F16> {
  static constexpr int kBlk = 32;
  typedef i32x4 Frag;
  typedef f32x16 Acc;
  static __device__ __forceinline__ void mfma_inplace(Frag x, Frag y, Acc& c) {
    asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+a"(c) : "v"(x), "v"(y));
  }
};

template <class G>
__global__ __launch_bounds__(256, 1) void mfma_ceiling(const uint8_t* a, const uint8_t* b, size_t a_bytes,
                                                       size_t b_bytes, int iters, float* sink) {
  typedef typename G::Frag Frag;
  typedef typename G::Acc Acc;
  constexpr int kN = 128 / G::kBlk;   // blocks per side of the wave's 128 x 128 outputs
  Frag fa[kN], fb[kN];
  Acc acc[kN][kN];
  // Fragment i of this lane: sizeof(Frag) bytes of the operand, a different place for every lane,
  // wave, workgroup and i (wrapping around inside the buffer).
  const size_t lane_id = (size_t)blockIdx.x * 256 + threadIdx.x;
#pragma unroll
  for (int i = 0; i < kN; ++i) {
    const size_t at = (lane_id * kN + i) * sizeof(Frag);
    fa[i] = *(const Frag*)(a + at % (a_bytes - sizeof(Frag) + 1) / sizeof(Frag) * sizeof(Frag));
    fb[i] = *(const Frag*)(b + at % (b_bytes - sizeof(Frag) + 1) / sizeof(Frag) * sizeof(Frag));
  }
#pragma unroll
  for (int i = 0; i < kN; ++i)
#pragma unroll
    for (int j = 0; j < kN; ++j)
#pragma unroll
      for (int r = 0; r < (int)(sizeof(Acc) / 4); ++r) acc[i][j][r] = 0.f;
  for (int it = 0; it < iters; ++it) {
    static_for<kN * kN>([&](auto uc) __attribute__((always_inline)) {
      constexpr int u = decltype(uc)::value;
      G::mfma_inplace(fb[u % kN], fa[u / kN], acc[u / kN][u % kN]);
    });
  }
  // The MFMAs are inline assembly: the compiler does not know how long their results take.
  asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < kN; ++i)
#pragma unroll
    for (int j = 0; j < kN; ++j) {
      Acc c = acc[i][j];
      asm volatile("" : "+a"(c));
      s += c[0];
    }
  sink[lane_id] = s;
}

__global__ __launch_bounds__(256) void read_ceiling(const u32x4* src, size_t chunks, uint32_t* sink) {
  u32x4 x = {0, 0, 0, 0};
  const size_t stride = (size_t)gridDim.x * 256;
  for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < chunks; i += stride) x ^= __builtin_nontemporal_load(src + i);
  sink[(size_t)blockIdx.x * 256 + threadIdx.x] = x[0] ^ x[1] ^ x[2] ^ x[3];
}

// out[w][0][0] = XCD of wave w, out[w][1][0] = 0; out[w][0][1 + s] = shader cycles and out[w][1][1 + s] = 10 ns ticks
// at sample s (uint64 out[waves][2][samples + 1]).  s_memtime counts shader cycles on this GPU (a chain of
// dependent MFMAs reads the same difference whatever the clock), s_memrealtime counts at 100 MHz.  Every loop is
// bounded by the arguments.
__global__ __launch_bounds__(64) void clock_probe(uint64_t* out, int samples, int pause) {
  uint32_t xcc;
  asm volatile("s_getreg_b32 %0, hwreg(HW_REG_XCC_ID)" : "=s"(xcc));
  // One lane writes, in 4-byte pieces: nothing here is worth the care wider stores' data registers need.
  volatile uint32_t* cycles_of = (volatile uint32_t*)(out + (size_t)blockIdx.x * 2 * (size_t)(samples + 1));
  volatile uint32_t* ticks_of = cycles_of + 2 * (size_t)(samples + 1);
  auto put = [](volatile uint32_t* at, uint64_t x) __attribute__((always_inline)) {
    at[0] = (uint32_t)x;
    at[1] = (uint32_t)(x >> 32);
  };
  if (threadIdx.x == 0) {
    put(cycles_of, xcc & 15u);
    put(ticks_of, 0);
  }
  for (int s = 0; s < samples; ++s) {
    const uint64_t cycles = __builtin_readcyclecounter(), ticks = __builtin_amdgcn_s_memrealtime();
    if (threadIdx.x == 0) {
      put(cycles_of + 2 * (size_t)(1 + s), cycles);
      put(ticks_of + 2 * (size_t)(1 + s), ticks);
    }
    for (int p = 0; p < pause; ++p) __builtin_amdgcn_s_sleep(127);
  }
}

}  // namespace
}  // namespace mi355

extern "C" {

size_t mi355_calibrate_sink_bytes(void) { return (size_t)4096 * 256 * 4; }

int mi355_calibrate_mfma_shape(int in_dtype, int wide_blocks, const void* a, size_t a_bytes, const void* b, size_t b_bytes,
                               int iters, void* sink, double* flops, void* stream) {
  using namespace mi355;
  if (!a || !b || !sink || !flops) return MI355_ERR_NULL;
  if (in_dtype != MI355_BF16 && in_dtype != MI355_F16 && in_dtype != MI355_E4M3) return MI355_ERR_DTYPE;
  if (wide_blocks != 0 && wide_blocks != 1) return MI355_ERR_VARIANT;
  if (iters <= 0 || a_bytes < 4096 || b_bytes < 4096) return MI355_ERR_SHAPE;
  if ((uintptr_t)a % 32 != 0 || (uintptr_t)b % 32 != 0 || (uintptr_t)sink % 4 != 0) return MI355_ERR_ALIGN;
  const int cus = compute_units();
  if (cus > 4096) return MI355_ERR_LAUNCH;
  hipStream_t s = (hipStream_t)stream;
  const uint8_t* pa = (const uint8_t*)a;
  const uint8_t* pb = (const uint8_t*)b;
  // Every shape covers the wave's 128 x 128 outputs once per pass over its blocks, with a K extent
  // of 32 or 16 elements (16-bit, 16- or 32-wide blocks) or 128 or 64 elements (fp8).
  const double k_extent = in_dtype == MI355_E4M3 ? (wide_blocks ? 64.0 : 128.0) : (wide_blocks ? 16.0 : 32.0);
  *flops = 2.0 * 128.0 * 128.0 * k_extent * (double)iters * 4.0 * (double)cus;
  const dim3 grid(cus), block(256);
  float* out = (float*)sink;
  if (!wide_blocks) {
    if (in_dtype == MI355_BF16) hipLaunchKernelGGL(mfma_ceiling<Geo<BF16>>, grid, block, 0, s, pa, pb, a_bytes, b_bytes, iters, out);
    else if (in_dtype == MI355_F16) hipLaunchKernelGGL(mfma_ceiling<Geo<F16>>, grid, block, 0, s, pa, pb, a_bytes, b_bytes, iters, out);
    else hipLaunchKernelGGL(mfma_ceiling<GeoE4M3Rows>, grid, block, 0, s, pa, pb, a_bytes, b_bytes, iters, out);
  } else {
    if (in_dtype == MI355_BF16) hipLaunchKernelGGL(mfma_ceiling<Geo32<BF16>>, grid, block, 0, s, pa, pb, a_bytes, b_bytes, iters, out);
    else if (in_dtype == MI355_F16) hipLaunchKernelGGL(mfma_ceiling<Geo32<F16>>, grid, block, 0, s, pa, pb, a_bytes, b_bytes, iters, out);
    else hipLaunchKernelGGL(mfma_ceiling<Geo<E4M3>>, grid, block, 0, s, pa, pb, a_bytes, b_bytes, iters, out);
  }
  return hipGetLastError() == hipSuccess ? MI355_OK : MI355_ERR_LAUNCH;
}

int mi355_calibrate_mfma(int in_dtype, const void* a, size_t a_bytes, const void* b, size_t b_bytes, int iters,
                         void* sink, double* flops, void* stream) {
  return mi355_calibrate_mfma_shape(in_dtype, 0, a, a_bytes, b, b_bytes, iters, sink, flops, stream);
}

int mi355_calibrate_read(const void* src, size_t bytes, void* sink, void* stream) {
  using namespace mi355;
  if (!src || !sink) return MI355_ERR_NULL;
  if (bytes < 16) return MI355_ERR_SHAPE;
  if ((uintptr_t)src % 16 != 0 || (uintptr_t)sink % 4 != 0) return MI355_ERR_ALIGN;
  const int cus = compute_units();
  const unsigned blocks = (unsigned)(cus * 16 < 4096 ? cus * 16 : 4096);
  hipLaunchKernelGGL(read_ceiling, dim3(blocks), dim3(256), 0, (hipStream_t)stream, (const u32x4*)src, bytes / 16,
                     (uint32_t*)sink);
  return hipGetLastError() == hipSuccess ? MI355_OK : MI355_ERR_LAUNCH;
}

size_t mi355_clock_probe_bytes(int waves, int samples) {
  if (waves < 1 || waves > 1024 || samples < 2 || samples > 4096) return 0;
  return (size_t)waves * (size_t)(samples + 1) * 2 * sizeof(uint64_t);
}

int mi355_clock_probe(int waves, int samples, int pause, void* out, void* stream) {
  using namespace mi355;
  if (!out) return MI355_ERR_NULL;
  // at most 65536 sleeps of 127 x 64 cycles per wave: a quarter of a second at 2 GHz
  if (mi355_clock_probe_bytes(waves, samples) == 0 || pause < 1 || (int64_t)samples * pause > 65536) return MI355_ERR_SHAPE;
  if ((uintptr_t)out % 8 != 0) return MI355_ERR_ALIGN;
  hipLaunchKernelGGL(clock_probe, dim3((unsigned)waves), dim3(64), 0, (hipStream_t)stream, (uint64_t*)out, samples, pause);
  return hipGetLastError() == hipSuccess ? MI355_OK : MI355_ERR_LAUNCH;
}

}  // extern "C"
