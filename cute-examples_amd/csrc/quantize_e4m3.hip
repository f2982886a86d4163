// Per-tensor fp8 quantisation on the device: the step in front of the fp8 GEMM.
//
//   amax  = max |x|                       (atomic max over the fp32 bit patterns of |x|)
//   scale = amax / 448  (1 if amax == 0)  (OCP e4m3 has no infinities; 448 is its largest value)
//   x_q   = e4m3_rne(clamp(x / scale, -448, 448))
//
// so that x ~= scale * x_q.  Three launches on the caller's stream, no host synchronisation: the
// scale stays in device memory and the GEMM reads it from there.  The reference has no fp8 path;
// the contract is the benchmark configuration's (operands quantised with per-tensor fp32 scales
// amax/448) and is checked against torch's float8_e4m3fn cast and the C restatement in the tests.
#include "cdna4_primitives.h"
#include "gemm_launch.h"
#include "quantize_convert.h"

namespace mi355 {
namespace {

constexpr float kE4m3Max = 448.0f;

__global__ void amax_init(float* out) { out[0] = 1.0f; out[1] = 0.0f; }

// out[1] accumulates amax: for non-negative floats the unsigned order of the bit patterns is the
// numeric order, so an integer atomic max does it.
template <class In>
__global__ __launch_bounds__(256) void amax_kernel(const void* x, int64_t n, float* out) {
  float m = 0.f;
  const int64_t stride = (int64_t)gridDim.x * 256 * 8;
  int64_t i = ((int64_t)blockIdx.x * 256 + threadIdx.x) * 8;
  for (; i + 3 * stride + 8 <= n; i += 4 * stride) {   // four loads in flight per thread: few workgroups run this
    float v[4][8];
#pragma unroll
    for (int u = 0; u < 4; ++u) Load8<In>::run(x, i + u * stride, v[u]);
#pragma unroll
    for (int u = 0; u < 4; ++u)
#pragma unroll
      for (int k = 0; k < 8; ++k) m = __builtin_fmaxf(m, __builtin_fabsf(v[u][k]));
  }
  for (; i + 8 <= n; i += stride) {
    float v[8];
    Load8<In>::run(x, i, v);
#pragma unroll
    for (int k = 0; k < 8; ++k) m = __builtin_fmaxf(m, __builtin_fabsf(v[k]));
  }
  for (; i < n; ++i) m = __builtin_fmaxf(m, __builtin_fabsf(Load8<In>::one(x, i)));  // at most one thread: the tail
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) m = __builtin_fmaxf(m, __shfl_xor(m, off));
  __shared__ float wave_max[4];
  if ((threadIdx.x & 63) == 0) wave_max[threadIdx.x >> 6] = m;
  __syncthreads();
  if (threadIdx.x == 0) {
    m = __builtin_fmaxf(__builtin_fmaxf(wave_max[0], wave_max[1]), __builtin_fmaxf(wave_max[2], wave_max[3]));
    // Thousands of atomics on one address take tens of microseconds, one after the other.  The maximum only grows, so a
    // workgroup whose own maximum is not above what it reads there has nothing to add; on ordinary data a handful are.
    const unsigned mine = __builtin_bit_cast(unsigned, m);
    if (mine > __hip_atomic_load((unsigned*)(out + 1), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT))
      atomicMax((unsigned*)(out + 1), mine);
  }
}

template <class In>
__global__ __launch_bounds__(256) void quantize_kernel(const void* x, int64_t n, uint8_t* q, float* out) {
  const float amax = out[1];
  const float scale = amax > 0.f ? amax / kE4m3Max : 1.0f;
  if (blockIdx.x == 0 && threadIdx.x == 0) out[0] = scale;
  const int64_t stride = (int64_t)gridDim.x * 256 * 8;
  int64_t i = ((int64_t)blockIdx.x * 256 + threadIdx.x) * 8;
  for (; i + 8 <= n; i += stride) {
    float v[8];
    Load8<In>::run(x, i, v);
    const uint32_t lo = to_e4m3x4(v[0] / scale, v[1] / scale, v[2] / scale, v[3] / scale);
    const uint32_t hi = to_e4m3x4(v[4] / scale, v[5] / scale, v[6] / scale, v[7] / scale);
    *(u32x2*)(q + i) = (u32x2){lo, hi};
  }
  for (; i < n; ++i) q[i] = (uint8_t)to_e4m3(Load8<In>::one(x, i) / scale);
}

template <class In>
int run(const void* x, int64_t n, void* q, float* out, hipStream_t stream) {
  const int64_t want = (n / 8 + 255) / 256;
  const unsigned blocks = (unsigned)(want < 1 ? 1 : want > 4096 ? 4096 : want);
  hipLaunchKernelGGL(amax_init, dim3(1), dim3(1), 0, stream, out);
  // Few workgroups for the maximum: those that finish together all find the accumulator still low and all add to it,
  // one atomic after the other (12 ns each: 4096 workgroups 50 us, 512 at most 6); 512 read as fast as 4096 do.
  hipLaunchKernelGGL((amax_kernel<In>), dim3(blocks < 512 ? blocks : 512), dim3(256), 0, stream, x, n, out);
  hipLaunchKernelGGL((quantize_kernel<In>), dim3(blocks), dim3(256), 0, stream, x, n, (uint8_t*)q, out);
  return hipGetLastError() == hipSuccess ? 0 : -1;
}

}  // namespace

// in_dtype: 0 bf16, 1 fp16, 3 fp32.
int launch_quantize_e4m3(const void* x, int in_dtype, int64_t n, void* q, float* scale_amax, hipStream_t stream) {
  switch (in_dtype) {
    case 0: return run<BF16>(x, n, q, scale_amax, stream);
    case 1: return run<F16>(x, n, q, scale_amax, stream);
    case 3: return run<float>(x, n, q, scale_amax, stream);
  }
  return -1;
}

}  // namespace mi355
