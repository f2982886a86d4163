// One thread per output element: C[m][n] = rne(scale * sum_k A[m][k] * B[n][k]) with a serial
// fp32 fused-multiply-add chain over k.  Handles every shape, stride and dtype the ABI accepts;
// it is the library's on-device cross-check for the MFMA kernels and the path for shapes they
// reject.  Also here: the two copy kernels with which the library repacks such a problem into an
// aligned one when the caller lends it the memory (gemm_api.hip).  Counterpart in the reference:
// none (its only kernel rejects such shapes, kernels/gemm_kernels/sm90a/gemm_test.cu:33-41).
#include "cdna4_primitives.h"
#include "gemm_launch.h"

namespace mi355 {
namespace {

template <class T, class OutT>
__global__ __launch_bounds__(256) void gemm_tn_simple(GemmArgs g) {
  // 16 x 16 outputs per workgroup; the workgroups walk the blocks of C in one dimension (the y and z
  // dimensions of a grid hold 65535 entries only), striding when there are more than 2^31 - 1.
  const int64_t blocks_n = (g.N + 15) / 16, blocks = blocks_n * ((g.M + 15) / 16);
  for (int64_t b = blockIdx.x; b < blocks; b += gridDim.x) {
    const int64_t n = (b % blocks_n) * 16 + (threadIdx.x & 15);
    const int64_t m = (b / blocks_n) * 16 + (threadIdx.x >> 4);
    if (m >= g.M || n >= g.N) continue;
    const int64_t a0 = m * g.lda, b0 = n * g.ldb;
    float acc = 0.f;
    for (int64_t k = 0; k < g.K; ++k)
      acc = __builtin_fmaf(Decode<T>::run(g.A, a0 + k), Decode<T>::run(g.B, b0 + k), acc);
    ((uint16_t*)g.C)[m * g.ldc + n] = Pack4<OutT>::one(acc * output_scale(g));
  }
}

// One thread per 16-byte chunk of the destination.  The source has only element alignment, so it is
// read element by element (the loads of neighbouring threads still coalesce).
template <class E>
__global__ __launch_bounds__(256) void repack_rows(const uint8_t* __restrict__ src, int64_t rows, int64_t row_bytes,
                                                   int64_t src_ld, uint8_t* __restrict__ dst, int64_t dst_rows,
                                                   int64_t dst_ld) {
  constexpr int kPer = 16 / (int)sizeof(E);
  const int64_t chunks_per_row = dst_ld / 16;
  const int64_t id = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (id >= dst_rows * chunks_per_row) return;
  const int64_t row = id / chunks_per_row, at = (id % chunks_per_row) * 16;
  E v[kPer];
#pragma unroll
  for (int i = 0; i < kPer; ++i) {
    const int64_t byte = at + i * (int64_t)sizeof(E);
    v[i] = row < rows && byte < row_bytes ? *(const E*)(src + row * src_ld + byte) : (E)0;
  }
  u32x4 out;
  __builtin_memcpy(&out, v, 16);
  *(u32x4*)(dst + row * dst_ld + at) = out;
}

// One thread per four columns: the source rows are 8-byte aligned (src_ld % 4 == 0), the
// destination has only element alignment.
__global__ __launch_bounds__(256) void copy_out(const uint16_t* __restrict__ src, int64_t rows, int64_t cols,
                                                int64_t src_ld, uint16_t* __restrict__ dst, int64_t dst_ld) {
  const int64_t quads = (cols + 3) / 4;
  const int64_t id = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (id >= rows * quads) return;
  const int64_t row = id / quads, col = (id % quads) * 4;
  const u32x2 v = *(const u32x2*)(src + row * src_ld + col);
  uint16_t* d = dst + row * dst_ld + col;
  d[0] = (uint16_t)v[0];
  if (col + 1 < cols) d[1] = (uint16_t)(v[0] >> 16);
  if (col + 2 < cols) d[2] = (uint16_t)v[1];
  if (col + 3 < cols) d[3] = (uint16_t)(v[1] >> 16);
}

template <class T, class OutT>
int launch(const GemmArgs& g, hipStream_t stream) {
  const int64_t blocks = ((g.N + 15) / 16) * ((g.M + 15) / 16);
  const int64_t grid = blocks < 0x7fffffff ? blocks : 0x7fffffff;
  hipLaunchKernelGGL((gemm_tn_simple<T, OutT>), dim3((unsigned)grid), dim3(256), 0, stream, g);
  return hipGetLastError() == hipSuccess ? 0 : -1;
}

}  // namespace

int launch_repack_rows(const void* src, int64_t rows, int64_t row_bytes, int64_t src_ld, void* dst, int64_t dst_rows,
                       int64_t dst_ld, int elem_bytes, hipStream_t stream) {
  const int64_t chunks = dst_rows * (dst_ld / 16);
  if (chunks == 0) return 0;
  const int64_t blocks = (chunks + 255) / 256;
  if (blocks >= ((int64_t)1 << 31) || dst_ld % 16 != 0) return -1;
  if (elem_bytes == 2)
    hipLaunchKernelGGL(repack_rows<uint16_t>, dim3((unsigned)blocks), dim3(256), 0, stream, (const uint8_t*)src, rows,
                       row_bytes, src_ld, (uint8_t*)dst, dst_rows, dst_ld);
  else
    hipLaunchKernelGGL(repack_rows<uint8_t>, dim3((unsigned)blocks), dim3(256), 0, stream, (const uint8_t*)src, rows,
                       row_bytes, src_ld, (uint8_t*)dst, dst_rows, dst_ld);
  return hipGetLastError() == hipSuccess ? 0 : -1;
}

int launch_copy_out(const void* src, int64_t rows, int64_t cols, int64_t src_ld, void* dst, int64_t dst_ld,
                    hipStream_t stream) {
  const int64_t n = rows * ((cols + 3) / 4);
  if (n == 0) return 0;
  const int64_t blocks = (n + 255) / 256;
  if (blocks >= ((int64_t)1 << 31) || src_ld % 4 != 0 || (uintptr_t)src % 8 != 0) return -1;
  hipLaunchKernelGGL(copy_out, dim3((unsigned)blocks), dim3(256), 0, stream, (const uint16_t*)src, rows, cols, src_ld,
                     (uint16_t*)dst, dst_ld);
  return hipGetLastError() == hipSuccess ? 0 : -1;
}

int launch_simple(const GemmArgs& g, int in_dtype, int out_dtype, hipStream_t stream) {
  const bool out_bf16 = out_dtype == 0;
  switch (in_dtype) {
    case 0: return out_bf16 ? launch<BF16, BF16>(g, stream) : launch<BF16, F16>(g, stream);
    case 1: return out_bf16 ? launch<F16, BF16>(g, stream) : launch<F16, F16>(g, stream);
    case 2: return out_bf16 ? launch<E4M3, BF16>(g, stream) : launch<E4M3, F16>(g, stream);
  }
  return -1;
}

}  // namespace mi355
