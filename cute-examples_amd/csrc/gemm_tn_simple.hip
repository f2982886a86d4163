// One thread per output element: C[m][n] = rne(scale * sum_k A[m][k] * B[n][k]) with a serial
// fp32 fused-multiply-add chain over k.  Handles every shape, stride and dtype the ABI accepts;
// it is the library's on-device cross-check for the MFMA kernels and the path for shapes they
// reject.  Counterpart in the reference: none (its only kernel rejects such shapes,
// kernels/gemm_kernels/sm90a/gemm_test.cu:33-41).
#include "cdna4_primitives.h"
#include "gemm_launch.h"

namespace mi355 {
namespace {

template <class T, class OutT>
__global__ __launch_bounds__(256) void gemm_tn_simple(GemmArgs g) {
  const int64_t n = (int64_t)blockIdx.x * 16 + (threadIdx.x & 15);
  const int64_t m = (int64_t)blockIdx.y * 16 + (threadIdx.x >> 4);
  if (m >= g.M || n >= g.N) return;
  const int64_t a0 = m * g.lda, b0 = n * g.ldb;
  float acc = 0.f;
  for (int64_t k = 0; k < g.K; ++k)
    acc = __builtin_fmaf(Decode<T>::run(g.A, a0 + k), Decode<T>::run(g.B, b0 + k), acc);
  ((uint16_t*)g.C)[m * g.ldc + n] = Pack4<OutT>::one(acc * output_scale(g));
}

template <class T, class OutT>
int launch(const GemmArgs& g, hipStream_t stream) {
  dim3 grid((unsigned)((g.N + 15) / 16), (unsigned)((g.M + 15) / 16));
  hipLaunchKernelGGL((gemm_tn_simple<T, OutT>), grid, dim3(256), 0, stream, g);
  return hipGetLastError() == hipSuccess ? 0 : -1;
}

}  // namespace

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
