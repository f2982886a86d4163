/*
 * gemm_oracle.c — TEST INFRASTRUCTURE, NOT PRODUCT CODE.
 *
 * CPU restatement of what the reference's GEMM path computes, used only by tests/, by
 * __graft_entry__.smoke() and by bench.py's cpu_baseline leg as the checker.  Nothing in the
 * shipped library links, loads or calls this file.
 *
 * The reference kernel (kernels/gemm_kernels/sm90a/gemm.cuh:352-377) computes, per output
 * element, sum_k A[m][k]*B[n][k] with exact bf16*bf16 products accumulated in fp32 by the
 * tensor core and rounds the sum to bf16 with round-to-nearest-even
 * (NumericArrayConverter<bf16,float,2>, gemm.cuh:375-377).  Its own ground truth is
 * torch.matmul(A.float(), B.float().T) in fp32 (kernels/tests/gemm_test.py:36).  The
 * multiply-accumulate itself is the Hopper wgmma instruction reached through NVIDIA/cutlass
 * (git submodule libs/cutlass, .gitmodules:1-3, not vendored, pinned commit not recoverable);
 * its summation order is unspecified, so this oracle accumulates in double (exact to well below
 * fp32 rounding) and the parity tests compare within the tolerance the reference's test uses
 * (gemm_test.py:10) rather than bit-for-bit.
 *
 * Pinning: every function here is checked in tests/test_oracle.py against an independent
 * source — exhaustive bit-pattern sweeps against torch's dtype casts for the decoders and
 * rounders, torch.matmul in fp32 and a numpy float64 product for the GEMM, and closed forms
 * (identity, all-ones, one-hot, exact small-integer products) stored under tests/golden/.
 */
#include <math.h>
#include <stdint.h>
#include <string.h>

enum { ORACLE_BF16 = 0, ORACLE_F16 = 1, ORACLE_E4M3 = 2 };

static float bits_to_f32(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }
static uint32_t f32_to_bits(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }

/* bf16 is the upper half of an IEEE binary32 (inputs of gemm_test.cu:26-28). */
float oracle_bf16_to_f32(uint16_t h) { return bits_to_f32((uint32_t)h << 16); }

/* IEEE binary16: 1 sign, 5 exponent (bias 15), 10 mantissa bits. */
float oracle_f16_to_f32(uint16_t h) {
  uint32_t s = (uint32_t)(h >> 15) << 31, e = (h >> 10) & 31, m = h & 1023;
  if (e == 31) return bits_to_f32(s | 0x7f800000u | (m << 13));
  if (e == 0) {
    float v = ldexpf((float)m, -24);
    return s ? -v : v;
  }
  return bits_to_f32(s | ((e + 112) << 23) | (m << 13));
}

/* OCP FP8 E4M3 ("e4m3fn"): bias 7, no infinities, S.1111.111 is NaN, max finite 448. */
float oracle_e4m3_to_f32(uint8_t b) {
  int s = b >> 7, e = (b >> 3) & 15, m = b & 7;
  float v;
  if (e == 15 && m == 7) return NAN;
  if (e == 0) v = ldexpf((float)m, -9);
  else v = ldexpf(1.0f + (float)m / 8.0f, e - 7);
  return s ? -v : v;
}

/* fp32 -> bf16, round to nearest even (the epilogue conversion, gemm.cuh:368-377). */
uint16_t oracle_f32_to_bf16(float f) {
  uint32_t u = f32_to_bits(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x0040u); /* quiet NaN */
  uint32_t round = 0x7fffu + ((u >> 16) & 1u);
  return (uint16_t)((u + round) >> 16);
}

/* fp32 -> binary16, round to nearest even, overflow to infinity, gradual underflow. */
uint16_t oracle_f32_to_f16(float f) {
  uint32_t u = f32_to_bits(f);
  uint16_t s = (uint16_t)((u >> 16) & 0x8000u);
  uint32_t a = u & 0x7fffffffu;
  if (a > 0x7f800000u) return (uint16_t)(s | 0x7e00u);
  if (a >= 0x477ff000u) return (uint16_t)(s | 0x7c00u); /* >= 65520 rounds to inf */
  if (a < 0x33000001u) return s;                         /* <= 2^-25 rounds to zero */
  int e = (int)(a >> 23) - 127;
  uint32_t m = (a & 0x7fffffu) | 0x800000u; /* 24-bit significand */
  int shift = e < -14 ? 13 + (-14 - e) : 13; /* bits dropped */
  uint32_t kept = m >> shift;
  uint32_t rem = m & ((1u << shift) - 1u);
  uint32_t halfway = 1u << (shift - 1);
  if (rem > halfway || (rem == halfway && (kept & 1u))) kept++;
  uint32_t out;
  if (e < -14) out = kept; /* subnormal; a carry into bit 10 yields the smallest normal */
  else out = ((uint32_t)(e + 15) << 10) + (kept - 0x400u); /* carry propagates into exponent */
  return (uint16_t)(s | out);
}

/* fp32 -> e4m3fn, round to nearest even, saturating at +-448; NaN -> 0x7f. */
uint8_t oracle_f32_to_e4m3_sat(float f) {
  if (isnan(f)) return 0x7f;
  uint8_t s = signbit(f) ? 0x80 : 0;
  float a = fabsf(f);
  if (a >= 448.0f) return (uint8_t)(s | 0x7e);
  if (a < ldexpf(1.0f, -6)) { /* subnormal range: multiples of 2^-9 */
    float q = nearbyintf(a * 512.0f); /* default rounding mode = nearest even */
    return (uint8_t)(s | (uint8_t)q); /* q == 8 encodes the smallest normal, 0x08 */
  }
  int e;
  float fr = frexpf(a, &e); /* a = fr * 2^e, fr in [0.5, 1) */
  float q = nearbyintf(fr * 16.0f); /* 8..16 */
  e -= 1;
  if (q == 16.0f) { q = 8.0f; e += 1; }
  uint8_t out = (uint8_t)(((e + 7) << 3) | ((int)q - 8));
  if (out > 0x7e) out = 0x7e;
  return (uint8_t)(s | out);
}

static float decode(const void *p, int64_t i, int dtype) {
  switch (dtype) {
    case ORACLE_BF16: return oracle_bf16_to_f32(((const uint16_t *)p)[i]);
    case ORACLE_F16: return oracle_f16_to_f32(((const uint16_t *)p)[i]);
    default: return oracle_e4m3_to_f32(((const uint8_t *)p)[i]);
  }
}

/*
 * C32[m][n] = (float)(scale * sum_k A[m][k]*B[n][k]), A (M,K) and B (N,K) K-contiguous with row
 * strides lda/ldb — the contraction of gemm_test.py:36 (B is (N,K) and enters transposed).
 * Products of two bf16/fp16/e4m3 values are exact in double; the sum is accumulated in double.
 * Returns 0, or -1 for a bad dtype.
 */
int oracle_gemm_tn_f32(const void *A, const void *B, float *C32, int64_t M, int64_t N, int64_t K,
                       int64_t lda, int64_t ldb, int64_t ldc, int in_dtype, float scale) {
  if (in_dtype < 0 || in_dtype > 2) return -1;
#pragma omp parallel for schedule(static)
  for (int64_t m = 0; m < M; ++m) {
    for (int64_t n = 0; n < N; ++n) {
      double acc = 0.0;
      for (int64_t k = 0; k < K; ++k)
        acc += (double)decode(A, m * lda + k, in_dtype) * (double)decode(B, n * ldb + k, in_dtype);
      C32[m * ldc + n] = (float)(acc * (double)scale);
    }
  }
  return 0;
}

/* Same contraction followed by the epilogue's down-conversion to bf16 or fp16. */
int oracle_gemm_tn(const void *A, const void *B, uint16_t *C, int64_t M, int64_t N, int64_t K,
                   int64_t lda, int64_t ldb, int64_t ldc, int in_dtype, int out_dtype, float scale) {
  if (in_dtype < 0 || in_dtype > 2 || out_dtype < 0 || out_dtype > 1) return -1;
#pragma omp parallel for schedule(static)
  for (int64_t m = 0; m < M; ++m) {
    for (int64_t n = 0; n < N; ++n) {
      double acc = 0.0;
      for (int64_t k = 0; k < K; ++k)
        acc += (double)decode(A, m * lda + k, in_dtype) * (double)decode(B, n * ldb + k, in_dtype);
      float r = (float)(acc * (double)scale);
      C[m * ldc + n] = out_dtype == ORACLE_BF16 ? oracle_f32_to_bf16(r) : oracle_f32_to_f16(r);
    }
  }
  return 0;
}

/* Vector forms of the scalar converters, for exhaustive sweeps from Python. */
void oracle_decode_array(const void *src, float *dst, int64_t n, int dtype) {
  for (int64_t i = 0; i < n; ++i) dst[i] = decode(src, i, dtype);
}
void oracle_round_array(const float *src, void *dst, int64_t n, int dtype) {
  for (int64_t i = 0; i < n; ++i) {
    if (dtype == ORACLE_BF16) ((uint16_t *)dst)[i] = oracle_f32_to_bf16(src[i]);
    else if (dtype == ORACLE_F16) ((uint16_t *)dst)[i] = oracle_f32_to_f16(src[i]);
    else ((uint8_t *)dst)[i] = oracle_f32_to_e4m3_sat(src[i]);
  }
}
