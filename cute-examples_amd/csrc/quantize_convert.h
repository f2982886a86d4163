// Element loads and the fp32 -> e4m3 conversion shared by the fp8 quantisers.
#pragma once
#include "cdna4_primitives.h"

namespace mi355 {

template <class In> struct Load8;  // 8 consecutive elements -> 8 floats
template <> struct Load8<float> {
  static __device__ __forceinline__ void run(const void* p, int64_t i, float* v) {
    const f32x4 a = ((const f32x4*)((const float*)p + i))[0], b = ((const f32x4*)((const float*)p + i))[1];
    v[0] = a[0]; v[1] = a[1]; v[2] = a[2]; v[3] = a[3]; v[4] = b[0]; v[5] = b[1]; v[6] = b[2]; v[7] = b[3];
  }
  static __device__ __forceinline__ float one(const void* p, int64_t i) { return ((const float*)p)[i]; }
};
template <> struct Load8<BF16> {
  static __device__ __forceinline__ void run(const void* p, int64_t i, float* v) {
    const u32x4 a = *(const u32x4*)((const uint16_t*)p + i);
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      v[2 * k] = __builtin_bit_cast(float, a[k] << 16);
      v[2 * k + 1] = __builtin_bit_cast(float, a[k] & 0xffff0000u);
    }
  }
  static __device__ __forceinline__ float one(const void* p, int64_t i) { return Decode<BF16>::run(p, i); }
};
template <> struct Load8<F16> {
  static __device__ __forceinline__ void run(const void* p, int64_t i, float* v) {
    const f16x8 a = *(const f16x8*)((const _Float16*)p + i);
#pragma unroll
    for (int k = 0; k < 8; ++k) v[k] = (float)a[k];
  }
  static __device__ __forceinline__ float one(const void* p, int64_t i) { return Decode<F16>::run(p, i); }
};

// fp32 -> e4m3 (OCP), round to nearest even, saturating at +-448, NaN -> 0x7f.
__device__ __forceinline__ uint32_t to_e4m3(float f) {
  const uint32_t u = __builtin_bit_cast(uint32_t, f);
  const uint32_t sign = (u >> 24) & 0x80u;
  const uint32_t a = u & 0x7fffffffu;
  if (a > 0x7f800000u) return 0x7fu;                       // NaN
  if (a >= 0x43e00000u) return sign | 0x7eu;               // >= 448 (and inf) saturate
  uint32_t code;
  if (a < 0x3c800000u) {                                   // < 2^-6: multiples of 2^-9
    code = (uint32_t)__builtin_rintf(__builtin_bit_cast(float, a) * 512.0f);  // 8 encodes the smallest normal
  } else {
    const uint32_t r = a + 0x7ffffu + ((a >> 20) & 1u);    // RNE to 3 mantissa bits, carry into the exponent
    code = (r >> 20) - (120u << 3);                        // rebias 127 -> 7
    if (code > 0x7eu) code = 0x7eu;
  }
  return sign | code;
}

// Four fp32 -> four e4m3 codes in one word (a in the lowest byte), bit for bit what to_e4m3 gives: the hardware
// conversion (v_cvt_pk_fp8_f32, OCP e4m3 on this GPU, round to nearest even) behind an explicit clamp to +-448.  A NaN
// is carried around the clamp, which would turn it into a number, and comes out of the conversion as a code whose
// low seven bits are all ones, as no number does; the sign of such codes is cleared afterwards.
__device__ __forceinline__ uint32_t to_e4m3x4(float a, float b, float c, float d) {
  const auto clamped = [](float f) __attribute__((always_inline)) {
    const float inside = __builtin_amdgcn_fmed3f(f, -448.0f, 448.0f);
    return f != f ? f : inside;
  };
  int w = __builtin_amdgcn_cvt_pk_fp8_f32(clamped(a), clamped(b), 0, false);
  w = __builtin_amdgcn_cvt_pk_fp8_f32(clamped(c), clamped(d), w, true);
  const uint32_t u = (uint32_t)w;
  const uint32_t nan_sign = ((u & 0x7f7f7f7fu) + 0x01010101u) & 0x80808080u;   // bit 7 of the bytes that hold 0x7f or 0xff
  return u & ~nan_sign;
}

}  // namespace mi355
