// OCP MX block scaling for the fp8 GEMM: the quantiser and the scale shuffle.
//
// An MX-quantised matrix X (rows, K), K % 32 == 0, is a pair
//   x_q     (rows, K)      e4m3 elements
//   scales  (rows, K/32)   one E8M0 byte per block of 32 consecutive elements of a row,
//                          value 2^(byte - 127)
// with X ~= x_q * scale of its block.  The quantiser follows the OCP Microscaling Formats (MX)
// specification v1.0, section 6.3: the shared exponent of a block is floor(log2(amax)) - 8 (8 is
// the exponent of the largest e4m3 binade), elements are x / 2^shared rounded to nearest even and
// saturated at +-448.  A block of zeros gets the scale 1.  NaN and infinity are not supported.
// The reference has no fp8 path; this is the block-scaled variant of the quantiser in
// quantize_e4m3.hip, and the format the scaled MFMA of gfx950 consumes.
//
// The GEMM kernel reads scales in a "shuffled" layout (gemm_tn_ring.h: kMxUnitBytes), produced
// here from the natural row-major one: one 512-byte unit per (group of 128 rows, k-step of 128
// elements), units ordered [row group][k-step], 8 bytes per lane: byte i of lane l is the scale of
// row 16*i + l%16 of the group for block 4*kstep + l/16.  Rows are padded to whole 256-row tiles
// with the scale 1 (their elements read as zeros).
#include "cdna4_primitives.h"
#include "gemm_launch.h"
#include "quantize_convert.h"

namespace mi355 {
namespace {

constexpr int kMxBlock = 32;

// One operand's scale bytes and where its shuffled copy goes.
struct MxOperand {
  const uint8_t* scales;
  int64_t rows, ld;
  uint64_t slots;  // 8-byte lane slots of the shuffled layout
  uint8_t* out;
};

// Shuffles one operand, or two in one launch (second.slots == 0 if there is only one): thread ids
// below first.slots work on the first operand, the rest on the second.
__global__ __launch_bounds__(256) void mx_shuffle_kernel(MxOperand first, MxOperand second, uint32_t k_steps) {
  uint64_t id = (uint64_t)blockIdx.x * 256 + threadIdx.x;  // one lane slot of 8 bytes
  const bool is_second = id >= first.slots;
  if (is_second) id -= first.slots;
  const MxOperand& op = is_second ? second : first;
  if (id >= op.slots) return;
  const uint8_t* __restrict__ scales = op.scales;
  uint8_t* __restrict__ out = op.out;
  const int64_t rows = op.rows, ld = op.ld;
  const uint32_t lane = (uint32_t)(id & 63u);
  const uint64_t unit = id >> 6;
  const uint64_t group = unit / k_steps;
  const uint32_t kstep = (uint32_t)(unit % k_steps);
  const int64_t block = 4 * (int64_t)kstep + lane / 16;
  uint32_t w[2] = {0, 0};
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const int64_t row = (int64_t)group * 128 + 16 * i + lane % 16;
    const uint32_t b = row < rows ? scales[row * ld + block] : 127u;
    w[i / 4] |= b << (8 * (i % 4));
  }
  *(u32x2*)(out + id * 8) = (u32x2){w[0], w[1]};
}

// Where the scale of (row, block) lives in the shuffled layout.
__device__ __forceinline__ int64_t shuffled_index(int64_t row, int64_t blk, int64_t blocks_per_row) {
  const int64_t unit = (row / 128) * (blocks_per_row / 4) + blk / 4;
  const int64_t lane = row % 16 + 16 * (blk % 4);
  return unit * 512 + lane * 8 + (row % 128) / 16;
}

// One thread per block of 32 elements.  kShuffled: the scales are written straight into the layout
// the GEMM reads (rows padded to a multiple of 256 with the scale 1), which saves the shuffle launch.
template <class In, bool kShuffled>
__global__ __launch_bounds__(256) void mx_quantize_kernel(const void* __restrict__ x, int64_t rows, int64_t blocks_per_row,
                                                          int64_t ldx, uint8_t* __restrict__ q,
                                                          uint8_t* __restrict__ scales) {
  const int64_t id = (int64_t)blockIdx.x * 256 + threadIdx.x;
  const int64_t padded_rows = kShuffled ? (rows + 255) / 256 * 256 : rows;
  if (id >= padded_rows * blocks_per_row) return;
  const int64_t row = id / blocks_per_row, blk = id % blocks_per_row;
  if (kShuffled && row >= rows) {
    scales[shuffled_index(row, blk, blocks_per_row)] = 127;
    return;
  }
  const int64_t at = row * ldx + blk * kMxBlock;
  float v[kMxBlock];
#pragma unroll
  for (int i = 0; i < kMxBlock; i += 8) Load8<In>::run(x, at + i, v + i);
  float amax = 0.f;
#pragma unroll
  for (int i = 0; i < kMxBlock; ++i) amax = __builtin_fmaxf(amax, __builtin_fabsf(v[i]));
  // floor(log2(amax)) is the exponent field of amax minus 127 (fields below 8, including the
  // fp32 subnormals, clamp to the smallest scale).
  const uint32_t field = __builtin_bit_cast(uint32_t, amax) >> 23;
  const uint32_t byte = amax == 0.f ? 127u : (field > 8u ? field - 8u : 0u);
  const float inv = __builtin_bit_cast(float, (254u - byte) << 23);  // 2^(127 - byte), exact
  uint32_t w[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) w[i] = to_e4m3x4(v[4 * i] * inv, v[4 * i + 1] * inv, v[4 * i + 2] * inv, v[4 * i + 3] * inv);
  u32x4* dst = (u32x4*)(q + row * blocks_per_row * kMxBlock + blk * kMxBlock);
  dst[0] = (u32x4){w[0], w[1], w[2], w[3]};
  dst[1] = (u32x4){w[4], w[5], w[6], w[7]};
  scales[kShuffled ? shuffled_index(row, blk, blocks_per_row) : id] = (uint8_t)byte;
}

// The quantiser that writes the shuffled layout, by patches of 128 rows x 8 blocks (two 512-byte units of scales):
// eight neighbouring threads read 512 contiguous bytes of a row, the 1024 scale bytes of the patch are put in place
// in LDS, and 256 threads write them out four bytes each, instead of every thread writing one byte to a line of its own
// (bf16 8192 x 8192: 35.8 -> 30 us, what the natural layout takes).  Rows past the end get the scale 1.
template <class In>
__global__ __launch_bounds__(1024) void mx_quantize_shuffled_kernel(const void* __restrict__ x, int64_t rows,
                                                                    int64_t blocks_per_row, int64_t ldx,
                                                                    uint8_t* __restrict__ q, uint8_t* __restrict__ scales) {
  __shared__ uint32_t patch[256];
  const int t = threadIdx.x;
  const int64_t row = (int64_t)blockIdx.y * 128 + t / 8, blk = (int64_t)blockIdx.x * 8 + t % 8;
  uint32_t byte = 127u;
  if (row < rows && blk < blocks_per_row) {
    const int64_t at = row * ldx + blk * kMxBlock;
    float v[kMxBlock];
#pragma unroll
    for (int i = 0; i < kMxBlock; i += 8) Load8<In>::run(x, at + i, v + i);
    float amax = 0.f;
#pragma unroll
    for (int i = 0; i < kMxBlock; ++i) amax = __builtin_fmaxf(amax, __builtin_fabsf(v[i]));
    const uint32_t field = __builtin_bit_cast(uint32_t, amax) >> 23;     // as in mx_quantize_kernel
    byte = amax == 0.f ? 127u : (field > 8u ? field - 8u : 0u);
    const float inv = __builtin_bit_cast(float, (254u - byte) << 23);
    uint32_t w[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) w[i] = to_e4m3x4(v[4 * i] * inv, v[4 * i + 1] * inv, v[4 * i + 2] * inv, v[4 * i + 3] * inv);
    u32x4* dst = (u32x4*)(q + row * blocks_per_row * kMxBlock + blk * kMxBlock);
    dst[0] = (u32x4){w[0], w[1], w[2], w[3]};
    dst[1] = (u32x4){w[4], w[5], w[6], w[7]};
  }
  // Byte of (row, block) inside its unit: lane (row % 16 + 16 * (block % 4)) x 8 + (row % 128) / 16 (shuffled_index).
  const int r = t / 8, b = t % 8;
  ((uint8_t*)patch)[(b / 4) * 512 + (r % 16 + 16 * (b % 4)) * 8 + r / 16] = (uint8_t)byte;
  __syncthreads();
  if (t < 256) {
    const int64_t unit_blk = (int64_t)blockIdx.x * 8 + (t / 128) * 4;      // first block of the unit this thread writes to
    if (unit_blk < blocks_per_row) {
      const int64_t unit = (int64_t)blockIdx.y * (blocks_per_row / 4) + unit_blk / 4;
      ((uint32_t*)(scales + unit * 512))[t % 128] = patch[t];
    }
  }
}

template <class In>
int run_quantize(const void* x, int64_t rows, int64_t K, int64_t ldx, void* q, uint8_t* scales, bool shuffled,
                 hipStream_t stream) {
  const int64_t n = (shuffled ? (rows + 255) / 256 * 256 : rows) * (K / kMxBlock);
  if (n == 0) return 0;
  const int64_t blocks = (n + 255) / 256;
  if (blocks >= ((int64_t)1 << 31)) return -1;
  if (shuffled) {
    const int64_t bpr = K / kMxBlock, gx = (bpr + 7) / 8, gy = (rows + 255) / 256 * 2;   // rows padded to 256: whole patches
    if (gy > 65535 || gx >= ((int64_t)1 << 31))      // more than 8 million rows: the one-byte stores
      hipLaunchKernelGGL((mx_quantize_kernel<In, true>), dim3((unsigned)blocks), dim3(256), 0, stream, x, rows, bpr, ldx,
                         (uint8_t*)q, scales);
    else
      hipLaunchKernelGGL((mx_quantize_shuffled_kernel<In>), dim3((unsigned)gx, (unsigned)gy), dim3(1024), 0, stream, x, rows,
                         bpr, ldx, (uint8_t*)q, scales);
  } else
    hipLaunchKernelGGL((mx_quantize_kernel<In, false>), dim3((unsigned)blocks), dim3(256), 0, stream, x, rows,
                       K / kMxBlock, ldx, (uint8_t*)q, scales);
  return hipGetLastError() == hipSuccess ? 0 : -1;
}

}  // namespace

size_t mx_shuffled_bytes(int64_t rows, int64_t K) {
  if (rows <= 0 || K <= 0) return 0;
  return (size_t)((rows + 255) / 256 * 256) * (size_t)(K / kMxBlock);
}

int launch_mx_shuffle(const uint8_t* scales, int64_t rows, int64_t K, int64_t ld, uint8_t* out, hipStream_t stream) {
  return launch_mx_shuffle2(scales, rows, ld, out, nullptr, 0, 0, nullptr, K, stream);
}

// Both operands of a GEMM in one launch (rows_b == 0: only the first).
int launch_mx_shuffle2(const uint8_t* scales_a, int64_t rows_a, int64_t ld_a, uint8_t* out_a,
                       const uint8_t* scales_b, int64_t rows_b, int64_t ld_b, uint8_t* out_b, int64_t K,
                       hipStream_t stream) {
  const MxOperand a = {scales_a, rows_a, ld_a, mx_shuffled_bytes(rows_a, K) / 8, out_a};
  const MxOperand b = {scales_b, rows_b, ld_b, mx_shuffled_bytes(rows_b, K) / 8, out_b};
  if (a.slots + b.slots == 0) return 0;
  const uint64_t blocks = (a.slots + b.slots + 255) / 256;
  if (blocks >= ((uint64_t)1 << 31)) return -1;
  hipLaunchKernelGGL(mx_shuffle_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, a, b, (uint32_t)(K / 128));
  return hipGetLastError() == hipSuccess ? 0 : -1;
}

// in_dtype: 0 bf16, 1 fp16, 3 fp32.
int launch_quantize_mxfp8(const void* x, int in_dtype, int64_t rows, int64_t K, int64_t ldx, void* q,
                          uint8_t* scales, bool shuffled, hipStream_t stream) {
  switch (in_dtype) {
    case 0: return run_quantize<BF16>(x, rows, K, ldx, q, scales, shuffled, stream);
    case 1: return run_quantize<F16>(x, rows, K, ldx, q, scales, shuffled, stream);
    case 3: return run_quantize<float>(x, rows, K, ldx, q, scales, shuffled, stream);
  }
  return -1;
}

}  // namespace mi355
