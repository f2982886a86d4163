// C ABI of the library (declared in include/mi355_gemm.h): argument validation, variant
// selection and dispatch.  Validation runs before any HIP call so that it can be exercised on a
// machine without a GPU.  Counterpart in the reference: the host launcher
// test::gemm_tn_test, kernels/gemm_kernels/sm90a/gemm_test.cu:12-92.
#include "../../include/mi355_gemm.h"

#include "gemm_launch.h"
#include "tile_map.h"

#include <atomic>

namespace {

int elem_bytes(int dtype) { return dtype == MI355_E4M3 ? 1 : 2; }

bool valid_in(int d) { return d == MI355_BF16 || d == MI355_F16 || d == MI355_E4M3; }  // MI355_F32: quantiser only
bool valid_out(int d) { return d == MI355_BF16 || d == MI355_F16; }

// Sizes far beyond what 288 GB of HBM can hold are refused up front, so that none of the size
// arithmetic below (byte counts, tile counts, workspace sizes) can leave 64 bits: every extent and
// row stride is at most 2^40 and every array has at most 2^50 elements.
constexpr int64_t kMaxExtent = (int64_t)1 << 40;
constexpr double kMaxElements = 1125899906842624.0;  // 2^50
bool array_ok(int64_t rows, int64_t ld) {
  return rows <= kMaxExtent && ld <= kMaxExtent && (double)rows * (double)ld <= kMaxElements;
}
bool extents_ok(int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb, int64_t ldc) {
  return K <= kMaxExtent && array_ok(M, lda) && array_ok(N, ldb) && array_ok(M, ldc) && array_ok(M, N) &&
         array_ok(M, K) && array_ok(N, K);
}

// Constraints of the 256x256-tile kernels beyond the generic ones.
bool tile256_ok(int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb, int64_t ldc, int in_dtype) {
  const int64_t es = elem_bytes(in_dtype);
  if (M <= 0 || N <= 0 || K <= 0) return false;
  if ((K * es) % 16 != 0) return false;                     // rows are moved in 16-byte chunks
  if ((lda * es) % 16 != 0 || (ldb * es) % 16 != 0) return false;
  if (N % 4 != 0 || ldc % 4 != 0) return false;             // 8-byte output stores
  // A 256-row panel must stay below 2 GiB: offsets from 2^31 up mark chunks to be dropped.
  if (256 * lda * es >= (int64_t)1 << 31 || 256 * ldb * es >= (int64_t)1 << 31) return false;
  // 32-bit offsets inside a 256-row tile of C and of an fp32 split-K plane (row stride N <= ldc)
  if (256 * ldc * 4 >= (int64_t)1 << 31) return false;
  return true;
}

// Constraints of the small-M streaming kernel.  It wins up to M = 64 ...
constexpr int64_t kSkinnyAutoMaxM = 64;
// ... and up to M = 128 while the 64-column tiles fit the 256 CUs in one round (N <= 16384) and the
// rows of A, which every one of those tiles reads again, stay in an XCD's 4 MiB L2 beside the
// streaming weights (M*K*elem_bytes <= 2.2 MB): measured on 72 bf16 and fp8 problems with M = 96 and
// 128 (N = 2048...16384), -6 % in the geometric mean where the rule applies, from -22 % to +10 %;
// with more tiles the tile kernel is 14-20 % faster, with more bytes of A up to 40 % faster.
// Of those, problems with enough columns and k-steps go to the tile kernel's nine-slot ring instead
// (ring_one_row_deep).
bool auto_streams(int64_t M, int64_t N, int64_t K, int64_t es) {
  if (M <= kSkinnyAutoMaxM) return true;
  if (mi355::ring_one_row_deep(M, N, K, (int)es)) return false;
  return M <= 128 && (N + 63) / 64 <= 256 && M * K * es <= 2200000;
}
// Two workgroups per CU on 256 x 128 tiles, one storing while the other computes: where a tile is
// nearly all epilogue.  The kernel copies 1.5 times the bytes per flop of the 256 x 256 tile and a CU
// takes in no more than about 44 bytes per cycle, so its k loop is 13-17 % slower than the single
// group's (bf16 8192^3: 1392 against 1625 TFLOP/s); what it hides is the store phase.  bf16, against
// the rest of the planner: K = 256 at 16384^2 / 8192 x 16384 / 4096 x 8192 / 8192^2 / 6144^2 14 / 12 /
// 10 / 7 / 1-5 % faster, K = 128 at 16384^2 / 8192^2 10 / 3 %; K = 320 and 384 (five and six k-steps)
// 2 % slower, K = 512 from 2 % faster (8192^2) to 7 % slower (16384 x 8192).  So: 16-bit inputs (the
// kernel has no fp8 form), at most four k-steps, at least two tiles per resident workgroup.
bool auto_alternates(int64_t M, int64_t N, int64_t K, int in_dtype) {
  if (in_dtype == MI355_E4M3) return false;
  const int64_t k_steps = (K * 2 + 127) / 128, tiles = ((M + 255) / 256) * ((N + 127) / 128);
  return k_steps >= 1 && k_steps <= 4 && tiles >= 1024;
}
// Whether the tile kernels write C with non-temporal stores (nt sc1) or keep it in the caches on its way out (sc1).
// Kept when the output (16-bit) is at most 192 MiB and operands and output together at most 288 MiB, a little more
// than the 256 MB Infinity Cache.  Measured, kept against streamed: fp8 8192^3 2-3 % faster, 8192^2 x 1024..2048 6 %,
// bf16 8192^2 x 4096 1.6 %, the two-workgroup kernel at K <= 256 with outputs up to 192 MiB 9-16 %; bf16 8192^3
// (384 MiB in all) 0-0.9 % slower, outputs of 256 MiB and more 0.6-5.7 % slower (that kernel: 22-34 %).
int32_t c_streams(int64_t M, int64_t N, int64_t K, int elem_bytes) {
  const double mib = 1024.0 * 1024.0, out = (double)M * (double)N * 2.0;
  const double total = ((double)M + (double)N) * (double)K * elem_bytes + out;
  return out <= 192.0 * mib && total <= 288.0 * mib ? 0 : 1;
}
bool skinny_ok(int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb, int64_t ldc, int in_dtype) {
  if (M > 256) return false;
  return tile256_ok(M, N, K, lda, ldb, ldc, in_dtype);
}

int check_common(int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb, int64_t ldc,
                 int in_dtype, int out_dtype, int variant) {
  if (!valid_in(in_dtype) || !valid_out(out_dtype)) return MI355_ERR_DTYPE;
  if (variant < MI355_VARIANT_AUTO || variant > MI355_VARIANT_ALTERNATE) return MI355_ERR_VARIANT;
  if (M < 0 || N < 0 || K < 0) return MI355_ERR_SHAPE;
  if (lda < K || ldb < K || ldc < N) return MI355_ERR_SHAPE;
  if (!extents_ok(M, N, K, lda, ldb, ldc)) return MI355_ERR_SHAPE;
  return MI355_OK;
}

int resolve(int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb, int64_t ldc, int in_dtype,
            int variant) {
  if (variant == MI355_VARIANT_AUTO) {
    if (!tile256_ok(M, N, K, lda, ldb, ldc, in_dtype)) return MI355_VARIANT_SIMPLE;
    // A few rows of activations against a large weight matrix: stream the weights.
    if (auto_streams(M, N, K, elem_bytes(in_dtype)) && skinny_ok(M, N, K, lda, ldb, ldc, in_dtype)) return MI355_VARIANT_SKINNY;
    if (auto_alternates(M, N, K, in_dtype)) return MI355_VARIANT_ALTERNATE;
    return MI355_VARIANT_BASIC;
  }
  if (variant == MI355_VARIANT_BASIC || variant == MI355_VARIANT_PINGPONG)
    return tile256_ok(M, N, K, lda, ldb, ldc, in_dtype) ? variant : MI355_ERR_SHAPE;
  if (variant == MI355_VARIANT_SKINNY)
    return skinny_ok(M, N, K, lda, ldb, ldc, in_dtype) ? variant : MI355_ERR_SHAPE;
  if (variant == MI355_VARIANT_ALTERNATE) {
    if (in_dtype == MI355_E4M3) return MI355_ERR_VARIANT;   // 16-bit inputs only
    return tile256_ok(M, N, K, lda, ldb, ldc, in_dtype) ? variant : MI355_ERR_SHAPE;
  }
  return variant;
}

// Repacking: MI355_VARIANT_AUTO turns a problem the tiled kernels cannot address (K*elem_bytes or
// a row stride not a multiple of 16, N or ldc not a multiple of 4, misaligned pointers) into an
// aligned one in the caller's workspace -- A and B copied to zero-padded 16-byte-aligned rows, C
// computed into a padded buffer and copied out -- when the workspace is large enough and the
// problem is big enough to pay for three more passes over the operands.  The generic kernel takes
// about a millisecond per GFLOP; the repacked problem runs at the tiled kernels' rate.
struct Repack {
  bool a, b, c;
  int64_t Kp, Np;                 // padded K (elements) and N
  int64_t ld_ab, ld_c;            // row strides (elements) of the repacked operands and of the padded C:
                                  // multiples of 128 bytes, so that no 128-byte piece of a row straddles
                                  // two cache lines (4096x4096x4104 bf16: 123 us with 8208-byte rows, 98 us
                                  // with 8320-byte rows)
  size_t bytes_a, bytes_b, bytes_c;
};

size_t round_up(size_t x, size_t to) { return (x + to - 1) / to * to; }

bool repack_plan(const void* A, const void* B, const void* C, int64_t M, int64_t N, int64_t K, int64_t lda,
                 int64_t ldb, int64_t ldc, int in_dtype, Repack* r) {
  const int64_t es = elem_bytes(in_dtype);
  if (M <= 0 || N <= 0 || K <= 0) return false;
  if (2.0 * (double)M * (double)N * (double)K < 134217728.0) return false;   // under ~0.1 ms on the generic kernel
  const int64_t per16 = 16 / es;
  r->Kp = (K + per16 - 1) / per16 * per16;
  r->Np = (N + 3) / 4 * 4;
  r->a = r->Kp != K || (lda * es) % 16 != 0 || (uintptr_t)A % 16 != 0;
  r->b = r->Kp != K || (ldb * es) % 16 != 0 || (uintptr_t)B % 16 != 0 || r->Np != N;
  r->c = r->Np != N || ldc % 4 != 0 || (uintptr_t)C % 8 != 0;
  if (!r->a && !r->b && !r->c) return false;
  r->ld_ab = (int64_t)round_up((size_t)(r->Kp * es), 128) / es;
  r->ld_c = (int64_t)round_up((size_t)r->Np, 64);
  r->bytes_a = r->a ? round_up((size_t)M * (size_t)r->ld_ab * (size_t)es, 256) : 0;
  r->bytes_b = r->b ? round_up((size_t)r->Np * (size_t)r->ld_ab * (size_t)es, 256) : 0;
  r->bytes_c = r->c ? round_up((size_t)M * (size_t)r->ld_c * 2, 256) : 0;
  // the repacked problem must be one the tiled kernels take
  return tile256_ok(M, r->Np, r->Kp, r->a ? r->ld_ab : lda, r->b ? r->ld_ab : ldb, r->c ? r->ld_c : ldc, in_dtype);
}

// How a call treats a workspace that is too small for what the plan wants.
//   kLenient    run without (tiles unsplit, generic kernel instead of repacking, ...), as documented
//               for mi355_gemm_tn
//   kStrict     refuse with MI355_ERR_SCRATCH: the workspace is the library's own fixed buffer, and
//               a caller who cannot allocate should hear that the problem is beyond it
//   kStrictDry  the same decisions and return codes, stopping before the first HIP call
enum WorkspaceMode { kLenient, kStrict, kStrictDry };

}  // namespace

// Scratch of mi355_gemm_tn_noalloc: one copy per GPU, held from the moment the code object is
// loaded on that GPU until the process ends.  In host code this name is only a handle for
// hipGetSymbolAddress; the device address differs per GPU and is kept in scratch_address[].
constexpr size_t kScratchBytes = (size_t)MI355_NOALLOC_SCRATCH_BYTES;
static __device__ __align__(256) unsigned char scratch[kScratchBytes];

namespace {

constexpr int kMaxDevices = 64;
std::atomic<void*> scratch_address[kMaxDevices];

// Device address of `scratch` on the current device, looked up once per device.
int scratch_of_current_device(void** out) {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return MI355_ERR_LAUNCH;
  void* p = scratch_address[dev].load(std::memory_order_acquire);
  if (!p) {
    if (hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)) != hipSuccess || !p) return MI355_ERR_LAUNCH;
    scratch_address[dev].store(p, std::memory_order_release);
  }
  *out = p;
  return MI355_OK;
}

int run_gemm(const void* A, const void* B, void* C, int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb,
             int64_t ldc, int in_dtype, int out_dtype, float scale, const float* scale_a, const float* scale_b,
             int variant, void* workspace, size_t workspace_bytes, void* stream, WorkspaceMode mode);

}  // namespace

extern "C" {

int mi355_gemm_version(void) { return (0 << 16) | 2; }

const char* mi355_gemm_strerror(int status) {
  switch (status) {
    case MI355_OK: return "success";
    case MI355_ERR_NULL: return "A, B and C must be non-null device pointers";
    case MI355_ERR_DTYPE: return "unsupported dtype: inputs bf16/fp16/e4m3, output bf16/fp16";
    case MI355_ERR_SHAPE:
      return "shape or leading dimension violates a constraint of the requested variant "
             "(need M,N,K >= 0, lda,ldb >= K, ldc >= N; tiled variants need K*elem_bytes % 16 == 0, "
             "16-byte aligned rows and N % 4 == 0; skinny needs M <= 256)";
    case MI355_ERR_VARIANT: return "unknown variant, or variant not available for this shape/dtype";
    case MI355_ERR_WORKSPACE: return "workspace is NULL or smaller than mi355_gemm_workspace_bytes()";
    case MI355_ERR_LAUNCH: return "HIP runtime rejected the kernel launch";
    case MI355_ERR_ALIGN: return "A and B must be 16-byte aligned and C 8-byte aligned for the tiled variants";
    case MI355_ERR_SCRATCH:
      return "mi355_gemm_tn_noalloc: the problem wants more scratch than the library's built-in buffer of "
             "MI355_NOALLOC_SCRATCH_BYTES holds; call mi355_gemm_tn with a workspace of "
             "mi355_gemm_workspace_bytes() instead";
  }
  return "unknown status code";
}

int mi355_gemm_tile_coord(int64_t block, int64_t tiles_m, int64_t tiles_n, int64_t* tile_m,
                          int64_t* tile_n) {
  if (!tile_m || !tile_n) return MI355_ERR_NULL;
  if (tiles_m <= 0 || tiles_n <= 0 || block < 0) return MI355_ERR_SHAPE;
  if (tiles_m > ((int64_t)1 << 60) / tiles_n) return MI355_ERR_SHAPE;   // the map's arithmetic stays inside 64 bits
  if (block >= tiles_m * tiles_n) return MI355_ERR_SHAPE;
  mi355::tile_coord(block, tiles_m, tiles_n, tile_m, tile_n);
  return MI355_OK;
}

int mi355_gemm_check(int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb, int64_t ldc,
                     int in_dtype, int out_dtype, int variant) {
  int st = check_common(M, N, K, lda, ldb, ldc, in_dtype, out_dtype, variant);
  if (st != MI355_OK) return st;
  int v = resolve(M, N, K, lda, ldb, ldc, in_dtype, variant);
  return v < 0 ? v : MI355_OK;
}

int mi355_gemm_select_variant(int64_t M, int64_t N, int64_t K, int in_dtype) {
  if (!valid_in(in_dtype)) return MI355_ERR_DTYPE;
  if (M < 0 || N < 0 || K < 0 || !extents_ok(M, N, K, K, K, N)) return MI355_ERR_SHAPE;
  return resolve(M, N, K, K, K, N, in_dtype, MI355_VARIANT_AUTO);
}

int mi355_gemm_plan(int64_t M, int64_t N, int64_t K, int in_dtype, int variant, int* tile_rows, int* tile_cols,
                    int* k_splits, int* tail_tiles, int* tail_splits) {
  if (!valid_in(in_dtype)) return MI355_ERR_DTYPE;
  if (variant < MI355_VARIANT_AUTO || variant > MI355_VARIANT_ALTERNATE) return MI355_ERR_VARIANT;
  if (M < 0 || N < 0 || K < 0 || !extents_ok(M, N, K, K, K, N)) return MI355_ERR_SHAPE;
  const int v = resolve(M, N, K, K, K, N, in_dtype, variant);
  if (v < 0) return v;
  int rows = 0, cols = 0, splits = 1, tt = 0, ts = 1;
  const int es = elem_bytes(in_dtype);
  if (v == MI355_VARIANT_SKINNY) {
    rows = M <= 16 ? 16 : M <= 32 ? 32 : M <= 64 ? 64 : M <= 128 ? 128 : 256;
    cols = mi355::stream_tile_cols(M, N, K, es);
    if (cols == 128) rows = 64;   // the wide tile exists with 64 rows only
    splits = mi355::stream_splits(M, N, K, es);
  } else if (v == MI355_VARIANT_PINGPONG) {
    rows = cols = 256;
  } else if (v == MI355_VARIANT_ALTERNATE) {
    rows = 256;
    cols = 128;
  } else if (v == MI355_VARIANT_BASIC) {
    int64_t pm = M, pn = N;   // of two launches (mi355_gemm_pieces) the first one's plan
    if (variant == MI355_VARIANT_AUTO) {
      bool along_m = false;
      const int64_t first = mi355::ring_first_piece(M, N, K, es, &along_m);
      if (first > 0) (along_m ? pm : pn) = first;
    }
    const int tile = mi355::ring_tile_edge(pm, pn, K, es);
    rows = mi355::ring_tile_rows(tile);
    cols = mi355::ring_tile_cols(tile);
    splits = mi355::ring_splits(pm, pn, K, es);
    if (splits == 1) mi355::ring_tail(pm, pn, K, es, &tt, &ts);
  }
  if (tile_rows) *tile_rows = rows;
  if (tile_cols) *tile_cols = cols;
  if (k_splits) *k_splits = splits;
  if (tail_tiles) *tail_tiles = tt;
  if (tail_splits) *tail_splits = ts;
  return v;
}

int mi355_gemm_pieces(int64_t M, int64_t N, int64_t K, int in_dtype, int variant, int64_t* first_rows, int64_t* first_cols) {
  if (first_rows) *first_rows = M;
  if (first_cols) *first_cols = N;
  if (!valid_in(in_dtype) || M <= 0 || N <= 0 || K <= 0 || !extents_ok(M, N, K, K, K, N)) return MI355_ERR_SHAPE;
  if (variant < MI355_VARIANT_AUTO || variant > MI355_VARIANT_ALTERNATE) return MI355_ERR_VARIANT;
  if (variant != MI355_VARIANT_AUTO || resolve(M, N, K, K, K, N, in_dtype, variant) != MI355_VARIANT_BASIC) return 1;
  bool along_m = false;
  const int64_t first = mi355::ring_first_piece(M, N, K, elem_bytes(in_dtype), &along_m);
  if (first <= 0) return 1;
  if (along_m && first_rows) *first_rows = first;
  if (!along_m && first_cols) *first_cols = first;
  return 2;
}

size_t mi355_gemm_workspace_bytes(int64_t M, int64_t N, int64_t K, int in_dtype, int variant) {
  if (!valid_in(in_dtype) || M <= 0 || N <= 0 || K <= 0) return 0;
  if (variant < MI355_VARIANT_AUTO || variant > MI355_VARIANT_ALTERNATE) return 0;
  if (!extents_ok(M, N, K, K, K, N)) return 0;
  const int v = resolve(M, N, K, K, K, N, in_dtype, variant);
  if (v == MI355_VARIANT_SIMPLE && variant == MI355_VARIANT_AUTO) {
    // contiguous, aligned operands assumed: only K and N decide what is repacked
    Repack r;
    if (!repack_plan(nullptr, nullptr, nullptr, M, N, K, K, K, N, in_dtype, &r)) return 0;
    return r.bytes_a + r.bytes_b + r.bytes_c + mi355_gemm_workspace_bytes(M, r.Np, r.Kp, in_dtype, MI355_VARIANT_AUTO);
  }
  if (v == MI355_VARIANT_BASIC && variant == MI355_VARIANT_AUTO) {   // two launches: what the hungrier piece wants
    bool along_m = false;
    const int64_t first = mi355::ring_first_piece(M, N, K, elem_bytes(in_dtype), &along_m);
    if (first > 0) {
      const size_t a = mi355_gemm_workspace_bytes(along_m ? first : M, along_m ? N : first, K, in_dtype, MI355_VARIANT_BASIC);
      const size_t b = mi355_gemm_workspace_bytes(along_m ? M - first : M, along_m ? N : N - first, K, in_dtype, MI355_VARIANT_BASIC);
      return a > b ? a : b;
    }
  }
  int splits = 1;
  if (v == MI355_VARIANT_SKINNY) splits = mi355::stream_splits(M, N, K, elem_bytes(in_dtype));
  else if (v == MI355_VARIANT_BASIC) splits = mi355::ring_splits(M, N, K, elem_bytes(in_dtype));
  if (splits > 1) return (size_t)splits * (size_t)M * (size_t)N * sizeof(float);
  if (v == MI355_VARIANT_BASIC) {
    int tail_tiles, tail_splits;
    return mi355::ring_tail(M, N, K, elem_bytes(in_dtype), &tail_tiles, &tail_splits);
  }
  return 0;
}

int mi355_quantize_e4m3(const void* x, int x_dtype, int64_t n, void* x_q, float* scale_amax, void* stream) {
  if (x_dtype != MI355_BF16 && x_dtype != MI355_F16 && x_dtype != MI355_F32) return MI355_ERR_DTYPE;
  if (n < 0 || (double)n > kMaxElements) return MI355_ERR_SHAPE;
  if (!scale_amax || (n > 0 && (!x || !x_q))) return MI355_ERR_NULL;
  if ((uintptr_t)x % 16 != 0 || (uintptr_t)x_q % 8 != 0 || (uintptr_t)scale_amax % 4 != 0) return MI355_ERR_ALIGN;
  return mi355::launch_quantize_e4m3(x, x_dtype, n, x_q, scale_amax, (hipStream_t)stream) == 0 ? MI355_OK
                                                                                              : MI355_ERR_LAUNCH;
}

size_t mi355_mx_shuffled_bytes(int64_t rows, int64_t K) {
  if (rows <= 0 || K <= 0 || K % 128 != 0 || !array_ok(rows, K)) return 0;
  return mi355::mx_shuffled_bytes(rows, K);
}

int mi355_mx_shuffle_scales(const uint8_t* scales, int64_t rows, int64_t K, int64_t ld, uint8_t* out, void* stream) {
  if (rows < 0 || K < 0 || K % 128 != 0 || ld < K / 32) return MI355_ERR_SHAPE;
  if (!array_ok(rows, K) || !array_ok(rows, ld)) return MI355_ERR_SHAPE;
  if (rows == 0 || K == 0) return MI355_OK;
  if (!scales || !out) return MI355_ERR_NULL;
  if ((uintptr_t)out % 8 != 0) return MI355_ERR_ALIGN;
  return mi355::launch_mx_shuffle(scales, rows, K, ld, out, (hipStream_t)stream) == 0 ? MI355_OK : MI355_ERR_LAUNCH;
}

int mi355_quantize_mxfp8(const void* x, int x_dtype, int64_t rows, int64_t K, int64_t ldx, void* x_q,
                         uint8_t* scales, int scales_shuffled, void* stream) {
  if (x_dtype != MI355_BF16 && x_dtype != MI355_F16 && x_dtype != MI355_F32) return MI355_ERR_DTYPE;
  if (rows < 0 || K < 0 || K % 32 != 0 || ldx < K || !array_ok(rows, ldx)) return MI355_ERR_SHAPE;
  if (scales_shuffled && K % 128 != 0) return MI355_ERR_SHAPE;
  if (rows == 0 || K == 0) return MI355_OK;
  if (!x || !x_q || !scales) return MI355_ERR_NULL;
  const int64_t es = x_dtype == MI355_F32 ? 4 : 2;
  if ((uintptr_t)x % 16 != 0 || (ldx * es) % 16 != 0 || (uintptr_t)x_q % 16 != 0) return MI355_ERR_ALIGN;
  if (scales_shuffled && (uintptr_t)scales % 8 != 0) return MI355_ERR_ALIGN;   // as mi355_mx_shuffle_scales wants its output
  return mi355::launch_quantize_mxfp8(x, x_dtype, rows, K, ldx, x_q, scales, scales_shuffled != 0, (hipStream_t)stream) == 0
             ? MI355_OK : MI355_ERR_LAUNCH;
}

int mi355_gemm_mx_check(int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb, int64_t ldc, int out_dtype) {
  if (!valid_out(out_dtype)) return MI355_ERR_DTYPE;
  if (M < 0 || N < 0 || K < 0) return MI355_ERR_SHAPE;
  if (lda < K || ldb < K || ldc < N) return MI355_ERR_SHAPE;
  if (!extents_ok(M, N, K, lda, ldb, ldc)) return MI355_ERR_SHAPE;
  if (K % 128 != 0) return MI355_ERR_SHAPE;
  if (M == 0 || N == 0) return MI355_OK;
  if (K > 0 && !tile256_ok(M, N, K, lda, ldb, ldc, MI355_E4M3)) return MI355_ERR_SHAPE;
  // 32-bit offsets into the shuffled scale arrays
  if (mi355::mx_shuffled_bytes(M, K) >= ((size_t)1 << 31) || mi355::mx_shuffled_bytes(N, K) >= ((size_t)1 << 31))
    return MI355_ERR_SHAPE;
  return MI355_OK;
}

namespace {
// Partial results of the block-scaled GEMM's K split or tail split (the planner's, as for plain fp8).
// Whether a block-scaled problem goes to the streaming kernel, and with how many K splits.
int mx_stream_splits(int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb, int64_t ldc) {
  if (M > kSkinnyAutoMaxM || !skinny_ok(M, N, K, lda, ldb, ldc, MI355_E4M3)) return 0;
  return mi355::stream_splits(M, N, K, 1, true);
}

size_t mx_partial_bytes(int64_t M, int64_t N, int64_t K, int* splits, int* tail_tiles, int* tail_splits) {
  int s = mi355::ring_splits(M, N, K, 1, true), tt = 0, ts = 1;
  size_t bytes = s > 1 ? (size_t)s * (size_t)M * (size_t)N * sizeof(float) : mi355::ring_tail(M, N, K, 1, &tt, &ts, true);
  if (splits) *splits = s;
  if (tail_tiles) *tail_tiles = tt;
  if (tail_splits) *tail_splits = ts;
  return bytes;
}
}  // namespace

size_t mi355_gemm_mx_workspace_bytes(int64_t M, int64_t N, int64_t K, int scales_shuffled) {
  if (M <= 0 || N <= 0 || K <= 0 || K % 128 != 0 || !extents_ok(M, N, K, K, K, N)) return 0;
  const int ss = mx_stream_splits(M, N, K, K, K, N);
  size_t partial = ss ? (ss > 1 ? (size_t)ss * (size_t)M * (size_t)N * sizeof(float) : 0)
                      : mx_partial_bytes(M, N, K, nullptr, nullptr, nullptr);
  if (!ss) {   // two launches (as for plain operands): what the hungrier piece wants
    bool along_m = false;
    if (const int64_t first = mi355::ring_first_piece(M, N, K, 1, &along_m)) {
      const size_t a = mx_partial_bytes(along_m ? first : M, along_m ? N : first, K, nullptr, nullptr, nullptr);
      const size_t b = mx_partial_bytes(along_m ? M - first : M, along_m ? N : N - first, K, nullptr, nullptr, nullptr);
      partial = a > b ? a : b;
    }
  }
  return partial + (scales_shuffled ? 0 : mi355::mx_shuffled_bytes(M, K) + mi355::mx_shuffled_bytes(N, K));
}

int mi355_gemm_tn_mxfp8(const void* A_q, const void* B_q, void* C, int64_t M, int64_t N, int64_t K, int64_t lda,
                        int64_t ldb, int64_t ldc, const uint8_t* scale_a, int64_t ld_scale_a,
                        const uint8_t* scale_b, int64_t ld_scale_b, int scales_shuffled, int out_dtype,
                        void* workspace, size_t workspace_bytes, void* stream) {
  int st = mi355_gemm_mx_check(M, N, K, lda, ldb, ldc, out_dtype);
  if (st != MI355_OK) return st;
  if (M == 0 || N == 0) return MI355_OK;
  if (!C) return MI355_ERR_NULL;
  hipStream_t s = (hipStream_t)stream;
  mi355::GemmArgs g;
  g.A = A_q; g.B = B_q; g.C = C;
  g.M = M; g.N = N; g.K = K;
  g.lda = lda; g.ldb = ldb; g.ldc = ldc;
  g.scale = 1.0f;
  g.splits = 1;
  g.partial = nullptr;
  g.tail_tiles = 0;
  g.tail_splits = 1;
  g.scale_a = g.scale_b = nullptr;
  g.mx_a = g.mx_b = nullptr;
  g.c_streams = c_streams(M, N, K, 1);
  if (K == 0) {  // an empty sum: zeros, written by the generic kernel
    g.tiles_m = g.tiles_n = 0;
    return mi355::launch_simple(g, MI355_E4M3, out_dtype, s) == 0 ? MI355_OK : MI355_ERR_LAUNCH;
  }
  if (!A_q || !B_q || !scale_a || !scale_b) return MI355_ERR_NULL;
  if ((uintptr_t)A_q % 16 != 0 || (uintptr_t)B_q % 16 != 0 || (uintptr_t)C % 8 != 0) return MI355_ERR_ALIGN;
  size_t used = 0;  // bytes of the workspace taken by the shuffled scales
  if (scales_shuffled) {
    if ((uintptr_t)scale_a % 8 != 0 || (uintptr_t)scale_b % 8 != 0) return MI355_ERR_ALIGN;
    g.mx_a = scale_a;
    g.mx_b = scale_b;
  } else {
    if (ld_scale_a < K / 32 || ld_scale_b < K / 32) return MI355_ERR_SHAPE;
    if (!array_ok(M, ld_scale_a) || !array_ok(N, ld_scale_b)) return MI355_ERR_SHAPE;
    const size_t bytes_a = mi355::mx_shuffled_bytes(M, K), bytes_b = mi355::mx_shuffled_bytes(N, K);
    if (!workspace || workspace_bytes < bytes_a + bytes_b || (uintptr_t)workspace % 16 != 0) return MI355_ERR_WORKSPACE;
    uint8_t* wa = (uint8_t*)workspace;
    uint8_t* wb = wa + bytes_a;  // bytes_a is a multiple of 1024
    if (mi355::launch_mx_shuffle2(scale_a, M, ld_scale_a, wa, scale_b, N, ld_scale_b, wb, K, s) != 0) return MI355_ERR_LAUNCH;
    g.mx_a = wa;
    g.mx_b = wb;
    used = bytes_a + bytes_b;
  }
  // A few rows of activations: stream the weights, as for plain fp8 (when the workspace holds the
  // partial results of its K split, if it has one; otherwise the tile kernel below takes it).
  if (const int ss = mx_stream_splits(M, N, K, lda, ldb, ldc)) {
    const size_t need = ss > 1 ? (size_t)ss * (size_t)M * (size_t)N * sizeof(float) : 0;
    if (!need || (workspace && (uintptr_t)workspace % 16 == 0 && workspace_bytes >= used + need)) {
      g.tiles_m = g.tiles_n = 0;
      return mi355::launch_stream_mx(g, out_dtype, ss, (uint8_t*)workspace + used, s) == 0 ? MI355_OK : MI355_ERR_LAUNCH;
    }
  }
  // The tile kernel on rows [m0, m0 + m) of A and rows [n0, n0 + n) of B (multiples of 256 but for the last).
  // K split or tail split when the rest of the workspace holds the partial results (optional, as
  // for the other tiled kernels: without it the tiles run unsplit).
  const auto tiles_of_piece = [&](int64_t m0, int64_t m, int64_t n0, int64_t n) {
    mi355::GemmArgs p = g;
    p.A = (const uint8_t*)A_q + m0 * lda;
    p.B = (const uint8_t*)B_q + n0 * ldb;
    p.C = (uint8_t*)C + (m0 * ldc + n0) * 2;                              // 16-bit output
    p.mx_a = g.mx_a + (m0 / 128) * (K / 128) * 512;                       // one 512-byte unit per 128 rows and k-step
    p.mx_b = g.mx_b + (n0 / 128) * (K / 128) * 512;
    p.M = m;
    p.N = n;
    p.c_streams = c_streams(m, n, K, 1);
    int splits, tail_tiles, tail_splits;
    const size_t partial = mx_partial_bytes(m, n, K, &splits, &tail_tiles, &tail_splits);
    if (partial && workspace && (uintptr_t)workspace % 16 == 0 && workspace_bytes >= used + partial) {
      p.partial = (float*)((uint8_t*)workspace + used);  // used is a multiple of 1024
      p.splits = splits;
      p.tail_tiles = tail_tiles;
      p.tail_splits = tail_splits;
    }
    const int tile = mi355::ring_tile_edge(m, n, K, 1, true);
    p.tiles_m = (m + mi355::ring_tile_rows(tile) - 1) / mi355::ring_tile_rows(tile);
    p.tiles_n = (n + mi355::ring_tile_cols(tile) - 1) / mi355::ring_tile_cols(tile);
    return mi355::launch_tile_ring_mx(p, out_dtype, tile, s) == 0 ? MI355_OK : MI355_ERR_LAUNCH;
  };
  // Two launches where a cut spares a partly filled last round of workgroups, as for plain operands (ring_first_piece).
  bool along_m = false;
  const int64_t first = mi355::ring_first_piece(M, N, K, 1, &along_m);
  if (first <= 0) return tiles_of_piece(0, M, 0, N);
  st = along_m ? tiles_of_piece(0, first, 0, N) : tiles_of_piece(0, M, 0, first);
  if (st != MI355_OK) return st;
  return along_m ? tiles_of_piece(first, M - first, 0, N) : tiles_of_piece(0, M, first, N - first);
}

int mi355_gemm_tn(const void* A, const void* B, void* C, int64_t M, int64_t N, int64_t K,
                  int64_t lda, int64_t ldb, int64_t ldc, int in_dtype, int out_dtype, float scale,
                  int variant, void* workspace, size_t workspace_bytes, void* stream) {
  return mi355_gemm_tn_scaled(A, B, C, M, N, K, lda, ldb, ldc, in_dtype, out_dtype, scale, nullptr, nullptr,
                              variant, workspace, workspace_bytes, stream);
}

int mi355_gemm_tn_scaled(const void* A, const void* B, void* C, int64_t M, int64_t N, int64_t K,
                         int64_t lda, int64_t ldb, int64_t ldc, int in_dtype, int out_dtype, float scale,
                         const float* scale_a, const float* scale_b, int variant, void* workspace,
                         size_t workspace_bytes, void* stream) {
  return run_gemm(A, B, C, M, N, K, lda, ldb, ldc, in_dtype, out_dtype, scale, scale_a, scale_b, variant, workspace,
                  workspace_bytes, stream, kLenient);
}

int mi355_gemm_tn_noalloc(const void* A, const void* B, void* C, int64_t M, int64_t N, int64_t K,
                          int64_t lda, int64_t ldb, int64_t ldc, int in_dtype, int out_dtype, float scale,
                          int variant, void* stream) {
  // First the whole decision path without a HIP call (argument errors and MI355_ERR_SCRATCH come from
  // here, so they can be provoked on a machine without a GPU); the stand-in address only has to
  // be non-null and aligned like the real one.
  int st = run_gemm(A, B, C, M, N, K, lda, ldb, ldc, in_dtype, out_dtype, scale, nullptr, nullptr, variant,
                    (void*)(uintptr_t)256, kScratchBytes, stream, kStrictDry);
  if (st != MI355_OK || M == 0 || N == 0) return st;
  void* ws = nullptr;
  st = scratch_of_current_device(&ws);
  if (st != MI355_OK) return st;
  return run_gemm(A, B, C, M, N, K, lda, ldb, ldc, in_dtype, out_dtype, scale, nullptr, nullptr, variant, ws,
                  kScratchBytes, stream, kStrict);
}

}  // extern "C"

namespace {

int run_gemm(const void* A, const void* B, void* C, int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb,
             int64_t ldc, int in_dtype, int out_dtype, float scale, const float* scale_a, const float* scale_b,
             int variant, void* workspace, size_t workspace_bytes, void* stream, WorkspaceMode mode) {
  const bool strict = mode != kLenient, dry = mode == kStrictDry;
  int st = check_common(M, N, K, lda, ldb, ldc, in_dtype, out_dtype, variant);
  if (st != MI355_OK) return st;
  if (M == 0 || N == 0) return MI355_OK;  // nothing to write
  if (!C || (K > 0 && (!A || !B))) return MI355_ERR_NULL;  // K == 0 reads no operand
  int v = resolve(M, N, K, lda, ldb, ldc, in_dtype, variant);
  if (v < 0) return v;

  mi355::GemmArgs g;
  g.A = A; g.B = B; g.C = C;
  g.M = M; g.N = N; g.K = K;
  g.lda = lda; g.ldb = ldb; g.ldc = ldc;
  g.scale = scale;
  g.splits = 1;
  g.partial = nullptr;
  g.tail_tiles = 0;
  g.tail_splits = 1;
  g.scale_a = scale_a;
  g.scale_b = scale_b;
  g.mx_a = g.mx_b = nullptr;
  g.c_streams = c_streams(M, N, K, in_dtype == MI355_E4M3 ? 1 : 2);
  hipStream_t s = (hipStream_t)stream;

  if (v == MI355_VARIANT_BASIC || v == MI355_VARIANT_PINGPONG || v == MI355_VARIANT_SKINNY || v == MI355_VARIANT_ALTERNATE) {
    const bool aligned = ((uintptr_t)A % 16 == 0) && ((uintptr_t)B % 16 == 0) && ((uintptr_t)C % 8 == 0);
    if (!aligned) {
      if (variant != MI355_VARIANT_AUTO) return MI355_ERR_ALIGN;
      v = MI355_VARIANT_SIMPLE;
    }
  }
  if (v == MI355_VARIANT_SIMPLE && variant == MI355_VARIANT_AUTO && workspace && (uintptr_t)workspace % 256 == 0) {
    Repack r;
    if (repack_plan(A, B, C, M, N, K, lda, ldb, ldc, in_dtype, &r)) {
      const size_t packed = r.bytes_a + r.bytes_b + r.bytes_c;
      // What the repacked (aligned) problem wants for its own splits.  The streaming kernel insists
      // on the workspace of its K split, so a lenient call repacks only when the rest covers it.
      const size_t inner = mi355_gemm_workspace_bytes(M, r.Np, r.Kp, in_dtype, MI355_VARIANT_AUTO);
      const bool inner_streams = mi355_gemm_select_variant(M, r.Np, r.Kp, in_dtype) == MI355_VARIANT_SKINNY;
      const bool fits = workspace_bytes >= packed && (workspace_bytes - packed >= inner || (!strict && !inner_streams));
      if (strict && !fits) return MI355_ERR_SCRATCH;
      if (fits) {
        if (dry) return MI355_OK;
        const int64_t es = elem_bytes(in_dtype);
        uint8_t* wa = (uint8_t*)workspace;
        uint8_t* wb = wa + r.bytes_a;
        uint8_t* wc = wb + r.bytes_b;
        uint8_t* rest = wc + r.bytes_c;
        const size_t rest_bytes = workspace_bytes - packed;
        if (r.a && mi355::launch_repack_rows(A, M, K * es, lda * es, wa, M, r.ld_ab * es, (int)es, s) != 0) return MI355_ERR_LAUNCH;
        if (r.b && mi355::launch_repack_rows(B, N, K * es, ldb * es, wb, r.Np, r.ld_ab * es, (int)es, s) != 0) return MI355_ERR_LAUNCH;
        st = run_gemm(r.a ? wa : A, r.b ? wb : B, r.c ? (void*)wc : C, M, r.Np, r.Kp, r.a ? r.ld_ab : lda,
                      r.b ? r.ld_ab : ldb, r.c ? r.ld_c : ldc, in_dtype, out_dtype, scale, scale_a, scale_b,
                      MI355_VARIANT_AUTO, rest_bytes ? rest : nullptr, rest_bytes, stream, mode);
        if (st != MI355_OK) return st;
        if (r.c && mi355::launch_copy_out(wc, M, N, r.ld_c, C, ldc, s) != 0) return MI355_ERR_LAUNCH;
        return MI355_OK;
      }
    }
  }
  if (variant == MI355_VARIANT_AUTO && v == MI355_VARIANT_BASIC) {
    // Two launches where the planner finds a cut that spares a partly filled last round (ring_first_piece): each
    // piece is the single-group kernel's problem of its own, with its own tile, splits and store policy, one after
    // the other on the stream and through the same workspace.
    bool along_m = false;
    const int64_t first = mi355::ring_first_piece(M, N, K, elem_bytes(in_dtype), &along_m);
    if (first > 0) {
      const int64_t es = elem_bytes(in_dtype);
      st = run_gemm(A, B, C, along_m ? first : M, along_m ? N : first, K, lda, ldb, ldc, in_dtype, out_dtype, scale, scale_a,
                    scale_b, MI355_VARIANT_BASIC, workspace, workspace_bytes, stream, mode);
      if (st != MI355_OK) return st;
      const uint8_t* a2 = (const uint8_t*)A + (along_m ? first * lda * es : 0);
      const uint8_t* b2 = (const uint8_t*)B + (along_m ? 0 : first * ldb * es);
      uint8_t* c2 = (uint8_t*)C + (along_m ? first * ldc : first) * 2;   // 16-bit output
      return run_gemm(a2, b2, c2, along_m ? M - first : M, along_m ? N : N - first, K, lda, ldb, ldc, in_dtype, out_dtype, scale,
                      scale_a, scale_b, MI355_VARIANT_BASIC, workspace, workspace_bytes, stream, mode);
    }
  }
  int rc;
  // The streaming kernel's split count depends on the shape only, never on the leading dimensions,
  // so it matches what mi355_gemm_workspace_bytes reported.  Its K split needs the workspace: an
  // explicit MI355_VARIANT_SKINNY without it is an error, MI355_VARIANT_AUTO goes to the tile
  // kernel instead, whose split is optional.
  const int stream_s = v == MI355_VARIANT_SKINNY ? mi355::stream_splits(M, N, K, elem_bytes(in_dtype)) : 1;
  const size_t stream_need = stream_s > 1 ? (size_t)stream_s * (size_t)M * (size_t)N * sizeof(float) : 0;
  if (stream_need && (!workspace || workspace_bytes < stream_need || (uintptr_t)workspace % 16 != 0)) {
    if (strict) return MI355_ERR_SCRATCH;
    if (variant != MI355_VARIANT_AUTO) return MI355_ERR_WORKSPACE;
    v = MI355_VARIANT_BASIC;   // whatever the streaming kernel takes the tile kernel takes too
  }
  if (v == MI355_VARIANT_SKINNY) {
    if (dry) return MI355_OK;
    const int splits = stream_s;
    g.tiles_m = g.tiles_n = 0;
    rc = mi355::launch_stream(g, in_dtype, out_dtype, splits, workspace, s);
  } else if (v == MI355_VARIANT_BASIC || v == MI355_VARIANT_PINGPONG) {
    const int tile = v == MI355_VARIANT_PINGPONG ? 256 : mi355::ring_tile_edge(M, N, K, elem_bytes(in_dtype));
    if (v == MI355_VARIANT_BASIC) {
      // Both kinds of K split are optional for this kernel: without a (large enough, aligned)
      // workspace a lenient call runs the same tiles unsplit, slower but with the same result contract.
      const auto usable = [&](size_t need) {
        return need && workspace && workspace_bytes >= need && (uintptr_t)workspace % 16 == 0;
      };
      const int splits = mi355::ring_splits(M, N, K, elem_bytes(in_dtype));
      g.partial = (float*)workspace;
      if (splits > 1) {
        const size_t need = (size_t)splits * (size_t)M * (size_t)N * sizeof(float);
        if (usable(need)) g.splits = splits;
        else if (strict) return MI355_ERR_SCRATCH;
      } else {
        int tail_tiles, tail_splits;
        const size_t need = mi355::ring_tail(M, N, K, elem_bytes(in_dtype), &tail_tiles, &tail_splits);
        if (usable(need)) {
          g.tail_tiles = tail_tiles;
          g.tail_splits = tail_splits;
        } else if (strict && need) {
          return MI355_ERR_SCRATCH;
        }
      }
    }
    if (dry) return MI355_OK;
    g.tiles_m = (M + mi355::ring_tile_rows(tile) - 1) / mi355::ring_tile_rows(tile);
    g.tiles_n = (N + mi355::ring_tile_cols(tile) - 1) / mi355::ring_tile_cols(tile);
    rc = v == MI355_VARIANT_PINGPONG ? mi355::launch_tile256_pingpong(g, in_dtype, out_dtype, s)
                                     : mi355::launch_tile_ring(g, in_dtype, out_dtype, tile, s);
  } else if (v == MI355_VARIANT_ALTERNATE) {
    if (dry) return MI355_OK;
    g.tiles_m = (M + 255) / 256;
    g.tiles_n = (N + 127) / 128;
    rc = mi355::launch_tile_alternate(g, in_dtype, out_dtype, s);
  } else {
    if (dry) return MI355_OK;
    g.tiles_m = g.tiles_n = 0;
    rc = mi355::launch_simple(g, in_dtype, out_dtype, s);
  }
  return rc == 0 ? MI355_OK : MI355_ERR_LAUNCH;
}

}  // namespace
