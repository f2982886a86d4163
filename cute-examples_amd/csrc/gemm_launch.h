// Host-side plumbing shared by the kernel translation units and the C ABI.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace mi355 {

// Kernel argument block.  Leading dimensions are in elements.
struct GemmArgs {
  const void* A;
  const void* B;
  void* C;
  int64_t M, N, K;
  int64_t lda, ldb, ldc;
  int64_t tiles_m, tiles_n;
  float scale;
  // K split: with splits > 1 every (tile, split) pair is a work item that covers k-steps
  // [split*steps/splits, (split+1)*steps/splits) and writes its unscaled fp32 partial tile to
  // partial[split][M][N]; launch_splitk_reduce then adds the splits in order, scales and rounds.
  int32_t splits;
  float* partial;
  // Tail split (single-group tile kernel only, splits == 1): the last tail_tiles tiles in tile-map
  // order are cut tail_splits ways along K, so that the last, partly filled round of workgroups
  // takes 1/tail_splits of a tile's time.  Their fp32 partial tiles go to
  // partial[split][tail tile][tile edge][tile edge] and launch_tail_reduce writes those tiles of C.
  int32_t tail_tiles, tail_splits;
  // Optional device-resident factors (one float each, or null) multiplied into scale by the
  // kernel that writes C, so that per-tensor fp8 scales never have to visit the host.
  const float* scale_a;
  const float* scale_b;
  // Non-zero when operands and output together exceed what the Infinity Cache holds: the tile kernels then write C
  // with non-temporal stores (tile_store.h).
  int32_t c_streams;
  // Block scales (MX) of A and of B in the shuffled layout, or null.
  const uint8_t* mx_a;
  const uint8_t* mx_b;
};

// Effective output scale; wave-uniform, read once per workgroup.
#if defined(__HIPCC__)
__device__ __forceinline__ float output_scale(const GemmArgs& g) {
  float s = g.scale;
  if (g.scale_a) s *= *g.scale_a;
  if (g.scale_b) s *= *g.scale_b;
  return s;
}
#endif

// Each returns 0 after a successful enqueue, non-zero if the runtime rejected the launch.
// in_dtype / out_dtype use the numbering of enum mi355_dtype.
int launch_tile256_pingpong(const GemmArgs& g, int in_dtype, int out_dtype, hipStream_t stream);
// Two workgroups per CU on 256x128 tiles (g.tiles_n counts 128-column tiles); bf16 / fp16 inputs only.
int launch_tile_alternate(const GemmArgs& g, int in_dtype, int out_dtype, hipStream_t stream);
// Single-wave-group ring kernel.  `tile` is 256 or 128 (square tiles) or kRingTile256x128 (256 rows
// of A by 128 rows of B); ring_tile_edge, ring_splits and ring_tail are pure host heuristics.
constexpr int kRingTile256x128 = 384;
// 128 x 128 tile on the nine-slot ring (four k-steps of copies in flight, one workgroup per CU).
constexpr int kRingTile128Deep = 129;
// The same ring without the staggered start of the k-steps: for tiles that share rows of A and B through the L2.
constexpr int kRingTile128DeepPlain = 130;
// One row of 128 x 128 tiles that the tile kernel runs on the nine-slot ring, also where the streaming kernel could
// take the problem (pure host function).
bool ring_one_row_deep(int64_t M, int64_t N, int64_t K, int elem_bytes);
inline int ring_tile_rows(int tile) { return tile == 128 || tile == kRingTile128Deep || tile == kRingTile128DeepPlain ? 128 : 256; }
inline int ring_tile_cols(int tile) { return tile == 256 ? 256 : 128; }
// block_scaled: for the kernel with block scales, which exists on the five-slot ring only.
int ring_tile_edge(int64_t M, int64_t N, int64_t K, int elem_bytes, bool block_scaled = false);
int ring_splits(int64_t M, int64_t N, int64_t K, int elem_bytes, bool block_scaled = false);
// Whether MI355_VARIANT_AUTO runs the problem as two launches of the single-group kernel: the first piece's extent
// along N (along M with *along_m set), or 0 for one launch.  Pure host heuristic; plain operands only.
int64_t ring_first_piece(int64_t M, int64_t N, int64_t K, int elem_bytes, bool* along_m);
// C = rne(scale * sum_s partial[s]) for partial laid out [splits][M][N] in fp32.
int launch_splitk_reduce(const float* partial, const GemmArgs& g, int out_dtype, hipStream_t stream);
int launch_tile_ring(const GemmArgs& g, int in_dtype, int out_dtype, int tile, hipStream_t stream);
// Tail split the single-group kernel would use for this problem (pure host heuristic): returns the
// workspace bytes it needs (0 = no tail split) and sets *tail_tiles, *tail_splits.
size_t ring_tail(int64_t M, int64_t N, int64_t K, int elem_bytes, int* tail_tiles, int* tail_splits, bool block_scaled = false);
int launch_tile_ring_mx(const GemmArgs& g, int out_dtype, int tile, hipStream_t stream);
// Per-input-type halves of launch_tile_ring (one translation unit each).
int launch_tile_ring_bf16(const GemmArgs& g, int out_dtype, int tile, hipStream_t stream);
int launch_tile_ring_f16(const GemmArgs& g, int out_dtype, int tile, hipStream_t stream);
int launch_tile_ring_e4m3(const GemmArgs& g, int out_dtype, int tile, hipStream_t stream);
// Block scales: bytes of the shuffled layout for `rows` rows and K elements per row; the shuffle
// itself (natural (rows, K/32) row-major bytes -> shuffled); and the MX quantiser
// (x (rows, K) -> e4m3 elements + natural-layout E8M0 scales).
size_t mx_shuffled_bytes(int64_t rows, int64_t K);
int launch_mx_shuffle(const uint8_t* scales, int64_t rows, int64_t K, int64_t ld, uint8_t* out, hipStream_t stream);
int launch_mx_shuffle2(const uint8_t* scales_a, int64_t rows_a, int64_t ld_a, uint8_t* out_a, const uint8_t* scales_b,
                       int64_t rows_b, int64_t ld_b, uint8_t* out_b, int64_t K, hipStream_t stream);
int launch_quantize_mxfp8(const void* x, int in_dtype, int64_t rows, int64_t K, int64_t ldx, void* q,
                          uint8_t* scales, bool shuffled, hipStream_t stream);
// Skinny (small-M) weight-streaming kernel.  stream_splits is a pure host function.
int stream_splits(int64_t M, int64_t N, int64_t K, int elem_bytes, bool mx = false);  // mx: block scales ride along
int stream_tile_cols(int64_t M, int64_t N, int64_t K, int elem_bytes, bool mx = false);  // rows of W per workgroup: 64 or 128
int launch_stream_mx(const GemmArgs& g, int out_dtype, int splits, void* workspace, hipStream_t stream);
int launch_stream(const GemmArgs& g, int in_dtype, int out_dtype, int splits, void* workspace, hipStream_t stream);
// Per-tensor e4m3 quantisation (amax -> scale -> cast); scale_amax points to two floats.
int launch_quantize_e4m3(const void* x, int in_dtype, int64_t n, void* q, float* scale_amax, hipStream_t stream);
int launch_simple(const GemmArgs& g, int in_dtype, int out_dtype, hipStream_t stream);
// Repacking for problems the tiled kernels cannot address (gemm_tn_simple.hip): rows of `row_bytes`
// bytes with stride src_ld bytes -> 16-byte aligned rows with stride dst_ld bytes, the tail of every
// row and the rows from `rows` up to dst_rows zero-filled; and a (rows x cols) block of 16-bit
// elements with row stride src_ld elements -> row stride dst_ld elements at any 2-byte alignment.
int launch_repack_rows(const void* src, int64_t rows, int64_t row_bytes, int64_t src_ld, void* dst, int64_t dst_rows,
                       int64_t dst_ld, int elem_bytes, hipStream_t stream);
int launch_copy_out(const void* src, int64_t rows, int64_t cols, int64_t src_ld, void* dst, int64_t dst_ld,
                    hipStream_t stream);

}  // namespace mi355
