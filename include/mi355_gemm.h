/*
 * mi355_gemm.h — C ABI of the MI355X (gfx950) dense GEMM library.
 *
 * Every entry point computes C[M,N] = scale * A[M,K] · B[N,K]^T with both operands
 * K-contiguous ("TN"), fp32 accumulation on the matrix cores and a round-to-nearest-even
 * down-conversion of the result.  Pointers are device pointers; nothing here allocates,
 * synchronises or touches global mutable state, so calls are re-entrant and may be issued
 * from several host threads on different streams.
 *
 * The functions replace the reference's host launcher
 *   test::gemm_tn_test(const torch::Tensor A, const torch::Tensor B, torch::Tensor C)
 *   (kernels/gemm_kernels/sm90a/gemm_test.cu:12-92, bound at
 *    kernels/gemm_kernels/__init__.cpp:7-8)
 * with plain pointers and sizes so that any host language can bind them.
 */
#ifndef MI355_GEMM_H
#define MI355_GEMM_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Element types.  Inputs: BF16, F16, E4M3 (OCP e4m3fn, max 448).  Outputs: BF16, F16. */
enum mi355_dtype {
  MI355_BF16 = 0,
  MI355_F16 = 1,
  MI355_E4M3 = 2,
  MI355_F32 = 3   /* accepted by mi355_quantize_e4m3 only */
};

/* Kernel families.  AUTO picks by shape; the others force one family (and fail with
 * MI355_ERR_SHAPE when the shape does not meet that family's constraints). */
enum mi355_variant {
  MI355_VARIANT_AUTO = 0,
  MI355_VARIANT_BASIC = 1,    /* 256x256, 256x128 or 128x128 tile, one wave group, LDS ring   */
  MI355_VARIANT_PINGPONG = 2, /* same tile, two wave groups alternating MFMA and load phases   */
  MI355_VARIANT_SKINNY = 3,   /* small-M weight-streaming kernel with split-K                  */
  MI355_VARIANT_SIMPLE = 4,   /* one thread per output element; any shape; slow; self-check    */
  MI355_VARIANT_ALTERNATE = 5 /* 256x128 tiles, two workgroups per CU alternating whole tiles: one
                                 workgroup's stores run under the other's MFMAs; bf16/fp16 inputs   */
};

/* Status codes (0 = success, negative = error; see mi355_gemm_strerror). */
enum mi355_status {
  MI355_OK = 0,
  MI355_ERR_NULL = -1,      /* a required pointer is NULL                                   */
  MI355_ERR_DTYPE = -2,     /* unsupported input/output dtype combination                   */
  MI355_ERR_SHAPE = -3,     /* M, N, K or a leading dimension violates a constraint         */
  MI355_ERR_VARIANT = -4,   /* unknown variant, or variant cannot run this shape/dtype      */
  MI355_ERR_WORKSPACE = -5, /* workspace missing or smaller than mi355_gemm_workspace_bytes */
  MI355_ERR_LAUNCH = -6,    /* the HIP runtime refused the launch                           */
  MI355_ERR_ALIGN = -7,     /* a pointer or leading dimension is not 16-byte aligned        */
  MI355_ERR_SCRATCH = -8    /* mi355_gemm_tn_noalloc: the problem is beyond the built-in scratch */
};

/*
 * C = scale * A · B^T.
 *
 *   A         device pointer, M rows of K elements, row stride lda (elements)
 *   B         device pointer, N rows of K elements, row stride ldb (elements)
 *   C         device pointer, M rows of N elements, row stride ldc (elements)
 *   in_dtype  element type of A and B (enum mi355_dtype)
 *   out_dtype element type of C: MI355_BF16 or MI355_F16
 *   scale     fp32 factor applied to the fp32 accumulator before the down-conversion
 *             (1.0f for bf16/fp16; scale_a*scale_b for per-tensor-scaled fp8)
 *   variant   enum mi355_variant
 *   workspace device scratch of at least mi355_gemm_workspace_bytes(...) bytes, or NULL when
 *             that function returns 0; contents need not be initialised.  An explicit skinny
 *             variant needs it for its K split (MI355_ERR_WORKSPACE otherwise); the tiled variant
 *             runs without its K split or tail split, i.e. slower, when it is NULL or too small,
 *             and MI355_VARIANT_AUTO then uses the tiled variant also where it would stream.
 *             MI355_VARIANT_AUTO also uses it (256-byte aligned) to repack a large problem the
 *             tiled kernels cannot address (K*elem_bytes % 16, N % 4, strides, pointers) into
 *             an aligned one; without it such a problem runs on the slow generic kernel
 *   stream    hipStream_t on which the kernels are enqueued (NULL = the null stream)
 *
 * Replaces test::gemm_tn_test (kernels/gemm_kernels/sm90a/gemm_test.cu:12-92): same operand
 * layout and the argument checks of :15-41, plus checks of C the reference omits; divisibility
 * by the tile is not required (the tiled variants need K*elem_bytes % 16 == 0, row strides that
 * are multiples of 16 bytes, N % 4 == 0, ldc % 4 == 0, 256 rows of A and of B below 2 GiB and
 * 256*ldc below 2^29 elements; MI355_VARIANT_AUTO routes anything else to the generic kernel).
 * Every entry point of this header refuses (MI355_ERR_SHAPE, or 0 from the size queries) an
 * extent or row stride above 2^40 and an array of more than 2^50 elements, so that its size
 * arithmetic stays inside 64 bits.
 * Asynchronous: returns after enqueueing.
 */
int mi355_gemm_tn(const void *A, const void *B, void *C,
                  int64_t M, int64_t N, int64_t K,
                  int64_t lda, int64_t ldb, int64_t ldc,
                  int in_dtype, int out_dtype, float scale, int variant,
                  void *workspace, size_t workspace_bytes, void *stream);

/*
 * mi355_gemm_tn with two more factors that live in device memory: C = scale * (*scale_a) *
 * (*scale_b) * A · B^T.  Either pointer may be NULL (factor 1).  They are read by the kernel that
 * writes C, so the per-tensor scales produced by mi355_quantize_e4m3 never visit the host.
 * Counterpart in the reference: none (no fp8 path); same launcher contract as mi355_gemm_tn.
 */
int mi355_gemm_tn_scaled(const void *A, const void *B, void *C,
                         int64_t M, int64_t N, int64_t K,
                         int64_t lda, int64_t ldb, int64_t ldc,
                         int in_dtype, int out_dtype, float scale,
                         const float *scale_a, const float *scale_b, int variant,
                         void *workspace, size_t workspace_bytes, void *stream);

/*
 * mi355_gemm_tn for callers that cannot allocate device memory (code under HIP graph capture,
 * tight serving loops, harnesses that forbid hipMalloc): the same computation, kernels and plan,
 * with the workspace replaced by a buffer of MI355_NOALLOC_SCRATCH_BYTES that is part of the
 * library's code object.  The call allocates and frees nothing and hands over no workspace.
 * No counterpart in the reference (its launcher, kernels/gemm_kernels/sm90a/gemm_test.cu:12-92,
 * has no workspace at all).
 *
 *   - Each GPU the library runs on holds its own copy of the buffer from the first use of the
 *     library on that GPU until the process ends.  Its address on a GPU is looked up on the first
 *     call made with that GPU current (no allocation, but a one-time runtime query: make one call
 *     outside a graph capture first).
 *   - A problem whose plan wants more than the buffer holds is refused with MI355_ERR_SCRATCH; it
 *     is never silently run on a slower path.  K-split partial planes and tail-split partial tiles
 *     always fit (a plan has at most 256 split items of at most 256 x 256 floats = 64 MiB), and
 *     problems that want no workspace have no size limit, so in practice the limit applies to the
 *     repacked operands of a large misaligned problem (K*elem_bytes % 16, N % 4, strides, pointers;
 *     mi355_gemm_workspace_bytes reports the figure for contiguous operands).
 *   - All calls on one GPU share that GPU's buffer, which keeps the last call's contents (nothing
 *     in it needs to start at zero).  Calls that may overlap on one GPU (different streams, or
 *     several host threads) race on it: serialise them, or use mi355_gemm_tn with a workspace each.
 * Argument checks and their status codes are those of mi355_gemm_tn and run before any HIP call.
 */
#define MI355_NOALLOC_SCRATCH_BYTES 67108864 /* 64 MiB */
int mi355_gemm_tn_noalloc(const void *A, const void *B, void *C,
                          int64_t M, int64_t N, int64_t K,
                          int64_t lda, int64_t ldb, int64_t ldc,
                          int in_dtype, int out_dtype, float scale, int variant,
                          void *stream);

/*
 * Per-tensor fp8 quantisation, the step in front of the fp8 GEMM: amax = max|x|,
 * scale = amax/448 (1 if amax is 0), x_q[i] = e4m3(x[i]/scale) rounded to nearest even and
 * saturated at +-448, so that x ~= scale * x_q.
 *
 *   x          device pointer, n contiguous elements of x_dtype (MI355_BF16, MI355_F16, MI355_F32),
 *              16-byte aligned
 *   x_q        device pointer, n bytes (e4m3), 8-byte aligned
 *   scale_amax device pointer to two floats: [0] receives scale, [1] is scratch (receives amax)
 *
 * Asynchronous on `stream` (three launches, no host synchronisation).  Counterpart in the
 * reference: none; the contract is the fp8 benchmark configuration's (per-tensor fp32 scales
 * amax/448).
 */
int mi355_quantize_e4m3(const void *x, int x_dtype, int64_t n, void *x_q,
                        float *scale_amax, void *stream);

/*
 * OCP MX block scaling (MXFP8): C = A · B^T where every block of 32 consecutive elements of a row
 * of A or of B shares one E8M0 scale byte (value 2^(byte-127)):
 *   A[m,k] = A_q[m,k] * 2^(scale_a[m, k/32] - 127),  A_q e4m3; the same for B.
 * The block scales are applied by the scaled matrix-core instruction of gfx950 inside the k loop.
 *
 *   scale_a, scale_b   device pointers to the scale bytes.  With scales_shuffled == 0 they are in
 *                      the natural layout, (M, K/32) and (N, K/32) row-major with row strides
 *                      ld_scale_a / ld_scale_b (bytes); the call then re-lays them into the
 *                      workspace first (one small kernel per operand).  With scales_shuffled == 1
 *                      they are the output of mi355_mx_shuffle_scales (ld_scale_* ignored) and no
 *                      workspace is needed: do this once for weights.
 *   workspace          mi355_gemm_mx_workspace_bytes(M, N, K, scales_shuffled) bytes, 16-byte
 *                      aligned: the shuffled scales (required when scales_shuffled == 0) followed
 *                      by the partial results of a K split or tail split (optional: with less
 *                      room the tiles run unsplit, and a problem of at most 64 rows runs on the
 *                      tiled kernel instead of the weight-streaming one).
 * Constraints: K % 128 == 0; A, B 16-byte aligned with row strides that are multiples of 16;
 * N % 4 == 0, ldc % 4 == 0, C 8-byte aligned; the size limits of the tiled variants.  Runs the
 * weight-streaming kernel (MI355_VARIANT_SKINNY) for M <= 64 and otherwise the tiled kernel
 * (MI355_VARIANT_BASIC) with the planner's choice of tile and splits among the tiles this kernel
 * has: what mi355_gemm_plan reports for MI355_E4M3 operands of this shape and that variant,
 * except where plain operands get the nine-slot ring of 128 x 128 tiles (one row or column of
 * tiles, or tiles that make a single round), which the block-scaled kernel does not have.
 * Counterpart in the reference: none (it has no fp8 path); same launcher contract as
 * mi355_gemm_tn (kernels/gemm_kernels/sm90a/gemm_test.cu:12-92), block format per the OCP
 * Microscaling Formats (MX) specification v1.0.
 */
int mi355_gemm_tn_mxfp8(const void *A_q, const void *B_q, void *C,
                        int64_t M, int64_t N, int64_t K,
                        int64_t lda, int64_t ldb, int64_t ldc,
                        const uint8_t *scale_a, int64_t ld_scale_a,
                        const uint8_t *scale_b, int64_t ld_scale_b,
                        int scales_shuffled, int out_dtype,
                        void *workspace, size_t workspace_bytes, void *stream);

/* Workspace mi355_gemm_tn_mxfp8 wants: shuffled scales (unless already shuffled) + split partials. */
size_t mi355_gemm_mx_workspace_bytes(int64_t M, int64_t N, int64_t K, int scales_shuffled);

/* Argument check of mi355_gemm_tn_mxfp8 without pointers; runs without a GPU. */
int mi355_gemm_mx_check(int64_t M, int64_t N, int64_t K,
                        int64_t lda, int64_t ldb, int64_t ldc, int out_dtype);

/*
 * Re-lay the scale bytes of one operand, (rows, K/32) row-major with row stride ld bytes, into
 * the layout the kernel reads: `out` receives mi355_mx_shuffled_bytes(rows, K) bytes (rows padded
 * to a multiple of 256 with the scale 1).  K % 128 == 0; out 8-byte aligned.
 * Counterpart in the reference: none.
 */
int mi355_mx_shuffle_scales(const uint8_t *scales, int64_t rows, int64_t K, int64_t ld,
                            uint8_t *out, void *stream);
size_t mi355_mx_shuffled_bytes(int64_t rows, int64_t K);

/*
 * MX quantiser: x (rows, K) of x_dtype (BF16, F16 or F32), row stride ldx elements, K % 32 == 0
 * -> x_q (rows, K) contiguous e4m3 and the E8M0 scale bytes: (rows, K/32) contiguous in the natural
 * layout, or, with scales_shuffled != 0 (K % 128 == 0), mi355_mx_shuffled_bytes(rows, K) bytes in the
 * layout mi355_gemm_tn_mxfp8 takes with scales_shuffled == 1 (no shuffle launch then).  Per block: scale = 2^(floor(log2(amax)) - 8) (1 for a block of zeros), elements
 * x/scale rounded to nearest even, saturated at +-448.  x 16-byte aligned with ldx*elem_bytes
 * % 16 == 0, x_q 16-byte aligned, shuffled scales 8-byte aligned.  NaN and infinity are not supported.
 * Counterpart in the reference: none; OCP MX specification v1.0, section 6.3.
 */
int mi355_quantize_mxfp8(const void *x, int x_dtype, int64_t rows, int64_t K, int64_t ldx,
                         void *x_q, uint8_t *scales, int scales_shuffled, void *stream);

/* Scratch bytes mi355_gemm_tn wants for this problem and variant (0 for most shapes).
 * Counterpart: none in the reference (it has no split-K); sizes the split-K partials that
 * replace the reference's single-pass accumulation (gemm.cuh:352-367) on skinny shapes and in
 * the last round of tiles when that round would leave more than half of the CUs idle. */
size_t mi355_gemm_workspace_bytes(int64_t M, int64_t N, int64_t K,
                                  int in_dtype, int variant);

/* What mi355_gemm_tn would launch for this problem: the resolved variant (return value, or a
 * negative mi355_status), and for the tiled variants the tile (rows of A x rows of B per
 * workgroup), the uniform K split and the tail split (tiles of the last round cut along K;
 * 0 tiles / 1 split when there is none).  For the skinny variant its tile (rows of A x 64 or 128 rows of B) and its K split.
 * Any output pointer may be NULL.  Pure host function.  Counterpart in the reference: the
 * compile-time DefaultConfig (kernels/gemm_kernels/sm90a/gemm.cuh:420-451). */
int mi355_gemm_plan(int64_t M, int64_t N, int64_t K, int in_dtype, int variant,
                    int *tile_rows, int *tile_cols, int *k_splits,
                    int *tail_tiles, int *tail_splits);

/* How many launches of the GEMM kernel a call makes for this problem: 1, or 2 where MI355_VARIANT_AUTO cuts a
 * problem of the tiled kernel along N or M so that the first piece fills a whole number of rounds of workgroups and
 * the rest runs as a problem of its own (mi355_gemm_plan then describes the first piece; the second is what
 * MI355_VARIANT_BASIC plans for its shape).  *first_rows x *first_cols receive the first piece's extent (M x N for one
 * launch); either may be NULL.  Explicit variants never cut; mi355_gemm_tn_mxfp8 cuts where this function says so for
 * MI355_E4M3 operands (and M > 64).  Returns a negative mi355_status for bad arguments.
 * Pure host function.  Counterpart in the reference: none (its Scheduler walks one tile grid per launch,
 * kernels/gemm_kernels/sm90a/gemm.cuh:168-212). */
int mi355_gemm_pieces(int64_t M, int64_t N, int64_t K, int in_dtype, int variant,
                      int64_t *first_rows, int64_t *first_cols);

/* The variant MI355_VARIANT_AUTO resolves to for this problem (an enum mi355_variant value),
 * or a negative mi355_status.  Replaces the compile-time choice of kernel header at
 * kernels/gemm_kernels/sm90a/gemm_test.cu:7 / kernels/setup.py:12-15. */
int mi355_gemm_select_variant(int64_t M, int64_t N, int64_t K, int in_dtype);

/* Argument validation only, no HIP call: returns what mi355_gemm_tn would return before it
 * touches the device.  Mirrors the TORCH_CHECK block at gemm_test.cu:15-41. */
int mi355_gemm_check(int64_t M, int64_t N, int64_t K,
                     int64_t lda, int64_t ldb, int64_t ldc,
                     int in_dtype, int out_dtype, int variant);

/* Output tile a workgroup computes: block index -> (tile_m, tile_n) for a tiles_m x tiles_n
 * grid.  Pure integer function, callable without a GPU.  Replaces Scheduler::
 * get_swizzled_block_idx (kernels/gemm_kernels/sm90a/gemm.cuh:184-197): same contract
 * (a bijection onto the tile grid that keeps co-resident workgroups on neighbouring tiles),
 * re-derived for 8 XCDs with private L2s.  Returns 0, or MI355_ERR_SHAPE if block is out of
 * range. */
int mi355_gemm_tile_coord(int64_t block, int64_t tiles_m, int64_t tiles_n,
                          int64_t *tile_m, int64_t *tile_n);

/*
 * Measured ceilings of the GPU the call runs on, for a benchmark's roofline line.  No counterpart
 * in the reference, whose benchmark reads the peak from a table (kernels/tests/gemm_bench.py:592-599).
 *
 * mi355_calibrate_mfma enqueues ONE launch of a kernel that does nothing but matrix-core work: one
 * workgroup of four waves per compute unit, every wave running the tile kernel's MFMA pattern
 * (v_mfma_f32_16x16x32 for MI355_BF16 / MI355_F16, v_mfma_f32_16x16x128_f8f6f4 for MI355_E4M3;
 * 64 accumulator blocks) `iters` times on operand fragments it loads once from `a` and `b` (any
 * device data of that type, e.g. the operands of the GEMM being measured: the sustained clock
 * depends on the data; at least 4096 bytes each, 32-byte aligned).  *flops receives the flop count
 * of the launch; the caller times it.  `sink` is device memory of mi355_calibrate_sink_bytes().
 * mi355_calibrate_mfma_shape is the same with the choice of MFMA shape: wide_blocks == 0 is the
 * above, wide_blocks == 1 runs the loop on the 32-wide shapes the kernels do not use
 * (v_mfma_f32_32x32x16 for the 16-bit types, v_mfma_f32_32x32x64_f8f6f4 for MI355_E4M3; 16
 * accumulator blocks, the same 128 x 128 outputs per wave), so that a benchmark can report both.
 *
 * mi355_calibrate_read enqueues one launch that reads `bytes` bytes at `src` (16-byte aligned)
 * with plain 16-byte loads and nothing else.
 */
size_t mi355_calibrate_sink_bytes(void);
int mi355_calibrate_mfma(int in_dtype, const void *a, size_t a_bytes, const void *b, size_t b_bytes,
                         int iters, void *sink, double *flops, void *stream);
int mi355_calibrate_mfma_shape(int in_dtype, int wide_blocks, const void *a, size_t a_bytes,
                               const void *b, size_t b_bytes, int iters, void *sink, double *flops,
                               void *stream);
int mi355_calibrate_read(const void *src, size_t bytes, void *sink, void *stream);

/*
 * Shader clock under load, without a profiler.  No counterpart in the reference.
 * mi355_clock_probe enqueues ONE launch of `waves` single-wave workgroups (1..1024) that do nothing
 * but sleep and, `samples` times (2..4096) with `pause` sleeps of 127 x 64 cycles in between
 * (samples * pause <= 65536), read the shader-cycle counter and the constant 100 MHz counter.
 * Enqueued on a second stream while other work runs on the first (a wave of it needs 8 registers and
 * no LDS, so it finds room beside the tile kernels' workgroups), it yields the clock that work runs at.
 * (A stream's hardware queue is set up at its first launch, which disturbs whatever runs at that
 * moment: launch something small on the second stream once before the measurement.)
 * `out` is device memory of mi355_clock_probe_bytes(waves, samples) bytes, 8-byte aligned, read as
 * uint64 out[waves][2][samples + 1]: out[w][0][0] = XCD the wave ran on, out[w][1][0] = 0,
 * out[w][0][1 + s] = shader cycles and out[w][1][1 + s] = ticks of 10 ns at sample s; the clock
 * between two samples is the ratio of the differences.  mi355_clock_probe_bytes returns 0 for counts outside the ranges above.
 */
size_t mi355_clock_probe_bytes(int waves, int samples);
int mi355_clock_probe(int waves, int samples, int pause, void *out, void *stream);

/* Human-readable text for a status code; never NULL.  Replaces the TORCH_CHECK messages of
 * gemm_test.cu:15-41 and the stderr print of :88-90. */
const char *mi355_gemm_strerror(int status);

/* Library version, (major << 16) | minor. */
int mi355_gemm_version(void);

#ifdef __cplusplus
}
#endif
#endif /* MI355_GEMM_H */
