// "skinny" variant: weight-streaming GEMM for small M (LLM projections with a few tokens).
//
// C[M,N] = scale * X[M,K] · W[N,K]^T with M <= 256 is bound by reading W once from HBM, so the
// kernel is built around keeping many bytes of W in flight per CU rather than around MFMA issue:
//
//   * output tile TM x 64 with TM = 16/32/64/128/256 >= M, or 64 x 128 (see wide_tiles); the grid
//     is (tiles along N) x (K splits), several workgroups resident per CU (the LDS ring of one
//     workgroup is 30-120 KiB), or, when the tiles alone occupy most CUs, no K split and a deeper
//     ring (see unsplit_deep);
//   * per k-step (128 B of K per row) the TM rows of X and the 64 or 128 rows of W go global -> LDS with
//     full-cache-line direct-to-LDS loads into a ring of kDepth stages, kDepth-1 k-steps ahead;
//   * the four waves read MFMA fragments from LDS (same 16-byte-chunk swizzle as the big-tile
//     kernels) and run v_mfma_f32_16x16x32 (two per k-step and block pair) or, for fp8,
//     v_mfma_f32_16x16x128_f8f6f4 (one; with OCP MX block scales its scaled form, the scale bytes
//     riding through the ring behind the rows); W blocks are the MFMA rows, so every lane ends up
//     with four consecutive n of one m;
//   * workgroups start their k-steps at different points and wrap around, so that they do not all
//     read the same column of rows a power of two apart (the same memory channels) at once;
//   * with K split S ways the partial tiles go to an fp32 workspace [S][M][N] and a second kernel
//     adds them in a fixed order (deterministic), scales and rounds; with S = 1 the tile is
//     rounded and stored directly.
//
// Counterpart in the reference: none — its launcher rejects M not divisible by 256
// (kernels/gemm_kernels/sm90a/gemm_test.cu:33-35); the arithmetic contract is the same one
// (gemm.cuh:352-377: fp32 accumulation of exact products, round-to-nearest-even output).
#include "gemm_launch.h"
#include "ring_common.h"

#include <type_traits>

namespace mi355 {
namespace {

constexpr int kThreads = 256;
constexpr int kTileN = 64;
constexpr int kTileNWide = 128, kDepthWide = 3;   // the 64 x 128 tile of wide_tiles and its ring depth

// kMB x kNB 16x16 blocks per wave, kWM x kWN waves (kWM * kWN == 4).
// Geometry per input type: 16x16 blocks for all of them (fp8 on the 16x16x128 shape).
template <class T> struct StreamGeo { typedef Geo<T> type; };
template <> struct StreamGeo<E4M3> { typedef GeoE4M3Rows type; };
template <> struct StreamGeo<MxE4M3> { typedef GeoMxE4M3Rows type; };

// Block scales (MxE4M3) come in the layout the tile kernel reads too (mx_scales.hip): one 512-byte
// unit per (group of 128 rows, k-step), in which lane l owns the 8 bytes at 8*l: byte i is the scale
// of row 16*i + l%16 for K block 4*kstep + l/16, i.e. exactly what lane l of the scaled MFMA has
// to supply for the i-th 16-row block.  A 64-row tile is one half of a group, so one 4-byte copy
// per lane and k-step brings the scales of all four blocks of W, and another those of X; they
// travel through the ring like the operands (256 bytes each behind the rows of a stage).
constexpr uint32_t kMxUnit = 512;

template <class T, class OutT, int kMB, int kNB, int kWM, int kWN, int kDepth>
__global__ __launch_bounds__(kThreads) void gemm_tn_stream(GemmArgs g, float* partial, int splits) {
  typedef typename StreamGeo<T>::type G;
  typedef typename G::Frag Frag;
  static_assert(G::kBlk == 16 && kWM * kWN == 4, "16x16 MFMA blocks, four waves");
  constexpr int kSliceChunks = G::kGroups * G::kCpl;   // 16-byte chunks of a row one MFMA consumes
  constexpr int kSlices = 8 / kSliceChunks;            // MFMAs per k-step and block pair
  constexpr int kTm = 16 * kMB * kWM, kTn = 16 * kNB * kWN;
  constexpr bool kMx = G::kMx;
  static_assert(!kMx || (kWM == 1 && kWN == 4 && kNB == 1), "block scales: one 64-row half group per operand");
  constexpr int kDataBytes = (kTm + kTn) * kRowBytes;
  constexpr int kStageBytes = kDataBytes + (kMx ? 512 : 0);   // + the scales of W, then of X
  constexpr int kCopies = (kTm + kTn) / 8;          // 8-row copies per k-step
  constexpr int kCpw = (kCopies + 3) / 4;           // per wave (padded with repeats)
  constexpr int kXCopies = kTm / 8;
  constexpr int kVm = kCpw + (kMx ? 1 : 0);         // vector-memory instructions per wave and k-step
  static_assert(kVm * (kDepth - 1) < 64, "vmcnt is a 6-bit counter");
  __shared__ __attribute__((aligned(1024))) uint8_t ring[kDepth * kStageBytes];

  const uint32_t tid = threadIdx.x;
  const uint32_t lane = tid & 63u;
  const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const uint32_t wm = wave / kWN, wn = wave % kWN;

  const int64_t tiles_m = (g.M + kTm - 1) / kTm;
  const int64_t tile_m = blockIdx.x % tiles_m, tile_n = blockIdx.x / tiles_m;
  const int64_t m0 = tile_m * kTm, n0 = tile_n * kTn;
  const uint32_t split = blockIdx.y;

  const uint32_t ldx_b = (uint32_t)(g.lda * T::kBytes), ldw_b = (uint32_t)(g.ldb * T::kBytes);
  const uint32_t k_bytes = (uint32_t)(g.K * T::kBytes);
  // Split `split` of S takes k-steps [split*k/S, (split+1)*k/S): every step once, lengths within one
  // of each other when S does not divide them.  A ragged last k-step (K*elem_bytes not a multiple
  // of 128) is handled by fetching its missing chunks from an out-of-range offset.
  const uint32_t steps_total = (k_bytes + kRowBytes - 1) / kRowBytes;
  const uint32_t tail_bytes = __builtin_amdgcn_readfirstlane(k_bytes % kRowBytes);
  const uint32_t step0 = __builtin_amdgcn_readfirstlane(split * steps_total / (uint32_t)splits);
  const uint32_t steps = __builtin_amdgcn_readfirstlane((split + 1) * steps_total / (uint32_t)splits) - step0;
  const int64_t rows_x = g.M - m0 < kTm ? g.M - m0 : kTm;
  const int64_t rows_w = g.N - n0 < kTn ? g.N - n0 : kTn;
  const __amdgpu_buffer_rsrc_t rsrc_x = make_raw_buffer(
      (const uint8_t*)g.A + m0 * (int64_t)ldx_b, (uint32_t)((rows_x - 1) * ldx_b + k_bytes));
  const __amdgpu_buffer_rsrc_t rsrc_w = make_raw_buffer(
      (const uint8_t*)g.B + n0 * (int64_t)ldw_b, (uint32_t)((rows_w - 1) * ldw_b + k_bytes));

  // Scales: even waves copy those of W, odd waves those of X (twice each, so that every wave
  // issues the same number of instructions).
  const uint32_t scale_units = kMx ? (uint32_t)((g.M + 255) / 256) * 2u * steps_total * kMxUnit : 0u;
  const uint32_t scale_units_w = kMx ? (uint32_t)((g.N + 255) / 256) * 2u * steps_total * kMxUnit : 0u;
  const __amdgpu_buffer_rsrc_t rsrc_sx = make_raw_buffer(g.mx_a, scale_units);
  const __amdgpu_buffer_rsrc_t rsrc_sw = make_raw_buffer(g.mx_b, scale_units_w);
  const uint32_t voff_sx = (uint32_t)(m0 / 128) * steps_total * kMxUnit + lane * 8 + (uint32_t)(m0 % 128) / 64 * 4;
  const uint32_t voff_sw = (uint32_t)(n0 / 128) * steps_total * kMxUnit + lane * 8 + (uint32_t)(n0 % 128) / 64 * 4;

  // Copy c (0..kCopies-1) of a k-step moves 8 rows x 128 B: X rows first, then W rows; wave w
  // issues copies w, w+4, ...  (indices past the end repeat earlier copies so that every wave
  // issues the same number and one vmcnt value fits all).  Rows past the matrix edge are out of
  // the descriptor's range and read as zeros.
  const uint32_t r8 = lane >> 3, c8 = lane & 7u;
  const uint32_t ring0 = __builtin_amdgcn_readfirstlane(lds_address(ring));
  // Workgroups that run side by side walk their k-steps from different starting points (and wrap
  // around): started together at the same k they would all be reading the same 128-byte column of
  // rows that lie a power of two apart when K is one, i.e. the same few memory channels (fp8
  // 16x8192x8192 cut in two: 19.6 us, against 16.2 us for K = 8320).  Only the order of the fp32
  // additions inside a tile depends on it, and that order is fixed per tile.
  // The tiles' starting points are spread evenly over the k-steps (neighbouring tiles one n-th of the
  // way apart: of four spacings tried this was the best, 16x14336x4096 bf16 25.1 -> 21.9 us against
  // a stride of seven k-steps).
  // Tiles of 64 rows of X differ: a third to a half of what such a workgroup reads is its slice of X, which
  // all tiles of its K split read too.  Spread evenly, the four or eight of them that share an XCD's L2 pass
  // a given k-step so far apart in time that the rows of W streaming through have evicted it in between
  // (bf16 64x4096x14336: 164 MiB fetched by the L2s for 113 MiB of operands).  So there the XCDs start an
  // eighth of the k-steps apart and an XCD's tiles two k-steps apart: 31.5 -> 27.4 us on that problem,
  // 64x8192x28672 103 -> 91 us, 56x5120x13824 34.6 -> 31.9 us.  With many tiles per XCD (evenly spread
  // neighbours under three k-steps apart) and on the shorter tiles, where X is a small share, the even
  // spread stays: clustered, bf16 16x14336x4096 took 23.7 us against 21.4 and 64x14336x4096 28.0 against 26.3,
  // and 23x24388x8264 on the 64 x 128 tile (its lower rows out of range) 100.0 against 95.3.  Beyond 96 tile
  // columns it takes eight k-steps between neighbours for the cluster to pay: 64x20480x28672 (22 apart)
  // 239 -> 220 us, 64x18432x16384 (14) 127 -> 121 us, but 64x24388x8264 (5.4), 64x28672x8192 (4.6) and
  // 64x16384x7168 (3.5) 2-3 % slower.
  uint32_t first = blockIdx.x * steps / gridDim.x;
  if (kTm == 64 && rows_x > 32 && 8u * steps >= (gridDim.x > 96u ? 8u : 3u) * gridDim.x)
    first = ((blockIdx.x + gridDim.x * blockIdx.y) & 7u) * steps / 8u + (blockIdx.x >> 3) * 2u;
  const uint32_t rot = __builtin_amdgcn_readfirstlane((first + blockIdx.y * 3u) % steps);
  auto issue_step = [&](uint32_t stage, uint32_t kt) __attribute__((always_inline)) {
    uint32_t at = (kt < steps ? kt : steps - 1) + rot;   // steps past the end repeat the last one
    at = at >= steps ? at - steps : at;
    const uint32_t kk = step0 + at;
    const uint32_t soff = kk * kRowBytes;
    const bool ragged = tail_bytes != 0 && kk == steps_total - 1;
#pragma unroll
    for (int i = 0; i < kCpw; ++i) {
      const uint32_t c = (wave + 4 * i) % kCopies;
      const uint32_t row = c * 8 + r8;                   // row inside the stage: X rows, then W rows
      const uint32_t chunk = c8 ^ swizzle(row);
      const uint32_t dst = ring0 + stage * kStageBytes + c * 1024;
      const uint32_t drop = ragged && chunk * 16 >= tail_bytes ? 0x80000000u : 0u;  // panels are < 2 GiB
      if (c < kXCopies) dma_16B_to_lds(dst, (row * ldx_b + chunk * 16) | drop, rsrc_x, soff);   // c is wave-uniform
      else dma_16B_to_lds(dst, ((row - kTm) * ldw_b + chunk * 16) | drop, rsrc_w, soff);
    }
    if constexpr (kMx) {
      const uint32_t dst = ring0 + stage * kStageBytes + kDataBytes;
      if ((wave & 1u) == 0) dma_4B_to_lds(dst, voff_sw, rsrc_sw, kk * kMxUnit);
      else dma_4B_to_lds(dst + 256, voff_sx, rsrc_sx, kk * kMxUnit);
    }
  };

  // Fragment geometry: lane l supplies row l%16 of a block, lane group l/16 picks the chunk.
  const uint32_t rblk = lane & 15u, grp = lane >> 4;
  const uint32_t swz = swizzle(rblk);
  const uint32_t x_lane = (wm * kMB * 16 + rblk) * kRowBytes;
  const uint32_t w_lane = (kTm + wn * kNB * 16 + rblk) * kRowBytes;
  auto frag = [&](const uint8_t* rows, int blk, int s) __attribute__((always_inline)) -> Frag {
    const uint8_t* p = rows + blk * 16 * kRowBytes;
    if constexpr (G::kCpl == 1) {
      return *(const i32x4*)(p + (((uint32_t)(s * kSliceChunks) + grp) ^ swz) * 16);
    } else {
      // One MFMA spans the k-step: lane group g supplies chunks g and 4+g.  The scaled MFMA needs that
      // order of K; the plain one takes any order common to both operands, and this one has no LDS
      // bank conflicts where chunks 2g, 2g+1 have one per access (see chunk_off in gemm_tn_ring.h).
      static_assert(kSlices == 1, "a fragment of two chunks covers the whole k-step");
      const i32x4 lo = *(const i32x4*)(p + ((grp ^ swz) * 16));
      const i32x4 hi = *(const i32x4*)(p + (((grp + 4) ^ swz) * 16));
      return (i32x8){lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
    }
  };

  f32x4 acc[kMB][kNB];
#pragma unroll
  for (int i = 0; i < kMB; ++i)
#pragma unroll
    for (int j = 0; j < kNB; ++j) acc[i][j] = (f32x4){0.f, 0.f, 0.f, 0.f};

#pragma unroll
  for (int st = 0; st < kDepth - 1; ++st) issue_step(st, st);

  uint32_t stage = 0;
  for (uint32_t kt = 0; kt < steps; ++kt) {
    wait_vmcnt<kVm * (kDepth - 2)>();   // my copies of k-step kt have landed
    wait_lgkmcnt0();                    // my LDS reads of k-step kt-1 are back
    __builtin_amdgcn_s_barrier();       // everybody's are: stage of kt is full, stage of kt-1 is free
    const uint32_t refill = stage == 0 ? kDepth - 1 : stage - 1;
    issue_step(refill, kt + kDepth - 1);
    const uint8_t* st_base = ring + stage * kStageBytes;
#pragma unroll
    for (int s = 0; s < kSlices; ++s) {
      Frag fx[kMB], fw[kNB];
#pragma unroll
      for (int j = 0; j < kNB; ++j) fw[j] = frag(st_base + w_lane, j, s);
#pragma unroll
      for (int i = 0; i < kMB; ++i) fx[i] = frag(st_base + x_lane, i, s);
      if constexpr (kMx) {
        // this lane's four scale bytes of W (block wn is this wave's) and of X (block i)
        const uint32_t sw = *(const uint32_t*)(st_base + kDataBytes + lane * 4) >> (wn * 8);
        const uint32_t sx = *(const uint32_t*)(st_base + kDataBytes + 256 + lane * 4);
        static_for<kMB>([&](auto ic) __attribute__((always_inline)) {
          constexpr int i = decltype(ic)::value;
          G::template mfma_scaled_inplace<0, i>(fw[0], fx[i], acc[i][0], sw, sx);
        });
      } else {
#pragma unroll
        for (int i = 0; i < kMB; ++i)
#pragma unroll
          for (int j = 0; j < kNB; ++j) acc[i][j] = G::mfma(fw[j], fx[i], acc[i][j]);
      }
    }
    stage = stage + 1 == kDepth ? 0 : stage + 1;
  }
  wait_vmcnt<0>();
  // the scaled MFMAs are inline assembly: the compiler does not know how long their results take
  if constexpr (kMx) asm volatile("s_nop 15\n\ts_nop 15\n\ts_nop 15" ::: "memory");

  // acc[i][j][r] of lane l is the (partial) sum for
  //   m = m0 + (wm*kMB + i)*16 + l%16,   n = n0 + (wn*kNB + j)*16 + 4*(l/16) + r.
#pragma unroll
  for (int i = 0; i < kMB; ++i) {
    const int64_t m = m0 + (wm * kMB + i) * 16 + rblk;
    if (m >= g.M) continue;
#pragma unroll
    for (int j = 0; j < kNB; ++j) {
      const int64_t n = n0 + (wn * kNB + j) * 16 + grp * 4;
      if (n + 4 > g.N) continue;
      // A wave has at most sixteen of these stores: each one's data registers are simply held over
      // the wait states a wide store wants before they may be rewritten (see hold_previous).
      if (partial) {
        u32x4 data = __builtin_bit_cast(u32x4, acc[i][j]);
        asm volatile("" : "+v"(data));
        *(u32x4*)(partial + ((int64_t)split * g.M + m) * g.N + n) = data;
        hold_last(data);
      } else {
        const float sc = output_scale(g);
        u32x2 data = Pack4<OutT>::run(acc[i][j][0] * sc, acc[i][j][1] * sc, acc[i][j][2] * sc, acc[i][j][3] * sc);
        asm volatile("" : "+v"(data));
        *(u32x2*)((uint16_t*)g.C + m * g.ldc + n) = data;
        hold_last(data);
      }
    }
  }
}

// C[m][n..n+3] = rne(scale * (partial[0] + partial[1] + ... + partial[S-1])), summed in that order.
template <class OutT>
__global__ __launch_bounds__(256) void splitk_reduce(const float* partial, GemmArgs g) {
  uint16_t* C = (uint16_t*)g.C;
  const int64_t M = g.M, N = g.N, ldc = g.ldc;
  const int splits = g.splits;
  const float scale = output_scale(g);
  const int64_t quads_per_row = N / 4;
  const int64_t q = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (q >= M * quads_per_row) return;
  const int64_t m = q / quads_per_row, n = (q % quads_per_row) * 4;
  // Four planes per round: their loads go out together (a plane past the last one repeats the last and
  // is not added), the additions keep the order of the planes.
  const float* mine = partial + m * N + n;
  const int64_t plane = M * N;
  f32x4 sum = *(const f32x4*)mine;
  for (int s0 = 1; s0 < splits; s0 += 4) {
    f32x4 t[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) t[i] = *(const f32x4*)(mine + (int64_t)(s0 + i < splits ? s0 + i : splits - 1) * plane);
#pragma unroll
    for (int i = 0; i < 4; ++i) sum = s0 + i < splits ? sum + t[i] : sum;
  }
  *(u32x2*)(C + m * ldc + n) = Pack4<OutT>::run(sum[0] * scale, sum[1] * scale, sum[2] * scale, sum[3] * scale);
}

template <class T, class OutT, int kMB, int kNB, int kWM, int kWN, int kDepth>
int launch_cfg(const GemmArgs& g, int splits, float* ws, hipStream_t stream) {
  constexpr int kTm = 16 * kMB * kWM, kTn = 16 * kNB * kWN;
  const int64_t tiles = ((g.M + kTm - 1) / kTm) * ((g.N + kTn - 1) / kTn);
  float* partial = splits > 1 ? ws : nullptr;
  hipLaunchKernelGGL((gemm_tn_stream<T, OutT, kMB, kNB, kWM, kWN, kDepth>), dim3((unsigned)tiles, (unsigned)splits),
                     dim3(kThreads), 0, stream, g, partial, splits);
  if (hipGetLastError() != hipSuccess) return -1;
  if (splits > 1)
  {
    GemmArgs r = g;
    r.splits = splits;
    return launch_splitk_reduce(ws, r, std::is_same<OutT, BF16>::value ? 0 : 1, stream);
  }
  return 0;
}

// Ring depth (k-steps) per tile height.  Depths 3..6 measured the same on the LLM projection
// shapes; the shallow ones leave room for 3-4 workgroups per CU.
constexpr int kDepth16 = 4, kDepth32 = 4, kDepth64 = 3, kDepth128 = 4, kDepth256 = 3;
// Without a K split (enough tiles to give nearly every CU one) a workgroup has the CU to itself and
// keeps its bytes in flight with a deep ring instead of with neighbours: 16x14336x4096 bf16
// 27.7 us split four ways + reduce, 25.7 us unsplit with eight stages (27.1 us with fourteen); with
// the staggered start six stages are 2 % faster than eight over 36 problems.
constexpr int kDepthUnsplit = 6;
// That mode pays when the tiles occupy more than half of the 256 CUs and all of them are resident at once
// with the deep ring (two workgroups per CU at M <= 16, one above): measured on N = 12800...28672,
// bf16 and fp8, -7 to -20 % there; with more tiles than that (several rounds) the shallow ring with
// three or four workgroups per CU is 5-20 % faster again.
bool unsplit_deep(int64_t M, int64_t N, bool mx) {
  if (M > 64) return false;
  const int64_t tm = M <= 16 ? 16 : M <= 32 ? 32 : 64;
  const int64_t per_cu = 163840 / (kDepthUnsplit * ((tm + kTileN) * kRowBytes + (mx ? 512 : 0)));
  const int64_t tiles = (N + kTileN - 1) / kTileN;
  // (two per CU only for the lowest tile: fp8 32x28672x4096 measured 5 % slower that way than split)
  // From 150 tiles on for the two lower tiles (N = 11008 and 12288 at M <= 32: -16 to -18 % against the
  // split; with 128 tiles +25 %), from 200 for the 64-row tile (150...199 tiles: -10 % to +14 %).
  return tiles >= (tm <= 32 ? 150 : 200) && tiles <= 256 * (tm <= 16 ? per_cu : 1);
}

// 64 x 64 tile: the four waves as 2 x 2 (32 x 32 each: two fragments of X and two of W per wave and
// k-step instead of four and one; 3-9 % faster where the tile runs unsplit), except with block
// scales, whose layout wants one 64-row half group per operand and wave.
template <class T, class OutT, int kDepth>
int launch_64(const GemmArgs& g, int splits, float* ws, hipStream_t stream) {
  if constexpr (std::is_same<T, MxE4M3>::value) return launch_cfg<T, OutT, 4, 1, 1, 4, kDepth>(g, splits, ws, stream);
  else return launch_cfg<T, OutT, 2, 2, 2, 2, kDepth>(g, splits, ws, stream);
}

// K splits for tiles of tm x tn in a ring of `depth` stages: as many workgroups as can be resident at
// once (one wave of workgroups, no tail), each with enough k-steps.
int splits_for(int64_t M, int64_t N, int64_t K, int elem_bytes, bool mx, int64_t tm, int64_t tn, int depth) {
  const int64_t ring_bytes = depth * ((tm + tn) * kRowBytes + (mx ? 512 : 0));
  const int64_t per_cu = 163840 / ring_bytes < 8 ? 163840 / ring_bytes : 8;   // LDS-bound residency
  const int64_t slots = 256 * per_cu;  // MI355X has 256 CUs; a heuristic only, so no device query here
  const int64_t tiles = ((M + tm - 1) / tm) * ((N + tn - 1) / tn);
  const int64_t steps = (K * elem_bytes + kRowBytes - 1) / kRowBytes;
  // The workgroups of a CU share its bandwidth, and one of them already keeps it busy, so what counts
  // is the CU with the most k-steps to stream: ceil(workgroups / 256) workgroups of ceil(steps / S)
  // k-steps, each paying about four more to fill and drain its ring; splits beyond that only add
  // partial tiles.  Measured on 18 bf16 problems (M = 16 and 64, N = 2048...11008) with every S
  // forced: the choice is within 1 % of the best S on average (a rule that maximised the number
  // of workgroups: 10 %).  At least 8 k-steps per workgroup.
  int best = 1;
  double best_cost = 0;
  for (int s = 1; s <= 32; ++s) {
    if (tiles * s > slots) break;
    if (s > 1 && steps / s < 8) break;
    // On the 128-column tiles, which also serve thousands of columns, the partial planes count too: S x M x N
    // floats written and read back, priced in k-steps of a CU (3e-6 each; fifteen problems with every S forced:
    // all at their best S with 2e-6...4.4e-6; without the term 48x18432x2048 was cut in three, 23.1 us
    // against 21.5 unsplit).
    const double planes = tn == kTileNWide && s > 1 ? 3e-6 * (double)s * (double)M * (double)N : 0.0;
    const double cost = (double)((tiles * s + 255) / 256) * (double)((steps + s - 1) / s + 4) + 0.5 * s + planes;
    if (s == 1 || cost < best_cost) {
      best = s;
      best_cost = cost;
    }
  }
  return best;
}

int splits_narrow(int64_t M, int64_t N, int64_t K, int elem_bytes, bool mx) {
  if (unsplit_deep(M, N, mx)) return 1;
  const int64_t tm = M <= 16 ? 16 : M <= 32 ? 32 : M <= 64 ? 64 : M <= 128 ? 128 : 256;
  const int depth = M <= 16 ? kDepth16 : M <= 32 ? kDepth32 : M <= 64 ? kDepth64 : M <= 128 ? kDepth128 : kDepth256;
  return splits_for(M, N, K, elem_bytes, mx, tm, kTileN, depth);
}

// 64 x 128 tiles, made for 33...64 rows: a quarter fewer cache lines requested per output than 64 x 64 (192
// per 64 x 128 outputs and k-step against 2 x 128), paid for with half as many tiles to spread over the
// CUs.  Measured against the 64 x 64 tiles (M = 40...64, bf16, weights from HBM, each form with its own best
// split, the k-steps started as the kernel's `rot` says): 3-30 % faster with 129-256 wide tiles (the narrow
// ones no longer fit one round; N = 16896...32768, 16...448 k-steps), 2-17 % with 40-95 from 64 k-steps on
// and 2-28 % with 24-39 from 128 k-steps on; with fewer k-steps or fewer columns than that 1-17 % slower (the
// split that occupies the CUs leaves a workgroup too few k-steps); with 96-128 wide tiles, where the narrow
// ones make one unsplit round on the deep ring and the wide ones need a split, from 8 % faster to 21 %
// slower (K = 16384 at N = 13824 and 16384), so not there.  60 random problems inside the rule against the
// narrower one before it (160-256 tiles, 64-95 from 64 k-steps, 32-63 from 128): geometric mean -9 %,
// none more than 1 % slower; e4m3 on six -4...-13 %.
bool wide_tiles(int64_t M, int64_t N, int64_t K, int elem_bytes, bool mx) {
  if (mx || M > 64) return false;
  const int64_t tiles = (N + kTileNWide - 1) / kTileNWide;
  const int64_t steps = (K * elem_bytes + kRowBytes - 1) / kRowBytes;
  // Up to 32 rows the same tile (its lower half idle) wins only just above what the 64-column tiles
  // cover in one round: N = 17408...24576 at M = 16...32 and K = 2048...8192 2-18 % faster, N = 28672
  // the same, N = 32768 and N = 16384 0-4 % and 7-20 % slower.
  if (M <= 32) return tiles > 128 && tiles < 208;
  if (tiles > 128) return tiles <= 256;
  if (tiles >= 96) return false;
  if (tiles >= 40) return steps >= 64;
  return tiles >= 24 && steps >= 128;
}

template <class T, class OutT>
int launch_m(const GemmArgs& g, int splits, float* ws, hipStream_t stream) {
  if (wide_tiles(g.M, g.N, g.K, T::kBytes, std::is_same<T, MxE4M3>::value)) {
    if constexpr (!std::is_same<T, MxE4M3>::value) return launch_cfg<T, OutT, 2, 4, 2, 2, kDepthWide>(g, splits, ws, stream);
  }
  if (splits == 1 && unsplit_deep(g.M, g.N, std::is_same<T, MxE4M3>::value)) {
    if (g.M <= 16) return launch_cfg<T, OutT, 1, 1, 1, 4, kDepthUnsplit>(g, splits, ws, stream);
    if (g.M <= 32) return launch_cfg<T, OutT, 2, 1, 1, 4, kDepthUnsplit>(g, splits, ws, stream);
    return launch_64<T, OutT, kDepthUnsplit>(g, splits, ws, stream);
  }
  if (g.M <= 16) return launch_cfg<T, OutT, 1, 1, 1, 4, kDepth16>(g, splits, ws, stream);   //  16x64, 10 KiB/step
  if (g.M <= 32) return launch_cfg<T, OutT, 2, 1, 1, 4, kDepth32>(g, splits, ws, stream);   //  32x64, 12 KiB/step
  if (g.M <= 64) return launch_64<T, OutT, kDepth64>(g, splits, ws, stream);                 //  64x64, 16 KiB/step
  if constexpr (std::is_same<T, MxE4M3>::value) {
    return -1;   // block scales: up to 64 rows (the host routes taller problems to the tile kernel)
  } else {
    if (g.M <= 128) return launch_cfg<T, OutT, 4, 2, 2, 2, kDepth128>(g, splits, ws, stream);  // 128x64, 24 KiB/step
    return launch_cfg<T, OutT, 4, 4, 4, 1, kDepth256>(g, splits, ws, stream);                  // 256x64, 40 KiB/step
  }
}

}  // namespace

int stream_tile_cols(int64_t M, int64_t N, int64_t K, int elem_bytes, bool mx) {
  return wide_tiles(M, N, K, elem_bytes, mx) ? kTileNWide : kTileN;
}

int stream_splits(int64_t M, int64_t N, int64_t K, int elem_bytes, bool mx) {
  if (wide_tiles(M, N, K, elem_bytes, mx)) return splits_for(M, N, K, elem_bytes, mx, 64, kTileNWide, kDepthWide);
  return splits_narrow(M, N, K, elem_bytes, mx);
}

int launch_splitk_reduce(const float* partial, const GemmArgs& g, int out_dtype, hipStream_t stream) {
  const int64_t quads = g.M * (g.N / 4);
  const dim3 grid((unsigned)((quads + 255) / 256));
  if (out_dtype == 0) hipLaunchKernelGGL((splitk_reduce<BF16>), grid, dim3(256), 0, stream, partial, g);
  else hipLaunchKernelGGL((splitk_reduce<F16>), grid, dim3(256), 0, stream, partial, g);
  return hipGetLastError() == hipSuccess ? 0 : -1;
}

// Block-scaled fp8 (g.mx_a / g.mx_b in the shuffled layout), M <= 64.
int launch_stream_mx(const GemmArgs& g, int out_dtype, int splits, void* workspace, hipStream_t stream) {
  if (g.M > 64) return -1;
  return out_dtype == 0 ? launch_m<MxE4M3, BF16>(g, splits, (float*)workspace, stream)
                        : launch_m<MxE4M3, F16>(g, splits, (float*)workspace, stream);
}

int launch_stream(const GemmArgs& g, int in_dtype, int out_dtype, int splits, void* workspace, hipStream_t stream) {
  float* ws = (float*)workspace;
  const bool out_bf16 = out_dtype == 0;
  switch (in_dtype) {
    case 0: return out_bf16 ? launch_m<BF16, BF16>(g, splits, ws, stream) : launch_m<BF16, F16>(g, splits, ws, stream);
    case 1: return out_bf16 ? launch_m<F16, BF16>(g, splits, ws, stream) : launch_m<F16, F16>(g, splits, ws, stream);
    case 2: return out_bf16 ? launch_m<E4M3, BF16>(g, splits, ws, stream) : launch_m<E4M3, F16>(g, splits, ws, stream);
  }
  return -1;
}

}  // namespace mi355
