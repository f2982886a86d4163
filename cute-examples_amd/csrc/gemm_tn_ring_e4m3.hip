// Single-group tile kernel (gemm_tn_ring.h), e4m3 operands with per-tensor scales.
#include "gemm_tn_ring.h"

namespace mi355 {

int launch_tile_ring_e4m3(const GemmArgs& g, int out_dtype, int tile, hipStream_t stream) {
  return out_dtype == 0 ? launch<E4M3, BF16>(g, tile, stream) : launch<E4M3, F16>(g, tile, stream);
}

}  // namespace mi355
