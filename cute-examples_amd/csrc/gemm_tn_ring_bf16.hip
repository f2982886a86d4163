// Single-group tile kernel (gemm_tn_ring.h), bf16 operands.
#include "gemm_tn_ring.h"

namespace mi355 {

int launch_tile_ring_bf16(const GemmArgs& g, int out_dtype, int tile, hipStream_t stream) {
  return out_dtype == 0 ? launch<BF16, BF16>(g, tile, stream) : launch<BF16, F16>(g, tile, stream);
}

}  // namespace mi355
