// Single-group tile kernel (gemm_tn_ring.h), e4m3 operands with block scales in the shuffled
// layout (g.mx_a, g.mx_b).  build.py checks this unit's assembly.
#include "gemm_tn_ring.h"

namespace mi355 {

int launch_tile_ring_mx(const GemmArgs& g, int out_dtype, int tile, hipStream_t stream) {
  if (!g.mx_a || !g.mx_b) return -1;
  return out_dtype == 0 ? launch<MxE4M3, BF16>(g, tile, stream) : launch<MxE4M3, F16>(g, tile, stream);
}

}  // namespace mi355
