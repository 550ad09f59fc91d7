// Tile GEMM, one activation code per byte (activation widths above 4 bits).
#include "packed_gemm_kernel.h"

namespace oq {

int gemm_launch_bytes(const GemmArgs &g, int bits, int tile, hipStream_t stream) {
  return launch_mode<A_U8>(g, bits, tile, stream);
}

}  // namespace oq
