// The streaming kernel for 17 to 64 tokens: the body of packed_gemv_body.h with two or four blocks
// of sixteen token rows per workgroup (MB), so that the weights are still streamed and decoded
// once.  The tile kernel is the wrong tool there: its 128-row tiles are mostly padding, and a
// short-and-long matrix (4096 rows of 14336 values) gives it 32 workgroups for 256 CUs.
// Launch shapes (rows per workgroup, K-split) follow the rule of the sixteen-token launches, so a
// token row's sums do not depend on how many rows are computed with it.
#include "packed_gemv_body.h"

namespace oq {
namespace {

using namespace gemv;

template <bool BYTES, int BITS, int R, int WAVES, int MB>
__global__ __launch_bounds__(64 * WAVES) void packed_gemv_rows_kernel(GemvArgs g) {
  OQ_GEMV_TABLE_BLOCK(lds);
  packed_gemv_body<BYTES, BITS, R, WAVES, false, false, MB>(g, lds, blockIdx.x, [](auto) {});
}

template <bool BYTES, int BITS, int R, int WAVES, int MB>
int launch(const GemvArgs &g, hipStream_t stream) {
  const int64_t groups = (g.N + 16 * R - 1) / (16 * R);
  if (groups > 0x7fffffffLL) return fail(OQ_ERR_UNSUPPORTED, "packed_gemv: N too large");
  hipLaunchKernelGGL((packed_gemv_rows_kernel<BYTES, BITS, R, WAVES, MB>), dim3(static_cast<unsigned>(groups)),
                     dim3(64 * WAVES), 0, stream, g);
  return check_launch("packed_gemv_rows");
}

template <bool BYTES, int BITS, int MB>
int launch_shape(const GemvArgs &g, hipStream_t stream) {
  const int waves = gemv_waves(g.N, g.K);
  if (waves == 16) return launch<BYTES, BITS, 1, 16, MB>(g, stream);
  if (g.N <= 16 * 512) return launch<BYTES, BITS, 1, 8, MB>(g, stream);
  return launch<BYTES, BITS, 2, 8, MB>(g, stream);
}

template <bool BYTES, int BITS>
int launch_blocks(const GemvArgs &g, hipStream_t stream) {
  if (g.M <= 32) return launch_shape<BYTES, BITS, 2>(g, stream);
  return launch_shape<BYTES, BITS, 4>(g, stream);
}

}  // namespace

// 16 < g.M <= 64; everything else as checked by gemv_supported().
int gemv_rows_dispatch(const gemv::GemvArgs &g, int bits, bool bytes, hipStream_t stream) {
#define OQ_GEMV_BITS(BYTES)                                                   \
  switch (bits) {                                                             \
    case 2: return launch_blocks<BYTES, 2>(g, stream);                        \
    case 3: return launch_blocks<BYTES, 3>(g, stream);                        \
    case 4: return launch_blocks<BYTES, 4>(g, stream);                        \
    case 6: return launch_blocks<BYTES, 6>(g, stream);                        \
    case 8: return launch_blocks<BYTES, 8>(g, stream);                        \
    default: return fail(OQ_ERR_UNSUPPORTED, "packed_gemv: weight width %d", bits); \
  }
  if (!bytes) { OQ_GEMV_BITS(false) }
  OQ_GEMV_BITS(true)
#undef OQ_GEMV_BITS
}

}  // namespace oq
