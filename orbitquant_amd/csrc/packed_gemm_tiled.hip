// Tile GEMM on bf16 activation VALUES (the generic float-activation contract at large M): the
// activations are first rewritten into the matrix core's operand order (one small pass over M*K
// values), then the tile kernel of packed_gemm_kernel.h runs with its activation operands loaded
// straight into registers, 1 KB of consecutive bytes per wavefront load, and only the weights go
// through the lookup tables: 4 FN lookups per FM*FN MFMAs instead of 4 (FM + FN), and no
// workgroup-wide staging of an activation slab between barriers.
#include <utility>

#include "packed_gemm_kernel.h"

namespace oq {
namespace {

// piece ((row_tile * steps + k_step) * 4 + q) * 64 + 32 g + r  <-  x[32 row_tile + r][64 k_step + 32 g + 8 q .. + 7].
// A wavefront moves a quarter (eight rows) of one 32-row x 64-value block: lane l reads 16-byte chunk l % 8 of row
// 8 j + l / 8 (whole 128-byte lines in) and writes it as piece (q = chunk % 4, g = chunk / 4, r) (whole lines out).
__global__ __launch_bounds__(256) void tile_activations_kernel(const uint16_t *x, int64_t M, int64_t K, uint4 *tiled) {
  // workgroup (four k_steps, row_tile); a wavefront moves one block, eight rows per load
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int64_t steps = K / 64, ks = static_cast<int64_t>(blockIdx.x) * 4 + wave, rt = blockIdx.y;
  if (ks >= steps) return;
  const int chunk = lane & 7;
  uint4 v[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int64_t row = rt * 32 + 8 * j + (lane >> 3);
    v[j] = row < M ? *reinterpret_cast<const uint4 *>(x + row * K + ks * 64 + chunk * 8) : make_uint4(0u, 0u, 0u, 0u);
  }
  uint4 *out = tiled + ((rt * steps + ks) * 4 + (chunk & 3)) * 64 + (chunk >> 2) * 32 + (lane >> 3);
#pragma unroll
  for (int j = 0; j < 4; ++j) out[8 * j] = v[j];
}

// The operand-order copy lives in a buffer the library keeps per (device, stream) and grows on demand: calls on one
// stream are ordered, so they can share it; it is released when the process ends.
template <int BITS>
int launch_tiled(const GemmArgs &g, int tile, hipStream_t stream) {
  if (tile == 4) return launch_cfg<A_TILED, BITS, 4, 3, 4>(g, stream);
  if (tile == 3) return launch_cfg<A_TILED, BITS, 4, 3>(g, stream);
  if (tile == 1 || tile == 2) return launch_cfg<A_TILED, BITS, 2, 4>(g, stream);
  return launch_cfg<A_TILED, BITS, 2, 2>(g, stream);
}

}  // namespace

int gemm_choose_tile(int64_t M, int64_t N, int64_t K, int bits);  // packed_gemm.hip

// Bytes of the operand-order copy of [M, K] bf16 activations (whole row tiles of 32).
uint64_t gemm_tiled_workspace_bytes(int64_t M, int64_t K) {
  const int64_t row_tiles = (M + 31) / 32, pieces = row_tiles * (K / 64) * 256;
  return row_tiles > 65535 ? 0u : static_cast<uint64_t>(pieces) * 16u;
}

// x: bf16 [M, K], 16-byte aligned rows (K % 64 == 0).  `workspace`: the caller's buffer for the operand-order
// copy, gemm_tiled_workspace_bytes(M, K) bytes, 16-byte aligned; -1 (the caller takes the kernel that needs no
// buffer) when it is absent or too small.
int gemm_tiled_dispatch(const void *x, const float *token_scale, const uint8_t *w, int bits, const uint16_t *row_norms,
                        const float *w_cents, const void *bias, int bias_dtype, int64_t M, int64_t N, int64_t K, void *out,
                        int out_dtype, void *workspace, uint64_t workspace_bytes, hipStream_t stream) {
  const int64_t row_tiles = (M + 31) / 32;
  const uint64_t need = gemm_tiled_workspace_bytes(M, K);
  void *tiled = workspace;
  if (tiled == nullptr || need == 0 || workspace_bytes < need || (reinterpret_cast<uintptr_t>(tiled) & 15u) != 0) return -1;
  hipLaunchKernelGGL(tile_activations_kernel, dim3(static_cast<unsigned>((K / 64 + 3) / 4), static_cast<unsigned>(row_tiles)), dim3(256), 0, stream,
                     static_cast<const uint16_t *>(x), M, K, static_cast<uint4 *>(tiled));
  int rc = check_launch("tile_activations");
  if (rc == OQ_OK) {
    GemmArgs g{};
    g.a = static_cast<const uint8_t *>(tiled); g.row_scale = token_scale; g.act_cents = w_cents; g.a_levels = 0;
    g.w = w; g.row_norms = row_norms; g.w_cents = w_cents; g.bias = bias; g.bias_dtype = bias_dtype;
    g.M = M; g.N = N; g.K = K; g.out = out; g.out_dtype = out_dtype;
    g.out_map = OutMap{nullptr, -1};
    const int tile = gemm_choose_tile(M, N, K, bits);
    switch (bits) {
      case 2: rc = launch_tiled<2>(g, tile, stream); break;
      case 3: rc = launch_tiled<3>(g, tile, stream); break;
      case 4: rc = launch_tiled<4>(g, tile, stream); break;
      case 6: rc = launch_tiled<6>(g, tile, stream); break;
      case 8: rc = launch_tiled<8>(g, tile, stream); break;
      default: rc = fail(OQ_ERR_UNSUPPORTED, "packed_gemm: weight width %d", bits);
    }
  }
  return rc;
}

}  // namespace oq
