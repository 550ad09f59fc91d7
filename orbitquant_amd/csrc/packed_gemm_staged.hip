// Tile GEMM on bf16 activation VALUES read as the caller has them (no pass, no buffer): the A_STAGED mode of
// packed_gemm_kernel.h, in which every wavefront stages the K-step pieces of its own rows through a private slab
// of LDS.  Same sums as the other modes; about as fast as the operand-order pass + kernel at the DiT shapes
// (39 us at 2048 x 4608 x 1152), 10-15 % slower on large problems; what oq_matmul_packed_weight takes when it may
// not allocate (stream capture) or cannot.
#include "packed_gemm_kernel.h"

namespace oq {

int gemm_choose_tile(int64_t M, int64_t N, int64_t K, int bits);  // packed_gemm.hip

// x: bf16 [M, K] as it is; M * K * 2 < 4 GB, 16-byte aligned rows.  No pass, no buffer.
int gemm_staged_dispatch(const void *x, const float *token_scale, const uint8_t *w, int bits, const uint16_t *row_norms,
                         const float *w_cents, const void *bias, int bias_dtype, int64_t M, int64_t N, int64_t K, void *out,
                         int out_dtype, hipStream_t stream) {
  GemmArgs g{};
  g.a = static_cast<const uint8_t *>(x); g.row_scale = token_scale; g.act_cents = w_cents; g.a_levels = 0;
  g.w = w; g.row_norms = row_norms; g.w_cents = w_cents; g.bias = bias; g.bias_dtype = bias_dtype;
  g.M = M; g.N = N; g.K = K; g.out = out; g.out_dtype = out_dtype;
  g.out_map = OutMap{nullptr, -1};
  const int tile = gemm_choose_tile(M, N, K, bits);
  auto go = [&](auto bits_c) {
    constexpr int BITS = decltype(bits_c)::value;
    if (tile == 4) return launch_cfg<A_STAGED, BITS, 4, 3, 4>(g, stream);
    if (tile == 3 || tile == 2) return launch_cfg<A_STAGED, BITS, 4, 3>(g, stream);
    if (tile == 1) return launch_cfg<A_STAGED, BITS, 2, 4>(g, stream);
    return launch_cfg<A_STAGED, BITS, 2, 2>(g, stream);
  };
  switch (bits) {
    case 2: return go(std::integral_constant<int, 2>{});
    case 3: return go(std::integral_constant<int, 3>{});
    case 4: return go(std::integral_constant<int, 4>{});
    case 6: return go(std::integral_constant<int, 6>{});
    case 8: return go(std::integral_constant<int, 8>{});
    default: return fail(OQ_ERR_UNSUPPORTED, "packed_gemm: weight width %d", bits);
  }
}

}  // namespace oq
