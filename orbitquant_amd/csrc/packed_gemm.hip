// Tile GEMM, two-4-bit-codes-per-byte activations; tile choice and dispatch for both code formats.
#include <stdlib.h>

#include "packed_gemm_kernel.h"

namespace oq {

int gemm_launch_bytes(const GemmArgs &g, int bits, int tile, hipStream_t stream);  // packed_gemm_bytes.hip

// Tile choice by a small cost model.  A launch runs in rounds of as many workgroups as fit on
// the chip at once (256; 512 for the 128x128 tile, which fits two to a CU) plus one partial
// round; a workgroup costs a fixed prologue + epilogue and a time per K-step of 64.  The
// constants are microseconds measured on an MI355X: the "busy" set for launches long enough
// to run at sustained clocks with every CU occupied, the other for short launches; weight
// widths other than 4 pay for their longer index extraction, least on the largest tile.
int gemm_choose_tile(int64_t M, int64_t N, int64_t K, int bits) {
  const bool can_split = K % 256 == 0;  // a quarter of the K-steps per wavefront
  const char *force = debug_env(ENV_GEMM_TILE);
  if (force != nullptr && force[0] >= '0' && force[0] <= '3') return force[0] - '0';
  if (force != nullptr && force[0] == '4' && can_split) return 4;
  struct Shape { int tm, tn; double fixed, step_short, step_busy, other_bits; };
  static const Shape shapes[4] = {{128, 128, 4.5, 0.8, 1.19, 1.28}, {128, 256, 5.5, 1.0, 1.0, 1.34},
                                  {256, 256, 7.0, 1.5, 1.68, 1.13}, {256, 192, 6.0, 1.15, 1.24, 1.30}};
  const double steps = static_cast<double>(K / 64);
  const bool busy = 2.0 * static_cast<double>(M) * static_cast<double>(N) * static_cast<double>(K) > 2.0e11;
  int best = 0;
  double best_cost = 0.0;
  for (int t = 0; t < 4; ++t) {
    const Shape &sh = shapes[t];
    const int64_t tiles = ((M + sh.tm - 1) / sh.tm) * ((N + sh.tn - 1) / sh.tn);
    const int64_t capacity = t == 0 ? 512 : 256;
    const double width = bits == 4 ? 1.0 : sh.other_bits;
    const double per_step = (busy ? sh.step_busy : sh.step_short) * width;
    const int64_t full = tiles / capacity, rest = tiles % capacity;
    // a 128x128 workgroup alone on its CU has the LDS to itself
    const double rest_step = (t == 0 && rest <= 256) ? (busy ? 0.75 : 0.5) * width : per_step;
    const double cost = static_cast<double>(full) * (sh.fixed + steps * per_step) +
                        (rest > 0 ? sh.fixed + steps * rest_step : 0.0);
    if (t == 0 || cost < best_cost) {
      best = t;
      best_cost = cost;
    }
  }
  if (can_split) {  // 128x96 tiles, four wavefronts share the K range (+ about 1.5 us of reduction)
    const int64_t tiles = ((M + 127) / 128) * ((N + 95) / 96);
    const double per_step = (busy ? shapes[3].step_busy : shapes[3].step_short) * (bits == 4 ? 1.0 : shapes[3].other_bits);
    const double cost = static_cast<double>((tiles + 255) / 256) * (7.5 + steps / 4.0 * per_step);
    if (cost < best_cost) best = 4;
  }
  return best;
}

bool gemm_supported(int64_t K, int bits) {
  return K % 64 == 0 && (bits == 2 || bits == 3 || bits == 4 || bits == 6 || bits == 8);
}

// a_mode: 0 nibble codes, 1 bf16 values, 2 fp16 values
int gemm_dispatch(int a_mode, const void *a, const float *row_scale, const float *act_cents, int a_levels,
                  const uint8_t *w, int bits, const uint16_t *row_norms, const float *w_cents,
                  const void *bias, int bias_dtype, int64_t M, int64_t N, int64_t K, void *out,
                  int out_dtype, const uint16_t *out_map, hipStream_t stream) {
  GemmArgs g{};
  g.a = static_cast<const uint8_t *>(a); g.row_scale = row_scale; g.act_cents = act_cents; g.a_levels = a_levels;
  g.w = w; g.row_norms = row_norms; g.w_cents = w_cents; g.bias = bias; g.bias_dtype = bias_dtype;
  g.M = M; g.N = N; g.K = K; g.out = out; g.out_dtype = out_dtype;
  g.out_map = OutMap{out_map, out_map != nullptr && out_dtype == OQ_BF16 ? kWideLoBf16 : -1};
  const int tile = gemm_choose_tile(M, N, K, bits);
  if (a_mode == A_NIBBLE) return launch_mode<A_NIBBLE>(g, bits, tile, stream);
  if (a_mode == A_U8) return gemm_launch_bytes(g, bits, tile, stream);
  return fail(OQ_ERR_INVALID, "packed_gemm: a_mode %d", a_mode);
}

}  // namespace oq
