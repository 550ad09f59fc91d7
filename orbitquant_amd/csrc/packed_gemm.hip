// Tile GEMM, two-4-bit-codes-per-byte activations; tile choice and dispatch for both code formats.
#include <stdlib.h>

#include "packed_gemm_kernel.h"

namespace oq {

int gemm_launch_bytes(const GemmArgs &g, int bits, int tile, hipStream_t stream);  // packed_gemm_bytes.hip

// Tile choice by a small cost model: a launch runs in `rounds` of as many workgroups as fit
// on the chip at once; a workgroup costs a fixed prologue + epilogue and a time per K-step
// of 64 (both measured on an MI355X, microseconds).  128x128 tiles fit two to a CU.
int gemm_choose_tile(int64_t M, int64_t N, int64_t K) {
  const char *force = getenv("OQ_GEMM_TILE");
  const bool can_split = K % 256 == 0;  // a quarter of the K-steps per wavefront
  if (force != nullptr && force[0] >= '0' && force[0] <= '3') return force[0] - '0';
  if (force != nullptr && force[0] == '4' && can_split) return 4;
  struct Shape { int tm, tn; double fixed, per_step; };
  static const Shape shapes[4] = {{128, 128, 4.5, 0.8}, {128, 256, 5.5, 1.0}, {256, 256, 7.0, 1.5}, {256, 192, 6.0, 1.15}};
  const double steps = static_cast<double>(K / 64);
  int best = 0;
  double best_cost = 0.0;
  for (int t = 0; t < 4; ++t) {
    const int64_t tiles = ((M + shapes[t].tm - 1) / shapes[t].tm) * ((N + shapes[t].tn - 1) / shapes[t].tn);
    double per_step = shapes[t].per_step;
    int64_t capacity = 256;
    if (t == 0) {
      if (tiles <= 256) per_step = 0.5;  // one workgroup per CU: no LDS contention
      else capacity = 512;
    }
    const double rounds = static_cast<double>((tiles + capacity - 1) / capacity);
    const double cost = rounds * (shapes[t].fixed + steps * per_step);
    if (t == 0 || cost < best_cost) {
      best = t;
      best_cost = cost;
    }
  }
  if (can_split) {  // 128x96 tiles, four wavefronts share the K range (+ about 1.5 us of reduction)
    const int64_t tiles = ((M + 127) / 128) * ((N + 95) / 96);
    const double cost = static_cast<double>((tiles + 255) / 256) * (7.5 + steps / 4.0 * 1.15);
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
                  int out_dtype, hipStream_t stream) {
  GemmArgs g{};
  g.a = static_cast<const uint8_t *>(a); g.row_scale = row_scale; g.act_cents = act_cents; g.a_levels = a_levels;
  g.w = w; g.row_norms = row_norms; g.w_cents = w_cents; g.bias = bias; g.bias_dtype = bias_dtype;
  g.M = M; g.N = N; g.K = K; g.out = out; g.out_dtype = out_dtype;
  const int tile = gemm_choose_tile(M, N, K);
  if (a_mode == A_NIBBLE) return launch_mode<A_NIBBLE>(g, bits, tile, stream);
  if (a_mode == A_U8) return gemm_launch_bytes(g, bits, tile, stream);
  return fail(OQ_ERR_INVALID, "packed_gemm: a_mode %d", a_mode);
}

}  // namespace oq
