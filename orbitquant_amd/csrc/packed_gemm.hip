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
// byte_codes: one activation code per byte (eight single lookups per operand instead of four pair lookups);
// a K-step then costs 1.07-1.23 times as much, least on the tiles with many columns per activation row.
static int choose_tile_with_cost(int64_t M, int64_t N, int64_t K, int bits, double *cost_out, bool byte_codes = false) {
  const bool can_split = K % 256 == 0;  // a quarter of the K-steps per wavefront
  const char *force = debug_env(ENV_GEMM_TILE);
  if (force != nullptr && force[0] >= '0' && force[0] <= '3') return force[0] - '0';
  if (force != nullptr && force[0] == '4' && can_split) return 4;
  struct Shape { int tm, tn; double fixed, step_short, step_busy, other_bits, bytes; };
  static const Shape shapes[4] = {{128, 128, 4.5, 0.8, 1.19, 1.28, 1.20}, {128, 256, 5.5, 1.0, 1.0, 1.34, 1.07},
                                  {256, 256, 7.0, 1.5, 1.68, 1.13, 1.10}, {256, 192, 6.0, 1.15, 1.24, 1.30, 1.23}};
  const double steps = static_cast<double>(K / 64);
  const bool busy = 2.0 * static_cast<double>(M) * static_cast<double>(N) * static_cast<double>(K) > 5.0e10;  // some 50 us of work
  int best = 0;
  double best_cost = 0.0;
  for (int t = 0; t < 4; ++t) {
    const Shape &sh = shapes[t];
    const int64_t tiles = ((M + sh.tm - 1) / sh.tm) * ((N + sh.tn - 1) / sh.tn);
    const int64_t capacity = t == 0 ? 512 : 256;
    const double width = (bits == 4 ? 1.0 : sh.other_bits) * (byte_codes ? sh.bytes : 1.0);
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
    const double per_step = (busy ? shapes[3].step_busy : shapes[3].step_short) * (bits == 4 ? 1.0 : shapes[3].other_bits) *
                            (byte_codes ? shapes[3].bytes : 1.0);
    const double cost = static_cast<double>((tiles + 255) / 256) * (7.5 + steps / 4.0 * per_step);
    if (cost < best_cost) {
      best = 4;
      best_cost = cost;
    }
  }
  if (cost_out != nullptr) *cost_out = best_cost;
  return best;
}

int gemm_choose_tile(int64_t M, int64_t N, int64_t K, int bits) { return choose_tile_with_cost(M, N, K, bits, nullptr); }

int gemm_splitk_reduce(const float *partials, int splits, int64_t M, int64_t N, const float *row_scale,
                       const uint16_t *row_norms, const void *bias, int bias_dtype, void *out, int out_dtype,
                       hipStream_t stream);  // packed_gemm_splitk.hip
int apply_value_map(void *out, int64_t count, const uint16_t *table, hipStream_t stream);

// Short-and-long problems at a few hundred tokens (128 x 4096 outputs over K = 14336) have a few dozen tiles
// for 256 CUs, each with hundreds of K-steps.  Such a launch shares K between workgroups: `splits`
// workgroups per 128x128 tile, each over its part of the K-steps, raw fp32 partial tiles into a buffer, and a
// small second launch that adds them in order and applies the epilogue.  Returns the number of parts (1:
// none), chosen with the cost model above plus the second launch (3 us and the partial tiles, written and
// read back, at 3 TB/s):
// every part keeps at least sixteen K-steps, the partial tiles stay within 64 MB, and the split has to
// promise 15 % over the best single launch.  OQ_GEMM_WG_SPLIT overrides (1 = never).
int gemm_choose_splits(int64_t M, int64_t N, int64_t K, int bits) {
  const int64_t tiles = ((M + 127) / 128) * ((N + 127) / 128), steps = K / 64;
  auto allowed = [&](int s) { return s >= 2 && s <= 8 && steps / s >= 16 && M * N * 4 * s <= (64ll << 20); };
  if (const char *force = debug_env(ENV_GEMM_WG_SPLIT)) {
    int s = atoi(force);
    while (s > 1 && !allowed(s)) --s;
    return s < 1 ? 1 : s;
  }
  if (debug_env(ENV_GEMM_TILE) != nullptr) return 1;  // a forced tile is a forced single launch
  double single = 0.0;
  choose_tile_with_cost(M, N, K, bits, &single);
  const double width = bits == 4 ? 1.0 : 1.28;
  int best = 1;
  double best_cost = 0.85 * single;
  for (int s = 2; s <= 8; ++s) {
    if (!allowed(s)) continue;
    const int64_t groups = tiles * s;
    const double per_step = (groups <= 256 ? 0.5 : 0.8) * width;
    const double rounds = static_cast<double>((groups + 511) / 512);
    const double cost = rounds * (4.5 + static_cast<double>(steps / s) * per_step) + 3.0 +
                        static_cast<double>(M) * static_cast<double>(N) * (8.0 * s + 2.0) / 3.0e6;  // partial tiles written, then read
    if (cost < best_cost) {
      best = s;
      best_cost = cost;
    }
  }
  return best;
}

bool gemm_supported(int64_t K, int bits) {
  return K % 64 == 0 && (bits == 2 || bits == 3 || bits == 4 || bits == 6 || bits == 8);
}

// a_mode: 0 nibble codes, 1 bf16 values, 2 fp16 values
// Bytes of partial tiles a launch of this shape would like to have (0: it is a single launch anyway).
uint64_t gemm_workspace_bytes(int64_t M, int64_t N, int64_t K, int bits) {
  const int splits = gemm_choose_splits(M, N, K, bits);
  return splits > 1 ? static_cast<uint64_t>(M) * static_cast<uint64_t>(N) * 4u * static_cast<uint64_t>(splits) : 0u;
}

// `workspace` (the caller's; NULL or too small: the single launch, whatever the stream is doing) holds the
// partial tiles of a launch that shares K between workgroups.
int gemm_dispatch(int a_mode, const void *a, const float *row_scale, const float *act_cents, int a_levels,
                  const uint8_t *w, int bits, const uint16_t *row_norms, const float *w_cents,
                  const void *bias, int bias_dtype, int64_t M, int64_t N, int64_t K, void *out,
                  int out_dtype, const uint16_t *out_map, void *workspace, uint64_t workspace_bytes, hipStream_t stream) {
  GemmArgs g{};
  g.a = static_cast<const uint8_t *>(a); g.row_scale = row_scale; g.act_cents = act_cents; g.a_levels = a_levels;
  g.w = w; g.row_norms = row_norms; g.w_cents = w_cents; g.bias = bias; g.bias_dtype = bias_dtype;
  g.M = M; g.N = N; g.K = K; g.out = out; g.out_dtype = out_dtype;
  g.out_map = OutMap{out_map, out_map != nullptr && out_dtype == OQ_BF16 ? kWideLoBf16 : -1};
  int tile = choose_tile_with_cost(M, N, K, bits, nullptr, a_mode == A_U8);
  if (a_mode != A_NIBBLE && a_mode != A_U8) return fail(OQ_ERR_INVALID, "packed_gemm: a_mode %d", a_mode);
  g.k_splits = 1;
  if (const char *where = debug_env(ENV_GEMM_STAMPS)) g.stamps = reinterpret_cast<uint64_t *>(strtoull(where, nullptr, 0));  // builds with -DOQ_GEMM_STAMPS: a device buffer for the kernel's phase stamps
  const int splits = gemm_choose_splits(M, N, K, bits);
  if (splits > 1 && workspace != nullptr && (reinterpret_cast<uintptr_t>(workspace) & 15u) == 0 &&
      workspace_bytes >= static_cast<uint64_t>(M) * static_cast<uint64_t>(N) * 4u * static_cast<uint64_t>(splits)) {
    g.k_splits = splits;
    g.partials = static_cast<float *>(workspace);
    tile = 0;  // 128x128 tiles, two workgroups per CU
  }
  const int rc = a_mode == A_NIBBLE ? launch_mode<A_NIBBLE>(g, bits, tile, stream) : gemm_launch_bytes(g, bits, tile, stream);
  if (rc != OQ_OK || g.k_splits == 1) return rc;
  if (int rc2 = gemm_splitk_reduce(g.partials, g.k_splits, M, N, row_scale, row_norms, bias, bias_dtype, out, out_dtype, stream))
    return rc2;
  return out_map == nullptr ? OQ_OK : apply_value_map(out, M * N, out_map, stream);
}

}  // namespace oq
