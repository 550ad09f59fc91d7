// Arguments of the small-M kernel that serves several matrices in one launch
// (packed_gemv_group.hip): up to four matrices that read the same activation codes, the
// workgroups of the grid dealt to them in order.
#pragma once

#include "packed_gemv_body.h"

namespace oq {
namespace gemv {

constexpr int kMaxGroup = 4;

struct GroupArgs {
  GemvArgs m[kMaxGroup];
  int bits[kMaxGroup];
  int first[kMaxGroup + 1];  // first workgroup of every matrix; first[count] is the grid size
  int count;
};

// The matrix workgroup `b` works on (a uniform choice: every lane takes the same one), written
// with constant indices so that the arguments stay in scalar registers.
__device__ __forceinline__ void group_member(const GroupArgs &ga, int b, GemvArgs &g, int &bits, int &first) {
  g = ga.m[0];
  bits = ga.bits[0];
  first = 0;
#pragma unroll
  for (int j = 1; j < kMaxGroup; ++j) {
    if (j < ga.count && b >= ga.first[j]) {
      g = ga.m[j];
      bits = ga.bits[j];
      first = ga.first[j];
    }
  }
}

// The group's arguments from the caller's arrays (count entries each; `bias` may be NULL).
inline void group_fill(GroupArgs &ga, const void *codes, const float *row_scale, const float *act_cents, int a_levels,
                       int count, const uint8_t *const *w, const int *bits, const uint16_t *const *row_norms,
                       const float *const *w_cents, const void *const *bias, int bias_dtype, int64_t M,
                       const int64_t *N, int64_t K, void *const *out, int out_dtype) {
  ga = GroupArgs{};
  ga.count = count;
  for (int i = 0; i < count; ++i) {
    GemvArgs &g = ga.m[i];
    g.a = static_cast<const uint8_t *>(codes); g.row_scale = row_scale; g.act_cents = act_cents; g.a_levels = a_levels;
    g.w = w[i]; g.row_norms = row_norms[i]; g.w_cents = w_cents[i]; g.bias = bias != nullptr ? bias[i] : nullptr;
    g.bias_dtype = bias_dtype; g.M = static_cast<int>(M); g.N = N[i]; g.K = K; g.out = out[i]; g.out_dtype = out_dtype;
    ga.bits[i] = bits[i];
  }
}

// Whether `count` matrices can share a launch, and the K-split they all take: two to four
// matrices of 2-, 3- or 4-bit weights, 16-byte aligned, that a launch of their own would all
// split over the same number of wavefronts.  Returns 0 when they cannot.
inline int group_waves(int count, const uint8_t *const *w, const int *bits, const int64_t *N, int64_t K, int64_t *rows) {
  if (count < 2 || count > kMaxGroup || K % 128 != 0) return 0;
  const int waves = gemv_waves(N[0], K);
  *rows = 0;
  for (int i = 0; i < count; ++i) {
    if ((bits[i] != 2 && bits[i] != 3 && bits[i] != 4) || N[i] < 1 || gemv_waves(N[i], K) != waves ||
        (reinterpret_cast<uintptr_t>(w[i]) & 15u) != 0)
      return 0;
    *rows += N[i];
  }
  return waves;
}

// Deals the grid: fills `first` for R-row steps of 16 rows and returns the number of workgroups.
inline int64_t group_grid(GroupArgs &ga, int rows_per_step) {
  int64_t total = 0;
  for (int i = 0; i < ga.count; ++i) {
    ga.first[i] = static_cast<int>(total);
    total += (ga.m[i].N + 16 * rows_per_step - 1) / (16 * rows_per_step);
    if (total > 0x7fffffffLL) return -1;
  }
  for (int i = ga.count; i <= kMaxGroup; ++i) ga.first[i] = static_cast<int>(total);
  return total;
}

// Rows per workgroup step (16*R rows): enough that the grid is about one workgroup per CU; the
// results do not depend on it.  OQ_GEMV_GROUP_R overrides, for experiments.
inline int group_rows_per_step(int64_t rows) {
  int r = rows <= 16 * 256 ? 1 : rows <= 32 * 256 ? 2 : 4;
  if (const char *cfg = debug_env(ENV_GEMV_GROUP_R)) {
    const int cr = atoi(cfg);
    if (cr == 1 || cr == 2 || cr == 4) r = cr;
  }
  return r;
}

}  // namespace gemv
}  // namespace oq
