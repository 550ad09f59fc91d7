// Several small-M packed linears that read the SAME activation codes (the q, k and v projections
// of an attention block; the gate and up projections of an MLP) in one launch.  At decode sizes a
// launch of the streaming kernel is mostly fixed cost (start-up, table build, the cross-wave sum):
// three matrices of a few MB each take little longer in one grid than one of them does alone.
//
// A workgroup finds its matrix from its index (a uniform choice: every lane of the workgroup takes
// the same one) and runs the streaming kernel's body (packed_gemv_body.h) on it, with the weight
// width switched at run time between the 2-, 3- and 4-bit instances.  The K-split (WAVES) is the
// one a launch of each matrix alone would take, so every output equals that launch's bit for bit;
// the rows per workgroup (R) do not enter the sums.
#include "packed_gemv_group.h"

namespace oq {
namespace {

using namespace gemv;

template <int R, int WAVES, bool ASTAGE, int MB = 1>
__global__ __launch_bounds__(64 * WAVES) void packed_gemv_group_kernel(GroupArgs ga) {
  OQ_GEMV_TABLE_BLOCK(lds);
  GemvArgs g;
  int bits, first;
  group_member(ga, blockIdx.x, g, bits, first);
  const int64_t group = static_cast<int>(blockIdx.x) - first;
  if (bits == 2) packed_gemv_body<false, 2, R, WAVES, false, ASTAGE, MB>(g, lds, group, [](auto) {});
  else if (bits == 3) packed_gemv_body<false, 3, R, WAVES, false, ASTAGE, MB>(g, lds, group, [](auto) {});
  else packed_gemv_body<false, 4, R, WAVES, false, ASTAGE, MB>(g, lds, group, [](auto) {});
}

template <int R, int WAVES, int MB = 1>
int launch_group(GroupArgs &ga, hipStream_t stream) {
  const int64_t total = group_grid(ga, R);
  if (total < 0) return fail(OQ_ERR_UNSUPPORTED, "packed_linear_group: too many rows");
  auto kern = packed_gemv_group_kernel<R, WAVES, false, MB>;
  if constexpr (MB == 1) {
    if (gemv_stages_activations(ga.m[0].M, ga.m[0].K)) kern = packed_gemv_group_kernel<R, WAVES, true>;
  }
  hipLaunchKernelGGL(kern, dim3(static_cast<unsigned>(total)), dim3(64 * WAVES), 0, stream, ga);
  return check_launch("packed_linear_group");
}

}  // namespace

// One launch for `count` matrices, or *launched = false (nothing done) when the group does not
// qualify: nibble codes, at most 32 tokens, 2-, 3- or 4-bit weights, two to four matrices
// that a launch of their own would all split over the same number of wavefronts, and 16-byte
// aligned operands.
int gemv_group_dispatch(const void *codes, int code_format, const float *row_scale, const float *act_cents, int a_levels,
                        int count, const uint8_t *const *w, const int *bits, const uint16_t *const *row_norms,
                        const float *const *w_cents, const void *const *bias, int bias_dtype, int64_t M,
                        const int64_t *N, int64_t K, void *const *out, int out_dtype, hipStream_t stream, bool *launched) {
  *launched = false;
  auto aligned16 = [](const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; };
  if (debug_env(ENV_NO_GEMV_GROUP) != nullptr) return OQ_OK;
  // (beyond 32 tokens a group measured no faster than its members' own launches)
  if (code_format != OQ_CODES_NIBBLE || a_levels > 16 || M < 1 || M > 32 || M > gemv_max_tokens() || !aligned16(codes)) return OQ_OK;
  int64_t rows = 0;
  const int waves = group_waves(count, w, bits, N, K, &rows);
  if (waves == 0) return OQ_OK;
  GroupArgs ga;
  group_fill(ga, codes, row_scale, act_cents, a_levels, count, w, bits, row_norms, w_cents, bias, bias_dtype, M, N, K, out, out_dtype);
  int r = group_rows_per_step(rows);
  *launched = true;
  if (M > 16) {
    // 17 to 32 tokens: two blocks of sixteen token rows per workgroup; the partial sums of a workgroup
    // (wavefronts x row blocks x row steps KB) have to fit the 64 KB table block
    const int r_max = 64 / (waves * 2);
    if (r > r_max) r = r_max;
    if (waves == 16) return r == 1 ? launch_group<1, 16, 2>(ga, stream) : launch_group<2, 16, 2>(ga, stream);
    if (r == 1) return launch_group<1, 8, 2>(ga, stream);
    return r == 2 ? launch_group<2, 8, 2>(ga, stream) : launch_group<4, 8, 2>(ga, stream);
  }
  if (waves == 16) {
    if (r == 1) return launch_group<1, 16>(ga, stream);
    if (r == 2) return launch_group<2, 16>(ga, stream);
    return launch_group<4, 16>(ga, stream);
  }
  if (r == 1) return launch_group<1, 8>(ga, stream);
  if (r == 2) return launch_group<2, 8>(ga, stream);
  return launch_group<4, 8>(ga, stream);
}

}  // namespace oq
