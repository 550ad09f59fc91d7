// Small-M (decode-sized, M <= 16; up to 64 through packed_gemv_rows.hip) packed-weight linear on
// activation codes: kernel, launch configuration and argument checks.  The arithmetic is in
// packed_gemv_body.h.
#include "packed_gemv_body.h"

namespace oq {
namespace {

using namespace gemv;

// The arguments come one by one, the ones the first loads need first: the first sixteen dwords of a
// kernel's arguments can be handed over in scalar registers when the wavefront starts (the build asks for
// that with -mllvm -amdgpu-kernarg-preload-count=16), and then the weight stream is requested without
// waiting for a load of the argument block (0.6-0.8 us at the head of a 9 us launch).  A struct passed by
// value is never handed over that way.
template <bool BYTES, int BITS, int R, int WAVES, bool ASTAGE = false>
__global__ __launch_bounds__(64 * WAVES) void packed_gemv_kernel(const uint8_t *w, const uint8_t *a, const float *w_cents,
                                                                 const float *act_cents, int64_t K, int64_t N,
                                                                 const uint16_t *row_norms, int M, int a_levels,
                                                                 const float *row_scale, const void *bias, int bias_dtype,
                                                                 void *out, int out_dtype) {
  OQ_GEMV_TABLE_BLOCK(lds);
  GemvArgs g;
  g.a = a; g.row_scale = row_scale; g.act_cents = act_cents; g.a_levels = a_levels; g.w = w; g.row_norms = row_norms;
  g.w_cents = w_cents; g.bias = bias; g.bias_dtype = bias_dtype; g.M = M; g.N = N; g.K = K; g.out = out; g.out_dtype = out_dtype;
  packed_gemv_body<BYTES, BITS, R, WAVES, false, ASTAGE>(g, lds, blockIdx.x, [](auto) {});
}

template <bool BYTES, int BITS, int R, int WAVES>
int launch(const GemvArgs &g, hipStream_t stream) {
  const int64_t groups = (g.N + 16 * R - 1) / (16 * R);
  if (groups > 0x7fffffffLL) return fail(OQ_ERR_UNSUPPORTED, "packed_gemv: N too large");
  auto kern = packed_gemv_kernel<BYTES, BITS, R, WAVES>;
  // few tokens of nibble codes: the variant that decodes the activation values once per workgroup
  // (same sums)
  if constexpr (!BYTES) {
    if (gemv_stages_activations(g.M, g.K)) kern = packed_gemv_kernel<BYTES, BITS, R, WAVES, true>;
  }
  hipLaunchKernelGGL(kern, dim3(static_cast<unsigned>(groups)), dim3(64 * WAVES), 0, stream, g.w, g.a, g.w_cents, g.act_cents, g.K,
                     g.N, g.row_norms, g.M, g.a_levels, g.row_scale, g.bias, g.bias_dtype, g.out, g.out_dtype);
  return check_launch("packed_gemv");
}

template <bool BYTES, int BITS, int R>
int launch_waves(const GemvArgs &g, int waves, hipStream_t stream) {
  if constexpr (R == 1) {
    if (waves == 16) return launch<BYTES, BITS, R, 16>(g, stream);
  }
  if constexpr (!BYTES) {  // the other wavefront counts exist for experiments with OQ_GEMV_CFG only
    if (waves == 4) return launch<BYTES, BITS, R, 4>(g, stream);
    if (waves == 16) return launch<BYTES, BITS, R, 16>(g, stream);
  }
  return launch<BYTES, BITS, R, 8>(g, stream);
}

template <bool BYTES, int BITS>
int launch_bits(const GemvArgs &g, hipStream_t stream) {
  // rows per workgroup (16*R) and K-split (wavefronts per workgroup); OQ_GEMV_CFG="R,WAVES" overrides
  int r = g.N <= 16 * 512 ? 1 : 2, waves = gemv_waves(g.N, g.K);
  if (const char *cfg = debug_env(ENV_GEMV_CFG)) {
    int cr = 0, cw = 0;
    if (sscanf(cfg, "%d,%d", &cr, &cw) == 2 && (cr == 1 || cr == 2 || cr == 4) && (cw == 4 || cw == 8 || cw == 16)) {
      r = cr;
      waves = cw;
    }
  }
  if (r == 1) return launch_waves<BYTES, BITS, 1>(g, waves, stream);
  if constexpr (!BYTES) {
    if (r == 4) return launch_waves<BYTES, BITS, 4>(g, waves, stream);
  }
  return launch_waves<BYTES, BITS, 2>(g, waves, stream);
}

}  // namespace

int gemv_rows_dispatch(const gemv::GemvArgs &g, int bits, bool bytes, hipStream_t stream);  // packed_gemv_rows.hip

bool gemv_supported(int64_t M, int64_t K, int bits, int code_format, int a_levels) {
  const bool codes_ok = code_format == OQ_CODES_NIBBLE ? a_levels <= 16 : a_levels <= 256;
  return M >= 1 && M <= gemv_max_tokens() && K % 128 == 0 && codes_ok && (bits == 2 || bits == 3 || bits == 4 || bits == 6 || bits == 8);
}

int gemv_dispatch(const void *codes, int code_format, const float *row_scale, const float *act_cents, int a_levels,
                  const uint8_t *w, int bits, const uint16_t *row_norms, const float *w_cents,
                  const void *bias, int bias_dtype, int64_t M, int64_t N, int64_t K, void *out,
                  int out_dtype, hipStream_t stream) {
  GemvArgs g{};
  g.a = static_cast<const uint8_t *>(codes); g.row_scale = row_scale; g.act_cents = act_cents; g.a_levels = a_levels;
  g.w = w; g.row_norms = row_norms; g.w_cents = w_cents; g.bias = bias; g.bias_dtype = bias_dtype;
  g.M = static_cast<int>(M); g.N = N; g.K = K; g.out = out; g.out_dtype = out_dtype;
  if (M > 16) return gemv_rows_dispatch(g, bits, code_format != OQ_CODES_NIBBLE, stream);
#define OQ_GEMV_BITS(BYTES)                                                   \
  switch (bits) {                                                             \
    case 2: return launch_bits<BYTES, 2>(g, stream);                          \
    case 3: return launch_bits<BYTES, 3>(g, stream);                          \
    case 4: return launch_bits<BYTES, 4>(g, stream);                          \
    case 6: return launch_bits<BYTES, 6>(g, stream);                          \
    case 8: return launch_bits<BYTES, 8>(g, stream);                          \
    default: return fail(OQ_ERR_UNSUPPORTED, "packed_gemv: weight width %d", bits); \
  }
  if (code_format == OQ_CODES_NIBBLE) { OQ_GEMV_BITS(false) }
  OQ_GEMV_BITS(true)
#undef OQ_GEMV_BITS
}

}  // namespace oq
