// Dispatch of the one-token quantized linear (token_linear_impl.h): decides whether the single
// launch applies, and builds the arguments of its two halves.
#include "packed_gemv_body.h"
#include "rotate_quantize_row.h"

namespace oq {

int token_linear_launch_w2(const rq::RqArgs &q, const gemv::GemvArgs &g, int x_dtype, size_t rq_bytes, hipStream_t stream);
int token_linear_launch_w3(const rq::RqArgs &q, const gemv::GemvArgs &g, int x_dtype, size_t rq_bytes, hipStream_t stream);
int token_linear_launch_w4(const rq::RqArgs &q, const gemv::GemvArgs &g, int x_dtype, size_t rq_bytes, hipStream_t stream);

namespace {
constexpr size_t kLdsPerWorkgroup = 160 * 1024;  // gfx950
}  // namespace

// One token, 16-bit input, nibble activation codes, a weight width the streaming kernel has a
// single-launch variant for, K a multiple of 128 up to 8192 and N up to 8192 (measured: for
// longer rows every workgroup spends longer quantizing than a second launch costs, and more
// output rows than 32 per CU lose more by running one workgroup per CU than the launch
// saves) and 16-byte aligned operands.
bool token_linear_supported(int x_dtype, int64_t M, int64_t N, int64_t K, int levels, int bits, const void *x,
                            const int32_t *perm, const int8_t *signs) {
  auto aligned16 = [](const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; };
  if (debug_env(ENV_NO_TOKEN_LINEAR) != nullptr) return false;
  return M == 1 && (x_dtype == OQ_BF16 || x_dtype == OQ_F16) && levels <= 16 && K % 128 == 0 &&
         K <= 8192 && N <= 8192 && (bits == 2 || bits == 3 || bits == 4) &&
         aligned16(x) && aligned16(perm) && aligned16(signs);
}

int token_linear_dispatch(const void *x, int x_dtype, const uint16_t *input_map, int64_t K, const int32_t *perm,
                          const int8_t *signs, const float *boundaries, const float *act_cents, int levels,
                          int64_t block, float eps, float inv_sqrt_block, const uint8_t *packed_w, int bits,
                          const uint16_t *row_norms, const float *w_cents, const void *bias, int bias_dtype,
                          int64_t N, void *out, int out_dtype, hipStream_t stream, bool *launched) {
  *launched = false;
  rq::RqArgs q;
  bool vec = false;
  // codes and norm live in LDS; the placeholders only have to look like aligned buffers to the checks
  const int rc = rotate_quantize_prepare(x, x_dtype, 1, K, perm, signs, boundaries, nullptr, levels, block, eps,
                                         inv_sqrt_block, reinterpret_cast<void *>(16), OQ_CODES_NIBBLE, nullptr,
                                         OQ_VALUES_NONE, reinterpret_cast<float *>(16), input_map, &q, &vec);
  if (rc != OQ_OK) return rc;
  if (!vec) return OQ_OK;
  // the quantizer runs on all wavefronts of the streaming workgroup: 2 or 4 groups of 256 threads
  const int waves = N <= 16 * 256 ? gemv::gemv_waves(N, K) : 8;
  const size_t rq_bytes = rq::lds_bytes(q, x_dtype, true, waves * 64 / rq::kThreads);
  const size_t dynamic = rq_bytes + K / 2 + 32;
  if (static_cast<size_t>(gemv::kGemvTableBytes) + dynamic > kLdsPerWorkgroup) return OQ_OK;  // the caller takes two launches
  gemv::GemvArgs g{};
  g.act_cents = act_cents; g.a_levels = levels; g.w = packed_w; g.row_norms = row_norms; g.w_cents = w_cents;
  g.bias = bias; g.bias_dtype = bias_dtype; g.M = 1; g.N = N; g.K = K; g.out = out; g.out_dtype = out_dtype;
  *launched = true;
  switch (bits) {
    case 2: return token_linear_launch_w2(q, g, x_dtype, rq_bytes, stream);
    case 3: return token_linear_launch_w3(q, g, x_dtype, rq_bytes, stream);
    default: return token_linear_launch_w4(q, g, x_dtype, rq_bytes, stream);
  }
}

}  // namespace oq
