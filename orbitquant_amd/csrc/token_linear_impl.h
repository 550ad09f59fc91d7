// The quantized linear for ONE token in a single launch: every workgroup of the small-M
// streaming kernel builds its lookup tables, then rotates and quantizes the token row itself
// (all workgroups compute the same codes), requesting its share of the packed weights as soon
// as the quantizer has its own inputs, and goes on exactly like the streaming kernel, reading
// the activation codes and the token norm from LDS.  What this saves is the second launch.
// Both halves are the device functions the two separate kernels are made of, so the result is
// the one of oq_rotate_quantize followed by oq_packed_linear, bit for bit.
//
// Included by token_linear_w<BITS>.hip with OQ_TOKEN_LINEAR_BITS defined: one translation
// unit per weight width keeps the build parallel.
#include "packed_gemv_body.h"
#include "rotate_quantize_row.h"

namespace oq {
namespace {

// Dynamic LDS: [0, codes_offset) is the quantizer's scratch, then K/2 bytes of nibble codes and
// the norm (the streaming part's 64 KB table block is static).
// WAVES as the streaming kernel picks them (gemv_waves): 512 or 1024 threads = two or four pass
// groups of the quantizer.
template <int DT, int LOG_G, int BITS, int R, int WAVES>
__global__ __launch_bounds__(64 * WAVES) void token_linear_kernel(rq::RqArgs q, gemv::GemvArgs g, int codes_offset) {
  extern __shared__ __align__(16) unsigned char smem[];
  uint8_t *codes = smem + codes_offset;
  float *norm = reinterpret_cast<float *>(codes + ((q.K / 2 + 15) & ~static_cast<int64_t>(15)));
  q.codes = codes;
  q.norms = norm;
  g.a = codes;
  g.row_scale = norm;
  const int tid = threadIdx.x;
  OQ_GEMV_TABLE_BLOCK(tables);
  gemv::packed_gemv_body<false, BITS, R, WAVES, true>(g, tables, blockIdx.x, [&](auto issue_weights) {
    rq::rotate_quantize_row<DT, true, LOG_G, true>(q, smem, 0, tid, 64 * WAVES, issue_weights);
  });
}

template <int DT, int LOG_G, int BITS, int R, int WAVES>
int launch_token_waves(const rq::RqArgs &q, const gemv::GemvArgs &g, size_t rq_bytes, hipStream_t stream) {
  const size_t scratch = rq_bytes;
  const size_t smem = scratch + static_cast<size_t>((q.K / 2 + 15) & ~static_cast<int64_t>(15)) + 16;
  auto kern = token_linear_kernel<DT, LOG_G, BITS, R, WAVES>;
  if (!reserve_dynamic_lds(reinterpret_cast<const void *>(kern), smem))
    return fail(OQ_ERR_LAUNCH, "token_linear: cannot reserve %zu bytes of LDS", smem);
  const int64_t groups = (g.N + 16 * R - 1) / (16 * R);
  hipLaunchKernelGGL(kern, dim3(static_cast<unsigned>(groups)), dim3(64 * WAVES), smem, stream, q, g,
                     static_cast<int>(scratch));
  return check_launch("token_linear");
}

template <int DT, int LOG_G, int BITS, int R>
int launch_token(const rq::RqArgs &q, const gemv::GemvArgs &g, size_t rq_bytes, hipStream_t stream) {
  if constexpr (R == 1) {
    if (gemv::gemv_waves(g.N, g.K) == 16) return launch_token_waves<DT, LOG_G, BITS, R, 16>(q, g, rq_bytes, stream);
  }
  return launch_token_waves<DT, LOG_G, BITS, R, 8>(q, g, rq_bytes, stream);
}

template <int DT, int BITS, int R>
int launch_token_block(const rq::RqArgs &q, const gemv::GemvArgs &g, size_t rq_bytes, hipStream_t stream) {
  switch (rq::log2_groups(q)) {
    case 0: return launch_token<DT, 0, BITS, R>(q, g, rq_bytes, stream);
    case 1: return launch_token<DT, 1, BITS, R>(q, g, rq_bytes, stream);
    case 2: return launch_token<DT, 2, BITS, R>(q, g, rq_bytes, stream);
    case 3: return launch_token<DT, 3, BITS, R>(q, g, rq_bytes, stream);
    case 4: return launch_token<DT, 4, BITS, R>(q, g, rq_bytes, stream);
    case 5: return launch_token<DT, 5, BITS, R>(q, g, rq_bytes, stream);
    default: return fail(OQ_ERR_UNSUPPORTED, "token_linear: block %d is larger than 16384", q.block);
  }
}

}  // namespace

#define OQ_TOKEN_FN_CAT(a, b) a##b
#define OQ_TOKEN_FN(bits) OQ_TOKEN_FN_CAT(token_linear_launch_w, bits)

// x_dtype is OQ_F16 or OQ_BF16; the caller has checked token_linear_supported().
int OQ_TOKEN_FN(OQ_TOKEN_LINEAR_BITS)(const rq::RqArgs &q, const gemv::GemvArgs &g, int x_dtype, size_t rq_bytes,
                                      hipStream_t stream) {
  constexpr int BITS = OQ_TOKEN_LINEAR_BITS;
  // Rows per workgroup (the results do not depend on it): at most one workgroup per CU has room,
  // so the grid should not exceed the 256 CUs; the dispatcher only sends N up to 8192 here.
  const bool two = g.N > 16 * 256;
  if (x_dtype == OQ_BF16)
    return two ? launch_token_block<OQ_BF16, BITS, 2>(q, g, rq_bytes, stream)
               : launch_token_block<OQ_BF16, BITS, 1>(q, g, rq_bytes, stream);
  return two ? launch_token_block<OQ_F16, BITS, 2>(q, g, rq_bytes, stream)
             : launch_token_block<OQ_F16, BITS, 1>(q, g, rq_bytes, stream);
}

}  // namespace oq
