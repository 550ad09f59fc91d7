// Second half of a tile GEMM whose K range was shared between workgroups (GemmArgs::k_splits):
// adds the raw fp32 partial tiles in a fixed order and applies the epilogue,
//   out[m, n] = ((p_0 + p_1 + ... )[m, n] * scale[m]) * r_w[n] + bias[n],
// the expression of gemm_epilogue.h.  Memory-bound: k_splits * M * N * 4 bytes in, one output out.
#include "oq_common.h"

namespace oq {
namespace {

template <int OUT_DT>
__global__ __launch_bounds__(256) void splitk_reduce_kernel(const float *__restrict__ partials, int splits, int64_t M, int64_t N,
                                                            const float *__restrict__ row_scale,
                                                            const uint16_t *__restrict__ row_norms,
                                                            const void *__restrict__ bias, int bias_dtype,
                                                            void *__restrict__ out) {
  const int64_t quads = M * (N / 4);  // N is a multiple of 8
  const int64_t plane = M * N;
  for (int64_t q = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; q < quads;
       q += static_cast<int64_t>(gridDim.x) * blockDim.x) {
    const int64_t m = q / (N / 4), n = (q % (N / 4)) * 4;
    float4 sum = *reinterpret_cast<const float4 *>(partials + m * N + n);
    for (int z = 1; z < splits; ++z) {
      const float4 p = *reinterpret_cast<const float4 *>(partials + z * plane + m * N + n);
      sum.x += p.x; sum.y += p.y; sum.z += p.z; sum.w += p.w;
    }
    const float sc = row_scale != nullptr ? row_scale[m] : 1.0f;
    const float v[4] = {sum.x, sum.y, sum.z, sum.w};
    float y[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const float rn = bf16_bits_to_f32(row_norms[n + e]);
      const float bv = bias != nullptr ? load_dyn_f32(bias, bias_dtype, n + e) : 0.0f;
      y[e] = (v[e] * sc) * rn + bv;
    }
    if constexpr (OUT_DT == OQ_F32) {
      *reinterpret_cast<float4 *>(static_cast<float *>(out) + m * N + n) = make_float4(y[0], y[1], y[2], y[3]);
    } else {
      uint16_t h[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) h[e] = OUT_DT == OQ_BF16 ? f32_to_bf16_bits(y[e]) : f32_to_f16_bits(y[e]);
      *reinterpret_cast<uint2 *>(static_cast<uint16_t *>(out) + m * N + n) =
          make_uint2(h[0] | (static_cast<uint32_t>(h[1]) << 16), h[2] | (static_cast<uint32_t>(h[3]) << 16));
    }
  }
}

}  // namespace

int gemm_splitk_reduce(const float *partials, int splits, int64_t M, int64_t N, const float *row_scale,
                       const uint16_t *row_norms, const void *bias, int bias_dtype, void *out, int out_dtype,
                       hipStream_t stream) {
  const int64_t quads = M * (N / 4);
  const unsigned blocks = static_cast<unsigned>(quads / 256 + 1 < 4096 ? quads / 256 + 1 : 4096);
#define OQ_REDUCE(DT) hipLaunchKernelGGL(splitk_reduce_kernel<DT>, dim3(blocks), dim3(256), 0, stream, partials, splits, M, N, \
                                         row_scale, row_norms, bias, bias_dtype, out)
  if (out_dtype == OQ_BF16) OQ_REDUCE(OQ_BF16);
  else if (out_dtype == OQ_F16) OQ_REDUCE(OQ_F16);
  else OQ_REDUCE(OQ_F32);
#undef OQ_REDUCE
  return check_launch("splitk_reduce");
}

}  // namespace oq
