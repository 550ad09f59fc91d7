// Epilogue shared by the MFMA GEMM kernels:  out = acc * scale[m] * r_w[n] + bias[n].
//
// Accumulator e of lane l in a 32x32 MFMA tile is row 8*(e/4) + 4*(l/32) + e%4,
// column l%32.  Per-row and per-column factors are loaded before any store is
// issued, so the stores do not serialize behind loads they might alias.
#pragma once

#include "packed_decode.h"

namespace oq {

template <int FM, int FN, int OUT_DT>
__device__ __forceinline__ void gemm_epilogue_typed(const f32x16 (&acc)[FM][FN], int64_t m_base, int64_t n_base,
                                                    int r, int grp, int64_t M, int64_t N,
                                                    const float *__restrict__ row_scale,
                                                    const uint16_t *__restrict__ row_norms,
                                                    const void *__restrict__ bias, int bias_dtype,
                                                    void *__restrict__ out) {
  float rn[FN], bv[FN];
#pragma unroll
  for (int j = 0; j < FN; ++j) {
    const int64_t n = min(n_base + 32 * j + r, N - 1);
    rn[j] = bf16_bits_to_f32(row_norms[n]);
    bv[j] = bias != nullptr ? load_dyn_f32(bias, bias_dtype, n) : 0.0f;
  }
#pragma unroll
  for (int i = 0; i < FM; ++i) {
    float sc[16];
#pragma unroll
    for (int e = 0; e < 16; ++e) {
      const int64_t m = min(m_base + 32 * i + 8 * (e >> 2) + 4 * grp + (e & 3), M - 1);
      sc[e] = row_scale != nullptr ? row_scale[m] : 1.0f;
    }
#pragma unroll
    for (int e = 0; e < 16; ++e) {
      const int64_t m = m_base + 32 * i + 8 * (e >> 2) + 4 * grp + (e & 3);
      if (m < M) {
#pragma unroll
        for (int j = 0; j < FN; ++j) {
          const int64_t n = n_base + 32 * j + r;
          if (n < N) store_from_f32<OUT_DT>(out, m * N + n, acc[i][j][e] * sc[e] * rn[j] + bv[j]);
        }
      }
    }
  }
}

template <int FM, int FN>
__device__ __forceinline__ void gemm_epilogue(const f32x16 (&acc)[FM][FN], int64_t m_base, int64_t n_base, int r,
                                              int grp, int64_t M, int64_t N, const float *row_scale,
                                              const uint16_t *row_norms, const void *bias, int bias_dtype,
                                              void *out, int out_dtype) {
  if (out_dtype == OQ_BF16)
    gemm_epilogue_typed<FM, FN, OQ_BF16>(acc, m_base, n_base, r, grp, M, N, row_scale, row_norms, bias, bias_dtype, out);
  else if (out_dtype == OQ_F16)
    gemm_epilogue_typed<FM, FN, OQ_F16>(acc, m_base, n_base, r, grp, M, N, row_scale, row_norms, bias, bias_dtype, out);
  else
    gemm_epilogue_typed<FM, FN, OQ_F32>(acc, m_base, n_base, r, grp, M, N, row_scale, row_norms, bias, bias_dtype, out);
}

}  // namespace oq
