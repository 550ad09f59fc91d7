// Epilogue shared by the MFMA GEMM kernels:  out = acc * scale[m] * r_w[n] + bias[n].
//
// The kernels issue their MFMAs with the WEIGHT fragment as the first operand, so
// an accumulator tile is the transpose of the output tile: value e of lane l is
//   token row   m = 32*i + l%32
//   output col  n = 32*j + 8*(e/4) + 4*(l/32) + e%4
// i.e. every lane holds runs of four consecutive columns of one output row.  The
// fast path scales a run, packs it (8 bytes of bf16/fp16, 16 of fp32) and parks it
// in a wavefront-private LDS tile; the tile is then read back row-wise, 16 bytes
// per lane, so the global stores are whole 128-byte (or longer) row segments
// instead of 2-byte scatters.  Per-column factors (row norm, bias) are staged in
// LDS once per workgroup.
#pragma once

#include "packed_decode.h"

namespace oq {

constexpr int kEpiFactorBytes = 2048;                 // r_w[256] + bias[256] as fp32
constexpr int kEpiWavePitchMax = 32 * 2 * 4 + 16;     // two 32-column tiles of fp32 + padding
constexpr int kEpiWaveBytes = 32 * kEpiWavePitchMax;  // 8704
constexpr int kEpiLdsBytes = kEpiFactorBytes + 4 * kEpiWaveBytes;

// Per-thread epilogue factors, loaded at kernel start so their latency hides behind the main loop:
// thread t < tile_n owns output column n_tile + t; every lane owns the token rows wm + 32*i + lane%32.
template <int FM> struct EpiFactors {
  float rn, bv;
  float sc[FM];
};

template <int FM>
__device__ __forceinline__ void gemm_epilogue_prefetch(EpiFactors<FM> &f, int64_t m_tile, int64_t n_tile, int wm,
                                                       int tile_n, int tid, int64_t M, int64_t N,
                                                       const float *__restrict__ row_scale,
                                                       const uint16_t *__restrict__ row_norms,
                                                       const void *__restrict__ bias, int bias_dtype) {
  f.rn = 0.0f;
  f.bv = 0.0f;
  if (tid < tile_n) {
    const int64_t n = min(n_tile + tid, N - 1);
    f.rn = bf16_bits_to_f32(row_norms[n]);
    if (bias != nullptr) f.bv = load_dyn_f32(bias, bias_dtype, n);
  }
#pragma unroll
  for (int i = 0; i < FM; ++i)
    f.sc[i] = row_scale != nullptr ? row_scale[min(m_tile + wm + 32 * i + (tid & 31), M - 1)] : 1.0f;
}

template <int OUT_DT>
__device__ __forceinline__ void pack_run(const float (&y)[4], unsigned char *dst) {
  if constexpr (OUT_DT == OQ_F32) {
    *reinterpret_cast<float4 *>(dst) = make_float4(y[0], y[1], y[2], y[3]);
  } else if constexpr (OUT_DT == OQ_BF16) {
    uint2 v;
    v.x = static_cast<uint32_t>(f32_to_bf16_bits(y[0])) | (static_cast<uint32_t>(f32_to_bf16_bits(y[1])) << 16);
    v.y = static_cast<uint32_t>(f32_to_bf16_bits(y[2])) | (static_cast<uint32_t>(f32_to_bf16_bits(y[3])) << 16);
    *reinterpret_cast<uint2 *>(dst) = v;
  } else {
    uint2 v;
    v.x = static_cast<uint32_t>(f32_to_f16_bits(y[0])) | (static_cast<uint32_t>(f32_to_f16_bits(y[1])) << 16);
    v.y = static_cast<uint32_t>(f32_to_f16_bits(y[2])) | (static_cast<uint32_t>(f32_to_f16_bits(y[3])) << 16);
    *reinterpret_cast<uint2 *>(dst) = v;
  }
}

// Fast path.  `lds` = start of kEpiLdsBytes of LDS nobody else uses any more (the caller
// has put a barrier between the main loop and this call).  Needs N % 8 == 0 and a
// 16-byte aligned `out`.
template <int FM, int FN, int OUT_DT>
__device__ __forceinline__ void gemm_epilogue_lds(const f32x16 (&acc)[FM][FN], int64_t m_tile, int64_t n_tile,
                                                  int wm, int wn, int tile_n, int tid, int64_t M, int64_t N,
                                                  const EpiFactors<FM> &pre, void *__restrict__ out,
                                                  unsigned char *lds) {
  constexpr int ES = OUT_DT == OQ_F32 ? 4 : 2;
  constexpr int JC = FN >= 2 ? 2 : 1;             // 32-column tiles per pass
  constexpr int ROW_BYTES = 32 * JC * ES;
  constexpr int PITCH = ROW_BYTES + 16;
  constexpr int LPR = ROW_BYTES / 16;             // lanes per row when reading back
  constexpr int RPI = 64 / LPR;                   // rows per read instruction
  const int lane = tid & 63, wave = tid >> 6, r = lane & 31, grp = lane >> 5;

  float *rn_s = reinterpret_cast<float *>(lds);
  float *bv_s = rn_s + 256;
  if (tid < tile_n) {
    rn_s[tid] = pre.rn;
    bv_s[tid] = pre.bv;
  }
  __syncthreads();
  unsigned char *tile = lds + kEpiFactorBytes + wave * kEpiWaveBytes;

#pragma unroll
  for (int i = 0; i < FM; ++i) {
    const float sc = pre.sc[i];
#pragma unroll
    for (int jc = 0; jc < FN; jc += JC) {
#pragma unroll
      for (int jj = 0; jj < JC; ++jj) {
#pragma unroll
        for (int a = 0; a < 4; ++a) {
          const int col = 32 * jj + 8 * a + 4 * grp;  // inside this pass
          const float4 rn = *reinterpret_cast<const float4 *>(rn_s + wn + 32 * jc + col);
          const float4 bv = *reinterpret_cast<const float4 *>(bv_s + wn + 32 * jc + col);
          const float y[4] = {acc[i][jc + jj][4 * a + 0] * sc * rn.x + bv.x, acc[i][jc + jj][4 * a + 1] * sc * rn.y + bv.y,
                              acc[i][jc + jj][4 * a + 2] * sc * rn.z + bv.z, acc[i][jc + jj][4 * a + 3] * sc * rn.w + bv.w};
          pack_run<OUT_DT>(y, tile + r * PITCH + col * ES);
        }
      }
      // read the [32 x 32*JC] tile back row-wise and store whole row segments
#pragma unroll
      for (int t = 0; t < 32 / RPI; ++t) {
        const int row = t * RPI + lane / LPR, c = lane % LPR;
        const uint4 v = *reinterpret_cast<const uint4 *>(tile + row * PITCH + c * 16);
        const int64_t mm = m_tile + wm + 32 * i + row;
        const int64_t nn = n_tile + wn + 32 * jc + c * (16 / ES);
        if (mm < M && nn < N)
          *reinterpret_cast<uint4 *>(static_cast<unsigned char *>(out) + (mm * N + nn) * ES) = v;
      }
    }
  }
}

// Fallback for unaligned outputs / N not a multiple of 8: one store per value.
template <int FM, int FN, int OUT_DT>
__device__ __forceinline__ void gemm_epilogue_scalar(const f32x16 (&acc)[FM][FN], int64_t m_base, int64_t n_base,
                                                     int r, int grp, int64_t M, int64_t N,
                                                     const float *__restrict__ row_scale,
                                                     const uint16_t *__restrict__ row_norms,
                                                     const void *__restrict__ bias, int bias_dtype,
                                                     void *__restrict__ out) {
#pragma unroll
  for (int i = 0; i < FM; ++i) {
    const int64_t m = m_base + 32 * i + r;
    const float sc = row_scale != nullptr ? row_scale[min(m, M - 1)] : 1.0f;
#pragma unroll
    for (int j = 0; j < FN; ++j) {
#pragma unroll 1
      for (int e = 0; e < 16; ++e) {
        const int64_t n = n_base + 32 * j + 8 * (e >> 2) + 4 * grp + (e & 3);
        if (m < M && n < N) {
          const float rn = bf16_bits_to_f32(row_norms[n]);
          const float bv = bias != nullptr ? load_dyn_f32(bias, bias_dtype, n) : 0.0f;
          store_from_f32<OUT_DT>(out, m * N + n, acc[i][j][e] * sc * rn + bv);
        }
      }
    }
  }
}

// Entry used by the kernels (after their own __syncthreads()).
template <int FM, int FN>
__device__ __forceinline__ void gemm_epilogue(const f32x16 (&acc)[FM][FN], int64_t m_tile, int64_t n_tile, int wm,
                                              int wn, int tile_n, int tid, int64_t M, int64_t N,
                                              const float *row_scale, const uint16_t *row_norms,
                                              const void *bias, int bias_dtype, const EpiFactors<FM> &pre,
                                              void *out, int out_dtype, unsigned char *lds) {
  const int lane = tid & 63, r = lane & 31, grp = lane >> 5;
  const bool fast = (N % 8 == 0) && ((reinterpret_cast<uintptr_t>(out) & 15u) == 0);
  if (fast) {
    if (out_dtype == OQ_BF16)
      gemm_epilogue_lds<FM, FN, OQ_BF16>(acc, m_tile, n_tile, wm, wn, tile_n, tid, M, N, pre, out, lds);
    else if (out_dtype == OQ_F16)
      gemm_epilogue_lds<FM, FN, OQ_F16>(acc, m_tile, n_tile, wm, wn, tile_n, tid, M, N, pre, out, lds);
    else
      gemm_epilogue_lds<FM, FN, OQ_F32>(acc, m_tile, n_tile, wm, wn, tile_n, tid, M, N, pre, out, lds);
  } else {
    if (out_dtype == OQ_BF16)
      gemm_epilogue_scalar<FM, FN, OQ_BF16>(acc, m_tile + wm, n_tile + wn, r, grp, M, N, row_scale, row_norms, bias, bias_dtype, out);
    else if (out_dtype == OQ_F16)
      gemm_epilogue_scalar<FM, FN, OQ_F16>(acc, m_tile + wm, n_tile + wn, r, grp, M, N, row_scale, row_norms, bias, bias_dtype, out);
    else
      gemm_epilogue_scalar<FM, FN, OQ_F32>(acc, m_tile + wm, n_tile + wn, r, grp, M, N, row_scale, row_norms, bias, bias_dtype, out);
  }
}

}  // namespace oq
