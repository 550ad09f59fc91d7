// Epilogue shared by the MFMA GEMM kernels:  out = acc * scale[m] * r_w[n] + bias[n].
//
// The kernels issue their MFMAs with the WEIGHT fragment as the first operand, so
// an accumulator tile is the transpose of the output tile: value e of lane l is
//   token row   m = 32*i + l%32
//   output col  n = 32*j + 8*(e/4) + 4*(l/32) + e%4
// i.e. every lane holds runs of four consecutive columns of one output row.
//
// A wavefront moves its tiles to memory in passes of [32 rows x 64 columns]
// through a private fp32 staging tile in LDS:
//   1. every lane writes its raw accumulator runs (16 bytes per ds_write, straight
//      from the accumulator registers) - no arithmetic, no reads, nothing to wait for;
//   2. the tile is read back row-wise, each lane taking eight consecutive columns
//      of one row; it multiplies by the token factor of that row (staged in LDS)
//      and the row norms and adds the bias (both held in registers for the whole
//      column block), converts and stores 16 bytes (bf16 / fp16; 2 x 16 for fp32),
//      so a store instruction writes whole 128-byte row segments.
// LDS operations of one wavefront execute in program order, so step 2 of a pass
// needs no barrier after step 1, and step 1 of the next pass may be issued as soon
// as the reads of step 2 have been issued.  The cost is instruction issue: about
// 2.5 vector instructions per output value.
//
// An output map (the activation function that follows the linear, as a table) is applied
// to the packed 16-bit words right before the store: a lookup in a 16 KB window of the
// table kept in LDS behind the staging tiles, the full table in memory for the rare value
// outside the window.
//
// Needs N % 8 == 0 and a 16-byte aligned `out` (the dispatcher sends other
// shapes to the shape-agnostic kernels).
#pragma once

#include <type_traits>

#include "packed_decode.h"
#include "value_map.h"

namespace oq {

constexpr int kEpiFactorBytes = 3072;            // r_w[256] + bias[256] + token factor[256] as fp32
constexpr int kEpiPitch = 64 * 4 + 16;           // one staged row: 64 fp32 + padding
constexpr int kEpiWaveBytes = 32 * kEpiPitch;    // 8704
constexpr int kEpiMapOffset = kEpiFactorBytes + 4 * kEpiWaveBytes;  // window of an output map (value_map.h)
constexpr int kEpiLdsBytes = kEpiMapOffset + kWideBytes;

// Optional elementwise function applied to the 16-bit outputs before they are stored, as a
// table (value_map.h): table == nullptr means none; lo < 0 means no LDS window (fp16).
struct OutMap {
  const uint16_t *table;
  int lo;
};

inline bool gemm_output_ok(int64_t N, const void *out) {
  return (N % 8 == 0) && ((reinterpret_cast<uintptr_t>(out) & 15u) == 0);
}

// Per-thread epilogue factors, loaded at kernel start so their latency hides behind the main loop:
// thread t < tile_n owns output column n_tile + t; every lane owns the token rows wm + 32*i + lane%32.
template <int FM> struct EpiFactors {
  float rn, bv;
  float sc[FM];
};

// The same values as the loads left them.  A wavefront's loads return in order and the compiler
// waits for a load where its value is first touched, so the requests are branch-free (clamped
// indices, a readable stand-in address for an absent operand: no value is produced on one side of
// a branch only) and nothing looks at the bits before the main loop is over: a conversion at
// kernel start would be a full memory round trip in front of the first operand load.
template <int FM> struct EpiRaw {
  uint32_t rn_bits, bias_lo, bias_hi;
  float sc[FM];
};

template <int FM>
__device__ __forceinline__ void gemm_epilogue_request(EpiRaw<FM> &f, int64_t m_tile, int64_t n_tile, int wm,
                                                      int tid, int64_t M, int64_t N,
                                                      const float *__restrict__ row_scale,
                                                      const uint16_t *__restrict__ row_norms,
                                                      const void *__restrict__ bias, int bias_dtype,
                                                      const float *__restrict__ stand_in) {
  const int64_t n = min(n_tile + tid, N - 1);
  const bool has_bias = bias != nullptr;
  const int bias_size = has_bias ? dtype_size(bias_dtype) : 2;
  const uint8_t *bias_at = (has_bias ? static_cast<const uint8_t *>(bias) : reinterpret_cast<const uint8_t *>(row_norms)) + n * bias_size;
  f.rn_bits = row_norms[n];
  f.bias_lo = *reinterpret_cast<const uint16_t *>(bias_at);
  f.bias_hi = *reinterpret_cast<const uint16_t *>(bias_at + (bias_size - 2));
  const float *scale_at = row_scale != nullptr ? row_scale : stand_in;
#pragma unroll
  for (int i = 0; i < FM; ++i) f.sc[i] = scale_at[row_scale != nullptr ? min(m_tile + wm + 32 * i + (tid & 31), M - 1) : 0];
}

template <int FM>
__device__ __forceinline__ void gemm_epilogue_factors(EpiFactors<FM> &f, const EpiRaw<FM> &raw, int tile_n, int tid,
                                                      bool has_scale, bool has_bias, int bias_dtype) {
  f.rn = 0.0f;
  f.bv = 0.0f;
  if (tid < tile_n) {
    f.rn = bf16_bits_to_f32(static_cast<uint16_t>(raw.rn_bits));
    if (has_bias) f.bv = dyn_bits_to_f32(dtype_size(bias_dtype) == 4 ? (raw.bias_lo | (raw.bias_hi << 16)) : raw.bias_lo, bias_dtype);
  }
#pragma unroll
  for (int i = 0; i < FM; ++i) f.sc[i] = has_scale ? raw.sc[i] : 1.0f;
}

typedef float f32x2_t __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef _Float16 f16x2_t __attribute__((ext_vector_type(2)));

// two fp32 -> one dword of two 16-bit floats (round to nearest even), one conversion instruction
template <int OUT_DT>
__device__ __forceinline__ uint32_t pack_pair(float lo, float hi) {
  const f32x2_t v = {lo, hi};
  if constexpr (OUT_DT == OQ_BF16) return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2_t));
  else return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, f16x2_t));
}

// 16 bytes of output, as a streaming (non-temporal) store.  An output tile is written once and read by
// another kernel: kept as ordinary write-back lines, a launch's whole output sits dirty in the L2s until
// the kernel ends and is written back then, after the last wavefront, which the next launch waits for
// (2048 x 4608 bf16: 26.2 -> 25.0 us per launch with streaming stores, measured interleaved).
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
__device__ __forceinline__ void store_out16(unsigned char *p, const uint4 v) {
  __builtin_nontemporal_store(u32x4_t{v.x, v.y, v.z, v.w}, reinterpret_cast<u32x4_t *>(p));
}

// `lds` = start of kEpiLdsBytes of LDS nobody else uses any more (the caller has put a
// barrier between its main loop and this call).
// GUARD = false: the workgroup's tile lies wholly inside the output, no store is predicated
// (one straight-line block, so LDS reads, arithmetic and stores of different rows overlap).
template <int FM, int FN, int OUT_DT, bool GUARD>
__device__ __forceinline__ void gemm_epilogue_typed(const f32x16 (&acc)[FM][FN], int64_t m_tile, int64_t n_tile,
                                                    int wm, int wn, int tile_n, int tid, int64_t M, int64_t N,
                                                    const EpiFactors<FM> &pre, void *__restrict__ out,
                                                    unsigned char *lds, const OutMap map, const uint16_t *hot_ready) {
  const int lane = tid & 63, wave = tid >> 6, r = lane & 31, grp = lane >> 5;
  const bool mapped = OUT_DT != OQ_F32 && map.table != nullptr;
  // the window: filled by the caller before its main loop (hot_ready, anywhere in LDS), or here
  uint16_t *hot_lds = reinterpret_cast<uint16_t *>(lds + kEpiMapOffset);
  const uint16_t *hot = mapped && map.lo >= 0 ? (hot_ready != nullptr ? hot_ready : hot_lds) : nullptr;
  if (hot != nullptr && hot_ready == nullptr) fill_map_window<kWideLog2>(hot_lds, map.table, map.lo, tid, 256);  // published by the barrier below

  constexpr int ES = OUT_DT == OQ_F32 ? 4 : 2;
  float *rn_s = reinterpret_cast<float *>(lds);
  float *bv_s = rn_s + 256;
  float *sc_s = rn_s + 512;
  if (tid < tile_n) {
    rn_s[tid] = pre.rn;
    bv_s[tid] = pre.bv;
  }
  if (wn == 0 && grp == 0) {
#pragma unroll
    for (int i = 0; i < FM; ++i) sc_s[wm + 32 * i + r] = pre.sc[i];
  }
  __syncthreads();
  unsigned char *tile = lds + kEpiFactorBytes + wave * kEpiWaveBytes;
  const int64_t row_pitch = N * ES;  // bytes between output rows

#pragma unroll
  for (int jc = 0; jc < FN; jc += 2) {
    constexpr int kTwo = 2;
    const int JC = (FN - jc) < kTwo ? 1 : 2;     // 32-column tiles in this pass (compile-time after unrolling)
    const int LPR = 4 * JC;                      // lanes per row when reading back (8 columns each)
    const int RPI = 64 / LPR;                    // rows per read instruction
    const int row0 = lane / LPR, c = lane % LPR;
    // this lane's eight columns of the block: factors stay in registers for every row tile
    const float4 rn0 = *reinterpret_cast<const float4 *>(rn_s + wn + 32 * jc + 8 * c);
    const float4 rn1 = *reinterpret_cast<const float4 *>(rn_s + wn + 32 * jc + 8 * c + 4);
    const float4 bv0 = *reinterpret_cast<const float4 *>(bv_s + wn + 32 * jc + 8 * c);
    const float4 bv1 = *reinterpret_cast<const float4 *>(bv_s + wn + 32 * jc + 8 * c + 4);
    const int64_t nn = n_tile + wn + 32 * jc + 8 * c;
    const int64_t m_first = m_tile + wm + row0;
    unsigned char *dst = static_cast<unsigned char *>(out) + m_first * row_pitch + nn * ES;
    const int rows_left = static_cast<int>(min(static_cast<int64_t>(FM * 32), M - m_first));  // rows m_first+k, k < rows_left, exist
    const bool col_ok = nn < N;
    // Software pipeline over the row tiles: the staging writes and read-backs of tile i are issued
    // before the arithmetic and stores of tile i-1, so LDS latency hides behind them (LDS
    // operations of a wavefront execute in order, so re-using the one staging tile is safe).
    constexpr int kReads = 4;  // read instructions per tile at most (32 / RPI with RPI >= 8)
    float4 v0[2][kReads], v1[2][kReads];
    float sc[2][kReads];
    auto stage = [&](int i, int buf) {
#pragma unroll
      for (int jj = 0; jj < JC; ++jj)
#pragma unroll
        for (int a = 0; a < 4; ++a) {
          const int col = 32 * jj + 8 * a + 4 * grp;
          *reinterpret_cast<float4 *>(tile + r * kEpiPitch + col * 4) =
              make_float4(acc[i][jc + jj][4 * a + 0], acc[i][jc + jj][4 * a + 1], acc[i][jc + jj][4 * a + 2],
                          acc[i][jc + jj][4 * a + 3]);
        }
#pragma unroll
      for (int t = 0; t < 32 / RPI; ++t) {
        const int row = t * RPI + row0;
        v0[buf][t] = *reinterpret_cast<const float4 *>(tile + row * kEpiPitch + c * 32);
        v1[buf][t] = *reinterpret_cast<const float4 *>(tile + row * kEpiPitch + c * 32 + 16);
        sc[buf][t] = sc_s[wm + 32 * i + row];
      }
    };
    auto finish_groups = [&](int i, int buf, auto groups) {
      constexpr int T = decltype(groups)::value;   // row groups of this tile: 32 / RPI
      float y[kReads][8];
#pragma unroll
      for (int t = 0; t < T; ++t) {
        const float4 a0 = v0[buf][t], a1 = v1[buf][t];
        const float s = sc[buf][t];
        y[t][0] = (a0.x * s) * rn0.x + bv0.x; y[t][1] = (a0.y * s) * rn0.y + bv0.y;
        y[t][2] = (a0.z * s) * rn0.z + bv0.z; y[t][3] = (a0.w * s) * rn0.w + bv0.w;
        y[t][4] = (a1.x * s) * rn1.x + bv1.x; y[t][5] = (a1.y * s) * rn1.y + bv1.y;
        y[t][6] = (a1.z * s) * rn1.z + bv1.z; y[t][7] = (a1.w * s) * rn1.w + bv1.w;
      }
      if constexpr (OUT_DT == OQ_F32) {
#pragma unroll
        for (int t = 0; t < T; ++t) {
          if (!GUARD || (col_ok && 32 * i + t * RPI < rows_left)) {
            unsigned char *o = dst + (32 * i + t * RPI) * row_pitch;
            store_out16(o, make_uint4(__float_as_uint(y[t][0]), __float_as_uint(y[t][1]), __float_as_uint(y[t][2]), __float_as_uint(y[t][3])));
            store_out16(o + 16, make_uint4(__float_as_uint(y[t][4]), __float_as_uint(y[t][5]), __float_as_uint(y[t][6]), __float_as_uint(y[t][7])));
          }
        }
      } else {
        uint4 words[T];
#pragma unroll
        for (int t = 0; t < T; ++t)
          words[t] = make_uint4(pack_pair<OUT_DT>(y[t][0], y[t][1]), pack_pair<OUT_DT>(y[t][2], y[t][3]),
                                pack_pair<OUT_DT>(y[t][4], y[t][5]), pack_pair<OUT_DT>(y[t][6], y[t][7]));
        if (mapped) map_words8_many<OUT_DT, T, kWideLog2>(words, map.table, hot, map.lo);
#pragma unroll
        for (int t = 0; t < T; ++t) {
          if (!GUARD || (col_ok && 32 * i + t * RPI < rows_left))
            store_out16(dst + (32 * i + t * RPI) * row_pitch, words[t]);
        }
      }
    };
    auto finish = [&](int i, int buf) {
      if (JC == 2) finish_groups(i, buf, std::integral_constant<int, 4>{});
      else finish_groups(i, buf, std::integral_constant<int, 2>{});
    };
    stage(0, 0);
#pragma unroll
    for (int i = 1; i < FM; ++i) {
      stage(i, i & 1);
      finish(i - 1, (i - 1) & 1);
    }
    finish(FM - 1, (FM - 1) & 1);
  }
}

// Entry used by the kernels (after their own __syncthreads()).
template <int FM, int FN>
__device__ __forceinline__ void gemm_epilogue(const f32x16 (&acc)[FM][FN], int64_t m_tile, int64_t n_tile, int wm,
                                              int wn, int tile_n, int tid, int64_t M, int64_t N,
                                              const float *row_scale, const uint16_t *row_norms,
                                              const void *bias, int bias_dtype, const EpiFactors<FM> &pre,
                                              void *out, int out_dtype, unsigned char *lds, const OutMap map,
                                              int tile_m = 64 * FM, const uint16_t *hot_ready = nullptr) {
  (void)row_scale; (void)row_norms; (void)bias; (void)bias_dtype;
  const bool interior = m_tile + tile_m <= M && n_tile + tile_n <= N;  // uniform over the workgroup
#define OQ_EPILOGUE_CASE(DT)                                                                                   \
  if (interior) gemm_epilogue_typed<FM, FN, DT, false>(acc, m_tile, n_tile, wm, wn, tile_n, tid, M, N, pre, out, lds, map, hot_ready); \
  else gemm_epilogue_typed<FM, FN, DT, true>(acc, m_tile, n_tile, wm, wn, tile_n, tid, M, N, pre, out, lds, map, hot_ready)
  if (out_dtype == OQ_BF16) { OQ_EPILOGUE_CASE(OQ_BF16); }
  else if (out_dtype == OQ_F16) { OQ_EPILOGUE_CASE(OQ_F16); }
  else { OQ_EPILOGUE_CASE(OQ_F32); }
#undef OQ_EPILOGUE_CASE
}

}  // namespace oq
