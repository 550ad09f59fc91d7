// Lookup-table decode of packed low-bit indices into 16-bit MFMA operands,
// shared by the tiled GEMM and the small-M streaming kernel.
#pragma once

#include "oq_common.h"

namespace oq {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

// ---- lookup-table geometry ---------------------------------------------------
template <int BITS> struct WLut {
  static constexpr int kPairBits = BITS == 8 ? 8 : 2 * BITS;      // 8-bit: single-code table
  static constexpr int kEntries = 1 << kPairBits;
  static constexpr int kLogRep = kEntries <= 256 ? 5 : 0;        // replicate small tables x32
  static constexpr int kDwords = kEntries << kLogRep;
};
constexpr int kALutLogRep = 5;
constexpr int kALutDwords = 256 << kALutLogRep;

__device__ __forceinline__ uint32_t bf16_pair(float lo, float hi) {
  return static_cast<uint32_t>(f32_to_bf16_bits(lo)) | (static_cast<uint32_t>(f32_to_bf16_bits(hi)) << 16);
}
__device__ __forceinline__ uint32_t f16_pair(float lo, float hi) {
  return static_cast<uint32_t>(f32_to_f16_bits(lo)) | (static_cast<uint32_t>(f32_to_f16_bits(hi)) << 16);
}

// Fill a (possibly replicated) pair table: entry p holds (c[p & mask], c[p >> bits]).
template <bool F16>
__device__ __forceinline__ void fill_pair_lut(uint32_t *lut, const float *cents, int bits, int levels,
                                              int pair_bits, int log_rep, bool single) {
  const int total = (1 << pair_bits) << log_rep;
  const int mask = (1 << bits) - 1;
  for (int i = threadIdx.x; i < total; i += blockDim.x) {
    const int p = i >> log_rep;
    const int c0 = p & mask, c1 = single ? 0 : (p >> bits);
    const float v0 = c0 < levels ? cents[c0] : 0.0f;
    const float v1 = (!single && c1 < levels) ? cents[c1] : 0.0f;
    lut[i] = F16 ? f16_pair(v0, v1) : bf16_pair(v0, v1);
  }
}

// ---- weight decode: dwords of one lane's 32-value run -> operand of MFMA q ------
template <int BITS>
__device__ __forceinline__ uint4 decode_w(const uint32_t (&w)[BITS], int q, const uint32_t *lut, int rl) {
  constexpr int LR = WLut<BITS>::kLogRep;
  uint32_t o[4];
  if constexpr (BITS == 4) {
    const uint32_t f = w[q];
#pragma unroll
    for (int p = 0; p < 4; ++p) o[p] = lut[(((f >> (8 * p)) & 0xffu) << LR) + rl];
  } else if constexpr (BITS == 2) {
    const uint32_t f = (w[q >> 1] >> (16 * (q & 1))) & 0xffffu;
#pragma unroll
    for (int p = 0; p < 4; ++p) o[p] = lut[(((f >> (4 * p)) & 0xfu) << LR) + rl];
  } else if constexpr (BITS == 3) {
    uint32_t f;
    if (q == 0) f = w[0];
    else if (q == 1) f = __builtin_amdgcn_alignbit(w[1], w[0], 24);
    else if (q == 2) f = __builtin_amdgcn_alignbit(w[2], w[1], 16);
    else f = w[2] >> 8;
#pragma unroll
    for (int p = 0; p < 4; ++p) o[p] = lut[(((f >> (6 * p)) & 0x3fu) << LR) + rl];
  } else if constexpr (BITS == 6) {
    // 48-bit field at bit 48q of six dwords
    uint64_t f;
    if (q == 0) f = static_cast<uint64_t>(w[0]) | (static_cast<uint64_t>(w[1]) << 32);
    else if (q == 1) f = static_cast<uint64_t>(w[1] >> 16) | (static_cast<uint64_t>(w[2]) << 16);
    else if (q == 2) f = static_cast<uint64_t>(w[3]) | (static_cast<uint64_t>(w[4]) << 32);
    else f = static_cast<uint64_t>(w[4] >> 16) | (static_cast<uint64_t>(w[5]) << 16);
#pragma unroll
    for (int p = 0; p < 4; ++p) o[p] = lut[static_cast<uint32_t>(f >> (12 * p)) & 0xfffu];
  } else {  // 8 bits: one code per table entry (value in the low half)
    const uint32_t lo = w[2 * q], hi = w[2 * q + 1];
#pragma unroll
    for (int p = 0; p < 4; ++p) {
      const uint32_t src = p < 2 ? lo : hi;
      const uint32_t e0 = lut[(((src >> (16 * (p & 1))) & 0xffu) << LR) + rl] & 0xffffu;
      const uint32_t e1 = lut[(((src >> (16 * (p & 1) + 8)) & 0xffu) << LR) + rl] << 16;
      o[p] = e0 | e1;
    }
  }
  return make_uint4(o[0], o[1], o[2], o[3]);
}

__device__ __forceinline__ uint4 decode_a_nibble(uint32_t f, const uint32_t *lut, int rl) {
  uint32_t o[4];
#pragma unroll
  for (int p = 0; p < 4; ++p) o[p] = lut[(((f >> (8 * p)) & 0xffu) << kALutLogRep) + rl];
  return make_uint4(o[0], o[1], o[2], o[3]);
}

template <int BITS>
__device__ __forceinline__ void load_w(const uint8_t *p, uint32_t (&w)[BITS]) {
  if constexpr (BITS == 4) {
    const uint4 v = *reinterpret_cast<const uint4 *>(p);
    w[0] = v.x; w[1] = v.y; w[2] = v.z; w[3] = v.w;
  } else if constexpr (BITS == 2) {
    const uint2 v = *reinterpret_cast<const uint2 *>(p);
    w[0] = v.x; w[1] = v.y;
  } else if constexpr (BITS == 8) {
    const uint4 v0 = reinterpret_cast<const uint4 *>(p)[0], v1 = reinterpret_cast<const uint4 *>(p)[1];
    w[0] = v0.x; w[1] = v0.y; w[2] = v0.z; w[3] = v0.w; w[4] = v1.x; w[5] = v1.y; w[6] = v1.z; w[7] = v1.w;
  } else {
    const uint32_t *d = reinterpret_cast<const uint32_t *>(p);
#pragma unroll
    for (int i = 0; i < BITS; ++i) w[i] = d[i];
  }
}


}  // namespace oq
