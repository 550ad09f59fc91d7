// An elementwise function of a 16-bit value as a table: entry[bits of x] = bits of f(x), 65536
// entries.  The quantizer applies such a table to its inputs and the tile kernels' epilogue to
// its outputs, so an activation function between two quantized linears costs neither a kernel
// nor a round trip of the activations through memory, and its results are the framework's own
// (the table is filled by applying the framework's f to every bit pattern).
#pragma once

#include "oq_common.h"

namespace oq {

constexpr int kHotHalf = 2048;                  // entries per sign: 16 binades of bf16
constexpr int kHotBytes = 2 * kHotHalf * 2;     // 8 KB of LDS
constexpr int kHotLoBf16 = 117 << 7;            // the window holds |x| in [2^-10, 2^6): exponent field 117 .. 132
// The tile kernels' epilogue has room for a window twice as deep: 32 binades, |x| in [2^-26, 2^6).
// A lone wavefront per SIMD cannot hide the memory latency of a value outside the window, and
// with 2048 values per lookup call even |x| < 2^-10 would be hit by most calls.
constexpr int kWideLog2 = 12;
constexpr int kWideBytes = (2 << kWideLog2) * 2;  // 16 KB of LDS
constexpr int kWideLoBf16 = 101 << 7;

// Copy the window of a bf16 table (both signs) into LDS: 16 bytes per thread and step.  The
// caller puts a barrier between this and the first lookup.
// LOGH: log2 of the entries per sign (11: the 8 KB window above; 12: 32 binades, 16 KB).
template <int LOGH = 11>
__device__ __forceinline__ void fill_map_window(uint16_t *hot_lds, const uint16_t *table, int lo, int tid, int nthreads) {
  constexpr int kChunksPerSign = (2 << LOGH) / 16;
  for (int i = tid; i < 2 * kChunksPerSign; i += nthreads) {
    const int sign = i / kChunksPerSign, j = i % kChunksPerSign;
    reinterpret_cast<uint4 *>(hot_lds)[i] = reinterpret_cast<const uint4 *>(table + (sign << 15) + lo)[j];
  }
}

// The mapped value of eight 16-bit values (four dwords of two).  bf16 values inside the window
// (|x| in 16 binades starting at bits `lo`, both signs) are served from the copy in LDS (`hot`);
// a wavefront with any value outside it also reads the full table in memory for those.  Other
// dtypes (hot == nullptr) read the full table for every value.
template <int DT>
__device__ __forceinline__ uint4 map_words8(const uint4 raw, const uint16_t *table, const uint16_t *hot, int lo) {
  typedef unsigned short u16x2 __attribute__((ext_vector_type(2)));
  const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
  uint32_t out[4];
  if (DT == OQ_BF16 && hot != nullptr) {
    const uint32_t lo2 = static_cast<uint32_t>(lo) * 0x10001u;
    uint32_t outside = 0;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      // per half: t = bits - lo (16-bit wrap); inside the window <=> (t & 0x7fff) < 2048; slot = (t & 0x7ff) + 2048 * sign
      const uint32_t t = __builtin_bit_cast(uint32_t, __builtin_bit_cast(u16x2, w[j]) - __builtin_bit_cast(u16x2, lo2));
      outside |= t;
      const uint32_t slot = (t & 0x07ff07ffu) | ((t >> 4) & 0x08000800u);
      out[j] = static_cast<uint32_t>(hot[slot & 0xffffu]) | (static_cast<uint32_t>(hot[slot >> 16]) << 16);
    }
    if (__builtin_amdgcn_ballot_w64((outside & 0x78007800u) != 0) != 0) {
      // all sixteen-bit loads are issued before any is used; values inside the window read entry 0 and drop it
      uint32_t far[8];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const uint32_t t = __builtin_bit_cast(uint32_t, __builtin_bit_cast(u16x2, w[j]) - __builtin_bit_cast(u16x2, lo2));
        far[2 * j] = table[(t & 0x00007800u) ? (w[j] & 0xffffu) : 0u];
        far[2 * j + 1] = table[(t & 0x78000000u) ? (w[j] >> 16) : 0u];
      }
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const uint32_t t = __builtin_bit_cast(uint32_t, __builtin_bit_cast(u16x2, w[j]) - __builtin_bit_cast(u16x2, lo2));
        if (t & 0x00007800u) out[j] = (out[j] & 0xffff0000u) | far[2 * j];
        if (t & 0x78000000u) out[j] = (out[j] & 0x0000ffffu) | (far[2 * j + 1] << 16);
      }
    }
  } else {
#pragma unroll
    for (int j = 0; j < 4; ++j)
      out[j] = static_cast<uint32_t>(table[w[j] & 0xffffu]) | (static_cast<uint32_t>(table[w[j] >> 16]) << 16);
  }
  return make_uint4(out[0], out[1], out[2], out[3]);
}

// The same for T groups of eight values at once: every lookup of every group is issued before
// any result is used and the window check is taken once, so a wavefront that has nothing else
// to run meanwhile (the epilogue of a tile kernel: one wavefront per SIMD) pays the LDS latency
// once per call instead of once per group.
template <int DT, int T, int LOGH = 11>
__device__ __forceinline__ void map_words8_many(uint4 (&words)[T], const uint16_t *table, const uint16_t *hot, int lo) {
  typedef unsigned short u16x2 __attribute__((ext_vector_type(2)));
  constexpr uint32_t kIn = (1u << LOGH) - 1u;                 // slot inside a sign's half
  constexpr uint32_t kOut = 0x7fffu & ~kIn;                   // any of these bits: outside the window
  constexpr uint32_t kIn2 = kIn * 0x10001u, kSign2 = (1u << LOGH) * 0x10001u, kOut2 = kOut * 0x10001u;
  uint32_t w[T][4], out[T][4];
#pragma unroll
  for (int g = 0; g < T; ++g) {
    w[g][0] = words[g].x; w[g][1] = words[g].y; w[g][2] = words[g].z; w[g][3] = words[g].w;
  }
  if (DT == OQ_BF16 && hot != nullptr) {
    const uint32_t lo2 = static_cast<uint32_t>(lo) * 0x10001u;
    uint32_t outside = 0, t[T][4];
#pragma unroll
    for (int g = 0; g < T; ++g)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        t[g][j] = __builtin_bit_cast(uint32_t, __builtin_bit_cast(u16x2, w[g][j]) - __builtin_bit_cast(u16x2, lo2));
        outside |= t[g][j];
      }
    uint32_t e0[T][4], e1[T][4];
#pragma unroll
    for (int g = 0; g < T; ++g)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const uint32_t slot = (t[g][j] & kIn2) | ((t[g][j] >> (15 - LOGH)) & kSign2);
        e0[g][j] = hot[slot & 0xffffu];
        e1[g][j] = hot[slot >> 16];
      }
#pragma unroll
    for (int g = 0; g < T; ++g)
#pragma unroll
      for (int j = 0; j < 4; ++j) out[g][j] = e0[g][j] | (e1[g][j] << 16);
    if (__builtin_amdgcn_ballot_w64((outside & kOut2) != 0) != 0) {
      uint32_t far[T][8];
#pragma unroll
      for (int g = 0; g < T; ++g)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          far[g][2 * j] = table[(t[g][j] & kOut) ? (w[g][j] & 0xffffu) : 0u];
          far[g][2 * j + 1] = table[(t[g][j] & (kOut << 16)) ? (w[g][j] >> 16) : 0u];
        }
#pragma unroll
      for (int g = 0; g < T; ++g)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          if (t[g][j] & kOut) out[g][j] = (out[g][j] & 0xffff0000u) | far[g][2 * j];
          if (t[g][j] & (kOut << 16)) out[g][j] = (out[g][j] & 0x0000ffffu) | (far[g][2 * j + 1] << 16);
        }
    }
  } else {
    uint32_t e0[T][4], e1[T][4];
#pragma unroll
    for (int g = 0; g < T; ++g)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        e0[g][j] = table[w[g][j] & 0xffffu];
        e1[g][j] = table[w[g][j] >> 16];
      }
#pragma unroll
    for (int g = 0; g < T; ++g)
#pragma unroll
      for (int j = 0; j < 4; ++j) out[g][j] = e0[g][j] | (e1[g][j] << 16);
  }
#pragma unroll
  for (int g = 0; g < T; ++g) words[g] = make_uint4(out[g][0], out[g][1], out[g][2], out[g][3]);
}

}  // namespace oq
