// Lookup-table decode of packed low-bit indices into 16-bit MFMA operands,
// shared by the tiled GEMM and the small-M streaming kernel.
//
// Every table lives in LDS and is replicated 32 times: entry e occupies 128
// bytes, copy c of it sits at byte e*128 + c*4, and lane l always reads copy
// l%32.  A wavefront therefore never presents two different addresses to one
// LDS bank, whatever indices its lanes hold.  A lookup costs two VALU
// instructions (bit-field extract, shift-add of the lane's base) and one
// ds_read_b32.
//
//   widths 2, 3, 4 : the table is indexed by a PAIR of codes (2*bits bits) and
//                    returns both 16-bit values in one dword
//   widths 6, 8    : one code per lookup; the entry holds the value in both
//                    halves so two lookups merge with one bit-select
#pragma once

#include "oq_common.h"

namespace oq {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

typedef __attribute__((address_space(3))) const uint32_t lds_cu32;

#if defined(__HIP_DEVICE_COMPILE__)
__device__ __forceinline__ uint32_t lds_read_u32(uint32_t byte_addr) { return *(lds_cu32 *)(byte_addr); }

__device__ __forceinline__ uint32_t lds_byte_address(const void *p) {
  return (uint32_t)(uintptr_t)(__attribute__((address_space(3))) const char *)p;
}
#else  // the host pass only needs the declarations to parse
__device__ uint32_t lds_read_u32(uint32_t byte_addr);
__device__ uint32_t lds_byte_address(const void *p);
#endif

// LR = log2(copies per entry): 5 for the MFMA-bound GEMM (no bank conflicts at all), 3 for the
// HBM-bound small-M kernel (smaller tables, more workgroups per CU, a few 2-way conflicts).
template <int BITS, int LR = 5> struct WLut {
  static constexpr bool kPair = BITS <= 4;
  static constexpr int kIndexBits = kPair ? 2 * BITS : BITS;
  static constexpr int kEntries = 1 << kIndexBits;
  static constexpr int kDwords = kEntries << LR;
};
constexpr int kALutDwords = 256 * 32;  // pair table of 4-bit activation codes, 32 copies
template <int LR> constexpr int alut_dwords() { return 256 << LR; }

__device__ __forceinline__ uint32_t pack16(float lo, float hi, bool f16) {
  const uint32_t a = f16 ? f32_to_f16_bits(lo) : f32_to_bf16_bits(lo);
  const uint32_t b = f16 ? f32_to_f16_bits(hi) : f32_to_bf16_bits(hi);
  return a | (b << 16);
}

// Fill a replicated table.  pair: entry e = (c[e & mask], c[e >> bits]); single: (c[e], c[e]).
template <int LR = 5>
__device__ __forceinline__ void fill_lut(uint32_t *lut, const float *cents, int bits, int levels, bool pair,
                                         bool f16) {
  const int entries = 1 << (pair ? 2 * bits : bits);
  const int mask = (1 << bits) - 1;
  for (int e = threadIdx.x; e < entries; e += blockDim.x) {
    const int c0 = pair ? (e & mask) : e;
    const int c1 = pair ? (e >> bits) : e;
    const float v0 = c0 < levels ? cents[c0] : 0.0f;
    const float v1 = c1 < levels ? cents[c1] : 0.0f;
    const uint32_t d = pack16(v0, v1, f16);
    uint4 *dst = reinterpret_cast<uint4 *>(lut + (e << LR));
    const uint4 v = make_uint4(d, d, d, d);
#pragma unroll
    for (int i = 0; i < (1 << LR) / 4; ++i) dst[i] = v;
  }
}

// `base` = LDS byte address of the table + 4 * (lane % copies)
template <int LR = 5>
__device__ __forceinline__ uint32_t lut_at(uint32_t base, uint32_t index) { return lds_read_u32((index << (LR + 2)) + base); }

// table lookup of the `width`-bit field of `word` at bit `pos` (both compile-time after unrolling)
template <int LR = 5>
__device__ __forceinline__ uint32_t lut_field(uint32_t base, uint32_t word, int pos, int width) {
  return lds_read_u32((__builtin_amdgcn_ubfe(word, pos, width) << (LR + 2)) + base);
}

// ---- weight decode: the dwords of one lane's 32-value run -> dword p (two values) of the operand of MFMA q ----
template <int BITS, int LR = 5>
__device__ __forceinline__ uint32_t decode_w_piece(const uint32_t (&w)[BITS], int q, int p, uint32_t base) {
  if constexpr (BITS == 4) {
    return lut_field<LR>(base, w[q], 8 * p, 8);
  } else if constexpr (BITS == 2) {
    return lut_field<LR>(base, w[q >> 1], 16 * (q & 1) + 4 * p, 4);
  } else if constexpr (BITS == 3) {
    uint32_t f;
    if (q == 0) f = w[0];
    else if (q == 1) f = __builtin_amdgcn_alignbit(w[1], w[0], 24);
    else if (q == 2) f = __builtin_amdgcn_alignbit(w[2], w[1], 16);
    else f = w[2] >> 8;
    return lut_field<LR>(base, f, 6 * p, 6);
  } else if constexpr (BITS == 6) {
    // 48-bit field at bit 48q of six dwords: eight 6-bit codes
    uint32_t lo, hi;  // lo: codes 0..4 and two bits of code 5; hi: the rest
    if (q == 0) { lo = w[0]; hi = w[1]; }
    else if (q == 1) { lo = __builtin_amdgcn_alignbit(w[2], w[1], 16); hi = w[2] >> 16; }
    else if (q == 2) { lo = w[3]; hi = w[4]; }
    else { lo = __builtin_amdgcn_alignbit(w[5], w[4], 16); hi = w[5] >> 16; }
    const uint32_t src = p < 2 ? lo : __builtin_amdgcn_alignbit(hi, lo, 24);  // codes 0..3 | codes 4..7
    const uint32_t c0 = (src >> (12 * (p & 1))) & 63u, c1 = (src >> (12 * (p & 1) + 6)) & 63u;
    return __builtin_amdgcn_perm(lut_at<LR>(base, c1), lut_at<LR>(base, c0), 0x07060100u);
  } else {  // 8 bits
    const uint32_t src = p < 2 ? w[2 * q] : w[2 * q + 1];
    const uint32_t e0 = lut_at<LR>(base, (src >> (16 * (p & 1))) & 0xffu);
    const uint32_t e1 = lut_at<LR>(base, (src >> (16 * (p & 1) + 8)) & 0xffu);
    return __builtin_amdgcn_perm(e1, e0, 0x07060100u);
  }
}

template <int BITS, int LR = 5>
__device__ __forceinline__ uint4 decode_w(const uint32_t (&w)[BITS], int q, uint32_t base) {
  return make_uint4(decode_w_piece<BITS, LR>(w, q, 0, base), decode_w_piece<BITS, LR>(w, q, 1, base),
                    decode_w_piece<BITS, LR>(w, q, 2, base), decode_w_piece<BITS, LR>(w, q, 3, base));
}

// eight 4-bit activation codes (one dword) -> operand of one MFMA
template <int LR = 5>
__device__ __forceinline__ uint4 decode_a_nibble(uint32_t f, uint32_t base) {
  uint32_t o[4];
#pragma unroll
  for (int p = 0; p < 4; ++p) o[p] = lut_field<LR>(base, f, 8 * p, 8);
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
