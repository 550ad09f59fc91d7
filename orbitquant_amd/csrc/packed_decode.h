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
typedef uint32_t lds_u32x4 __attribute__((ext_vector_type(4)));

#if defined(__HIP_DEVICE_COMPILE__)
__device__ __forceinline__ uint32_t lds_read_u32(uint32_t byte_addr) { return *(lds_cu32 *)(byte_addr); }
__device__ __forceinline__ uint4 lds_read_u128(uint32_t byte_addr) {  // 16-byte aligned
  const lds_u32x4 v = *(__attribute__((address_space(3))) const lds_u32x4 *)(byte_addr);
  return make_uint4(v[0], v[1], v[2], v[3]);
}

__device__ __forceinline__ uint32_t lds_byte_address(const void *p) {
  return (uint32_t)(uintptr_t)(__attribute__((address_space(3))) const char *)p;
}
#else  // the host pass only needs the declarations to parse
__device__ uint32_t lds_read_u32(uint32_t byte_addr);
__device__ uint4 lds_read_u128(uint32_t byte_addr);
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


// ---- the 64 KB table block shared by the tiled GEMM and the small-M kernel -------------------
// 256 rows of 256 bytes at a 65536-aligned LDS address.  Row e holds, 32 times each, the dword
// of weight-table entry e (bytes 0..127) and of activation-table entry e (bytes 128..255); lane l
// reads copy l%32, so the lanes of a wavefront never collide on a bank whatever codes they hold.
// The activation table and the 4-bit weight table are indexed by a whole byte of the packed
// stream (two codes) and return both bf16 values in one dword; because a row is 256 bytes the
// LDS address of such a lookup is "byte 0 = the lane's offset, byte 1 = the code byte", which one
// v_perm_b32 assembles.  Other weight widths index the same rows with a bit-field extract (pair
// tables for 2/3 bits, single-code tables for 6/8).
constexpr int kRowTableBytes = 65536;

__device__ __forceinline__ uint32_t row_address(uint32_t word, uint32_t lane_off, int p) {
  return __builtin_amdgcn_perm(word, lane_off, 0x03020400u + (static_cast<uint32_t>(p) << 8));
}

__device__ __forceinline__ uint4 decode_bytes(uint32_t f, uint32_t lane_off) {
  return make_uint4(lds_read_u32(row_address(f, lane_off, 0)), lds_read_u32(row_address(f, lane_off, 1)),
                    lds_read_u32(row_address(f, lane_off, 2)), lds_read_u32(row_address(f, lane_off, 3)));
}

// centroid i (i < COUNT <= 64) into lane i of one register.  The addresses are uniform, so the
// values come through scalar loads, which do not queue behind the wavefront's vector loads.
template <int COUNT>
__device__ __forceinline__ float lane_table(const float *__restrict__ cents, int valid) {
  const int lane = threadIdx.x & 63;
  float t = 0.0f;
#pragma unroll
  for (int i = 0; i < COUNT; ++i) {
    const float c = i < valid ? cents[i] : 0.0f;
    t = lane == i ? c : t;
  }
  return t;
}

// Build the block with WAVES wavefronts: wavefront w writes rows [w*256/WAVES, (w+1)*256/WAVES),
// four rows per 16-byte-per-lane store.  The caller puts a barrier between this and the first lookup.
// A_SINGLE: the activation half holds single-code entries (one code per byte, up to 256 levels)
// instead of the pair table of two 4-bit codes.
// W_ONLY: the activation half of every row is left alone (it then holds something else: the
// small-M kernel parks decoded activation values there).
template <int BITS, int WAVES, bool A_SINGLE = false, bool W_ONLY = false>
__device__ __forceinline__ void build_row_tables(uint32_t *lds, const float *__restrict__ w_cents,
                                                 const float *__restrict__ act_cents, int a_levels) {
  constexpr int kLevels = 1 << BITS;
  constexpr bool kPair = BITS <= 4;
  constexpr int kRowsPerWave = 256 / WAVES;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  float a_tab = 0.0f;
  if constexpr (!W_ONLY) a_tab = A_SINGLE ? lane_table<64>(act_cents, a_levels) : lane_table<16>(act_cents, a_levels);
  float w_tab = 0.0f;
  if constexpr (kLevels <= 64) w_tab = lane_table<kLevels>(w_cents, kLevels);
  if constexpr (W_ONLY) {
    // only the rows an index can reach (16, 64 or 256), eight rows per 16-byte-per-lane store
    // (a weight half is eight lanes wide), the groups of eight rows dealt round the wavefronts
    constexpr int kRows = kPair ? (kLevels * kLevels < 256 ? kLevels * kLevels : 256) : kLevels;
    constexpr int kGroups = (kRows + 7) / 8;
#pragma unroll
    for (int i = 0; i < (kGroups + WAVES - 1) / WAVES; ++i) {
      const int grp8 = wave + WAVES * i;
      if (grp8 >= kGroups) break;  // the same for the whole wavefront
      const int e = 8 * grp8 + (lane >> 3);
      uint32_t ew;
      if constexpr (kLevels <= 64) {
        if constexpr (kPair) ew = pack16(__shfl(w_tab, e & (kLevels - 1)), __shfl(w_tab, (e >> BITS) & (kLevels - 1)), false);
        else ew = pack16(__shfl(w_tab, e & (kLevels - 1)), __shfl(w_tab, e & (kLevels - 1)), false);
      } else {
        const float v = w_cents[e];
        ew = pack16(v, v, false);
      }
      *reinterpret_cast<uint4 *>(reinterpret_cast<unsigned char *>(lds) + e * 256 + (lane & 7) * 16) = make_uint4(ew, ew, ew, ew);
    }
    return;
  }
#pragma unroll
  for (int i = 0; i < kRowsPerWave / 4; ++i) {
    const int e = wave * kRowsPerWave + 4 * i + (lane >> 4);  // the row this lane writes to
    uint32_t ea;
    if constexpr (A_SINGLE) {
      float v = __shfl(a_tab, e & 63);
      if (a_levels > 64) v = e < a_levels ? act_cents[e] : 0.0f;  // wide tables: one vector load per row
      else if (e >= a_levels) v = 0.0f;
      ea = pack16(v, v, false);
    } else {
      ea = pack16(__shfl(a_tab, e & 15), __shfl(a_tab, e >> 4), false);
    }
    uint32_t ew;
    if constexpr (kLevels <= 64) {
      if constexpr (kPair) {
        ew = (e < kLevels * kLevels)
                 ? pack16(__shfl(w_tab, e & (kLevels - 1)), __shfl(w_tab, (e >> BITS) & (kLevels - 1)), false)
                 : 0u;
      } else {
        const float v = __shfl(w_tab, e & (kLevels - 1));
        ew = (e < kLevels) ? pack16(v, v, false) : 0u;
      }
    } else {
      const float v = w_cents[e];  // 256 single-code entries: one vector load per row
      ew = pack16(v, v, false);
    }
    const uint32_t d = (lane & 8) ? ea : ew;
    *reinterpret_cast<uint4 *>(reinterpret_cast<unsigned char *>(lds) + e * 256 + (lane & 15) * 16) = make_uint4(d, d, d, d);
  }
}

// The same block for a 256-thread workgroup whose thread t already holds the two dwords of row t
// (loaded with its first vector loads, before any bulk load): wavefront w writes rows 64w..64w+63;
// 16-byte chunk c of a row is a weight copy (c < 8) or an activation copy; lane l writes chunk l%16
// of row 64w + 4i + l/16.  Fewer shuffles than build_row_tables, at the price of a vector-load latency.
__device__ __forceinline__ void write_row_tables(uint32_t *lds, uint32_t my_w, uint32_t my_a) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    const int src = 4 * i + (lane >> 4);
    const uint32_t ew = __shfl(my_w, src), ea = __shfl(my_a, src);
    const uint32_t d = (lane & 8) ? ea : ew;
    *reinterpret_cast<uint4 *>(reinterpret_cast<unsigned char *>(lds) + (64 * wave + src) * 256 + (lane & 15) * 16) =
        make_uint4(d, d, d, d);
  }
}

// The same block without a lane exchange, for pair tables (weights of 2, 3 or 4 bits; activation codes two
// per byte or no activation table at all).  Lane l of wavefront w writes 16-byte chunk l % 16 of rows
// 64 w + 4 i + l / 16, i = 0..15: a weight copy (chunks 0..7) or an activation copy.  The entry of row e is
// (c[e mod L], c[(e >> bits) mod L]), and for the rows of one lane  e mod L = (4 i + l / 16) mod L  takes four
// values while  e >> bits  takes at most eight, the same for every lane of the wavefront: a lane loads those
// centroids itself (request_pair_seed, with the kernel's other first loads) and every entry is one conversion
// instruction.  (The exchange-based build is a chain of sixteen LDS round trips per wavefront: 0.8 us of a
// 25 us launch.)  Weight rows past L * L are never indexed and hold arbitrary entries.
template <int BITS, bool HAS_A>
__device__ __forceinline__ void request_pair_seed(float (&lo_w)[4], float (&hi_w)[8], float (&lo_a)[4], float (&hi_a)[4],
                                                  const float *__restrict__ w_cents,
                                                  const float *__restrict__ act_cents, int a_levels) {
  static_assert(BITS >= 2 && BITS <= 4, "pair tables");
  constexpr int L = 1 << BITS;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, g = lane >> 4;
#pragma unroll
  for (int j = 0; j < 4; ++j) lo_w[j] = w_cents[(4 * j + g) & (L - 1)];
  // e >> bits for rows 64 w + 4 i + g:  4 w + i / 4 (16 levels),  i / 2 (8 levels, rows below 64),  i (4 levels, rows below 16)
#pragma unroll
  for (int t = 0; t < 8; ++t) hi_w[t] = t < (BITS == 3 ? 8 : 4) ? w_cents[BITS == 4 ? ((4 * wave + t) & 15) : t] : 0.0f;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    lo_a[j] = HAS_A ? act_cents[min(4 * j + g, a_levels - 1)] : 0.0f;
    hi_a[j] = HAS_A ? act_cents[min(4 * wave + j, a_levels - 1)] : 0.0f;
  }
}

template <int BITS, bool HAS_A>
__device__ __forceinline__ void write_pair_tables(uint32_t *lds, const float (&lo_w)[4], const float (&hi_w)[8],
                                                  const float (&lo_a_raw)[4], const float (&hi_a_raw)[4], int a_levels) {
  typedef float f32x2_t __attribute__((ext_vector_type(2)));
  typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, g = lane >> 4;
  const bool is_a = (lane & 8) != 0;
  float lo_a[4], hi_a[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) {  // codes past the table read zero
    lo_a[j] = (HAS_A && 4 * j + g < a_levels) ? lo_a_raw[j] : 0.0f;
    hi_a[j] = (HAS_A && 4 * wave + j < a_levels) ? hi_a_raw[j] : 0.0f;
  }
  // a lane writes either weight or activation copies: choose the operands once
  float lo[4], hi[16];
#pragma unroll
  for (int j = 0; j < 4; ++j) lo[j] = is_a ? lo_a[j] : lo_w[j];
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    const int slot = BITS == 4 ? (i >> 2) : BITS == 3 ? (i >> 1) : (i & 3);
    if (BITS == 4 && (i & 3)) hi[i] = hi[i & ~3];
    else hi[i] = is_a ? hi_a[i >> 2] : hi_w[slot];
  }
  unsigned char *row0 = reinterpret_cast<unsigned char *>(lds) + (64 * wave + g) * 256 + (lane & 15) * 16;
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    const f32x2_t pair = {lo[i & 3], hi[i]};
    const uint32_t d = __builtin_bit_cast(uint32_t, __builtin_convertvector(pair, bf16x2_t));
    *reinterpret_cast<uint4 *>(row0 + i * 1024) = make_uint4(d, d, d, d);
  }
}

// The weight half of the block alone (W_ONLY above), for pair tables, without a lane exchange: lane l of
// wavefront w writes 16-byte chunk l % 8 of rows 8 (w + WAVES i) + l / 8 and loads the two centroids of each
// of its rows itself, with the kernel's first requests (request_w_rows); an entry is then one conversion.
template <int BITS, int WAVES> struct WRows {
  static constexpr int kLevels = 1 << BITS;
  static constexpr int kRows = kLevels * kLevels < 256 ? kLevels * kLevels : 256;
  static constexpr int kGroups = kRows / 8;
  static constexpr int kIters = (kGroups + WAVES - 1) / WAVES;  // at most 8 (four wavefronts, 256 rows)
};

template <int BITS, int WAVES>
__device__ __forceinline__ void request_w_rows(float (&lo)[8], float (&hi)[8],
                                               const float *__restrict__ w_cents) {
  typedef WRows<BITS, WAVES> W;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
#pragma unroll
  for (int i = 0; i < W::kIters; ++i) {
    const int e = (8 * (wave + WAVES * i) + (lane >> 3)) & (W::kRows - 1);  // (a wavefront past the last group reads a row it does not write)
    lo[i] = w_cents[e & (W::kLevels - 1)];
    hi[i] = w_cents[(e >> BITS) & (W::kLevels - 1)];
  }
}

template <int BITS, int WAVES>
__device__ __forceinline__ void write_w_rows(uint32_t *lds, const float (&lo)[8], const float (&hi)[8]) {
  typedef WRows<BITS, WAVES> W;
  typedef float f32x2_t __attribute__((ext_vector_type(2)));
  typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
#pragma unroll
  for (int i = 0; i < W::kIters; ++i) {
    const int grp8 = wave + WAVES * i;
    if (grp8 >= W::kGroups) break;  // the same for the whole wavefront
    const f32x2_t pair = {lo[i], hi[i]};
    const uint32_t d = __builtin_bit_cast(uint32_t, __builtin_convertvector(pair, bf16x2_t));
    *reinterpret_cast<uint4 *>(reinterpret_cast<unsigned char *>(lds) + (8 * grp8 + (lane >> 3)) * 256 + (lane & 7) * 16) =
        make_uint4(d, d, d, d);
  }
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
