// Fused RPBH rotate + per-token Lloyd-Max quantize for gfx950.
//
// One workgroup per token row: 256 threads, or fewer wavefronts when the row is shorter
// than 1536 elements (a wavefront covers 512).  The row is staged once in LDS as
// fp32 (coalesced 16-byte global loads), the sum of squares is taken in the
// fixed order the C header documents, then every thread gathers eight
// consecutive rotated slots from LDS (permutation), divides by (norm + eps),
// applies the sign and runs the Walsh-Hadamard butterflies:
//   distance 1,2,4        in registers (the thread's own eight values)
//   distance 8 .. 256     across the lanes of the wavefront (lane xor 1 .. 32: DPP lane
//                         exchanges up to 8, wavefront shuffles or lane-group swaps of register pairs for 16 and 32)
//   distance 512 ..       through LDS, regrouped so the stages are register-local
// Every butterfly output is one fp32 add or subtract of two values of the
// previous stage, so the result does not depend on this schedule.
//
// This file must be compiled without FMA contraction: every fp32 operation
// rounds once, exactly like the CPU statement of the algorithm.
//
// This header holds the whole computation of one row as a device function, so that the
// standalone kernel (rotate_quantize.hip) and the one-token linear (quantize and stream the
// packed weights in the same launch) run the very same arithmetic.
#pragma once
#pragma clang fp contract(off)

#include <stdlib.h>

#include <type_traits>

#include "oq_common.h"
#include "value_map.h"

namespace oq {
namespace rq {

constexpr int kThreads = 256;
constexpr int kChunk = 8;
constexpr int kPass = kThreads * kChunk;  // 2048 elements per pass
constexpr int kMaxPasses = 8;             // K <= 16384
constexpr int kLaneSpan = 64 * kChunk;    // 512 elements covered by one wavefront

struct RqArgs {
  const void *x;
  int64_t M, K;
  const int32_t *perm;
  const int8_t *signs;
  const float *bounds;
  const float *cents;
  int levels;       // number of codes
  int levels_pow2;  // next power of two >= levels
  int block;
  int passes;
  float eps;
  float inv_sqrt_block;
  uint8_t *codes;
  int code_format;
  void *values;
  int values_mode;
  float *norms;
  const uint16_t *map;  // optional elementwise map of 16-bit inputs: 65536 entries indexed by the input's bits
  int map_lo;           // bf16 only: first |bits| of the window of 2 x 2048 entries kept in LDS; < 0: no window
  int map_lds_offset;   // where the window starts in the dynamic LDS block (bytes, a multiple of 16)
};

// The mapped value of eight 16-bit inputs (value_map.h) for this kernel's arguments.
template <int DT>
__device__ __forceinline__ uint4 map_raw8(const uint4 raw, const RqArgs &a, const uint16_t *hot) {
  return map_words8<DT>(raw, a.map, hot, a.map_lo);
}

template <int DT, bool VEC>
__device__ __forceinline__ void load_chunk(const RqArgs &a, const uint16_t *hot, int64_t row_base, int64_t i0,
                                           float (&f)[kChunk]) {
  const void *x = a.x;
  const int64_t K = a.K;
  if constexpr (VEC) {
    if (i0 + kChunk <= K) {
      if constexpr (DT == OQ_F32) {
        const float4 *p = reinterpret_cast<const float4 *>(static_cast<const float *>(x) + row_base + i0);
        float4 a = p[0], b = p[1];
        f[0] = a.x; f[1] = a.y; f[2] = a.z; f[3] = a.w;
        f[4] = b.x; f[5] = b.y; f[6] = b.z; f[7] = b.w;
      } else {
        uint4 raw = *reinterpret_cast<const uint4 *>(static_cast<const uint16_t *>(x) + row_base + i0);
        if (a.map != nullptr) raw = map_raw8<DT>(raw, a, hot);
        const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const uint16_t lo = static_cast<uint16_t>(w[j] & 0xffffu), hi = static_cast<uint16_t>(w[j] >> 16);
          if constexpr (DT == OQ_BF16) {
            f[2 * j] = bf16_bits_to_f32(lo);
            f[2 * j + 1] = bf16_bits_to_f32(hi);
          } else {
            f[2 * j] = f16_bits_to_f32(lo);
            f[2 * j + 1] = f16_bits_to_f32(hi);
          }
        }
      }
      return;
    }
  }
#pragma unroll
  for (int e = 0; e < kChunk; ++e) {
    f[e] = 0.0f;
    if (i0 + e < K) {
      if constexpr (DT != OQ_F32) {
        if (a.map != nullptr) {
          const uint16_t bits = a.map[static_cast<const uint16_t *>(x)[row_base + i0 + e]];
          f[e] = DT == OQ_BF16 ? bf16_bits_to_f32(bits) : f16_bits_to_f32(bits);
          continue;
        }
      }
      f[e] = load_as_f32<DT>(x, row_base + i0 + e);
    }
  }
}

__device__ __forceinline__ int bucketize(const float *bnd, int levels_pow2, float v) {
  int code = 0;
  for (int step = levels_pow2 >> 1; step > 0; step >>= 1)
    if (bnd[code + step - 1] < v) code += step;
  return code;
}

// The same search for N values at once: the N reads of a step are independent, so their LDS
// latencies overlap (a thread of a decode-sized launch has nothing else to hide them behind).
template <int N>
__device__ __forceinline__ void bucketize_many(const float *bnd, int levels_pow2, const float (&v)[N], int (&code)[N]) {
#pragma unroll
  for (int e = 0; e < N; ++e) code[e] = 0;
  for (int step = levels_pow2 >> 1; step > 0; step >>= 1) {
    float b[N];
#pragma unroll
    for (int e = 0; e < N; ++e) b[e] = bnd[code[e] + step - 1];
#pragma unroll
    for (int e = 0; e < N; ++e)
      if (b[e] < v[e]) code[e] += step;
  }
}

// Faster bucketize for small codebooks: the interval [first boundary, last boundary] is cut
// into kCells(levels) uniform cells; cell c stores how many boundaries lie in lower cells and
// the one boundary inside it (+inf if none), so a value costs one LDS read and one compare:
//   code = table[cell(v)].below + (table[cell(v)].boundary < v)
// This is exact for ANY monotone cell(): boundaries in lower cells are < v, boundaries in
// higher cells are > v, and the one in v's own cell is compared directly.  The table is only
// used when no cell holds two boundaries (checked while it is built); otherwise, and for
// codebooks of more than 64 levels, the binary search above is used.
constexpr int kMaxCells = 512;
struct CellMap {
  float scale, offset;
  int cells;  // 0: table not usable
};
__device__ __forceinline__ int cell_of(const CellMap &m, float v) {
  const int c = __float2int_rd(__builtin_fmaf(v, m.scale, m.offset));
  return min(max(c, 0), m.cells - 1);
}
__device__ __forceinline__ int bucketize_cells(const uint2 *table, const CellMap &m, float v) {
  const uint2 e = table[cell_of(m, v)];
  return static_cast<int>(e.y) + (__uint_as_float(e.x) < v ? 1 : 0);
}

// Emit eight consecutive results (slots c0 .. c0+7 of `row`).
template <int DT, bool VEC, typename Args>
__device__ __forceinline__ void emit8(const Args &a, int64_t row, int64_t c0, const int (&code)[kChunk],
                                      const float *cent, float s) {
  const int64_t K = a.K;
  if (a.codes != nullptr) {
    if (a.code_format == OQ_CODES_U8) {
      uint8_t *dst = a.codes + row * K + c0;
      if (VEC && c0 + kChunk <= K) {
        uint2 w;
        w.x = code[0] | (code[1] << 8) | (code[2] << 16) | (code[3] << 24);
        w.y = code[4] | (code[5] << 8) | (code[6] << 16) | (code[7] << 24);
        *reinterpret_cast<uint2 *>(dst) = w;
      } else {
        for (int e = 0; e < kChunk; ++e)
          if (c0 + e < K) dst[e] = static_cast<uint8_t>(code[e]);
      }
    } else {
      uint8_t *dst = a.codes + row * (K / 2) + c0 / 2;
      if (VEC && c0 + kChunk <= K) {
        uint32_t w = 0;
#pragma unroll
        for (int e = 0; e < kChunk; ++e) w |= static_cast<uint32_t>(code[e]) << (4 * e);
        *reinterpret_cast<uint32_t *>(dst) = w;
      } else {
        for (int e = 0; e < kChunk; e += 2)
          if (c0 + e < K) dst[e / 2] = static_cast<uint8_t>(code[e] | (code[e + 1] << 4));
      }
    }
  }
  if (a.values_mode == OQ_VALUES_SCALED) {
    for (int e = 0; e < kChunk; ++e)
      if (c0 + e < K) store_from_f32<DT>(a.values, row * K + c0 + e, cent[code[e]] * s);
  } else if (a.values_mode == OQ_VALUES_UNIT_BF16) {
    uint16_t *dst = static_cast<uint16_t *>(a.values) + row * K + c0;
    if (VEC && c0 + kChunk <= K) {
      uint32_t w[4];
#pragma unroll
      for (int j = 0; j < 4; ++j)
        w[j] = f32_to_bf16_bits(cent[code[2 * j]]) | (static_cast<uint32_t>(f32_to_bf16_bits(cent[code[2 * j + 1]])) << 16);
      *reinterpret_cast<uint4 *>(dst) = make_uint4(w[0], w[1], w[2], w[3]);
    } else {
      for (int e = 0; e < kChunk; ++e)
        if (c0 + e < K) dst[e] = f32_to_bf16_bits(cent[code[e]]);
    }
  }
}

// Register butterflies over a power-of-two array, distance 1 first.
template <int N>
__device__ __forceinline__ void fwht_regs(float (&v)[N], int limit) {
#pragma unroll
  for (int d = 1; d < N; d <<= 1) {
    if (d < limit) {
#pragma unroll
      for (int j = 0; j < N; ++j) {
        if ((j & d) == 0) {
          const float l = v[j], r = v[j + d];
          v[j] = l + r;
          v[j + d] = l - r;
        }
      }
    }
  }
}

// Lane exchanges for the butterflies between lanes l and l xor J: DPP quad permutes (1, 2),
// masked row shifts (4), a row rotate (8); wavefront shuffles for 16 and 32 (see also swap_stage).
__device__ __forceinline__ float dpp_xor1(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, v), 0xB1, 0xF, 0xF, true));
}
__device__ __forceinline__ float dpp_xor2(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, v), 0x4E, 0xF, 0xF, true));
}
__device__ __forceinline__ float dpp_xor4(float v) {
  const int i = __builtin_bit_cast(int, v);
  int o = __builtin_amdgcn_update_dpp(i, i, 0x104, 0xF, 0x5, false);  // lanes 0-3, 8-11 of a row <- lane + 4
  o = __builtin_amdgcn_update_dpp(o, i, 0x114, 0xF, 0xA, false);      // lanes 4-7, 12-15 <- lane - 4
  return __builtin_bit_cast(float, o);
}
__device__ __forceinline__ float dpp_xor8(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, v), 0x128, 0xF, 0xF, true));
}
template <int J>
__device__ __forceinline__ float lane_xor(float v) {
  if constexpr (J == 1) return dpp_xor1(v);
  else if constexpr (J == 2) return dpp_xor2(v);
  else if constexpr (J == 4) return dpp_xor4(v);
  else if constexpr (J == 8) return dpp_xor8(v);
  else return __shfl_xor(v, J, 64);
}

// Butterflies between lanes l and l xor J for J = 16, 32 without LDS traffic, two registers at a
// time.  The swap instruction exchanges the upper half of each 2J-lane group of `a` with the
// lower half of the same group of `b`; afterwards a holds the lower-half values of both
// registers and b the upper-half values, lane for lane, so sum and difference are plain
// register operations, and a second swap puts them back where the butterfly wants them
// (lower lane: y + other, upper lane: other - y, the same two operands as with a lane exchange).
template <int J>
__device__ __forceinline__ void swap_stage(float (&y)[kChunk]) {
  typedef unsigned u32x2 __attribute__((ext_vector_type(2)));
  auto swap = [](float a, float b) -> u32x2 {
    if constexpr (J == 16) return __builtin_amdgcn_permlane16_swap(__float_as_uint(a), __float_as_uint(b), false, false);
    else return __builtin_amdgcn_permlane32_swap(__float_as_uint(a), __float_as_uint(b), false, false);
  };
#pragma unroll
  for (int e = 0; e < kChunk; e += 2) {
    const u32x2 r = swap(y[e], y[e + 1]);
    const float lo = __uint_as_float(r.x), hi = __uint_as_float(r.y);
    const u32x2 o = swap(lo + hi, lo - hi);
    y[e] = __uint_as_float(o.x);
    y[e + 1] = __uint_as_float(o.y);
  }
}

// x / (s + eps) is evaluated as q0 = x*r, then two residual corrections
// q <- fma(fma(-q, d, x), r, q) with r = 1/d correctly rounded: the first makes q a
// faithful quotient, the second rounds it correctly (Markstein), which is what the
// IEEE division of the specification returns.  Inputs for which a residual could
// underflow, or that are not finite, take the plain division instead.
__device__ __forceinline__ float divide_by_row_norm(float x, float d, float r) {
  float q = x * r;
  q = __builtin_fmaf(__builtin_fmaf(-q, d, x), r, q);
  q = __builtin_fmaf(__builtin_fmaf(-q, d, x), r, q);
  return q;
}
__device__ __forceinline__ bool needs_plain_division(float x) {
  const float ax = __builtin_fabsf(x);
  return !((ax > 1e-30f || ax == 0.0f) && ax < 1e30f);
}

// Where the row is staged in LDS: 16-bit inputs stay 16-bit (half the LDS, so twice the rows
// in flight per CU) unless the big-block path needs the buffer for fp32 intermediates.
template <int DT, bool VEC, int LOG_G> struct RqStage {
  static constexpr bool k16 = VEC && DT != OQ_F32 && LOG_G == 0;
  static constexpr int kBytes = k16 ? 2 : 4;
};

struct PermSigns {
  int4 pa, pb;
  uint2 sg;
};
__device__ __forceinline__ void load_perm_signs(const RqArgs &a, int64_t c0, PermSigns &ps) {
  if (c0 + kChunk <= a.K) {
    ps.pa = *reinterpret_cast<const int4 *>(a.perm + c0);
    ps.pb = *reinterpret_cast<const int4 *>(a.perm + c0 + 4);
    ps.sg = *reinterpret_cast<const uint2 *>(a.signs + c0);
  }
}

// One row: `smem` is the workgroup's scratch (rq_lds_bytes() bytes, 16-byte aligned), `tid` the
// thread's index in a workgroup of `block_threads` threads (64 * wavefronts, or 256 * pass
// groups), all of which must make this call.  Codes, values and the norm go where `a` points
// for row `row` (any address space reachable through a generic pointer).
// `after_loads()` is called once by every thread, as soon as its first pass has gathered its
// inputs: from there on the only global loads it still waits for are the permutation / sign
// prefetches of later passes (rows longer than one pass per thread).
// FEW: the launch has a handful of rows (decode).  Then building the cell table (a barrier and
// a microsecond of dependent LDS reads per workgroup) costs more than it saves, and the values
// of a thread are searched together instead.  Same codes either way.
template <int DT, bool VEC, int LOG_G, bool FEW, typename AfterLoads>
__device__ __forceinline__ void rotate_quantize_row(const RqArgs &a, unsigned char *smem, const int64_t row,
                                                    const int tid, const int block_threads, AfterLoads after_loads) {
  using Stage = RqStage<DT, VEC, LOG_G>;
  // Thread = (virtual lane t of the 256-lane pass structure, pass group pg).  With one group a
  // thread walks all passes of its lane; when few rows are in flight the launcher starts up to
  // four groups so that the passes of a long row run side by side (group pg takes passes
  // pg, pg + groups, ...).
  const int t = tid & (kThreads - 1);
  const int pg = tid >> 8, groups_n = block_threads > kThreads ? block_threads >> 8 : 1;
  const int lane = t & 63;
  const int wave = t >> 6;
  const int64_t K = a.K;
  const int Kp = a.passes * kPass;
  float *bnd = reinterpret_cast<float *>(smem);  // 256 floats
  float *cent = bnd + 256;                       // 256 floats
  float *red = cent + 256;                       // 4 floats
  uint2 *cells = reinterpret_cast<uint2 *>(red + 4);            // kMaxCells x (boundary, count below)
  int *cells_bad = reinterpret_cast<int *>(cells + kMaxCells);  // 4 ints (one used)
  float *xbuf = reinterpret_cast<float *>(cells_bad + 4);       // Kp elements of Stage::kBytes
  // The window of the input map sits behind everything else, so that no other LDS address depends on it.
  const bool windowed = a.map != nullptr && a.map_lo >= 0;     // bf16 only (the launcher decides)
  uint16_t *hot_lds = reinterpret_cast<uint16_t *>(smem + a.map_lds_offset);  // kHotBytes, only when windowed
  const uint16_t *hot = windowed ? hot_lds : nullptr;
  uint16_t *xbuf16 = reinterpret_cast<uint16_t *>(xbuf);
  uint8_t *cbuf = reinterpret_cast<uint8_t *>(xbuf) + static_cast<size_t>(Kp) * Stage::kBytes;  // Kp bytes, big-block path only
  float *psum = reinterpret_cast<float *>(cbuf + (LOG_G > 0 ? Kp : 0));  // [passes][256], only with several pass groups

  // Permutation and signs of the first pass: requested before anything else so their latency
  // overlaps the row load (loads of one wavefront return in order).
  PermSigns ps_cur, ps_nxt;
  if constexpr (VEC) load_perm_signs(a, static_cast<int64_t>(pg) * kPass + t * kChunk, ps_cur);

  // Tables: requested here, parked in LDS only after the row has been requested.  The loads are
  // branch-free (clamped index, the boundaries as a readable stand-in for absent centroids) and
  // their values are not touched before that, so nothing waits here: a wavefront's loads return
  // in order, and a store of a loaded value at this point would put a full memory round trip
  // in front of the row's own.
  const int nthreads = block_threads;  // 64 * (wavefronts that own a part of the row), or 256 * pass groups
  const float *cent_src = a.cents != nullptr ? a.cents : a.bounds;
  const int cent_last = a.cents != nullptr ? a.levels - 1 : a.levels - 2;
  // entry tid of the 256 (every entry a codebook of up to 64 levels has); the others, if any, at park time
  const float table_b0 = a.bounds[min(tid, a.levels - 2)], table_c0 = cent_src[min(tid, cent_last)];
  auto park_tables = [&] {
    for (int i = tid; i < 256; i += nthreads) {
      float bv = __builtin_inff(), cv = 0.0f;
      if (i < a.levels - 1) bv = i == tid ? table_b0 : a.bounds[i];
      if (a.cents != nullptr && i < a.levels) cv = i == tid ? table_c0 : a.cents[i];
      bnd[i] = bv;
      cent[i] = cv;
    }
  };
  if (tid == 0) cells_bad[0] = 0;
  if (windowed) {  // both signs of the window, 16 bytes per thread and step; the rows are mapped before the first barrier below
    for (int i = tid; i < kHotBytes / 16; i += nthreads) {
      const int sign = i / (kHotHalf * 2 / 16), j = i % (kHotHalf * 2 / 16);
      reinterpret_cast<uint4 *>(hot_lds)[i] = reinterpret_cast<const uint4 *>(a.map + (sign << 15) + a.map_lo)[j];
    }
    __syncthreads();
  }

  // ---- phase A: stage the row, sum of squares in the documented order --------
  const int64_t row_base = row * K;
  float q = 0.0f;
  auto square_sum = [&](const float (&f)[kChunk], int p) {
    float s[kChunk];
#pragma unroll
    for (int e = 0; e < kChunk; ++e) s[e] = f[e] * f[e];
    const float v8 = ((s[0] + s[1]) + (s[2] + s[3])) + ((s[4] + s[5]) + (s[6] + s[7]));
    if (groups_n == 1) q = (p == 0) ? v8 : q + v8;
    else psum[p * kThreads + t] = v8;
  };
  if constexpr (Stage::k16) {
    auto stage16 = [&](const uint4 rw, int p, int64_t i0) {
      *reinterpret_cast<uint4 *>(xbuf16 + i0) = rw;
      const uint32_t w[4] = {rw.x, rw.y, rw.z, rw.w};
      float f[kChunk];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        if constexpr (DT == OQ_BF16) {
          f[2 * j] = __uint_as_float(w[j] << 16);
          f[2 * j + 1] = __uint_as_float(w[j] & 0xffff0000u);
        } else {
          f[2 * j] = f16_bits_to_f32(static_cast<uint16_t>(w[j] & 0xffffu));
          f[2 * j + 1] = f16_bits_to_f32(static_cast<uint16_t>(w[j] >> 16));
        }
      }
      square_sum(f, p);
    };
    const uint16_t *xrow = static_cast<const uint16_t *>(a.x) + row_base;
    // Two loops on purpose: with the table lookup inside it, the compiler schedules the plain
    // loop (and the passes after it) measurably worse.
    if (a.map == nullptr) {
      for (int p = pg; p < a.passes; p += groups_n) {
        const int64_t i0 = static_cast<int64_t>(p) * kPass + t * kChunk;
        uint4 rw = make_uint4(0u, 0u, 0u, 0u);
        if (i0 + kChunk <= K) rw = *reinterpret_cast<const uint4 *>(xrow + i0);
        stage16(rw, p, i0);
      }
    } else {
      for (int p = pg; p < a.passes; p += groups_n) {
        const int64_t i0 = static_cast<int64_t>(p) * kPass + t * kChunk;
        uint4 rw = make_uint4(0u, 0u, 0u, 0u);
        if (i0 + kChunk <= K) rw = map_raw8<DT>(*reinterpret_cast<const uint4 *>(xrow + i0), a, hot);
        stage16(rw, p, i0);
      }
    }
  } else {
    for (int p = pg; p < a.passes; p += groups_n) {
      const int64_t i0 = static_cast<int64_t>(p) * kPass + t * kChunk;
      float f[kChunk];
      load_chunk<DT, VEC>(a, hot, row_base, i0, f);
      float4 *dst = reinterpret_cast<float4 *>(xbuf + i0);
      dst[0] = make_float4(f[0], f[1], f[2], f[3]);
      dst[1] = make_float4(f[4], f[5], f[6], f[7]);
      square_sum(f, p);
    }
  }
  park_tables();  // read after the barrier below
  if (groups_n > 1) {  // the lane's passes were summed by different threads: add them left to right
    __syncthreads();
    if (pg == 0) {
      q = psum[t];
      for (int p = 1; p < a.passes; ++p) q = q + psum[p * kThreads + t];
    }
  }
  q = q + lane_xor<1>(q);
  q = q + lane_xor<2>(q);
  q = q + lane_xor<4>(q);
  q = q + lane_xor<8>(q);
  q = q + lane_xor<16>(q);
  q = q + lane_xor<32>(q);
  if (lane == 0 && pg == 0) red[wave] = q;
  __syncthreads();
  const int nwaves = min(nthreads, kThreads) >> 6;  // wavefronts that were not launched own only padding: their sum is 0
  const float total = (red[0] + (nwaves > 1 ? red[1] : 0.0f)) + ((nwaves > 2 ? red[2] : 0.0f) + (nwaves > 3 ? red[3] : 0.0f));
  const float s_norm = sqrtf(total);  // IEEE-rounded (hipcc's default for fp32 sqrt and division)
  const float denom = s_norm + a.eps;
  const float recip = 1.0f / denom;
  const bool row_plain = !(denom > 1e-30f && denom < 1e30f);  // the reciprocal itself would lose bits
  if (tid == 0 && a.norms != nullptr) a.norms[row] = s_norm;

  // ---- bucketize table (the boundaries are in LDS since the barrier above) ----------------
  CellMap cmap;
  cmap.cells = !FEW && a.levels <= 64 && a.levels >= 3 ? 8 * a.levels_pow2 : 0;
  {
    const float lo = bnd[0], hi = bnd[a.levels - 2];
    cmap.scale = static_cast<float>(cmap.cells) / (hi - lo);
    cmap.offset = -lo * cmap.scale;
    if (!(hi > lo) || !(cmap.scale < 3.0e38f) || !(__builtin_fabsf(cmap.offset) < 3.0e38f)) cmap.cells = 0;
  }
  if (cmap.cells > 0) {
    const int nb = a.levels - 1;
    for (int c = tid; c < cmap.cells; c += nthreads) {
      // boundaries are ascending, so their cells are too: first boundary with cell >= c, first with cell > c
      int first = 0, last = 0;
      for (int step = a.levels_pow2; step > 0; step >>= 1) {
        if (first + step <= nb && cell_of(cmap, bnd[first + step - 1]) < c) first += step;
        if (last + step <= nb && cell_of(cmap, bnd[last + step - 1]) <= c) last += step;
      }
      if (last - first > 1) cells_bad[0] = 1;
      cells[c] = make_uint2(__float_as_uint(last > first ? bnd[first] : __builtin_inff()), static_cast<uint32_t>(first));
    }
    __syncthreads();
    if (cells_bad[0] != 0) cmap.cells = 0;
  }
  auto code_of = [&](float v) -> int {
    return cmap.cells > 0 ? bucketize_cells(cells, cmap, v) : bucketize(bnd, a.levels_pow2, v);
  };

  auto staged = [&](int i) -> float {
    if constexpr (Stage::k16) {
      if constexpr (DT == OQ_BF16) return bf16_bits_to_f32(xbuf16[i]);
      else return f16_bits_to_f32(xbuf16[i]);
    } else {
      return xbuf[i];
    }
  };

  // ---- phase B: gather, divide, sign, butterflies up to distance 256 ----------
  const int h = a.block;
  constexpr bool BIG = LOG_G > 0;
  float keep[BIG ? kMaxPasses : 1][kChunk];

#pragma unroll
  for (int pi = 0; pi < kMaxPasses; ++pi) {
    const int p = pg + pi * groups_n;
    // small blocks: a wavefront whose 512 slots of this pass all lie past the row has nothing to do
    if (p < a.passes && (BIG || static_cast<int64_t>(p) * kPass + (t & ~63) * kChunk < K)) {
      const int64_t c0 = static_cast<int64_t>(p) * kPass + t * kChunk;
      float y[kChunk];
      if constexpr (VEC) {
        if (p + groups_n < a.passes) load_perm_signs(a, c0 + static_cast<int64_t>(groups_n) * kPass, ps_nxt);  // one pass ahead
      }
      if (VEC && c0 + kChunk <= K) {
        const int idx[kChunk] = {ps_cur.pa.x, ps_cur.pa.y, ps_cur.pa.z, ps_cur.pa.w,
                                 ps_cur.pb.x, ps_cur.pb.y, ps_cur.pb.z, ps_cur.pb.w};
        const uint2 sg = ps_cur.sg;
        float xv[kChunk];
        bool plain = row_plain;
#pragma unroll
        for (int e = 0; e < kChunk; ++e) {
          xv[e] = staged(idx[e]);
          plain = plain || needs_plain_division(xv[e]);
          y[e] = divide_by_row_norm(xv[e], denom, recip);
        }
        if (__builtin_amdgcn_ballot_w64(plain) != 0) {  // rare, and uniform over the wavefront
#pragma unroll
          for (int e = 0; e < kChunk; ++e) y[e] = xv[e] / denom;
        }
#pragma unroll
        for (int e = 0; e < kChunk; ++e) {  // multiply by the sign (+1 / -1 = 0xff): flip the sign bit
          const uint32_t sw = e < 4 ? sg.x : sg.y;
          y[e] = __uint_as_float(__float_as_uint(y[e]) ^ ((sw << (24 - 8 * (e & 3))) & 0x80000000u));
        }
      } else if constexpr (VEC) {  // K is a multiple of the chunk there: the whole chunk lies past the row
#pragma unroll
        for (int e = 0; e < kChunk; ++e) y[e] = 0.0f;
      } else {
#pragma unroll
        for (int e = 0; e < kChunk; ++e) {
          if (c0 + e < K) y[e] = (staged(a.perm[c0 + e]) / denom) * static_cast<float>(a.signs[c0 + e]);
          else y[e] = 0.0f;
        }
      }
      if constexpr (VEC) {
        if (p + groups_n < a.passes) ps_cur = ps_nxt;  // same condition as the load: no wait where nothing was requested
      }
      if (pi == 0) after_loads();  // this thread's first permutation and signs have arrived and are used up
      fwht_regs<kChunk>(y, h);
      auto lane_stage = [&](auto jt) {
        constexpr int J = decltype(jt)::value;
        if (J * kChunk < h) {
          // upper lane of a pair: other - y = other + (-y); lower lane: y + other
          const uint32_t neg = (lane & J) ? 0x80000000u : 0u;
#pragma unroll
          for (int e = 0; e < kChunk; ++e) y[e] = lane_xor<J>(y[e]) + __uint_as_float(__float_as_uint(y[e]) ^ neg);
        }
      };
      lane_stage(std::integral_constant<int, 1>{});
      lane_stage(std::integral_constant<int, 2>{});
      lane_stage(std::integral_constant<int, 4>{});
      lane_stage(std::integral_constant<int, 8>{});
      if constexpr (BIG) {  // LDS is the busier unit on this path, the ALUs on the other
        swap_stage<16>(y);
        swap_stage<32>(y);
      } else {
        lane_stage(std::integral_constant<int, 16>{});
        lane_stage(std::integral_constant<int, 32>{});
      }
      if constexpr (!BIG) {
        int code[kChunk];
#pragma unroll
        for (int e = 0; e < kChunk; ++e) {
          if constexpr (!FEW) code[e] = code_of(y[e] * a.inv_sqrt_block);
        }
        if constexpr (FEW) {
          float sv[kChunk];
#pragma unroll
          for (int e = 0; e < kChunk; ++e) sv[e] = y[e] * a.inv_sqrt_block;
          bucketize_many<kChunk>(bnd, a.levels_pow2, sv, code);
        }
        if (c0 < K) emit8<DT, VEC>(a, row, c0, code, cent, s_norm);
      } else {
#pragma unroll
        for (int e = 0; e < kChunk; ++e) keep[pi][e] = y[e];
      }
    } else if (pi == 0) {
      after_loads();
    }
  }

  if constexpr (BIG) {
    // ---- phase C: distances 512 .. block/2 through LDS --------------------------
    __syncthreads();  // every gather has read xbuf
#pragma unroll
    for (int pi = 0; pi < kMaxPasses; ++pi) {
      const int p = pg + pi * groups_n;
      if (p < a.passes) {
        float4 *dst = reinterpret_cast<float4 *>(xbuf + static_cast<int64_t>(p) * kPass + t * kChunk);
        dst[0] = make_float4(keep[pi][0], keep[pi][1], keep[pi][2], keep[pi][3]);
        dst[1] = make_float4(keep[pi][4], keep[pi][5], keep[pi][6], keep[pi][7]);
      }
    }
    __syncthreads();
    constexpr int G = 1 << LOG_G;  // block / 512
    const int groups = static_cast<int>(K >> LOG_G);
    for (int gi = tid; gi < groups; gi += nthreads) {
      const int base = (gi >> 9) * h + (gi & (kLaneSpan - 1));
      float z[G];
#pragma unroll
      for (int v = 0; v < G; ++v) z[v] = xbuf[base + kLaneSpan * v];
      fwht_regs<G>(z, G);
      if constexpr (FEW) {
        float sv[G];
        int cd[G];
#pragma unroll
        for (int v = 0; v < G; ++v) sv[v] = z[v] * a.inv_sqrt_block;
        bucketize_many<G>(bnd, a.levels_pow2, sv, cd);
#pragma unroll
        for (int v = 0; v < G; ++v) cbuf[base + kLaneSpan * v] = static_cast<uint8_t>(cd[v]);
      } else {
#pragma unroll
        for (int v = 0; v < G; ++v)
          cbuf[base + kLaneSpan * v] = static_cast<uint8_t>(code_of(z[v] * a.inv_sqrt_block));
      }
    }
    __syncthreads();
    for (int64_t c0 = static_cast<int64_t>(tid) * kChunk; c0 < K; c0 += static_cast<int64_t>(max(nthreads, kThreads)) * kChunk) {
      const uint2 w = *reinterpret_cast<const uint2 *>(cbuf + c0);
      int code[kChunk];
#pragma unroll
      for (int e = 0; e < kChunk; ++e) code[e] = ((e < 4 ? w.x : w.y) >> (8 * (e & 3))) & 0xff;
      emit8<DT, VEC>(a, row, c0, code, cent, s_norm);
    }
  }
}


// Host side: bytes of scratch rotate_quantize_row needs for a workgroup of `pass_groups`
// groups of 256 threads (1: a single group, possibly of fewer wavefronts); sets the offset
// of the input-map window in `a` when there is one.
inline size_t lds_bytes(RqArgs &a, int x_dtype, bool vec, int pass_groups) {
  const size_t kp = static_cast<size_t>(a.passes) * kPass;
  const bool big = a.block > kLaneSpan;
  const bool stage16 = vec && x_dtype != OQ_F32 && !big;  // RqStage::k16
  size_t bytes = (256 + 256 + 4) * sizeof(float) + kMaxCells * 8 + 16 + kp * (stage16 ? 2 : 4) + (big ? kp : 0);
  if (pass_groups > 1) bytes += static_cast<size_t>(a.passes) * kThreads * sizeof(float);
  bytes = (bytes + 15) & ~static_cast<size_t>(15);
  if (a.map_lo >= 0) {
    a.map_lds_offset = static_cast<int>(bytes);
    bytes += kHotBytes;
  }
  return bytes;
}

inline int log2_groups(const RqArgs &a) {  // the LOG_G template argument for a block size
  int log_g = 0;
  for (int g = a.block / kLaneSpan; g > 1; g >>= 1) ++log_g;
  return log_g;
}

}  // namespace rq

// Checks the arguments of oq_rotate_quantize and fills `out`; `vec` tells whether every
// pointer and K allow the 16-byte access paths (the VEC template argument).  Returns OQ_OK,
// or the status to hand back (the message is set).  Defined in rotate_quantize.hip.
int rotate_quantize_prepare(const void *x, int x_dtype, int64_t M, int64_t K, const int32_t *perm,
                            const int8_t *signs, const float *boundaries, const float *centroids,
                            int levels, int64_t block, float eps, float inv_sqrt_block,
                            void *codes_out, int code_format, void *values_out, int values_mode,
                            float *norms_out, const uint16_t *input_map, rq::RqArgs *out, bool *vec);

}  // namespace oq
