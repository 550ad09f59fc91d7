// Fused RPBH rotate + per-token quantize with a rotate plan (rotate_plan.h): the throughput form
// of the kernel in rotate_quantize_row.h, same results bit for bit.
//
// The plain kernel is bound by instruction issue (about 90 vector instructions per value, against
// 78 issue slots per value at its measured speed), not by memory.  This one spends about a third:
//   * the block size is a template argument, so the butterfly stages are straight-line code;
//   * a row is cut into units of max(block, 512) values; a wavefront owns whole units and keeps a
//     unit in registers (block / 512 steps of 8 values per lane), so butterfly distances of 512
//     and more are register operations too and nothing is regrouped through LDS;
//   * lane exchanges are two instructions per value: DPP adds and subtracts restricted to the
//     lower / upper lanes of a pair by their bank masks (distances 4 and 8 lanes), an exclusive-or
//     plus a DPP add inside quads, lane-group swaps of register pairs for 16 and 32 lanes;
//   * permutation, sign, the 1/sqrt(block) factor and the bucketize table come from the plan;
//   * x / (s + eps) is four instructions: q = fma(x, rh, x * rl) with rh + rl = 1 / (s + eps) to
//     twice the working precision is a faithful quotient, and one residual correction
//     fma(fma(-q, d, x), rh, q) with rh the correctly rounded reciprocal rounds it correctly
//     (Markstein).  Rows whose magnitudes could make a residual inexact (a value below 2^-80, a
//     denominator outside [2^-80, 2^20], anything not finite) take the IEEE division instead;
//     the test is one packed instruction pair per two bf16 values while the row is read.
//
// The sum of squares keeps the documented order: [passes][256 lanes][8], tree over the lanes.
// Compiled without FMA contraction.
#pragma once
#pragma clang fp contract(off)

#include <type_traits>

#include "packed_decode.h"
#include "rotate_plan.h"
#include "rotate_quantize_row.h"
#include "value_map.h"

namespace oq {
namespace rqf {

using rq::kChunk;
using rq::kLaneSpan;
using rq::kPass;
using rq::kThreads;

struct FastArgs {
  const void *x;
  int64_t M, K;
  const unsigned char *plan;
  const float *cents;  // only for the values modes
  int levels, levels_pow2;
  int block;
  int passes;       // ceil(K / 2048)
  int units;        // units of max(block, 512) values per row
  float eps;
  uint8_t *codes;
  int code_format;
  void *values;
  int values_mode;
  float *norms;
  // EMIT_WEIGHT only
  const float *raw_bounds;   // the codebook's boundaries as they are (the plan's are folded with 1/sqrt(block))
  float inv_sqrt_block;
  int pack_bits;
  uint8_t *packed;           // flat bit stream of [M, K] indices
  uint16_t *norms_bf16;      // [M]
  // MAPPED only: a function of the 16-bit input as a table of 65536 entries (value_map.h), applied to
  // every value as it is read; what follows - norm, rotation, codes - is that of the mapped row
  const uint16_t *map;
};

// LDS: cells (2048) | thresholds (1024) | centroids (1024) | reduction slots (64) | staging
constexpr int kCellsAt = 0, kThrAt = 2048, kCentAt = 3072, kRedAt = 4096, kStageAt = plan::kStageAddress;  // kRedAt: four group sums, then one flag per wavefront

// staging: 4 bytes per value (fp32 once, 16-bit twice)
__host__ __device__ inline size_t fast_lds_bytes(int64_t K) { return static_cast<size_t>(kStageAt) + 4u * static_cast<size_t>(K); }
// ... and behind it, for a launch with an input map, the map's 16 KB window (value_map.h)
inline size_t fast_lds_bytes_mapped(int64_t K) { return fast_lds_bytes(K) + static_cast<size_t>(kWideBytes); }

// ---- lane-exchange butterflies, eight values per call -------------------------------------------
// y'[lane] = (lane & J) ? y[lane ^ J] - y[lane] : y[lane] + y[lane ^ J]
// The leading s_nop covers the two wait states a DPP read needs after a vector write of the same
// register (the values of the previous stage); inside a block eight other instructions separate
// a value's write from its next DPP read.
#define OQ_DPP_PAIR(ADD, SUB)                                                                      \
  asm("s_nop 1\n\t" ADD(0) SUB(0) ADD(1) SUB(1) ADD(2) SUB(2) ADD(3) SUB(3) ADD(4) SUB(4) ADD(5) SUB(5) ADD(6) SUB(6) ADD(7) SUB(7) \
      : "=&v"(d[0]), "=&v"(d[1]), "=&v"(d[2]), "=&v"(d[3]), "=&v"(d[4]), "=&v"(d[5]), "=&v"(d[6]), "=&v"(d[7])                 \
      : "v"(y[0]), "v"(y[1]), "v"(y[2]), "v"(y[3]), "v"(y[4]), "v"(y[5]), "v"(y[6]), "v"(y[7]))

__device__ __forceinline__ void stage_xor4(float (&y)[kChunk]) {
  float d[kChunk];
#define OQ_A(i) "v_add_f32_dpp %" #i ", %" OQ_IN(i) ", %" OQ_IN(i) " row_shl:4 row_mask:0xf bank_mask:0x5\n\t"
#define OQ_S(i) "v_sub_f32_dpp %" #i ", %" OQ_IN(i) ", %" OQ_IN(i) " row_shr:4 row_mask:0xf bank_mask:0xa\n\t"
#define OQ_IN(i) OQ_IN_##i
#define OQ_IN_0 "8"
#define OQ_IN_1 "9"
#define OQ_IN_2 "10"
#define OQ_IN_3 "11"
#define OQ_IN_4 "12"
#define OQ_IN_5 "13"
#define OQ_IN_6 "14"
#define OQ_IN_7 "15"
  OQ_DPP_PAIR(OQ_A, OQ_S);
#undef OQ_A
#undef OQ_S
#pragma unroll
  for (int e = 0; e < kChunk; ++e) y[e] = d[e];
}

__device__ __forceinline__ void stage_xor8(float (&y)[kChunk]) {
  float d[kChunk];
#define OQ_A(i) "v_add_f32_dpp %" #i ", %" OQ_IN(i) ", %" OQ_IN(i) " row_ror:8 row_mask:0xf bank_mask:0x3\n\t"
#define OQ_S(i) "v_sub_f32_dpp %" #i ", %" OQ_IN(i) ", %" OQ_IN(i) " row_ror:8 row_mask:0xf bank_mask:0xc\n\t"
  OQ_DPP_PAIR(OQ_A, OQ_S);
#undef OQ_A
#undef OQ_S
#pragma unroll
  for (int e = 0; e < kChunk; ++e) y[e] = d[e];
}

// Inside a quad no mask tells the lower lane of a pair from the upper one: the upper lane's own
// value is negated by an exclusive-or with `neg` (the sign bit in the upper lanes), then one DPP add.
#define OQ_QUAD_STAGE(NAME, PERM)                                                                                     \
  __device__ __forceinline__ void NAME(float (&y)[kChunk], uint32_t neg) {                                            \
    float d[kChunk];                                                                                                  \
    asm("v_xor_b32 %0, %16, %8\n\tv_xor_b32 %1, %16, %9\n\tv_xor_b32 %2, %16, %10\n\tv_xor_b32 %3, %16, %11\n\t"      \
        "v_xor_b32 %4, %16, %12\n\tv_xor_b32 %5, %16, %13\n\tv_xor_b32 %6, %16, %14\n\tv_xor_b32 %7, %16, %15\n\t"    \
        "v_add_f32_dpp %0, %8, %0 " PERM " row_mask:0xf bank_mask:0xf\n\t"                                            \
        "v_add_f32_dpp %1, %9, %1 " PERM " row_mask:0xf bank_mask:0xf\n\t"                                            \
        "v_add_f32_dpp %2, %10, %2 " PERM " row_mask:0xf bank_mask:0xf\n\t"                                           \
        "v_add_f32_dpp %3, %11, %3 " PERM " row_mask:0xf bank_mask:0xf\n\t"                                           \
        "v_add_f32_dpp %4, %12, %4 " PERM " row_mask:0xf bank_mask:0xf\n\t"                                           \
        "v_add_f32_dpp %5, %13, %5 " PERM " row_mask:0xf bank_mask:0xf\n\t"                                           \
        "v_add_f32_dpp %6, %14, %6 " PERM " row_mask:0xf bank_mask:0xf\n\t"                                           \
        "v_add_f32_dpp %7, %15, %7 " PERM " row_mask:0xf bank_mask:0xf\n\t"                                           \
        : "=&v"(d[0]), "=&v"(d[1]), "=&v"(d[2]), "=&v"(d[3]), "=&v"(d[4]), "=&v"(d[5]), "=&v"(d[6]), "=&v"(d[7])      \
        : "v"(y[0]), "v"(y[1]), "v"(y[2]), "v"(y[3]), "v"(y[4]), "v"(y[5]), "v"(y[6]), "v"(y[7]), "v"(neg));          \
    _Pragma("unroll") for (int e = 0; e < kChunk; ++e) y[e] = d[e];                                                   \
  }
OQ_QUAD_STAGE(stage_xor1, "quad_perm:[1,0,3,2]")
OQ_QUAD_STAGE(stage_xor2, "quad_perm:[2,3,0,1]")
#undef OQ_QUAD_STAGE
#undef OQ_DPP_PAIR
#undef OQ_IN
#undef OQ_IN_0
#undef OQ_IN_1
#undef OQ_IN_2
#undef OQ_IN_3
#undef OQ_IN_4
#undef OQ_IN_5
#undef OQ_IN_6
#undef OQ_IN_7

__device__ __forceinline__ uint16_t lds_read_u16(uint32_t byte_addr) {
  return *reinterpret_cast<__attribute__((address_space(3))) const uint16_t *>(static_cast<uintptr_t>(byte_addr));
}

// ---- the division -------------------------------------------------------------------------------
struct Reciprocal {
  float d, rh, rl;
  bool plain;  // this row takes the IEEE division
};
__device__ __forceinline__ float divide_fast(float x, const Reciprocal &r) {
  const float q = __builtin_fmaf(x, r.rh, x * r.rl);
  return __builtin_fmaf(__builtin_fmaf(-q, r.d, x), r.rh, q);
}

// code = entry.count + (entry.threshold < value) for eight values: the compares first, into eight
// scalar masks, then the eight carry additions (a mask must not be read right after it is written).
__device__ __forceinline__ void count_below(const uint2 (&ent)[kChunk], const float (&v)[kChunk], int (&code)[kChunk]) {
  uint64_t m0, m1, m2, m3, m4, m5, m6, m7;
  asm("v_cmp_lt_f32_e64 %8, %16, %24\n\tv_cmp_lt_f32_e64 %9, %17, %25\n\tv_cmp_lt_f32_e64 %10, %18, %26\n\t"
      "v_cmp_lt_f32_e64 %11, %19, %27\n\tv_cmp_lt_f32_e64 %12, %20, %28\n\tv_cmp_lt_f32_e64 %13, %21, %29\n\t"
      "v_cmp_lt_f32_e64 %14, %22, %30\n\tv_cmp_lt_f32_e64 %15, %23, %31\n\t"
      "v_addc_co_u32_e64 %0, %8, 0, %32, %8\n\tv_addc_co_u32_e64 %1, %9, 0, %33, %9\n\t"
      "v_addc_co_u32_e64 %2, %10, 0, %34, %10\n\tv_addc_co_u32_e64 %3, %11, 0, %35, %11\n\t"
      "v_addc_co_u32_e64 %4, %12, 0, %36, %12\n\tv_addc_co_u32_e64 %5, %13, 0, %37, %13\n\t"
      "v_addc_co_u32_e64 %6, %14, 0, %38, %14\n\tv_addc_co_u32_e64 %7, %15, 0, %39, %15"
      : "=&v"(code[0]), "=&v"(code[1]), "=&v"(code[2]), "=&v"(code[3]), "=&v"(code[4]), "=&v"(code[5]), "=&v"(code[6]),
        "=&v"(code[7]), "=&s"(m0), "=&s"(m1), "=&s"(m2), "=&s"(m3), "=&s"(m4), "=&s"(m5), "=&s"(m6), "=&s"(m7)
      : "v"(ent[0].x), "v"(ent[1].x), "v"(ent[2].x), "v"(ent[3].x), "v"(ent[4].x), "v"(ent[5].x), "v"(ent[6].x), "v"(ent[7].x),
        "v"(v[0]), "v"(v[1]), "v"(v[2]), "v"(v[3]), "v"(v[4]), "v"(v[5]), "v"(v[6]), "v"(v[7]),
        "v"(ent[0].y), "v"(ent[1].y), "v"(ent[2].y), "v"(ent[3].y), "v"(ent[4].y), "v"(ent[5].y), "v"(ent[6].y), "v"(ent[7].y));
}

// What a launch writes: EMIT_NIBBLE / EMIT_U8 are the two hot forms (codes only), EMIT_ANY reads
// the output arguments at run time (values modes, no codes, ...).  EMIT_WEIGHT is the weight side
// of the layer (src/orbitquant/layers.py:121-125,201-215 of the reference): the row is rotated
// as it is, multiplied by 1/sqrt(block), THEN divided by max(norm, eps) with the IEEE division,
// searched in the unfolded boundaries, and its indices are packed `pack_bits` wide into the flat
// little-endian stream; the norm is stored as bf16.
enum EmitMode { EMIT_NIBBLE = 0, EMIT_U8 = 1, EMIT_ANY = 2, EMIT_WEIGHT = 3 };

// One row.  `smem`: fast_lds_bytes(K) bytes, 16-byte aligned.  All 64 * waves threads of the
// workgroup make the call.
template <int DT, int LOG_H, int EMIT, bool MAPPED = false>
__device__ __forceinline__ void rotate_quantize_row_fast(const FastArgs &a, unsigned char *smem, const int64_t row,
                                                         const int tid, const int waves) {
  static_assert(!MAPPED || DT == OQ_BF16, "the input map's LDS window is one of bf16 bit patterns");
  constexpr int H = 1 << LOG_H;
  constexpr int G = H > kLaneSpan ? H / kLaneSpan : 1;  // steps of 512 values a unit is made of
  const int lane = tid & 63, wave = tid >> 6;
  const int64_t K = a.K;
  const plan::PlanHeader *hdr = reinterpret_cast<const plan::PlanHeader *>(a.plan);
  uint2 *cells = reinterpret_cast<uint2 *>(smem + kCellsAt);
  float *thr = reinterpret_cast<float *>(smem + kThrAt);
  float *cent = reinterpret_cast<float *>(smem + kCentAt);
  float *red = reinterpret_cast<float *>(smem + kRedAt);       // [0..3] group sums, [4..11] per-wavefront flags
  unsigned char *stage = smem + kStageAt;
  const uint32_t *gather = reinterpret_cast<const uint32_t *>(a.plan + plan::kGatherOffset) + (DT == OQ_F32 ? K : 0);

  // A plan built for another shape must not be walked.  No codes are written then, and the row's norm
  // is stored as NaN, so that the mismatch cannot pass for a result: every output computed from it is NaN.
  // (The gather entries are absolute LDS addresses, valid because this kernel's LDS block starts at 0.)
  if (hdr->magic != plan::kMagic || hdr->K != static_cast<uint32_t>(K) || hdr->block != static_cast<uint32_t>(H) ||
      hdr->levels != static_cast<uint32_t>(a.levels) || lds_byte_address(smem) != 0u) {
    if (tid == 0) {
      if (a.norms != nullptr) a.norms[row] = __builtin_nanf("");
      if constexpr (EMIT == EMIT_WEIGHT) a.norms_bf16[row] = 0x7fc0;
    }
    return;
  }
  const float cell_scale = hdr->cell_scale, cell_offset = hdr->cell_offset;

  // tables: entry tid is requested now and stored to LDS after the row has been requested (loads
  // return in order); workgroups of fewer than 256 threads fetch the rest when they store.
  const int nthreads = waves * 64;
  const int Ki = static_cast<int>(K);
  const int table_idx = min(tid, 255);
  const uint2 cell_v = reinterpret_cast<const uint2 *>(a.plan + plan::kCellsOffset)[table_idx];
  const float thr_v = EMIT == EMIT_WEIGHT ? (table_idx < a.levels - 1 ? a.raw_bounds[table_idx] : __builtin_inff())
                                          : reinterpret_cast<const float *>(a.plan + plan::kThresholdsOffset)[table_idx];
  const float cent_v = (EMIT == EMIT_ANY && a.cents != nullptr) ? a.cents[min(table_idx, a.levels - 1)] : 0.0f;

  // an input map's window goes to LDS first (every wavefront looks values up in it as it reads the row)
  const uint16_t *hot = nullptr;
  if constexpr (MAPPED) {
    uint16_t *window = reinterpret_cast<uint16_t *>(smem + fast_lds_bytes(K));
    fill_map_window<kWideLog2>(window, a.map, kWideLoBf16, tid, waves * 64);
    hot = window;
    __syncthreads();
  }

  // ---- phase A: stage the row (16-bit inputs as x and as -x), sum of squares -----------------
  // Virtual lane t of the documented [passes][256 lanes][8] order is lane t % 64 of group t / 64;
  // wavefront w owns the groups w, w + waves, ... with all their passes, and keeps four passes of
  // a group requested ahead of the one it is summing.  (Adding a lane's first pass to +0 is exact.)
  constexpr int kElem = DT == OQ_F32 ? 4 : 2;
  const unsigned char *xrow = static_cast<const unsigned char *>(a.x) + row * K * kElem;  // uniform
  typedef unsigned short u16x2 __attribute__((ext_vector_type(2)));
  uint32_t tiny_acc = 0xffffffffu;   // bf16: running minimum of (2 T - 1) - 2 |x| per half, T = bits of 2^-80
  bool tiny32 = false;               // fp32: a nonzero value below 2^-80 was seen
  const uint32_t kMadMul = 0xfffefffeu, kMadAdd = 0x2eff2effu;
  const int lane_first = lane * kChunk;
  constexpr int kBatch = 4;
#pragma nounroll
  for (int grp = wave; grp < 4; grp += waves) {  // uniform over the wavefront
    float q = 0.0f;
    uint4 raw_lo[kBatch], raw_hi[kBatch];  // a ring of requested chunks (fp32: both halves; 16-bit: raw_lo only)
    auto request = [&](int b, int p) {
      const int i0 = p * kPass + grp * kLaneSpan + lane_first;  // chunks past the row: i0 >= Ki
      raw_lo[b] = make_uint4(0u, 0u, 0u, 0u);
      raw_hi[b] = raw_lo[b];
      if (i0 < Ki) {
        const uint4 *src = reinterpret_cast<const uint4 *>(xrow + static_cast<uint32_t>(i0) * kElem);
        raw_lo[b] = src[0];
        if constexpr (DT == OQ_F32) raw_hi[b] = src[1];
      }
    };
#pragma unroll
    for (int b = 0; b < kBatch; ++b) request(b, b);
#pragma nounroll
    for (int pb = 0; pb < a.passes; pb += kBatch) {
#pragma unroll
      for (int b = 0; b < kBatch; ++b) {
        const int chunk0 = (pb + b) * kPass + grp * kLaneSpan;
        const int i0 = chunk0 + lane_first;
        if (chunk0 < Ki) {  // uniform over the wavefront; chunks wholly past the row would add +0
          float f[kChunk];
          if constexpr (DT == OQ_F32) {
            if (i0 < Ki) {
              uint4 *dst = reinterpret_cast<uint4 *>(stage + 4 * i0);
              dst[0] = raw_lo[b];
              dst[1] = raw_hi[b];
            }
            const uint32_t w[kChunk] = {raw_lo[b].x, raw_lo[b].y, raw_lo[b].z, raw_lo[b].w,
                                        raw_hi[b].x, raw_hi[b].y, raw_hi[b].z, raw_hi[b].w};
#pragma unroll
            for (int e = 0; e < kChunk; ++e) {
              f[e] = __uint_as_float(w[e]);
              tiny32 = tiny32 || (f[e] != 0.0f && __builtin_fabsf(f[e]) < 0x1p-80f);
            }
          } else {
            uint4 in = raw_lo[b];
            if constexpr (MAPPED) {
              // (lanes past the row's end look up an ordinary value instead of their zero padding, which lies
              // outside the window and would send the whole wavefront to the table in memory; they add +0 as before)
              const bool live = i0 < Ki;
              uint4 one[1] = {live ? in : make_uint4(0x3f803f80u, 0x3f803f80u, 0x3f803f80u, 0x3f803f80u)};
              map_words8_many<OQ_BF16, 1, kWideLog2>(one, a.map, hot, kWideLoBf16);
              in = live ? one[0] : make_uint4(0u, 0u, 0u, 0u);
            }
            const uint32_t w[4] = {in.x, in.y, in.z, in.w};
            if (i0 < Ki) {
              *reinterpret_cast<uint4 *>(stage + 2 * i0) = in;
              *reinterpret_cast<uint4 *>(stage + 2 * (Ki + i0)) =
                  make_uint4(w[0] ^ 0x80008000u, w[1] ^ 0x80008000u, w[2] ^ 0x80008000u, w[3] ^ 0x80008000u);
            }
#pragma unroll
            for (int j = 0; j < 4; ++j) {
              if constexpr (DT == OQ_BF16) {
                f[2 * j] = __uint_as_float(w[j] << 16);
                f[2 * j + 1] = __uint_as_float(w[j] & 0xffff0000u);
                uint32_t g;
                asm("v_pk_mad_u16 %0, %1, %2, %3" : "=v"(g) : "v"(w[j]), "v"(kMadMul), "v"(kMadAdd));
                tiny_acc = __builtin_bit_cast(uint32_t, __builtin_elementwise_min(__builtin_bit_cast(u16x2, tiny_acc),
                                                                                  __builtin_bit_cast(u16x2, g)));
              } else {
                f[2 * j] = f16_bits_to_f32(static_cast<uint16_t>(w[j] & 0xffffu));
                f[2 * j + 1] = f16_bits_to_f32(static_cast<uint16_t>(w[j] >> 16));
              }
            }
          }
#ifdef OQ_RQ_TIMING_NO_SUMSQ  // timing experiment only: what the pass would cost if the sums came from elsewhere
          q = q + f[0];
#else
          float sq[kChunk];
#pragma unroll
          for (int e = 0; e < kChunk; ++e) sq[e] = f[e] * f[e];
          q = q + (((sq[0] + sq[1]) + (sq[2] + sq[3])) + ((sq[4] + sq[5]) + (sq[6] + sq[7])));
#endif
        }
        if (pb + kBatch < a.passes) request(b, pb + b + kBatch);  // refill the slot: four passes stay in flight
      }
    }
    q = q + rq::lane_xor<1>(q);
    q = q + rq::lane_xor<2>(q);
    q = q + rq::lane_xor<4>(q);
    q = q + rq::lane_xor<8>(q);
    q = q + rq::lane_xor<16>(q);
    q = q + rq::lane_xor<32>(q);
    if (lane == 0) red[grp] = q;
  }
  bool tiny = tiny32;
  if constexpr (DT == OQ_BF16) tiny = min(tiny_acc & 0xffffu, tiny_acc >> 16) < 0x2effu;
  const bool wave_tiny = __builtin_amdgcn_ballot_w64(tiny) != 0;
  if (lane == 0) red[4 + wave] = wave_tiny ? 1.0f : 0.0f;
  if (tid < 256) {
    cells[tid] = cell_v;
    thr[tid] = thr_v;
    cent[tid] = cent_v;
  }
#pragma nounroll
  for (int idx = tid + nthreads; idx < 256; idx += nthreads) {  // workgroups of fewer than 256 threads only
    cells[idx] = reinterpret_cast<const uint2 *>(a.plan + plan::kCellsOffset)[idx];
    thr[idx] = EMIT == EMIT_WEIGHT ? (idx < a.levels - 1 ? a.raw_bounds[idx] : __builtin_inff())
                                   : reinterpret_cast<const float *>(a.plan + plan::kThresholdsOffset)[idx];
    cent[idx] = (EMIT == EMIT_ANY && a.cents != nullptr) ? a.cents[min(idx, a.levels - 1)] : 0.0f;
  }
  __syncthreads();
  const float total = (red[0] + red[1]) + (red[2] + red[3]);
  const float s_norm = sqrtf(total);
  Reciprocal rc;
  rc.d = s_norm + a.eps;
  rc.rh = 1.0f / rc.d;
  rc.rl = __builtin_fmaf(-rc.d, rc.rh, 1.0f) * rc.rh;
  bool row_plain = !(rc.d >= 0x1p-80f && rc.d <= 0x1p20f);
#pragma nounroll
  for (int w = 0; w < waves; ++w) row_plain = row_plain || red[4 + w] != 0.0f;
  if (tid == 0 && a.norms != nullptr) a.norms[row] = s_norm;
  const float weight_denominator = s_norm < a.eps ? a.eps : s_norm;  // clamp_min(eps): a NaN norm stays NaN
  if constexpr (EMIT == EMIT_WEIGHT) {
    if (tid == 0) a.norms_bf16[row] = f32_to_bf16_bits(s_norm);
  }

  // ---- phase B: units of max(H, 512) values, one wavefront each ---------------------------------
  // The two rare modes (IEEE division for this row, binary search instead of the cell table) pass
  // through an empty asm statement inside the loop on purpose: as loop invariants the compiler
  // clones the whole loop per combination.
  const uint32_t row_modes = __builtin_amdgcn_readfirstlane((row_plain ? 1u : 0u) | (hdr->cells != 0 ? 0u : 2u));
  uint8_t *codes_row = a.codes + row * (EMIT == EMIT_NIBBLE ? K / 2 : K);  // uniform; used by EMIT_NIBBLE / EMIT_U8 only
  const uint32_t neg1 = (lane & 1) ? 0x80000000u : 0u, neg2 = (lane & 2) ? 0x80000000u : 0u;
  // The gather entries of a step are requested one step ahead (past the last step: the row's
  // last chunk again, never used).
  int4 ea_next, eb_next;
  const unsigned char *gather_bytes = reinterpret_cast<const unsigned char *>(gather);  // uniform
  auto request_entries = [&](int first) {
    const uint32_t c = static_cast<uint32_t>(min(first + lane_first, Ki - kChunk));
    ea_next = *reinterpret_cast<const int4 *>(gather_bytes + c * 4u);
    eb_next = *reinterpret_cast<const int4 *>(gather_bytes + c * 4u + 16u);
  };
  request_entries(wave * (G * kLaneSpan));
  float xv[kChunk];  // the gathered inputs of a step
#pragma unroll
  for (int e = 0; e < kChunk; ++e) xv[e] = 0.0f;
#pragma nounroll
  for (int u = wave; u < a.units; u += waves) {
    float y[G][kChunk];
    const int unit_base = u * (G * kLaneSpan);
    uint32_t modes_now = row_modes;
    asm volatile("" : "+s"(modes_now));
    const bool plain = (modes_now & 1u) != 0u, searched = (modes_now & 2u) != 0u;
#pragma unroll
    for (int j = 0; j < G; ++j) {
      // Lanes past the end of the row (last unit of a row with H < 512 only) walk the row's last
      // chunk instead: their blocks are their own, and nothing of theirs is stored.
      const int4 ea = ea_next, eb = eb_next;
      request_entries(j + 1 < G ? unit_base + (j + 1) * kLaneSpan : unit_base + waves * (G * kLaneSpan));
      const uint32_t ent[kChunk] = {static_cast<uint32_t>(ea.x), static_cast<uint32_t>(ea.y), static_cast<uint32_t>(ea.z),
                                    static_cast<uint32_t>(ea.w), static_cast<uint32_t>(eb.x), static_cast<uint32_t>(eb.y),
                                    static_cast<uint32_t>(eb.z), static_cast<uint32_t>(eb.w)};
      if constexpr (DT == OQ_BF16) {
        // A bf16 value is the upper half of its fp32: the 16-bit LDS load that writes only the upper
        // half of its destination needs no conversion, as long as the lower halves are zero (xv was
        // zeroed before the loop and is only ever written by these loads).
        asm volatile("ds_read_u16_d16_hi %0, %8\n\tds_read_u16_d16_hi %1, %9\n\tds_read_u16_d16_hi %2, %10\n\t"
                     "ds_read_u16_d16_hi %3, %11\n\tds_read_u16_d16_hi %4, %12\n\tds_read_u16_d16_hi %5, %13\n\t"
                     "ds_read_u16_d16_hi %6, %14\n\tds_read_u16_d16_hi %7, %15\n\ts_waitcnt lgkmcnt(0)"
                     : "+v"(xv[0]), "+v"(xv[1]), "+v"(xv[2]), "+v"(xv[3]), "+v"(xv[4]), "+v"(xv[5]), "+v"(xv[6]), "+v"(xv[7])
                     : "v"(ent[0]), "v"(ent[1]), "v"(ent[2]), "v"(ent[3]), "v"(ent[4]), "v"(ent[5]), "v"(ent[6]), "v"(ent[7])
                     : "memory");
      } else {
#pragma unroll
        for (int e = 0; e < kChunk; ++e) {  // the entries are LDS addresses (the workgroup's LDS starts at 0)
          if constexpr (DT == OQ_F32) {
            const uint32_t raw = lds_read_u32(ent[e] & 0x7fffffffu);
            xv[e] = __uint_as_float(raw ^ (ent[e] & 0x80000000u));
          } else {
            xv[e] = f16_bits_to_f32(lds_read_u16(ent[e]));
          }
        }
      }
      if constexpr (EMIT == EMIT_WEIGHT) {
#pragma unroll
        for (int e = 0; e < kChunk; ++e) y[j][e] = xv[e];
      } else if (!plain) {
#pragma unroll
        for (int e = 0; e < kChunk; ++e) y[j][e] = divide_fast(xv[e], rc);
      } else {
#pragma unroll
        for (int e = 0; e < kChunk; ++e) y[j][e] = xv[e] / rc.d;
      }
      rq::fwht_regs<kChunk>(y[j], H);
      if constexpr (H > 8) stage_xor1(y[j], neg1);
      if constexpr (H > 16) stage_xor2(y[j], neg2);
      if constexpr (H > 32) stage_xor4(y[j]);
      if constexpr (H > 64) stage_xor8(y[j]);
      if constexpr (H > 128) rq::swap_stage<16>(y[j]);
      if constexpr (H > 256) rq::swap_stage<32>(y[j]);
    }
    // distances 512 and up: between the steps of the unit, in registers
#pragma unroll
    for (int dist = 1; dist < G; dist <<= 1) {
#pragma unroll
      for (int j = 0; j < G; ++j) {
        if ((j & dist) == 0) {
#pragma unroll
          for (int e = 0; e < kChunk; ++e) {
            const float l = y[j][e], r = y[j + dist][e];
            y[j][e] = l + r;
            y[j + dist][e] = l - r;
          }
        }
      }
    }
    // bucketize against the folded thresholds and emit
#pragma unroll
    for (int j = 0; j < G; ++j) {
      const int c0 = unit_base + j * kLaneSpan + lane_first;  // >= K: an idle lane of the row's last unit
      int code[kChunk];
      if constexpr (EMIT == EMIT_WEIGHT) {
        float unit[kChunk];
#pragma unroll
        for (int e = 0; e < kChunk; ++e) unit[e] = (y[j][e] * a.inv_sqrt_block) / weight_denominator;
        rq::bucketize_many<kChunk>(thr, a.levels_pow2, unit, code);
      } else if (!searched) {
        uint2 ent[kChunk];
#pragma unroll
        for (int e = 0; e < kChunk; ++e) ent[e] = cells[plan::cell_of(y[j][e], cell_scale, cell_offset)];
        count_below(ent, y[j], code);
      } else {
        rq::bucketize_many<kChunk>(thr, a.levels_pow2, y[j], code);
      }
      if (c0 < Ki) {
        if constexpr (EMIT == EMIT_NIBBLE) {
          uint32_t w = static_cast<uint32_t>(code[7]);
#pragma unroll
          for (int e = kChunk - 2; e >= 0; --e) w = (w << 4) | static_cast<uint32_t>(code[e]);  // one shift-or each
          *reinterpret_cast<uint32_t *>(codes_row + static_cast<uint32_t>(c0) / 2u) = w;
        } else if constexpr (EMIT == EMIT_U8) {
          uint2 w;
          w.x = ((((static_cast<uint32_t>(code[3]) << 8) | code[2]) << 8 | code[1]) << 8) | code[0];
          w.y = ((((static_cast<uint32_t>(code[7]) << 8) | code[6]) << 8 | code[5]) << 8) | code[4];
          *reinterpret_cast<uint2 *>(codes_row + static_cast<uint32_t>(c0)) = w;
        } else if constexpr (EMIT == EMIT_WEIGHT) {
          // eight indices = pack_bits whole bytes at a byte boundary of the stream (K is a multiple of 8)
          uint64_t word = 0;
#pragma unroll
          for (int e = 0; e < kChunk; ++e) word |= static_cast<uint64_t>(code[e]) << (a.pack_bits * e);
          uint8_t *dst = a.packed + (row * K + c0) / 8 * a.pack_bits;
#pragma unroll
          for (int b = 0; b < 8; ++b)
            if (b < a.pack_bits) dst[b] = static_cast<uint8_t>(word >> (8 * b));
        } else {
          rq::emit8<DT, true>(a, row, c0, code, cent, s_norm);
        }
      }
    }
  }
}

}  // namespace rqf
}  // namespace oq
