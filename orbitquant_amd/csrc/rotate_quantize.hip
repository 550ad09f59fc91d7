// Fused RPBH rotate + per-token Lloyd-Max quantize for gfx950.
//
// One 256-thread workgroup per token row.  The row is staged once in LDS as
// fp32 (coalesced 16-byte global loads), the sum of squares is taken in the
// fixed order the C header documents, then every thread gathers eight
// consecutive rotated slots from LDS (permutation), divides by (norm + eps),
// applies the sign and runs the Walsh-Hadamard butterflies:
//   distance 1,2,4        in registers (the thread's own eight values)
//   distance 8 .. 256     across the lanes of the wavefront (lane xor 1 .. 32)
//   distance 512 ..       through LDS, regrouped so the stages are register-local
// Every butterfly output is one fp32 add or subtract of two values of the
// previous stage, so the result does not depend on this schedule.
//
// This file must be compiled without FMA contraction: every fp32 operation
// rounds once, exactly like the CPU statement of the algorithm.
#pragma clang fp contract(off)

#include "oq_common.h"

namespace oq {
namespace {

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
};

template <int DT, bool VEC>
__device__ __forceinline__ void load_chunk(const void *x, int64_t row_base, int64_t i0, int64_t K,
                                           float (&f)[kChunk]) {
  if constexpr (VEC) {
    if (i0 + kChunk <= K) {
      if constexpr (DT == OQ_F32) {
        const float4 *p = reinterpret_cast<const float4 *>(static_cast<const float *>(x) + row_base + i0);
        float4 a = p[0], b = p[1];
        f[0] = a.x; f[1] = a.y; f[2] = a.z; f[3] = a.w;
        f[4] = b.x; f[5] = b.y; f[6] = b.z; f[7] = b.w;
      } else {
        const uint4 raw = *reinterpret_cast<const uint4 *>(static_cast<const uint16_t *>(x) + row_base + i0);
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
  for (int e = 0; e < kChunk; ++e) f[e] = (i0 + e < K) ? load_as_f32<DT>(x, row_base + i0 + e) : 0.0f;
}

__device__ __forceinline__ int bucketize(const float *bnd, int levels_pow2, float v) {
  int code = 0;
  for (int step = levels_pow2 >> 1; step > 0; step >>= 1)
    if (bnd[code + step - 1] < v) code += step;
  return code;
}

// Emit eight consecutive results (slots c0 .. c0+7 of `row`).
template <int DT, bool VEC>
__device__ __forceinline__ void emit8(const RqArgs &a, int64_t row, int64_t c0, const int (&code)[kChunk],
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

template <int DT, bool VEC, int LOG_G>
__global__ __launch_bounds__(kThreads) void rotate_quantize_kernel(RqArgs a) {
  extern __shared__ __align__(16) unsigned char smem[];
  const int t = threadIdx.x;
  const int lane = t & 63;
  const int wave = t >> 6;
  const int64_t row = blockIdx.x;
  const int64_t K = a.K;
  const int Kp = a.passes * kPass;
  float *xbuf = reinterpret_cast<float *>(smem);
  float *bnd = xbuf + Kp;        // 256 floats
  float *cent = bnd + 256;       // 256 floats
  float *red = cent + 256;       // 4 floats (+ pad to 16 B)
  uint8_t *cbuf = reinterpret_cast<uint8_t *>(red + 4);  // Kp bytes, big-block path only

  // tables
  bnd[t] = (t < a.levels - 1) ? a.bounds[t] : __builtin_inff();
  cent[t] = (a.cents != nullptr && t < a.levels) ? a.cents[t] : 0.0f;

  // ---- phase A: stage the row, sum of squares in the documented order --------
  const int64_t row_base = row * K;
  float q = 0.0f;
  for (int p = 0; p < a.passes; ++p) {
    const int64_t i0 = static_cast<int64_t>(p) * kPass + t * kChunk;
    float f[kChunk];
    load_chunk<DT, VEC>(a.x, row_base, i0, K, f);
    float4 *dst = reinterpret_cast<float4 *>(xbuf + i0);
    dst[0] = make_float4(f[0], f[1], f[2], f[3]);
    dst[1] = make_float4(f[4], f[5], f[6], f[7]);
    float s[kChunk];
#pragma unroll
    for (int e = 0; e < kChunk; ++e) s[e] = f[e] * f[e];
    const float v8 = ((s[0] + s[1]) + (s[2] + s[3])) + ((s[4] + s[5]) + (s[6] + s[7]));
    q = (p == 0) ? v8 : q + v8;
  }
#pragma unroll
  for (int off = 1; off < 64; off <<= 1) q = q + __shfl_xor(q, off, 64);
  if (lane == 0) red[wave] = q;
  __syncthreads();
  const float total = (red[0] + red[1]) + (red[2] + red[3]);
  const float s_norm = sqrtf(total);  // IEEE-rounded (hipcc's default for fp32 sqrt and division)
  const float denom = s_norm + a.eps;
  if (t == 0 && a.norms != nullptr) a.norms[row] = s_norm;

  // ---- phase B: gather, divide, sign, butterflies up to distance 256 ----------
  const int h = a.block;
  constexpr bool BIG = LOG_G > 0;
  float keep[BIG ? kMaxPasses : 1][kChunk];

#pragma unroll
  for (int p = 0; p < kMaxPasses; ++p) {
    if (p < a.passes) {
      const int64_t c0 = static_cast<int64_t>(p) * kPass + t * kChunk;
      float y[kChunk];
      if (VEC && c0 + kChunk <= K) {
        const int4 pa = *reinterpret_cast<const int4 *>(a.perm + c0);
        const int4 pb = *reinterpret_cast<const int4 *>(a.perm + c0 + 4);
        const int idx[kChunk] = {pa.x, pa.y, pa.z, pa.w, pb.x, pb.y, pb.z, pb.w};
        const uint2 sg = *reinterpret_cast<const uint2 *>(a.signs + c0);
#pragma unroll
        for (int e = 0; e < kChunk; ++e) {
          const uint32_t sw = e < 4 ? sg.x : sg.y;
          const float sign = static_cast<float>(static_cast<int8_t>((sw >> (8 * (e & 3))) & 0xff));
          y[e] = (xbuf[idx[e]] / denom) * sign;
        }
      } else {
#pragma unroll
        for (int e = 0; e < kChunk; ++e) {
          if (c0 + e < K) y[e] = (xbuf[a.perm[c0 + e]] / denom) * static_cast<float>(a.signs[c0 + e]);
          else y[e] = 0.0f;
        }
      }
      fwht_regs<kChunk>(y, h);
#pragma unroll
      for (int j = 1; j < 64; j <<= 1) {
        if (j * kChunk < h) {
          const bool upper = (lane & j) != 0;
#pragma unroll
          for (int e = 0; e < kChunk; ++e) {
            const float other = __shfl_xor(y[e], j, 64);
            y[e] = upper ? other - y[e] : y[e] + other;
          }
        }
      }
      if constexpr (!BIG) {
        int code[kChunk];
#pragma unroll
        for (int e = 0; e < kChunk; ++e) code[e] = bucketize(bnd, a.levels_pow2, y[e] * a.inv_sqrt_block);
        if (c0 < K) emit8<DT, VEC>(a, row, c0, code, cent, s_norm);
      } else {
#pragma unroll
        for (int e = 0; e < kChunk; ++e) keep[p][e] = y[e];
      }
    }
  }

  if constexpr (BIG) {
    // ---- phase C: distances 512 .. block/2 through LDS --------------------------
    __syncthreads();  // every gather has read xbuf
#pragma unroll
    for (int p = 0; p < kMaxPasses; ++p) {
      if (p < a.passes) {
        float4 *dst = reinterpret_cast<float4 *>(xbuf + static_cast<int64_t>(p) * kPass + t * kChunk);
        dst[0] = make_float4(keep[p][0], keep[p][1], keep[p][2], keep[p][3]);
        dst[1] = make_float4(keep[p][4], keep[p][5], keep[p][6], keep[p][7]);
      }
    }
    __syncthreads();
    constexpr int G = 1 << LOG_G;  // block / 512
    const int groups = static_cast<int>(K >> LOG_G);
    for (int gi = t; gi < groups; gi += kThreads) {
      const int base = (gi >> 9) * h + (gi & (kLaneSpan - 1));
      float z[G];
#pragma unroll
      for (int v = 0; v < G; ++v) z[v] = xbuf[base + kLaneSpan * v];
      fwht_regs<G>(z, G);
#pragma unroll
      for (int v = 0; v < G; ++v)
        cbuf[base + kLaneSpan * v] = static_cast<uint8_t>(bucketize(bnd, a.levels_pow2, z[v] * a.inv_sqrt_block));
    }
    __syncthreads();
    for (int64_t c0 = t * kChunk; c0 < K; c0 += kPass) {
      const uint2 w = *reinterpret_cast<const uint2 *>(cbuf + c0);
      int code[kChunk];
#pragma unroll
      for (int e = 0; e < kChunk; ++e) code[e] = ((e < 4 ? w.x : w.y) >> (8 * (e & 3))) & 0xff;
      emit8<DT, VEC>(a, row, c0, code, cent, s_norm);
    }
  }
}

template <int DT, bool VEC>
int launch_for_block(const RqArgs &a, size_t smem, hipStream_t stream) {
  int log_g = 0;
  for (int g = a.block / kLaneSpan; g > 1; g >>= 1) ++log_g;
  dim3 grid(static_cast<unsigned>(a.M)), block(kThreads);
#define OQ_RQ_CASE(LG)                                                                           \
  case LG: {                                                                                     \
    auto kern = rotate_quantize_kernel<DT, VEC, LG>;                                             \
    if (smem > 48 * 1024) {                                                                      \
      if (hipFuncSetAttribute(reinterpret_cast<const void *>(kern),                              \
                              hipFuncAttributeMaxDynamicSharedMemorySize,                        \
                              static_cast<int>(smem)) != hipSuccess)                            \
        return fail(OQ_ERR_LAUNCH, "rotate_quantize: cannot reserve %zu bytes of LDS", smem);    \
    }                                                                                            \
    hipLaunchKernelGGL(kern, grid, block, smem, stream, a);                                      \
    break;                                                                                       \
  }
  switch (log_g) {
    OQ_RQ_CASE(0)
    OQ_RQ_CASE(1)
    OQ_RQ_CASE(2)
    OQ_RQ_CASE(3)
    OQ_RQ_CASE(4)
    OQ_RQ_CASE(5)
    default:
      return fail(OQ_ERR_UNSUPPORTED, "rotate_quantize: block %d is larger than 16384", a.block);
  }
#undef OQ_RQ_CASE
  return check_launch("rotate_quantize");
}

}  // namespace

int rotate_quantize_dispatch(const void *x, int x_dtype, int64_t M, int64_t K, const int32_t *perm,
                             const int8_t *signs, const float *boundaries, const float *centroids,
                             int levels, int64_t block, float eps, float inv_sqrt_block,
                             void *codes_out, int code_format, void *values_out, int values_mode,
                             float *norms_out, hipStream_t stream) {
  if (M < 0 || K <= 0) return fail(OQ_ERR_INVALID, "rotate_quantize: M=%lld K=%lld", (long long)M, (long long)K);
  if (M == 0) return OQ_OK;
  if (x == nullptr || perm == nullptr || signs == nullptr || boundaries == nullptr)
    return fail(OQ_ERR_INVALID, "rotate_quantize: null input pointer");
  if (levels < 2 || levels > 256) return fail(OQ_ERR_INVALID, "rotate_quantize: levels=%d not in [2, 256]", levels);
  if (block <= 0 || (block & (block - 1)) != 0 || K % block != 0)
    return fail(OQ_ERR_INVALID, "rotate_quantize: block=%lld must be a power of two dividing K=%lld",
                (long long)block, (long long)K);
  if (K > static_cast<int64_t>(kMaxPasses) * kPass)
    return fail(OQ_ERR_UNSUPPORTED, "rotate_quantize: K=%lld exceeds %d", (long long)K, kMaxPasses * kPass);
  if (M > 0x7fffffffLL) return fail(OQ_ERR_UNSUPPORTED, "rotate_quantize: M=%lld exceeds the grid limit", (long long)M);
  if (codes_out != nullptr) {
    if (code_format != OQ_CODES_U8 && code_format != OQ_CODES_NIBBLE)
      return fail(OQ_ERR_INVALID, "rotate_quantize: unknown code_format %d", code_format);
    if (code_format == OQ_CODES_NIBBLE && (levels > 16 || (K & 1)))
      return fail(OQ_ERR_INVALID, "rotate_quantize: nibble codes need levels <= 16 and even K");
  }
  if (values_mode != OQ_VALUES_NONE) {
    if (values_mode != OQ_VALUES_SCALED && values_mode != OQ_VALUES_UNIT_BF16)
      return fail(OQ_ERR_INVALID, "rotate_quantize: unknown values_mode %d", values_mode);
    if (values_out == nullptr || centroids == nullptr)
      return fail(OQ_ERR_INVALID, "rotate_quantize: values_mode set but values_out/centroids is null");
  }

  RqArgs a;
  a.x = x; a.M = M; a.K = K; a.perm = perm; a.signs = signs; a.bounds = boundaries;
  a.cents = centroids; a.levels = levels;
  a.levels_pow2 = 2;
  while (a.levels_pow2 < levels) a.levels_pow2 <<= 1;
  a.block = static_cast<int>(block);
  a.passes = static_cast<int>((K + kPass - 1) / kPass);
  a.eps = eps; a.inv_sqrt_block = inv_sqrt_block;
  a.codes = static_cast<uint8_t *>(codes_out); a.code_format = code_format;
  a.values = values_mode == OQ_VALUES_NONE ? nullptr : values_out; a.values_mode = values_mode;
  a.norms = norms_out;

  const size_t kp = static_cast<size_t>(a.passes) * kPass;
  const bool big = block > kLaneSpan;
  const size_t smem = kp * sizeof(float) + (256 + 256 + 4) * sizeof(float) + (big ? kp : 0);

  auto aligned16 = [](const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; };
  const bool vec = (K % 8 == 0) && aligned16(x) && aligned16(perm) && aligned16(signs) &&
                   (codes_out == nullptr || aligned16(codes_out)) &&
                   (values_out == nullptr || aligned16(values_out));
  switch (x_dtype) {
    case OQ_F32: return vec ? launch_for_block<OQ_F32, true>(a, smem, stream) : launch_for_block<OQ_F32, false>(a, smem, stream);
    case OQ_F16: return vec ? launch_for_block<OQ_F16, true>(a, smem, stream) : launch_for_block<OQ_F16, false>(a, smem, stream);
    case OQ_BF16: return vec ? launch_for_block<OQ_BF16, true>(a, smem, stream) : launch_for_block<OQ_BF16, false>(a, smem, stream);
    default: return fail(OQ_ERR_INVALID, "rotate_quantize: unknown x_dtype %d", x_dtype);
  }
}

}  // namespace oq
