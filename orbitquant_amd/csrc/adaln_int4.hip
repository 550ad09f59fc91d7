// Packed INT4 group-scaled linear on bf16 activations: the AdaLN modulation linears of a DiT
// block, which the reference keeps out of the codebook path and quantizes round-to-nearest
// (src/orbitquant/adaln.py:17-35,319-425; kernels src/orbitquant/kernels/triton_cuda.py:682-819 and
// native-kernels/orbitquant-packed-matmul/orbitquant_packed_matmul_cpu/cpu_msvc_avx2.cpp:179-236):
//
//   w[n,k]   = bf16( (q[n,k] - 8) * float(scale[n, k / group]) )      q: 4-bit, two per byte, low nibble first,
//   out[m,n] = bf16( sum_k x[m,k] * w[n,k] + float(bias[n]) )         rows padded to whole groups in the stream
//
// Few tokens (the modulation input is one vector per sample), so the launch is a stream over the
// packed weights: a wavefront owns sixteen output rows for all of K, the tokens are the other
// side of v_mfma_f32_16x16x32_bf16 in blocks of sixteen, fp32 accumulation.
#include "oq_common.h"

namespace oq {
namespace {

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));

struct AdalnArgs {
  const uint16_t *x;       // bf16 [M, K]
  const uint8_t *packed;   // [N, padded_K / 2]
  const uint16_t *scales;  // bf16 [N, groups]
  const uint16_t *bias;    // bf16 [N] or NULL
  uint16_t *out;           // bf16 [M, N]
  int64_t M, N, K;
  int group, groups;       // values per scale, scales per row; padded_K = group * groups
};

// eight nibbles -> eight bf16 weights (as four dwords)
__device__ __forceinline__ uint4 decode8(uint32_t q, float scale) {
  uint32_t w[4];
#pragma unroll
  for (int p = 0; p < 4; ++p) {
    const float lo = static_cast<float>(static_cast<int>((q >> (8 * p)) & 15u) - 8) * scale;
    const float hi = static_cast<float>(static_cast<int>((q >> (8 * p + 4)) & 15u) - 8) * scale;
    w[p] = static_cast<uint32_t>(f32_to_bf16_bits(lo)) | (static_cast<uint32_t>(f32_to_bf16_bits(hi)) << 16);
  }
  return make_uint4(w[0], w[1], w[2], w[3]);
}

// K a multiple of 8, group a multiple of 8, x 16-byte aligned.
__global__ __launch_bounds__(256) void adaln_int4_mfma_kernel(AdalnArgs a) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int r = lane & 15, g = lane >> 4;
  const int64_t n = (static_cast<int64_t>(blockIdx.x) * 4 + wave) * 16 + r;
  const int64_t nc = min(n, a.N - 1);
  const int64_t row_bytes = static_cast<int64_t>(a.group) * a.groups / 2;
  const uint8_t *wrow = a.packed + nc * row_bytes;
  const uint16_t *srow = a.scales + nc * a.groups;
  const float bias = a.bias != nullptr ? bf16_bits_to_f32(a.bias[nc]) : 0.0f;
  for (int64_t m0 = 0; m0 < a.M; m0 += 16) {
    const int64_t m = m0 + r;  // the token whose values this lane feeds
    const uint16_t *xrow = a.x + min(m, a.M - 1) * a.K;
    f32x4 acc = {0.0f, 0.0f, 0.0f, 0.0f};
    for (int64_t k0 = 0; k0 < a.K; k0 += 32) {
      const int64_t k = k0 + 8 * g;
      uint4 xa = make_uint4(0u, 0u, 0u, 0u), wb = xa;
      if (k < a.K) {  // K is a multiple of 8: the eight values are all inside or all outside
        if (m < a.M) xa = *reinterpret_cast<const uint4 *>(xrow + k);
        const uint32_t q = *reinterpret_cast<const uint32_t *>(wrow + k / 2);
        wb = decode8(q, bf16_bits_to_f32(srow[k / a.group]));
      }
      acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, xa), __builtin_bit_cast(bf16x8, wb), acc, 0, 0, 0);
    }
    // accumulator e of lane l: token 4 * (l / 16) + e, output row l % 16
    if (n < a.N) {
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const int64_t mt = m0 + 4 * g + e;
        if (mt < a.M) a.out[mt * a.N + n] = f32_to_bf16_bits(acc[e] + bias);
      }
    }
  }
}

// The same linear as a stream in K-steps of 128: a workgroup owns sixteen output rows, its four wavefronts
// a quarter of the K-steps each; lane (r, g) loads the sixteen bytes that hold values 32g .. 32g+31 of its
// row's step (one load per lane and step instead of one dword per 32 values), the step after the one being
// multiplied is already requested, and the four partial tiles are added through LDS in wavefront order.
// (One wavefront walking all of K with one dword per lane and step is a chain of K / 32 dependent memory
// round trips: 13 us for the 1152 -> 6912 modulation linear of DiT-XL/2, a 4 MB matrix.)
// K a multiple of 8, group a multiple of 32, x and the packed rows 16-byte aligned.
__global__ __launch_bounds__(256) void adaln_int4_stream_kernel(AdalnArgs a) {
  __shared__ float part[4][64][4];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int r = lane & 15, g = lane >> 4;
  const int64_t n = static_cast<int64_t>(blockIdx.x) * 16 + r;
  const int64_t nc = min(n, a.N - 1);
  const int padded = a.group * a.groups;                 // values per row of the stream (K rounded up to whole groups)
  const int Ki = static_cast<int>(a.K);
  const uint8_t *wrow = a.packed + nc * (padded / 2);
  const uint16_t *srow = a.scales + nc * a.groups;
  const uint32_t bias_bits = a.bias != nullptr ? a.bias[nc] : 0u;
  const int steps = (Ki + 127) / 128;
  const int s_begin = steps * wave / 4, s_end = steps * (wave + 1) / 4;
  struct Step {
    uint4 w;
    uint32_t scale_bits;
    uint4 x[4];
  };
  for (int64_t m0 = 0; m0 < a.M; m0 += 16) {
    const int64_t m = m0 + r;  // the token whose values this lane feeds
    const uint16_t *xrow = a.x + min(m, a.M - 1) * a.K;
    // branch-free requests: clamped addresses, what lies past the row is zeroed when it is used
    auto fetch = [&](int s, Step &st) {
      const int k = 128 * min(s, steps - 1) + 32 * g;
      const int kw = min(k, padded - 32);
      st.w = *reinterpret_cast<const uint4 *>(wrow + kw / 2);
      st.scale_bits = srow[kw / a.group];
#pragma unroll
      for (int q = 0; q < 4; ++q) st.x[q] = *reinterpret_cast<const uint4 *>(xrow + min(k + 8 * q, Ki - 8));
    };
    f32x4 acc = {0.0f, 0.0f, 0.0f, 0.0f};
    auto multiply = [&](int s, const Step &st) {
      const int k = 128 * s + 32 * g;
      const float scale = bf16_bits_to_f32(static_cast<uint16_t>(st.scale_bits));
      const uint32_t wq[4] = {st.w.x, st.w.y, st.w.z, st.w.w};
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const bool live = k + 8 * q < Ki && m < a.M;   // K is a multiple of 8: eight values are all inside or all outside
        const uint4 xa = live ? st.x[q] : make_uint4(0u, 0u, 0u, 0u);
        const uint4 wb = decode8(k + 8 * q < padded ? wq[q] : 0x88888888u, scale);
        acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, xa), __builtin_bit_cast(bf16x8, wb), acc, 0, 0, 0);
      }
    };
    Step cur, next;
    if (s_begin < s_end) {
      fetch(s_begin, cur);
      for (int s = s_begin; s < s_end; ++s) {
        fetch(s + 1 < s_end ? s + 1 : s, next);   // (the last step asks for itself again: the caches hold it)
        multiply(s, cur);
        cur = next;
      }
    }
    *reinterpret_cast<float4 *>(&part[wave][lane][0]) = make_float4(acc[0], acc[1], acc[2], acc[3]);
    __syncthreads();
    // accumulator e of lane l: token 4 * (l / 16) + e, output row l % 16; wavefront 0 adds the four parts in order
    if (wave == 0 && n < a.N) {
      const float bias = a.bias != nullptr ? bf16_bits_to_f32(static_cast<uint16_t>(bias_bits)) : 0.0f;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const float sum = ((part[0][lane][e] + part[1][lane][e]) + part[2][lane][e]) + part[3][lane][e];
        const int64_t mt = m0 + 4 * g + e;
        if (mt < a.M) a.out[mt * a.N + n] = f32_to_bf16_bits(sum + bias);
      }
    }
    __syncthreads();
  }
}

// Any K, any group size, any alignment: one wavefront per (output row, token), lanes stride K.
__global__ __launch_bounds__(256) void adaln_int4_generic_kernel(AdalnArgs a) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int64_t n = blockIdx.x;
  const int64_t padded = static_cast<int64_t>(a.group) * a.groups;
  for (int64_t m = static_cast<int64_t>(blockIdx.y) * 4 + wave; m < a.M; m += static_cast<int64_t>(gridDim.y) * 4) {
    float acc = 0.0f;
    for (int64_t k = lane; k < a.K; k += 64) {
      const int64_t flat = n * padded + k;
      const uint32_t byte = a.packed[flat >> 1];
      const int q = static_cast<int>((flat & 1) ? (byte >> 4) : (byte & 15u)) - 8;
      const float w = bf16_bits_to_f32(f32_to_bf16_bits(static_cast<float>(q) * bf16_bits_to_f32(a.scales[n * a.groups + k / a.group])));
      acc = fmaf(bf16_bits_to_f32(a.x[m * a.K + k]), w, acc);
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) acc += __shfl_xor(acc, off, 64);
    if (lane == 0) a.out[m * a.N + n] = f32_to_bf16_bits(acc + (a.bias != nullptr ? bf16_bits_to_f32(a.bias[n]) : 0.0f));
  }
}


// The weight side (src/orbitquant/adaln.py:17-35 of the reference): a wavefront per (row, group):
// scale = max(absmax, 1e-12) / 7, code = clamp(round_half_even(w / scale), -8, 7) + 8, both IEEE
// fp32 operations (the division is the correctly rounded one), two codes per byte.  group even.
struct AdalnQuantArgs {
  const void *w;
  int w_dtype;
  int64_t N, K;
  int group, groups;
  uint8_t *packed;  // [N * groups * group / 2]
  float *scales;    // [N, groups]
};

__global__ __launch_bounds__(256) void adaln_quantize_kernel(AdalnQuantArgs a) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int64_t pairs = a.N * a.groups;
  for (int64_t pair = static_cast<int64_t>(blockIdx.x) * 4 + wave; pair < pairs; pair += static_cast<int64_t>(gridDim.x) * 4) {
    const int64_t n = pair / a.groups;
    const int g = static_cast<int>(pair - n * a.groups);
    const int64_t k0 = static_cast<int64_t>(g) * a.group;
    float top = 0.0f;
    for (int e = lane; e < a.group; e += 64) {
      const int64_t k = k0 + e;
      if (k < a.K) top = fmaxf(top, fabsf(load_dyn_f32(a.w, a.w_dtype, n * a.K + k)));
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) top = fmaxf(top, __shfl_xor(top, off, 64));
    const float scale = fmaxf(top, 1e-12f) / 7.0f;
    if (lane == 0) a.scales[pair] = scale;
    for (int e = 2 * lane; e < a.group; e += 128) {
      uint32_t byte = 0;
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        const int64_t k = k0 + e + h;
        const float v = k < a.K ? load_dyn_f32(a.w, a.w_dtype, n * a.K + k) : 0.0f;
        const float q = fminf(fmaxf(rintf(v / scale), -8.0f), 7.0f);
        byte |= static_cast<uint32_t>(static_cast<int>(q) + 8) << (4 * h);
      }
      a.packed[(pair * a.group + e) >> 1] = static_cast<uint8_t>(byte);
    }
  }
}

}  // namespace

int adaln_int4_dispatch(const uint16_t *x, const uint8_t *packed, const uint16_t *scales, const uint16_t *bias, int64_t M,
                        int64_t N, int64_t K, int64_t group, uint16_t *out, hipStream_t stream) {
  if (M < 0 || N <= 0 || K <= 0 || group <= 0) return fail(OQ_ERR_INVALID, "adaln_int4: M=%lld N=%lld K=%lld group=%lld", (long long)M, (long long)N, (long long)K, (long long)group);
  if (x == nullptr || packed == nullptr || scales == nullptr || (out == nullptr && M > 0)) return fail(OQ_ERR_INVALID, "adaln_int4: null pointer");
  if (M == 0) return OQ_OK;
  if (N > 0x7fffffffLL || group > 0x7fffffffLL || K > 0x7fffffffLL) return fail(OQ_ERR_UNSUPPORTED, "adaln_int4: shape exceeds the grid");
  AdalnArgs a{};
  a.x = x; a.packed = packed; a.scales = scales; a.bias = bias; a.out = out;
  a.M = M; a.N = N; a.K = K; a.group = static_cast<int>(group); a.groups = static_cast<int>((K + group - 1) / group);
  const bool fast = K % 8 == 0 && group % 8 == 0 && (reinterpret_cast<uintptr_t>(x) & 15u) == 0 &&
                    (reinterpret_cast<uintptr_t>(packed) & 3u) == 0;
  const bool stream_form = fast && group % 32 == 0 && K >= 32 && (reinterpret_cast<uintptr_t>(packed) & 15u) == 0 &&
                           (static_cast<int64_t>(a.group) * a.groups / 2) % 16 == 0;
  if (stream_form) {
    hipLaunchKernelGGL(adaln_int4_stream_kernel, dim3(static_cast<unsigned>((N + 15) / 16)), dim3(256), 0, stream, a);
  } else if (fast) {
    const int64_t blocks = (N + 63) / 64;
    hipLaunchKernelGGL(adaln_int4_mfma_kernel, dim3(static_cast<unsigned>(blocks)), dim3(256), 0, stream, a);
  } else {
    const int64_t row_groups = (M + 3) / 4;
    hipLaunchKernelGGL(adaln_int4_generic_kernel, dim3(static_cast<unsigned>(N), static_cast<unsigned>(row_groups < 65535 ? row_groups : 65535)),
                       dim3(256), 0, stream, a);
  }
  return check_launch("adaln_int4");
}

int adaln_quantize_dispatch(const void *w, int w_dtype, int64_t N, int64_t K, int64_t group, uint8_t *packed, float *scales,
                            hipStream_t stream) {
  if (N <= 0 || K <= 0 || group <= 0 || w == nullptr || packed == nullptr || scales == nullptr)
    return fail(OQ_ERR_INVALID, "adaln_quantize: N=%lld K=%lld group=%lld or a null pointer", (long long)N, (long long)K, (long long)group);
  if (w_dtype != OQ_F32 && w_dtype != OQ_F16 && w_dtype != OQ_BF16) return fail(OQ_ERR_INVALID, "adaln_quantize: w_dtype=%d", w_dtype);
  if (group % 2 != 0 || group > 0x7fffffffLL || K > 0x7fffffffLL) return fail(OQ_ERR_UNSUPPORTED, "adaln_quantize: group=%lld (even group sizes only)", (long long)group);
  AdalnQuantArgs a{};
  a.w = w; a.w_dtype = w_dtype; a.N = N; a.K = K; a.group = static_cast<int>(group); a.groups = static_cast<int>((K + group - 1) / group);
  a.packed = packed; a.scales = scales;
  const int64_t blocks = (N * a.groups + 3) / 4;
  hipLaunchKernelGGL(adaln_quantize_kernel, dim3(static_cast<unsigned>(blocks < 65536 ? blocks : 65536)), dim3(256), 0, stream, a);
  return check_launch("adaln_quantize");
}

}  // namespace oq
