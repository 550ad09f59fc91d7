// Shape-agnostic packed-weight kernels: any K, any bit width 1..8, any dtype.
// They are the correctness net under the tiled MFMA / streaming kernels (odd K,
// unusual widths, fp32 activations) and are not tuned: one wavefront per output
// element column strip, lanes striding K, per-element bit-stream decode.
#include "oq_common.h"

namespace oq {
namespace {

constexpr int kWaves = 4;

struct GenericArgs {
  const void *x;          // float activations [M,K] (x_dtype) or NULL
  int x_dtype;
  const uint8_t *codes;   // activation codes or NULL
  int code_format;
  const float *act_cents; // [a_levels] when codes != NULL
  int a_levels;
  const float *token_scale;  // [M] or NULL
  const uint8_t *packed_w;
  int bits;
  const uint16_t *row_norms;
  const float *w_cents;
  const void *bias;
  int bias_dtype;
  int64_t M, N, K;
  void *out;
  int out_dtype;
};

// grid = (N, min(ceil(M / kWaves), 65535)); block = 64 * kWaves; wave w handles rows blockIdx.y*kWaves + w, + gridDim.y*kWaves, ...
__global__ __launch_bounds__(64 * kWaves) void packed_generic_kernel(GenericArgs a) {
  __shared__ float wc[256];
  __shared__ float ac[256];
  const int t = threadIdx.x;
  wc[t] = (t < (1 << a.bits)) ? a.w_cents[t] : 0.0f;
  ac[t] = (a.codes != nullptr && t < a.a_levels) ? a.act_cents[t] : 0.0f;
  __syncthreads();
  const int lane = t & 63;
  const int64_t n = blockIdx.x;
  const int64_t nbytes = (a.N * a.K * a.bits + 7) / 8;
  // row groups beyond the grid's second dimension are walked by the same workgroups
  for (int64_t m = static_cast<int64_t>(blockIdx.y) * kWaves + (t >> 6); m < a.M; m += static_cast<int64_t>(gridDim.y) * kWaves) {
    float acc = 0.0f;
    for (int64_t k = lane; k < a.K; k += 64) {
      const float w = wc[unpack_index(a.packed_w, n * a.K + k, a.bits, nbytes)];
      float xv;
      if (a.codes != nullptr) {
        uint32_t code;
        if (a.code_format == OQ_CODES_U8) code = a.codes[m * a.K + k];
        else code = (a.codes[m * (a.K / 2) + (k >> 1)] >> ((k & 1) * 4)) & 0xfu;
        xv = ac[code];
      } else {
        xv = load_dyn_f32(a.x, a.x_dtype, m * a.K + k);
      }
      acc = fmaf(xv, w, acc);
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) acc += __shfl_xor(acc, off, 64);
    if (lane == 0) {
      // the same expression as the tiled and streaming kernels: (acc * token factor) * row norm + bias
      float y = a.token_scale != nullptr ? acc * a.token_scale[m] : acc;
      y = y * bf16_bits_to_f32(a.row_norms[n]);
      if (a.bias != nullptr) y += load_dyn_f32(a.bias, a.bias_dtype, n);
      const int64_t o = m * a.N + n;
      if (a.out_dtype == OQ_F32) store_from_f32<OQ_F32>(a.out, o, y);
      else if (a.out_dtype == OQ_F16) store_from_f32<OQ_F16>(a.out, o, y);
      else store_from_f32<OQ_BF16>(a.out, o, y);
    }
  }
}

__global__ __launch_bounds__(256) void unpack_kernel(const uint8_t *packed, int bits, int64_t count,
                                                     int64_t nbytes, uint8_t *out) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
  if (i < count) out[i] = static_cast<uint8_t>(unpack_index(packed, i, bits, nbytes));
}

int launch_generic(const GenericArgs &a, hipStream_t stream) {
  if (a.N > 0x7fffffffLL) return fail(OQ_ERR_UNSUPPORTED, "generic packed kernel: N=%lld exceeds the grid", (long long)a.N);
  const int64_t row_groups = (a.M + kWaves - 1) / kWaves;
  dim3 grid(static_cast<unsigned>(a.N), static_cast<unsigned>(row_groups < 65535 ? row_groups : 65535));
  hipLaunchKernelGGL(packed_generic_kernel, grid, dim3(64 * kWaves), 0, stream, a);
  return check_launch("packed_generic");
}

}  // namespace

int generic_matmul_float(const void *x, int x_dtype, const float *token_scale, const uint8_t *packed_w,
                         int bits, const uint16_t *row_norms, const float *w_cents, const void *bias,
                         int bias_dtype, int64_t M, int64_t N, int64_t K, void *out, int out_dtype,
                         hipStream_t stream) {
  GenericArgs a{};
  a.x = x; a.x_dtype = x_dtype; a.codes = nullptr; a.token_scale = token_scale;
  a.packed_w = packed_w; a.bits = bits; a.row_norms = row_norms; a.w_cents = w_cents;
  a.bias = bias; a.bias_dtype = bias_dtype; a.M = M; a.N = N; a.K = K; a.out = out; a.out_dtype = out_dtype;
  return launch_generic(a, stream);
}

int generic_linear_codes(const void *codes, int code_format, const float *token_norms,
                         const float *act_cents, int a_levels, const uint8_t *packed_w, int bits,
                         const uint16_t *row_norms, const float *w_cents, const void *bias,
                         int bias_dtype, int64_t M, int64_t N, int64_t K, void *out, int out_dtype,
                         hipStream_t stream) {
  GenericArgs a{};
  a.codes = static_cast<const uint8_t *>(codes); a.code_format = code_format; a.act_cents = act_cents; a.a_levels = a_levels;
  a.token_scale = token_norms; a.packed_w = packed_w; a.bits = bits; a.row_norms = row_norms;
  a.w_cents = w_cents; a.bias = bias; a.bias_dtype = bias_dtype; a.M = M; a.N = N; a.K = K;
  a.out = out; a.out_dtype = out_dtype;
  return launch_generic(a, stream);
}

int unpack_dispatch(const uint8_t *packed, int bits, int64_t count, uint8_t *out, hipStream_t stream) {
  if (count == 0) return OQ_OK;
  const int64_t nbytes = (count * bits + 7) / 8;
  const int64_t blocks = (count + 255) / 256;
  if (blocks > 0x7fffffffLL) return fail(OQ_ERR_UNSUPPORTED, "unpack: count too large");
  hipLaunchKernelGGL(unpack_kernel, dim3(static_cast<unsigned>(blocks)), dim3(256), 0, stream, packed, bits,
                     count, nbytes, out);
  return check_launch("unpack_lowbit");
}

// out[i] = table[out[i]] for 16-bit outputs: the output map of the kernels that do not apply it
// themselves (small-M and shape-agnostic paths, whose outputs are small).
__global__ void apply_value_map_kernel(uint16_t *out, int64_t count, const uint16_t *table) {
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < count;
       i += static_cast<int64_t>(gridDim.x) * blockDim.x)
    out[i] = table[out[i]];
}

int apply_value_map(void *out, int64_t count, const uint16_t *table, hipStream_t stream) {
  if (count <= 0) return OQ_OK;
  const int64_t blocks = (count + 255) / 256;
  hipLaunchKernelGGL(apply_value_map_kernel, dim3(static_cast<unsigned>(blocks < 4096 ? blocks : 4096)), dim3(256), 0, stream,
                     static_cast<uint16_t *>(out), count, table);
  return check_launch("apply_value_map");
}

}  // namespace oq
