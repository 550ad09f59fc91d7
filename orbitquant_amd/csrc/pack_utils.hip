// The bit-stream utilities of the weight format on the GPU: pack a stream of indices, and expand a
// packed weight to its dense (rotated-basis) values, centroid[index] * row_norm.  The reference has
// them as Triton kernels for its `dequant_bf16` debug mode (src/orbitquant/kernels/triton_cuda.py:523-547
// dequantize, 878-899 pack); the format is src/orbitquant/packing/lowbit.py: index i occupies bits
// [i * bits, (i + 1) * bits) of a little-endian stream, so eight indices fill exactly `bits` bytes.
// Both kernels are streams: a lane owns eight indices, i.e. `bits` whole bytes of the stream.
#include "oq_common.h"

namespace oq {
namespace {

__global__ __launch_bounds__(256) void pack_lowbit_kernel(const uint8_t *values, int bits, int64_t count, uint8_t *packed,
                                                          int64_t nbytes) {
  const uint64_t mask = (1ull << bits) - 1ull;
  const int64_t groups = (count + 7) / 8;
  for (int64_t g = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x; g < groups; g += static_cast<int64_t>(gridDim.x) * 256) {
    const int64_t first = g * 8;
    uint64_t word = 0;
#pragma unroll
    for (int i = 0; i < 8; ++i)
      if (first + i < count) word |= (static_cast<uint64_t>(values[first + i]) & mask) << (i * bits);
    const int64_t byte0 = g * bits;
    for (int b = 0; b < bits; ++b)
      if (byte0 + b < nbytes) packed[byte0 + b] = static_cast<uint8_t>(word >> (8 * b));
  }
}

template <int OUT>
__global__ __launch_bounds__(256) void dequantize_kernel(const uint8_t *packed, int bits, const uint16_t *row_norms,
                                                         const float *centroids, int64_t total, int64_t K, int64_t nbytes,
                                                         void *out) {
  const uint32_t mask = (1u << bits) - 1u;
  const int64_t groups = (total + 7) / 8;
  for (int64_t g = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x; g < groups; g += static_cast<int64_t>(gridDim.x) * 256) {
    const int64_t first = g * 8, byte0 = g * bits;
    uint64_t word = 0;
    for (int b = 0; b < bits; ++b)
      if (byte0 + b < nbytes) word |= static_cast<uint64_t>(packed[byte0 + b]) << (8 * b);
    int64_t row = first / K;
    int64_t row_end = (row + 1) * K;
    float norm = bf16_bits_to_f32(row_norms[row]);
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int64_t e = first + i;
      if (e >= total) break;
      while (e >= row_end) {  // K < 8: a group can span several rows
        ++row;
        row_end += K;
        norm = bf16_bits_to_f32(row_norms[row]);
      }
      const uint32_t idx = static_cast<uint32_t>(word >> (i * bits)) & mask;
      store_from_f32<OUT>(out, e, centroids[idx] * norm);
    }
  }
}

unsigned stream_blocks(int64_t groups) {
  const int64_t blocks = (groups + 255) / 256;
  return static_cast<unsigned>(blocks < 65536 ? (blocks > 0 ? blocks : 1) : 65536);
}

}  // namespace

int pack_lowbit_dispatch(const uint8_t *values, int bits, int64_t count, uint8_t *packed, hipStream_t stream) {
  if (count == 0) return OQ_OK;
  const int64_t nbytes = (count * bits + 7) / 8;
  hipLaunchKernelGGL(pack_lowbit_kernel, dim3(stream_blocks((count + 7) / 8)), dim3(256), 0, stream, values, bits, count, packed, nbytes);
  return check_launch("pack_lowbit");
}

int dequantize_dispatch(const uint8_t *packed, int bits, const uint16_t *row_norms, const float *centroids, int64_t N, int64_t K,
                        void *out, int out_dtype, hipStream_t stream) {
  const int64_t total = N * K;
  if (total == 0) return OQ_OK;
  const int64_t nbytes = (total * bits + 7) / 8;
  const dim3 grid(stream_blocks((total + 7) / 8));
  if (out_dtype == OQ_F32)
    hipLaunchKernelGGL(dequantize_kernel<OQ_F32>, grid, dim3(256), 0, stream, packed, bits, row_norms, centroids, total, K, nbytes, out);
  else if (out_dtype == OQ_F16)
    hipLaunchKernelGGL(dequantize_kernel<OQ_F16>, grid, dim3(256), 0, stream, packed, bits, row_norms, centroids, total, K, nbytes, out);
  else
    hipLaunchKernelGGL(dequantize_kernel<OQ_BF16>, grid, dim3(256), 0, stream, packed, bits, row_norms, centroids, total, K, nbytes, out);
  return check_launch("dequantize_packed_weight");
}

}  // namespace oq
