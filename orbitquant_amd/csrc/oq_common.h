// Shared host/device helpers for the gfx950 quantized-linear kernels.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/orbitquant_hip.h"

namespace oq {

// ---- error plumbing (host) -------------------------------------------------
void set_error(const char *fmt, ...);
int fail(oq_status code, const char *fmt, ...);
int check_launch(const char *what);
// Dynamic LDS above 48 KB has to be granted per kernel: asks the runtime the first time a
// (kernel, device) pair needs `bytes` or more than it was granted before, and answers from a
// small table afterwards.  False if the runtime refuses.
bool reserve_dynamic_lds(const void *kernel, size_t bytes);
// Experiment switches (environment variables) are read once per process, at first use.
const char *debug_env(int which);
enum DebugEnv { ENV_GEMM_TILE = 0, ENV_NO_TOKEN_LINEAR, ENV_RQ_ONE_GROUP, ENV_GEMV_CFG, ENV_RQ_WAVES, ENV_RQ_FAST_MIN_M, ENV_NO_GEMV_GROUP, ENV_GEMV_GROUP_R, ENV_GEMV_NO_ASTAGE, ENV_GEMV_MAX_M, ENV_GEMM_WG_SPLIT, ENV_FLOAT_GEMM_MIN_M, ENV_GEMM_STAMPS, ENV_COUNT };

inline hipStream_t as_stream(void *s) { return reinterpret_cast<hipStream_t>(s); }

// ---- dtype helpers (device) --------------------------------------------------
__device__ __forceinline__ float bf16_bits_to_f32(uint16_t b) {
  return __uint_as_float(static_cast<uint32_t>(b) << 16);
}

// round-to-nearest-even fp32 -> bf16 bits (the gfx950 conversion instruction)
__device__ __forceinline__ uint16_t f32_to_bf16_bits(float f) {
  return __builtin_bit_cast(uint16_t, static_cast<__bf16>(f));
}

__device__ __forceinline__ float f16_bits_to_f32(uint16_t b) {
  return static_cast<float>(__builtin_bit_cast(_Float16, b));
}

__device__ __forceinline__ uint16_t f32_to_f16_bits(float f) {
  return __builtin_bit_cast(uint16_t, static_cast<_Float16>(f));
}

template <int DT>
__device__ __forceinline__ float load_as_f32(const void *p, int64_t i) {
  if constexpr (DT == OQ_F32) return static_cast<const float *>(p)[i];
  else if constexpr (DT == OQ_F16) return f16_bits_to_f32(static_cast<const uint16_t *>(p)[i]);
  else return bf16_bits_to_f32(static_cast<const uint16_t *>(p)[i]);
}

template <int DT>
__device__ __forceinline__ void store_from_f32(void *p, int64_t i, float v) {
  if constexpr (DT == OQ_F32) static_cast<float *>(p)[i] = v;
  else if constexpr (DT == OQ_F16) static_cast<uint16_t *>(p)[i] = f32_to_f16_bits(v);
  else static_cast<uint16_t *>(p)[i] = f32_to_bf16_bits(v);
}

__device__ __forceinline__ float load_dyn_f32(const void *p, int dt, int64_t i) {
  if (dt == OQ_F32) return load_as_f32<OQ_F32>(p, i);
  if (dt == OQ_F16) return load_as_f32<OQ_F16>(p, i);
  return load_as_f32<OQ_BF16>(p, i);
}

// Conversion of a value loaded as raw bits (a 16-bit pattern in the low half), for kernels that
// request a value long before they use it.
__device__ __forceinline__ float dyn_bits_to_f32(uint32_t b, int dt) {
  if (dt == OQ_F32) return __builtin_bit_cast(float, b);
  if (dt == OQ_F16) return f16_bits_to_f32(static_cast<uint16_t>(b));
  return bf16_bits_to_f32(static_cast<uint16_t>(b));
}

__host__ __device__ inline int dtype_size(int dt) { return dt == OQ_F32 ? 4 : 2; }

// index `v` of a little-endian bit stream, `bits` wide (1..8)
__device__ __forceinline__ uint32_t unpack_index(const uint8_t *packed, int64_t v, int bits,
                                                 int64_t nbytes) {
  const int64_t bit = v * bits;
  const int64_t byte = bit >> 3;
  const uint32_t sh = static_cast<uint32_t>(bit & 7);
  uint32_t w = packed[byte];
  if (sh + bits > 8 && byte + 1 < nbytes) w |= static_cast<uint32_t>(packed[byte + 1]) << 8;
  return (w >> sh) & ((1u << bits) - 1u);
}

}  // namespace oq
