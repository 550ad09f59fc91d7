// extern "C" entry points: argument validation and kernel selection.
#include <stdarg.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <map>
#include <mutex>
#include <utility>

#include "gemm_epilogue.h"

namespace oq {

static thread_local char g_error[512] = "";

void set_error(const char *fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
}

int fail(oq_status code, const char *fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
  return static_cast<int>(code);
}

int check_launch(const char *what) {
  const hipError_t err = hipGetLastError();
  if (err != hipSuccess) return fail(OQ_ERR_LAUNCH, "%s: %s", what, hipGetErrorString(err));
  return OQ_OK;
}

bool reserve_dynamic_lds(const void *kernel, size_t bytes) {
  if (bytes <= 48 * 1024) return true;
  static std::mutex lock;
  static std::map<std::pair<const void *, int>, size_t> granted;
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) return false;
  std::lock_guard<std::mutex> guard(lock);
  size_t &have = granted[std::make_pair(kernel, dev)];
  if (bytes <= have) return true;
  if (hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(bytes)) != hipSuccess) return false;
  have = bytes;
  return true;
}

namespace {
const char *const kEnvNames[ENV_COUNT] = {"OQ_GEMM_TILE", "OQ_NO_TOKEN_LINEAR", "OQ_RQ_ONE_GROUP", "OQ_GEMV_CFG", "OQ_RQ_WAVES",
                                          "OQ_RQ_FAST_MIN_M", "OQ_NO_GEMV_GROUP", "OQ_GEMV_GROUP_R", "OQ_GEMV_NO_ASTAGE",
                                          "OQ_GEMV_MAX_M", "OQ_GEMM_WG_SPLIT", "OQ_FLOAT_GEMM_MIN_M", "OQ_GEMM_STAMPS"};
const char *env_values[ENV_COUNT];
bool overrides_allowed = false;  // ORBITQUANT_DEBUG=1 in the environment the process started with
void env_load() {
  static std::once_flag once;
  std::call_once(once, [] {
    for (int i = 0; i < ENV_COUNT; ++i) env_values[i] = getenv(kEnvNames[i]);
    const char *debug = getenv("ORBITQUANT_DEBUG");
    overrides_allowed = debug != nullptr && strcmp(debug, "1") == 0;
  });
}
}  // namespace

// The experiment switches: read from the environment once per process, then only changed through
// oq_debug_override.
const char *debug_env(int which) {
  env_load();
  return env_values[which];
}

int debug_env_set(const char *name, const char *value) {
  env_load();
  if (!overrides_allowed)  // a switch changes which kernel runs and so the bits of a result: not for a serving process
    return fail(OQ_ERR_INVALID, "debug_override: switches are fixed in this process (start it with ORBITQUANT_DEBUG=1 to change them at run time)");
  for (int i = 0; i < ENV_COUNT; ++i) {
    if (strcmp(name, kEnvNames[i]) == 0) {
      env_values[i] = value != nullptr ? strdup(value) : nullptr;  // a few bytes per call, never freed: readers may hold the old one
      return OQ_OK;
    }
  }
  return fail(OQ_ERR_INVALID, "debug_override: unknown switch %s", name);
}

// kernels (defined in the other translation units)
int rotate_quantize_dispatch(const void *x, int x_dtype, int64_t M, int64_t K, const int32_t *perm,
                             const int8_t *signs, const float *boundaries, const float *centroids,
                             int levels, int64_t block, float eps, float inv_sqrt_block,
                             void *codes_out, int code_format, void *values_out, int values_mode,
                             float *norms_out, const uint16_t *input_map, const void *plan, hipStream_t stream);
int rotate_plan_build(const int32_t *perm, const int8_t *signs, const float *boundaries, int levels, int64_t K,
                      int64_t block, float inv_sqrt_block, void *plan_out, hipStream_t stream);
int quantize_weight_fast(const void *w, int w_dtype, int64_t N, int64_t K, const void *plan, const float *boundaries,
                         int levels, int64_t block, float eps, float inv_sqrt_block, int bits, uint8_t *packed_out,
                         uint16_t *row_norms_out, hipStream_t stream);
int gemm_tiled_dispatch(const void *x, const float *token_scale, const uint8_t *w, int bits, const uint16_t *row_norms,
                        const float *w_cents, const void *bias, int bias_dtype, int64_t M, int64_t N, int64_t K, void *out,
                        int out_dtype, void *workspace, uint64_t workspace_bytes, hipStream_t stream);
uint64_t gemm_tiled_workspace_bytes(int64_t M, int64_t K);
uint64_t gemm_workspace_bytes(int64_t M, int64_t N, int64_t K, int bits);
int gemm_staged_dispatch(const void *x, const float *token_scale, const uint8_t *w, int bits, const uint16_t *row_norms,
                         const float *w_cents, const void *bias, int bias_dtype, int64_t M, int64_t N, int64_t K, void *out,
                         int out_dtype, hipStream_t stream);
int adaln_int4_dispatch(const uint16_t *x, const uint8_t *packed, const uint16_t *scales, const uint16_t *bias, int64_t M,
                        int64_t N, int64_t K, int64_t group, uint16_t *out, hipStream_t stream);
int adaln_quantize_dispatch(const void *w, int w_dtype, int64_t N, int64_t K, int64_t group, uint8_t *packed, float *scales,
                            hipStream_t stream);
int pack_lowbit_dispatch(const uint8_t *values, int bits, int64_t count, uint8_t *packed, hipStream_t stream);
int dequantize_dispatch(const uint8_t *packed, int bits, const uint16_t *row_norms, const float *centroids, int64_t N, int64_t K,
                        void *out, int out_dtype, hipStream_t stream);
bool token_linear_supported(int x_dtype, int64_t M, int64_t N, int64_t K, int levels, int bits, const void *x,
                            const int32_t *perm, const int8_t *signs);
int token_linear_dispatch(const void *x, int x_dtype, const uint16_t *input_map, int64_t K, const int32_t *perm,
                          const int8_t *signs, const float *boundaries, const float *act_cents, int levels,
                          int64_t block, float eps, float inv_sqrt_block, const uint8_t *packed_w, int bits,
                          const uint16_t *row_norms, const float *w_cents, const void *bias, int bias_dtype,
                          int64_t N, void *out, int out_dtype, hipStream_t stream, bool *launched);
int generic_matmul_float(const void *x, int x_dtype, const float *token_scale, const uint8_t *packed_w,
                         int bits, const uint16_t *row_norms, const float *w_cents, const void *bias,
                         int bias_dtype, int64_t M, int64_t N, int64_t K, void *out, int out_dtype,
                         hipStream_t stream);
int generic_linear_codes(const void *codes, int code_format, const float *token_norms,
                         const float *act_cents, int a_levels, const uint8_t *packed_w, int bits,
                         const uint16_t *row_norms, const float *w_cents, const void *bias,
                         int bias_dtype, int64_t M, int64_t N, int64_t K, void *out, int out_dtype,
                         hipStream_t stream);
int unpack_dispatch(const uint8_t *packed, int bits, int64_t count, uint8_t *out, hipStream_t stream);
bool gemm_supported(int64_t K, int bits);
int gemm_dispatch(int a_mode, const void *a, const float *row_scale, const float *act_cents, int a_levels,
                  const uint8_t *w, int bits, const uint16_t *row_norms, const float *w_cents,
                  const void *bias, int bias_dtype, int64_t M, int64_t N, int64_t K, void *out,
                  int out_dtype, const uint16_t *out_map, void *workspace, uint64_t workspace_bytes, hipStream_t stream);
int apply_value_map(void *out, int64_t count, const uint16_t *table, hipStream_t stream);
int gemm_choose_tile(int64_t M, int64_t N, int64_t K, int bits);
bool gemm_av_supported(int64_t K, int bits);
int gemm_av_dispatch(bool f16, const void *a, const float *row_scale, const uint8_t *w, int bits,
                     const uint16_t *row_norms, const float *w_cents, const void *bias, int bias_dtype,
                     int64_t M, int64_t N, int64_t K, void *out, int out_dtype, int tile, hipStream_t stream);
bool gemv_supported(int64_t M, int64_t K, int bits, int code_format, int a_levels);
int gemv_dispatch(const void *codes, int code_format, const float *row_scale, const float *act_cents, int a_levels,
                  const uint8_t *w, int bits, const uint16_t *row_norms, const float *w_cents,
                  const void *bias, int bias_dtype, int64_t M, int64_t N, int64_t K, void *out,
                  int out_dtype, hipStream_t stream);
int gemv_group_dispatch(const void *codes, int code_format, const float *row_scale, const float *act_cents, int a_levels,
                        int count, const uint8_t *const *w, const int *bits, const uint16_t *const *row_norms,
                        const float *const *w_cents, const void *const *bias, int bias_dtype, int64_t M,
                        const int64_t *N, int64_t K, void *const *out, int out_dtype, hipStream_t stream, bool *launched);
// Scratch of oq_quantized_linear_static: the activation codes and token norms that pass from the
// quantizer launch to the matmul launch.  One copy per GPU, at its own address there; host code
// only ever uses the address hipGetSymbolAddress returns for the current device.
constexpr size_t kStaticScratchBytes = OQ_STATIC_SCRATCH_BYTES;
static __device__ __attribute__((used)) __align__(256) unsigned char scratch[kStaticScratchBytes];

constexpr int kMaxDevices = 64;
static int static_scratch_address(unsigned char **out) {
  static std::mutex lock;
  static unsigned char *address[kMaxDevices];
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) return fail(OQ_ERR_LAUNCH, "no HIP device is current");
  if (dev < 0 || dev >= kMaxDevices) return fail(OQ_ERR_UNSUPPORTED, "device index %d is beyond %d", dev, kMaxDevices - 1);
  std::lock_guard<std::mutex> guard(lock);
  if (address[dev] == nullptr) {
    void *ptr = nullptr;
    const hipError_t err = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (err != hipSuccess || ptr == nullptr)
      return fail(OQ_ERR_LAUNCH, "cannot resolve the static scratch on device %d: %s", dev, hipGetErrorString(err));
    address[dev] = static_cast<unsigned char *>(ptr);
  }
  *out = address[dev];
  return OQ_OK;
}

static bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }
static bool valid_dtype(int dt) { return dt == OQ_F32 || dt == OQ_F16 || dt == OQ_BF16; }

static int check_matmul_common(const char *who, const uint8_t *packed_w, int bits, const uint16_t *row_norms,
                               const float *w_cents, const void *bias, int bias_dtype, int64_t M, int64_t N,
                               int64_t K, const void *out, int out_dtype) {
  if (M < 0 || N <= 0 || K <= 0) return fail(OQ_ERR_INVALID, "%s: M=%lld N=%lld K=%lld", who, (long long)M, (long long)N, (long long)K);
  if (bits < 1 || bits > 8) return fail(OQ_ERR_INVALID, "%s: bits=%d not in [1, 8]", who, bits);
  if (packed_w == nullptr || row_norms == nullptr || w_cents == nullptr || (out == nullptr && M > 0))
    return fail(OQ_ERR_INVALID, "%s: null pointer", who);
  if (!valid_dtype(out_dtype)) return fail(OQ_ERR_INVALID, "%s: out_dtype=%d", who, out_dtype);
  if (bias != nullptr && !valid_dtype(bias_dtype)) return fail(OQ_ERR_INVALID, "%s: bias_dtype=%d", who, bias_dtype);
  return OQ_OK;
}

}  // namespace oq

using namespace oq;

extern "C" {

const char *oq_last_error(void) { return g_error; }

const char *oq_version(void) { return "orbitquant-hip 0.1 (gfx950)"; }

int oq_device_ok(void) {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) return fail(OQ_ERR_LAUNCH, "no HIP device is current");
  hipDeviceProp_t prop;
  if (hipGetDeviceProperties(&prop, dev) != hipSuccess) return fail(OQ_ERR_LAUNCH, "cannot query device %d", dev);
  if (strncmp(prop.gcnArchName, "gfx950", 6) != 0)
    return fail(OQ_ERR_UNSUPPORTED, "device %d is %s; this library holds gfx950 code only", dev, prop.gcnArchName);
  unsigned char *unused = nullptr;
  return static_scratch_address(&unused);  // resolved here so that later calls (e.g. under graph capture) only look it up
}

int oq_rotate_quantize(const void *x, int x_dtype, int64_t M, int64_t K, const int32_t *perm,
                       const int8_t *signs, const float *boundaries, const float *centroids, int levels,
                       int64_t block, float eps, float inv_sqrt_block, const void *rotate_plan, void *codes_out,
                       int code_format, void *values_out, int values_mode, float *norms_out, void *stream) {
  return rotate_quantize_dispatch(x, x_dtype, M, K, perm, signs, boundaries, centroids, levels, block, eps,
                                  inv_sqrt_block, codes_out, code_format, values_out, values_mode, norms_out,
                                  nullptr, rotate_plan, as_stream(stream));
}

uint64_t oq_rotate_plan_bytes(int64_t K) { return K > 0 ? 3136u + 8u * static_cast<uint64_t>(K) : 0u; }

int oq_rotate_plan_build(const int32_t *perm, const int8_t *signs, const float *boundaries, int levels, int64_t K,
                         int64_t block, float inv_sqrt_block, void *plan_out, void *stream) {
  return rotate_plan_build(perm, signs, boundaries, levels, K, block, inv_sqrt_block, plan_out, as_stream(stream));
}

int oq_rotate_quantize_mapped(const void *x, int x_dtype, const uint16_t *input_map, int64_t M, int64_t K,
                              const int32_t *perm, const int8_t *signs, const float *boundaries,
                              const float *centroids, int levels, int64_t block, float eps, float inv_sqrt_block,
                              const void *rotate_plan, void *codes_out, int code_format, void *values_out,
                              int values_mode, float *norms_out, void *stream) {
  if (input_map == nullptr) return fail(OQ_ERR_INVALID, "rotate_quantize_mapped: input_map is null");
  return rotate_quantize_dispatch(x, x_dtype, M, K, perm, signs, boundaries, centroids, levels, block, eps,
                                  inv_sqrt_block, codes_out, code_format, values_out, values_mode, norms_out,
                                  input_map, rotate_plan, as_stream(stream));
}

int oq_quantize_weight(const void *w, int w_dtype, int64_t N, int64_t K, const void *rotate_plan,
                       const float *boundaries, int levels, int64_t block, float eps, float inv_sqrt_block, int bits,
                       uint8_t *packed_out, uint16_t *row_norms_out, void *stream) {
  const int rc = quantize_weight_fast(w, w_dtype, N, K, rotate_plan, boundaries, levels, block, eps, inv_sqrt_block, bits,
                                      packed_out, row_norms_out, as_stream(stream));
  return rc < 0 ? fail(OQ_ERR_UNSUPPORTED, "quantize_weight: no kernel for block %lld", (long long)block) : rc;
}

// oq_packed_linear with an optional output map (applied by the tile kernels' epilogue, by a
// small elementwise launch after the other kernels).
static int packed_linear_impl(const void *codes, int code_format, const float *token_norms,
                              const float *act_centroids, int a_bits, const uint8_t *packed_w, int w_bits,
                              const uint16_t *row_norms, const float *w_centroids, const void *bias, int bias_dtype,
                              int64_t M, int64_t N, int64_t K, void *out, int out_dtype, const uint16_t *out_map,
                              void *workspace, uint64_t workspace_bytes, void *stream) {
  if (int rc = check_matmul_common("packed_linear", packed_w, w_bits, row_norms, w_centroids, bias, bias_dtype, M, N, K, out, out_dtype)) return rc;
  if (M == 0) return OQ_OK;
  if (codes == nullptr || act_centroids == nullptr) return fail(OQ_ERR_INVALID, "packed_linear: null codes/centroids");
  if (a_bits < 1 || a_bits > 8) return fail(OQ_ERR_INVALID, "packed_linear: a_bits=%d", a_bits);
  if (code_format != OQ_CODES_U8 && code_format != OQ_CODES_NIBBLE) return fail(OQ_ERR_INVALID, "packed_linear: code_format=%d", code_format);
  if (code_format == OQ_CODES_NIBBLE && (a_bits > 4 || (K & 1))) return fail(OQ_ERR_INVALID, "packed_linear: nibble codes need a_bits <= 4 and even K");
  if (out_map != nullptr) {
    if (out_dtype == OQ_F32) return fail(OQ_ERR_INVALID, "packed_linear: an output map needs a 16-bit output dtype");
    if (!aligned16(out_map)) return fail(OQ_ERR_INVALID, "packed_linear: the output map must be 16-byte aligned");
  }
  const int a_levels = 1 << a_bits;
  hipStream_t s = as_stream(stream);
  const bool fast_ptrs = aligned16(codes) && aligned16(packed_w);
  const bool tiled_out = gemm_output_ok(N, out);  // the tiled kernels store 16-byte row segments
  int rc;
  if (fast_ptrs && gemv_supported(M, K, w_bits, code_format, a_levels)) {
    rc = gemv_dispatch(codes, code_format, token_norms, act_centroids, a_levels, packed_w, w_bits, row_norms, w_centroids,
                       bias, bias_dtype, M, N, K, out, out_dtype, s);
  } else if (fast_ptrs && tiled_out && gemm_supported(K, w_bits) && (code_format == OQ_CODES_NIBBLE || M > 16)) {
    return gemm_dispatch(code_format == OQ_CODES_NIBBLE ? 0 : 1, codes, token_norms, act_centroids, a_levels, packed_w, w_bits, row_norms, w_centroids,
                         bias, bias_dtype, M, N, K, out, out_dtype, out_map, workspace, workspace_bytes, s);
  } else {
    rc = generic_linear_codes(codes, code_format, token_norms, act_centroids, a_levels, packed_w, w_bits, row_norms,
                              w_centroids, bias, bias_dtype, M, N, K, out, out_dtype, s);
  }
  if (rc != OQ_OK || out_map == nullptr) return rc;
  return apply_value_map(out, M * N, out_map, s);
}

int oq_debug_override(const char *name, const char *value) {
  if (name == nullptr) return fail(OQ_ERR_INVALID, "debug_override: null name");
  return debug_env_set(name, value);
}

uint64_t oq_packed_linear_workspace_bytes(int64_t M, int64_t N, int64_t K, int w_bits, int code_format, int a_bits) {
  if (M <= 0 || N <= 0 || K <= 0 || a_bits < 1 || a_bits > 8) return 0;
  if (gemv_supported(M, K, w_bits, code_format, 1 << a_bits)) return 0;  // the streaming kernel
  if (N % 8 != 0 || !gemm_supported(K, w_bits) || !(code_format == OQ_CODES_NIBBLE || M > 16)) return 0;
  return gemm_workspace_bytes(M, N, K, w_bits);
}

uint64_t oq_matmul_packed_weight_workspace_bytes(int64_t M, int64_t N, int64_t K, int w_bits, int x_dtype) {
  if (M <= 0 || N <= 0 || K <= 0 || x_dtype != OQ_BF16 || K % 64 != 0 || N % 8 != 0 || !gemm_supported(K, w_bits)) return 0;
  return gemm_tiled_workspace_bytes(M, K);
}

int oq_packed_linear(const void *codes, int code_format, const float *token_norms, const float *act_centroids,
                     int a_bits, const uint8_t *packed_w, int w_bits, const uint16_t *row_norms,
                     const float *w_centroids, const void *bias, int bias_dtype, int64_t M, int64_t N,
                     int64_t K, void *out, int out_dtype, void *workspace, uint64_t workspace_bytes, void *stream) {
  return packed_linear_impl(codes, code_format, token_norms, act_centroids, a_bits, packed_w, w_bits, row_norms,
                            w_centroids, bias, bias_dtype, M, N, K, out, out_dtype, nullptr, workspace, workspace_bytes, stream);
}

int oq_packed_linear_group(const void *codes, int code_format, const float *token_norms, const float *act_centroids,
                           int a_bits, int count, const uint8_t *const *packed_w, const int *w_bits,
                           const uint16_t *const *row_norms, const float *const *w_centroids, const void *const *bias,
                           int bias_dtype, int64_t M, const int64_t *N, int64_t K, void *const *out, int out_dtype,
                           void *workspace, uint64_t workspace_bytes, void *stream) {
  if (count < 1 || count > 64) return fail(OQ_ERR_INVALID, "packed_linear_group: count=%d (1..64)", count);
  if (packed_w == nullptr || w_bits == nullptr || row_norms == nullptr || w_centroids == nullptr || N == nullptr || out == nullptr)
    return fail(OQ_ERR_INVALID, "packed_linear_group: null argument array");
  for (int i = 0; i < count; ++i)
    if (int rc = check_matmul_common("packed_linear_group", packed_w[i], w_bits[i], row_norms[i], w_centroids[i],
                                     bias != nullptr ? bias[i] : nullptr, bias_dtype, M, N[i], K, out[i], out_dtype))
      return rc;
  if (M == 0) return OQ_OK;
  if (codes == nullptr || act_centroids == nullptr) return fail(OQ_ERR_INVALID, "packed_linear_group: null codes/centroids");
  if (a_bits < 1 || a_bits > 8) return fail(OQ_ERR_INVALID, "packed_linear_group: a_bits=%d", a_bits);
  if (code_format != OQ_CODES_U8 && code_format != OQ_CODES_NIBBLE) return fail(OQ_ERR_INVALID, "packed_linear_group: code_format=%d", code_format);
  bool launched = false;
  if (int rc = gemv_group_dispatch(codes, code_format, token_norms, act_centroids, 1 << a_bits, count, packed_w, w_bits,
                                   row_norms, w_centroids, bias, bias_dtype, M, N, K, out, out_dtype, as_stream(stream),
                                   &launched))
    return rc;
  if (launched) return OQ_OK;
  for (int i = 0; i < count; ++i)
    if (int rc = packed_linear_impl(codes, code_format, token_norms, act_centroids, a_bits, packed_w[i], w_bits[i],
                                    row_norms[i], w_centroids[i], bias != nullptr ? bias[i] : nullptr, bias_dtype, M,
                                    N[i], K, out[i], out_dtype, nullptr, workspace, workspace_bytes, stream))
      return rc;
  return OQ_OK;
}

int oq_packed_linear_mapped(const void *codes, int code_format, const float *token_norms,
                            const float *act_centroids, int a_bits, const uint8_t *packed_w, int w_bits,
                            const uint16_t *row_norms, const float *w_centroids, const void *bias, int bias_dtype,
                            int64_t M, int64_t N, int64_t K, void *out, int out_dtype, const uint16_t *output_map,
                            void *workspace, uint64_t workspace_bytes, void *stream) {
  if (output_map == nullptr) return fail(OQ_ERR_INVALID, "packed_linear_mapped: output_map is null");
  return packed_linear_impl(codes, code_format, token_norms, act_centroids, a_bits, packed_w, w_bits, row_norms,
                            w_centroids, bias, bias_dtype, M, N, K, out, out_dtype, output_map, workspace, workspace_bytes, stream);
}

int oq_quantized_linear(const void *x, int x_dtype, const uint16_t *input_map, int64_t M, int64_t K,
                        const int32_t *perm, const int8_t *signs, const float *boundaries,
                        const float *act_centroids, int a_bits, int64_t block, float eps, float inv_sqrt_block,
                        const void *rotate_plan, const uint8_t *packed_w, int w_bits, const uint16_t *row_norms, const float *w_centroids,
                        const void *bias, int bias_dtype, int64_t N, void *codes_scratch, float *norms_scratch,
                        void *out, int out_dtype, const uint16_t *output_map, void *workspace, uint64_t workspace_bytes,
                        void *stream) {
  if (int rc = check_matmul_common("quantized_linear", packed_w, w_bits, row_norms, w_centroids, bias, bias_dtype, M, N, K, out, out_dtype)) return rc;
  if (M == 0) return OQ_OK;
  if (a_bits < 1 || a_bits > 8) return fail(OQ_ERR_INVALID, "quantized_linear: a_bits=%d", a_bits);
  if (act_centroids == nullptr) return fail(OQ_ERR_INVALID, "quantized_linear: null activation centroids");
  const int levels = 1 << a_bits;
  hipStream_t s = as_stream(stream);
  if (output_map != nullptr && (out_dtype == OQ_F32 || !aligned16(output_map)))
    return fail(OQ_ERR_INVALID, "quantized_linear: an output map needs a 16-bit output dtype and 16-byte alignment");
  if (aligned16(packed_w) && token_linear_supported(x_dtype, M, N, K, levels, w_bits, x, perm, signs)) {
    bool launched = false;
    const int rc = token_linear_dispatch(x, x_dtype, input_map, K, perm, signs, boundaries, act_centroids, levels, block,
                                         eps, inv_sqrt_block, packed_w, w_bits, row_norms, w_centroids, bias,
                                         bias_dtype, N, out, out_dtype, s, &launched);
    if (rc != OQ_OK) return rc;
    if (launched) return output_map == nullptr ? OQ_OK : apply_value_map(out, N, output_map, s);
  }
  if (codes_scratch == nullptr || norms_scratch == nullptr)
    return fail(OQ_ERR_INVALID, "quantized_linear: this shape takes two launches and needs the scratch buffers");
  const int fmt = (a_bits <= 4 && (K & 1) == 0) ? OQ_CODES_NIBBLE : OQ_CODES_U8;
  if (int rc = rotate_quantize_dispatch(x, x_dtype, M, K, perm, signs, boundaries, nullptr, levels, block, eps,
                                        inv_sqrt_block, codes_scratch, fmt, nullptr, OQ_VALUES_NONE, norms_scratch,
                                        input_map, rotate_plan, s))
    return rc;
  return packed_linear_impl(codes_scratch, fmt, norms_scratch, act_centroids, a_bits, packed_w, w_bits, row_norms,
                            w_centroids, bias, bias_dtype, M, N, K, out, out_dtype, output_map, workspace, workspace_bytes, stream);
}

int oq_quantized_linear_group(const void *x, int x_dtype, const uint16_t *input_map, int64_t M, int64_t K,
                              const int32_t *perm, const int8_t *signs, const float *boundaries,
                              const float *act_centroids, int a_bits, int64_t block, float eps, float inv_sqrt_block,
                              const void *rotate_plan, int count, const uint8_t *const *packed_w, const int *w_bits,
                              const uint16_t *const *row_norms, const float *const *w_centroids, const void *const *bias,
                              int bias_dtype, const int64_t *N, void *codes_scratch, float *norms_scratch,
                              void *const *out, int out_dtype, void *workspace, uint64_t workspace_bytes, void *stream) {
  if (count < 1 || count > 64) return fail(OQ_ERR_INVALID, "quantized_linear_group: count=%d (1..64)", count);
  if (packed_w == nullptr || w_bits == nullptr || row_norms == nullptr || w_centroids == nullptr || N == nullptr || out == nullptr)
    return fail(OQ_ERR_INVALID, "quantized_linear_group: null argument array");
  for (int i = 0; i < count; ++i)
    if (int rc = check_matmul_common("quantized_linear_group", packed_w[i], w_bits[i], row_norms[i], w_centroids[i],
                                     bias != nullptr ? bias[i] : nullptr, bias_dtype, M, N[i], K, out[i], out_dtype))
      return rc;
  if (M == 0) return OQ_OK;
  if (a_bits < 1 || a_bits > 8) return fail(OQ_ERR_INVALID, "quantized_linear_group: a_bits=%d", a_bits);
  if (act_centroids == nullptr) return fail(OQ_ERR_INVALID, "quantized_linear_group: null activation centroids");
  const int levels = 1 << a_bits;
  hipStream_t s = as_stream(stream);
  if (codes_scratch == nullptr || norms_scratch == nullptr)
    return fail(OQ_ERR_INVALID, "quantized_linear_group: null scratch buffers");
  const int fmt = (a_bits <= 4 && (K & 1) == 0) ? OQ_CODES_NIBBLE : OQ_CODES_U8;
  if (int rc = rotate_quantize_dispatch(x, x_dtype, M, K, perm, signs, boundaries, nullptr, levels, block, eps,
                                        inv_sqrt_block, codes_scratch, fmt, nullptr, OQ_VALUES_NONE, norms_scratch,
                                        input_map, rotate_plan, s))
    return rc;
  return oq_packed_linear_group(codes_scratch, fmt, norms_scratch, act_centroids, a_bits, count, packed_w, w_bits,
                                row_norms, w_centroids, bias, bias_dtype, M, N, K, out, out_dtype, workspace, workspace_bytes,
                                stream);
}

int oq_quantized_linear_static(const void *x, int x_dtype, const uint16_t *input_map, int64_t M, int64_t K,
                               const int32_t *perm, const int8_t *signs, const float *boundaries,
                               const float *act_centroids, int a_bits, int64_t block, float eps, float inv_sqrt_block,
                               const void *rotate_plan, const uint8_t *packed_w, int w_bits, const uint16_t *row_norms,
                               const float *w_centroids, const void *bias, int bias_dtype, int64_t N, void *out,
                               int out_dtype, const uint16_t *output_map, void *stream) {
  if (M < 0 || K <= 0) return fail(OQ_ERR_INVALID, "quantized_linear_static: M=%lld K=%lld", (long long)M, (long long)K);
  // layout of the scratch: codes (nibble or byte per value) rounded up to 256 bytes, then the norms
  const bool nibble = a_bits <= 4 && (K & 1) == 0;
  const uint64_t codes_bytes = static_cast<uint64_t>(M) * static_cast<uint64_t>(nibble ? K / 2 : K);
  const uint64_t norms_at = (codes_bytes + 255u) & ~static_cast<uint64_t>(255);
  if (static_cast<uint64_t>(K) > (1u << 20) || norms_at + 4u * static_cast<uint64_t>(M) > kStaticScratchBytes)
    return fail(OQ_ERR_UNSUPPORTED,
                "quantized_linear_static: %lld tokens of %lld values need %llu bytes of scratch, the static buffer holds %zu; "
                "use oq_quantized_linear with caller-owned scratch",
                (long long)M, (long long)K, (unsigned long long)(norms_at + 4u * static_cast<uint64_t>(M)), kStaticScratchBytes);
  unsigned char *base = nullptr;
  if (int rc = static_scratch_address(&base)) return rc;
  // (no workspace: the launch shapes that need no buffer beyond the scratch)
  return oq_quantized_linear(x, x_dtype, input_map, M, K, perm, signs, boundaries, act_centroids, a_bits, block, eps,
                             inv_sqrt_block, rotate_plan, packed_w, w_bits, row_norms, w_centroids, bias, bias_dtype, N, base,
                             reinterpret_cast<float *>(base + norms_at), out, out_dtype, output_map, nullptr, 0, stream);
}

int oq_matmul_packed_weight(const void *x, int x_dtype, const float *token_scale, const uint8_t *packed_w,
                            int bits, const uint16_t *row_norms, const float *w_centroids, const void *bias,
                            int bias_dtype, int64_t M, int64_t N, int64_t K, void *out, int out_dtype,
                            void *workspace, uint64_t workspace_bytes, void *stream) {
  if (int rc = check_matmul_common("matmul_packed_weight", packed_w, bits, row_norms, w_centroids, bias, bias_dtype, M, N, K, out, out_dtype)) return rc;
  if (M == 0) return OQ_OK;
  if (x == nullptr || !valid_dtype(x_dtype)) return fail(OQ_ERR_INVALID, "matmul_packed_weight: x / x_dtype");
  hipStream_t s = as_stream(stream);
  // bf16 activations take the tile kernel from two tokens on (one token on large matrices): measured against
  // the float-activation kernels below it is 3-4 times faster from 9 to 255 tokens (4096x4096 W4: 104 -> 28 us)
  // and up to 13 times at 2 to 8; only a single token on a small matrix is 2-3 us quicker on the
  // shape-agnostic kernel.  OQ_FLOAT_GEMM_MIN_M overrides, for measurements.
  int64_t tile_kernel_from = N * K >= (int64_t{32} << 20) ? 1 : 2;
  if (const char *v = debug_env(ENV_FLOAT_GEMM_MIN_M)) tile_kernel_from = atoi(v) > 1 ? atoi(v) : 1;
  if (x_dtype == OQ_BF16 && M >= tile_kernel_from && K % 64 == 0 && aligned16(x) && aligned16(packed_w) && gemm_output_ok(N, out) &&
      gemm_supported(K, bits)) {
    // Large M: the tile kernel of the code path on activation values.  Either one pass first puts the activations
    // into the matrix core's operand order (fastest on large problems; needs the caller's workspace), or every
    // wavefront stages its own rows through LDS (no buffer).
    const char *force = debug_env(ENV_GEMM_TILE);
    const bool force_staged = force != nullptr && force[0] != '\0' && force[1] == 's';
    if (!force_staged) {
      const int rc = gemm_tiled_dispatch(x, token_scale, packed_w, bits, row_norms, w_centroids, bias, bias_dtype, M, N, K, out, out_dtype,
                                         workspace, workspace_bytes, s);
      if (rc >= 0) return rc;
    }
    if (M * K * 2 < (int64_t{1} << 32))
      return gemm_staged_dispatch(x, token_scale, packed_w, bits, row_norms, w_centroids, bias, bias_dtype, M, N, K, out, out_dtype, s);
  }
  if (x_dtype != OQ_F32 && M > 8 && aligned16(x) && aligned16(packed_w) && gemm_output_ok(N, out) && gemm_av_supported(K, bits))
  {
    // The float-activation kernel has its own (measured) preference: 256x256 tiles once there are
    // at least half as many of them as CUs, 128x128 tiles below that; OQ_GEMM_TILE still overrides.
    const int64_t big_tiles = ((M + 255) / 256) * ((N + 255) / 256);
    const int tile = debug_env(ENV_GEMM_TILE) != nullptr ? gemm_choose_tile(M, N, K, bits) : (big_tiles >= 128 ? 2 : 0);
    return gemm_av_dispatch(x_dtype == OQ_F16, x, token_scale, packed_w, bits, row_norms, w_centroids, bias, bias_dtype,
                            M, N, K, out, out_dtype, tile, s);
  }
  return generic_matmul_float(x, x_dtype, token_scale, packed_w, bits, row_norms, w_centroids, bias, bias_dtype, M, N,
                              K, out, out_dtype, s);
}

int oq_matmul_packed_adaln_int4(const uint16_t *x, const uint8_t *packed_weight, const uint16_t *scales,
                                const uint16_t *bias, int64_t M, int64_t N, int64_t K, int64_t group_size, uint16_t *out,
                                void *stream) {
  return adaln_int4_dispatch(x, packed_weight, scales, bias, M, N, K, group_size, out, as_stream(stream));
}

int oq_quantize_adaln_weight(const void *w, int w_dtype, int64_t N, int64_t K, int64_t group_size, uint8_t *packed_out,
                             float *scales_out, void *stream) {
  return adaln_quantize_dispatch(w, w_dtype, N, K, group_size, packed_out, scales_out, as_stream(stream));
}

int oq_unpack_lowbit(const uint8_t *packed, int bits, int64_t count, uint8_t *out, void *stream) {
  if (bits < 1 || bits > 8 || count < 0) return fail(OQ_ERR_INVALID, "unpack_lowbit: bits=%d count=%lld", bits, (long long)count);
  if (count > 0 && (packed == nullptr || out == nullptr)) return fail(OQ_ERR_INVALID, "unpack_lowbit: null pointer");
  return unpack_dispatch(packed, bits, count, out, as_stream(stream));
}

int oq_pack_lowbit(const uint8_t *values, int bits, int64_t count, uint8_t *packed_out, void *stream) {
  if (bits < 1 || bits > 8 || count < 0) return fail(OQ_ERR_INVALID, "pack_lowbit: bits=%d count=%lld", bits, (long long)count);
  if (count > 0 && (values == nullptr || packed_out == nullptr)) return fail(OQ_ERR_INVALID, "pack_lowbit: null pointer");
  return pack_lowbit_dispatch(values, bits, count, packed_out, as_stream(stream));
}

int oq_dequantize_packed_weight(const uint8_t *packed_weight, int bits, const uint16_t *row_norms, const float *centroids,
                                int64_t N, int64_t K, void *out, int out_dtype, void *stream) {
  if (bits < 1 || bits > 8 || N < 0 || K < 0) return fail(OQ_ERR_INVALID, "dequantize_packed_weight: bits=%d N=%lld K=%lld", bits, (long long)N, (long long)K);
  if (out_dtype != OQ_F32 && out_dtype != OQ_F16 && out_dtype != OQ_BF16) return fail(OQ_ERR_INVALID, "dequantize_packed_weight: out_dtype=%d", out_dtype);
  if (N > 0 && K > 0 && (packed_weight == nullptr || row_norms == nullptr || centroids == nullptr || out == nullptr))
    return fail(OQ_ERR_INVALID, "dequantize_packed_weight: null pointer");
  return dequantize_dispatch(packed_weight, bits, row_norms, centroids, N, K, out, out_dtype, as_stream(stream));
}

}  // extern "C"
