// Rotate plan construction and the launcher of the plan-based rotate+quantize kernel
// (rotate_quantize_fast.h).
#include "rotate_quantize_fast.h"

namespace oq {
namespace {

using namespace rqf;

// ---- plan construction: one workgroup, once per layer ---------------------------------------------
// Floats in an order-preserving integer code, so that "the largest float t with RN(t * c) <= b" can
// be found by bisection over all of them.
__device__ __forceinline__ uint32_t float_to_ordered(float f) {
  const uint32_t u = __float_as_uint(f);
  return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}
__device__ __forceinline__ float ordered_to_float(uint32_t o) {
  return __uint_as_float((o & 0x80000000u) ? (o & 0x7fffffffu) : ~o);
}

__global__ __launch_bounds__(256) void rotate_plan_build_kernel(const int32_t *perm, const int8_t *signs,
                                                                 const float *boundaries, int levels, int K, int block,
                                                                 float c, unsigned char *out) {
  __shared__ float thr[256];
  __shared__ int bad;
  const int tid = threadIdx.x;
  const int nb = levels - 1;
  if (tid == 0) bad = 0;
  // thresholds: bisection between -inf and +inf in the ordered code (RN(t * c) is non-decreasing in t)
  float t = __builtin_inff();
  if (tid < nb) {
    const float b = boundaries[tid];
    if (b != b) {
      t = b;  // a NaN boundary is below nothing either way
    } else {
      uint32_t lo = float_to_ordered(-__builtin_inff()), hi = float_to_ordered(__builtin_inff());  // RN(lo * c) <= b always
      if (!(__builtin_inff() * c <= b)) {
        while (hi - lo > 1) {  // invariant: RN(lo * c) <= b < RN(hi * c)
          const uint32_t mid = lo + (hi - lo) / 2;
          if (ordered_to_float(mid) * c <= b) lo = mid;
          else hi = mid;
        }
      } else {
        lo = hi;
      }
      t = ordered_to_float(lo);
    }
  }
  thr[tid] = t;
  reinterpret_cast<float *>(out + plan::kThresholdsOffset)[tid] = t;
  __syncthreads();

  // cells over [first threshold, last threshold]
  const float lo = thr[0], hi = thr[nb > 0 ? nb - 1 : 0];
  float scale = static_cast<float>(plan::kCells) / (hi - lo);
  float offset = -lo * scale;
  bool usable = levels >= 3 && levels <= 64 && hi > lo && scale < 3.0e38f && __builtin_fabsf(offset) < 3.0e38f;
  if (usable) {
    // thresholds ascend, so their cells do: the first with cell >= tid, the first with cell > tid
    int first = 0, last = 0;
    for (int j = 0; j < nb; ++j) {
      const int cj = static_cast<int>(plan::cell_of(thr[j], scale, offset));
      if (cj < tid) first = j + 1;
      if (cj <= tid) last = j + 1;
      if (j > 0 && !(thr[j - 1] <= thr[j])) bad = 1;  // not ascending (or NaN): no table
    }
    if (last - first > 1) bad = 1;
    reinterpret_cast<uint2 *>(out + plan::kCellsOffset)[tid] =
        make_uint2(__float_as_uint(last > first ? thr[first] : __builtin_inff()), static_cast<uint32_t>(first));
  } else {
    reinterpret_cast<uint2 *>(out + plan::kCellsOffset)[tid] = make_uint2(__float_as_uint(__builtin_inff()), 0u);
  }
  __syncthreads();
  if (tid == 0) {
    plan::PlanHeader h{};
    h.magic = plan::kMagic;
    h.K = static_cast<uint32_t>(K);
    h.block = static_cast<uint32_t>(block);
    h.levels = static_cast<uint32_t>(levels);
    h.cells = (usable && bad == 0) ? plan::kCells : 0;
    h.cell_scale = scale;
    h.cell_offset = offset;
    h.inv_sqrt_block = c;
    *reinterpret_cast<plan::PlanHeader *>(out) = h;
  }
  // gather entries
  uint32_t *g16 = reinterpret_cast<uint32_t *>(out + plan::kGatherOffset);
  uint32_t *g32 = g16 + K;
  for (int i = tid; i < K; i += 256) {
    const uint32_t p = static_cast<uint32_t>(perm[i]);
    const bool negative = signs[i] < 0;
    g16[i] = plan::kStageAddress + 2u * p + (negative ? 2u * static_cast<uint32_t>(K) : 0u);
    g32[i] = (plan::kStageAddress + 4u * p) | (negative ? 0x80000000u : 0u);
  }
}

// ---- the kernel ------------------------------------------------------------------------------------
template <int DT, int LOG_H, int EMIT, bool MAPPED>
__global__ __launch_bounds__(512) void rotate_quantize_fast_kernel(FastArgs a) {
  extern __shared__ __align__(16) unsigned char smem[];
  rotate_quantize_row_fast<DT, LOG_H, EMIT, MAPPED>(a, smem, blockIdx.x, threadIdx.x, blockDim.x >> 6);
}

template <int DT, int LOG_H, int EMIT, bool MAPPED = false>
int launch_emit(const FastArgs &a, int waves, size_t smem, hipStream_t stream) {
  auto kern = rotate_quantize_fast_kernel<DT, LOG_H, EMIT, MAPPED>;
  if (!reserve_dynamic_lds(reinterpret_cast<const void *>(kern), smem))
    return fail(OQ_ERR_LAUNCH, "rotate_quantize: cannot reserve %zu bytes of LDS", smem);
  hipLaunchKernelGGL(kern, dim3(static_cast<unsigned>(a.M)), dim3(64 * waves), smem, stream, a);
  return check_launch("rotate_quantize (plan)");
}

template <int DT, int LOG_H>
int launch_one(const FastArgs &a, int waves, size_t smem, hipStream_t stream) {
  if (a.map != nullptr) {  // an input map: bf16 rows into codes only (the forms the layers use); -1 sends the rest to the plain kernel
    if constexpr (DT == OQ_BF16) {
      if (a.packed == nullptr && a.codes != nullptr && a.values == nullptr) {
        if (a.code_format == OQ_CODES_NIBBLE) return launch_emit<DT, LOG_H, EMIT_NIBBLE, true>(a, waves, smem, stream);
        return launch_emit<DT, LOG_H, EMIT_U8, true>(a, waves, smem, stream);
      }
    }
    return -1;
  }
  if (a.packed != nullptr) return launch_emit<DT, LOG_H, EMIT_WEIGHT>(a, waves, smem, stream);
  if (a.codes != nullptr && a.values == nullptr) {
    if (a.code_format == OQ_CODES_NIBBLE) return launch_emit<DT, LOG_H, EMIT_NIBBLE>(a, waves, smem, stream);
    return launch_emit<DT, LOG_H, EMIT_U8>(a, waves, smem, stream);
  }
  return launch_emit<DT, LOG_H, EMIT_ANY>(a, waves, smem, stream);
}

template <int DT>
int launch_dtype(const FastArgs &a, int log_h, int waves, size_t smem, hipStream_t stream) {
  switch (log_h) {
    case 3: return launch_one<DT, 3>(a, waves, smem, stream);
    case 4: return launch_one<DT, 4>(a, waves, smem, stream);
    case 5: return launch_one<DT, 5>(a, waves, smem, stream);
    case 6: return launch_one<DT, 6>(a, waves, smem, stream);
    case 7: return launch_one<DT, 7>(a, waves, smem, stream);
    case 8: return launch_one<DT, 8>(a, waves, smem, stream);
    case 9: return launch_one<DT, 9>(a, waves, smem, stream);
    case 10: return launch_one<DT, 10>(a, waves, smem, stream);
    case 11: return launch_one<DT, 11>(a, waves, smem, stream);
    case 12: return launch_one<DT, 12>(a, waves, smem, stream);
    default: return -1;
  }
}

}  // namespace

int rotate_plan_build(const int32_t *perm, const int8_t *signs, const float *boundaries, int levels, int64_t K,
                      int64_t block, float inv_sqrt_block, void *plan_out, hipStream_t stream) {
  if (perm == nullptr || signs == nullptr || boundaries == nullptr || plan_out == nullptr)
    return fail(OQ_ERR_INVALID, "rotate_plan_build: null pointer");
  if (levels < 2 || levels > 256) return fail(OQ_ERR_INVALID, "rotate_plan_build: levels=%d not in [2, 256]", levels);
  if (K <= 0 || K > 16384) return fail(OQ_ERR_UNSUPPORTED, "rotate_plan_build: K=%lld not in [1, 16384]", (long long)K);
  if (block <= 0 || (block & (block - 1)) != 0 || K % block != 0)
    return fail(OQ_ERR_INVALID, "rotate_plan_build: block=%lld must be a power of two dividing K=%lld", (long long)block, (long long)K);
  if (!(inv_sqrt_block > 0.0f) || !(inv_sqrt_block < 3.0e38f))
    return fail(OQ_ERR_INVALID, "rotate_plan_build: inv_sqrt_block must be positive and finite");
  if ((reinterpret_cast<uintptr_t>(plan_out) & 15u) != 0) return fail(OQ_ERR_INVALID, "rotate_plan_build: the plan must be 16-byte aligned");
  hipLaunchKernelGGL(rotate_plan_build_kernel, dim3(1), dim3(256), 0, stream, perm, signs, boundaries, levels,
                     static_cast<int>(K), static_cast<int>(block), inv_sqrt_block, static_cast<unsigned char *>(plan_out));
  return check_launch("rotate_plan_build");
}

static int launch_fast(FastArgs &a, int x_dtype, hipStream_t stream);

int quantize_weight_fast(const void *w, int w_dtype, int64_t N, int64_t K, const void *plan, const float *boundaries,
                         int levels, int64_t block, float eps, float inv_sqrt_block, int bits, uint8_t *packed_out,
                         uint16_t *row_norms_out, hipStream_t stream) {
  auto aligned16 = [](const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; };
  if (w == nullptr || plan == nullptr || boundaries == nullptr || packed_out == nullptr || row_norms_out == nullptr)
    return fail(OQ_ERR_INVALID, "quantize_weight: null pointer");
  if (w_dtype != OQ_F32 && w_dtype != OQ_F16 && w_dtype != OQ_BF16) return fail(OQ_ERR_INVALID, "quantize_weight: w_dtype=%d", w_dtype);
  if (N < 0 || K <= 0) return fail(OQ_ERR_INVALID, "quantize_weight: N=%lld K=%lld", (long long)N, (long long)K);
  if (bits < 1 || bits > 8 || levels < 2 || levels > (1 << bits))
    return fail(OQ_ERR_INVALID, "quantize_weight: bits=%d levels=%d", bits, levels);
  if (block <= 0 || (block & (block - 1)) != 0 || K % block != 0)
    return fail(OQ_ERR_INVALID, "quantize_weight: block=%lld must be a power of two dividing K=%lld", (long long)block, (long long)K);
  if (block < 8 || block > 4096 || K % 8 != 0 || K > 16384 || N > 0x7fffffffLL)
    return fail(OQ_ERR_UNSUPPORTED, "quantize_weight: needs 8 <= block <= 4096, K a multiple of 8 up to 16384 (block=%lld K=%lld)",
                (long long)block, (long long)K);
  if (!aligned16(w) || !aligned16(plan)) return fail(OQ_ERR_INVALID, "quantize_weight: w and the plan must be 16-byte aligned");
  if (N == 0) return OQ_OK;
  FastArgs a{};
  a.x = w; a.M = N; a.K = K; a.plan = static_cast<const unsigned char *>(plan);
  a.levels = levels; a.block = static_cast<int>(block); a.eps = eps;
  a.raw_bounds = boundaries; a.inv_sqrt_block = inv_sqrt_block; a.pack_bits = bits;
  a.packed = packed_out; a.norms_bf16 = row_norms_out;
  return launch_fast(a, w_dtype, stream);
}

int rotate_quantize_fast(const void *x, int x_dtype, int64_t M, int64_t K, const void *plan, int levels, int64_t block,
                         float eps, const float *centroids, void *codes_out, int code_format, void *values_out,
                         int values_mode, float *norms_out, const uint16_t *input_map, hipStream_t stream) {
  auto aligned16 = [](const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; };
  int log_h = 0;
  while ((int64_t{1} << log_h) < block) ++log_h;
  if (plan == nullptr || log_h < 3 || log_h > 12 || K % 8 != 0 || !aligned16(x) || !aligned16(plan) ||
      (codes_out != nullptr && !aligned16(codes_out)) || (values_out != nullptr && !aligned16(values_out)))
    return -1;
  FastArgs a{};
  a.x = x; a.M = M; a.K = K; a.plan = static_cast<const unsigned char *>(plan);
  a.cents = values_mode != OQ_VALUES_NONE ? centroids : nullptr;
  a.levels = levels;
  a.block = static_cast<int>(block);
  a.eps = eps;
  a.codes = static_cast<uint8_t *>(codes_out); a.code_format = code_format;
  a.values = values_mode == OQ_VALUES_NONE ? nullptr : values_out; a.values_mode = values_mode;
  a.norms = norms_out;
  a.map = input_map;
  return launch_fast(a, x_dtype, stream);
}

// Derived launch parameters and the launch itself; -1 when no kernel is instantiated for the block size.
static int launch_fast(FastArgs &a, int x_dtype, hipStream_t stream) {
  const int64_t K = a.K, block = a.block;
  int log_h = 0;
  while ((int64_t{1} << log_h) < block) ++log_h;
  a.levels_pow2 = 2;
  while (a.levels_pow2 < a.levels) a.levels_pow2 <<= 1;
  a.passes = static_cast<int>((K + kPass - 1) / kPass);
  const int64_t unit = block > kLaneSpan ? block : kLaneSpan;
  a.units = static_cast<int>((K + unit - 1) / unit);
  // Wavefronts per row (each owns whole units): four, which is also what staging the row uses,
  // eight for rows of sixteen units and more (measured: 5120 values in 5 units of 1024, 210 us on four
  // against 237 us on five; 13824 values in 27 units of 512, 608 us on eight against 655 us on four).
  int waves = a.units >= 16 ? 8 : (a.units < 4 ? a.units : 4);
  if (a.M <= 16) waves = a.units < 8 ? a.units : 8;  // few rows: every unit its own wavefront
  if (const char *forced = debug_env(ENV_RQ_WAVES)) {
    const int w = atoi(forced);
    if (w >= 1 && w <= 8) waves = w < a.units ? w : a.units;
  }
  const size_t smem = a.map != nullptr ? fast_lds_bytes_mapped(K) : fast_lds_bytes(K);
  if (smem > 160 * 1024) return -1;
  switch (x_dtype) {
    case OQ_F32: return launch_dtype<OQ_F32>(a, log_h, waves, smem, stream);
    case OQ_F16: return launch_dtype<OQ_F16>(a, log_h, waves, smem, stream);
    default: return launch_dtype<OQ_BF16>(a, log_h, waves, smem, stream);
  }
}

}  // namespace oq
