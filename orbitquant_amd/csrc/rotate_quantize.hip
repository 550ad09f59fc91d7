// Fused RPBH rotate + per-token Lloyd-Max quantize for gfx950: the kernel (one workgroup per
// token row), its launcher and the argument checks.  The arithmetic is in rotate_quantize_row.h.
#include "rotate_plan.h"
#include "rotate_quantize_row.h"

namespace oq {
namespace {

using namespace rq;

template <int DT, bool VEC, int LOG_G, bool FEW>
__global__ __launch_bounds__(4 * kThreads) void rotate_quantize_kernel(RqArgs a) {
  extern __shared__ __align__(16) unsigned char smem[];
  rotate_quantize_row<DT, VEC, LOG_G, FEW>(a, smem, blockIdx.x, threadIdx.x, blockDim.x, [] {});
}

template <int DT, bool VEC>
int launch_for_block(const RqArgs &a, hipStream_t stream) {
  const int log_g = log2_groups(a);
  // a wavefront owns 512 consecutive elements of a pass: launch only the wavefronts a single-pass row needs
  const int waves = a.K >= 3 * kLaneSpan ? 4 : static_cast<int>((a.K + kLaneSpan - 1) / kLaneSpan);
  // few rows (decode): the chip is empty anyway, so run the passes of a long row side by side
  const int pass_groups = (a.M <= 64 && a.passes >= 2 && debug_env(ENV_RQ_ONE_GROUP) == nullptr) ? (a.passes >= 3 ? 4 : 2) : 1;
  dim3 grid(static_cast<unsigned>(a.M)), block(pass_groups > 1 ? kThreads * pass_groups : 64 * waves);
  RqArgs args = a;
  const size_t smem = lds_bytes(args, DT, VEC, pass_groups);
  // the decode-sized variant exists for the 16-byte access paths only
  const bool few = VEC && a.M <= 16;
#define OQ_RQ_LAUNCH(KERN)                                                                       \
  {                                                                                              \
    auto kern = KERN;                                                                            \
    if (!reserve_dynamic_lds(reinterpret_cast<const void *>(kern), smem))                        \
      return fail(OQ_ERR_LAUNCH, "rotate_quantize: cannot reserve %zu bytes of LDS", smem);      \
    hipLaunchKernelGGL(kern, grid, block, smem, stream, args);                                   \
  }
#define OQ_RQ_CASE(LG)                                                                           \
  case LG:                                                                                       \
    if constexpr (VEC) {                                                                         \
      if (few) {                                                                                 \
        OQ_RQ_LAUNCH((rotate_quantize_kernel<DT, VEC, LG, true>))                                \
        break;                                                                                   \
      }                                                                                          \
    }                                                                                            \
    OQ_RQ_LAUNCH((rotate_quantize_kernel<DT, VEC, LG, false>))                                   \
    break;
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
#undef OQ_RQ_LAUNCH
  return check_launch("rotate_quantize");
}

}  // namespace

int rotate_quantize_prepare(const void *x, int x_dtype, int64_t M, int64_t K, const int32_t *perm,
                            const int8_t *signs, const float *boundaries, const float *centroids,
                            int levels, int64_t block, float eps, float inv_sqrt_block,
                            void *codes_out, int code_format, void *values_out, int values_mode,
                            float *norms_out, const uint16_t *input_map, rq::RqArgs *out, bool *vec_out) {
  if (M < 0 || K <= 0) return fail(OQ_ERR_INVALID, "rotate_quantize: M=%lld K=%lld", (long long)M, (long long)K);
  if (x_dtype != OQ_F32 && x_dtype != OQ_F16 && x_dtype != OQ_BF16)
    return fail(OQ_ERR_INVALID, "rotate_quantize: unknown x_dtype %d", x_dtype);
  if (M == 0) {  // nothing to do, nothing to check
    *out = rq::RqArgs{};
    *vec_out = false;
    return OQ_OK;
  }
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

  if (input_map != nullptr) {
    if (x_dtype != OQ_F16 && x_dtype != OQ_BF16)
      return fail(OQ_ERR_INVALID, "rotate_quantize: an input map needs 16-bit inputs (x_dtype %d)", x_dtype);
    if ((reinterpret_cast<uintptr_t>(input_map) & 15u) != 0)
      return fail(OQ_ERR_INVALID, "rotate_quantize: the input map must be 16-byte aligned");
  }

  RqArgs a;
  a.map = input_map;
  // bf16: |x| in [2^-10, 2^6) is served from LDS (exponent field 117 .. 132)
  a.map_lo = (input_map != nullptr && x_dtype == OQ_BF16) ? kHotLoBf16 : -1;
  a.map_lds_offset = 0;
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

  auto aligned16 = [](const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; };
  *vec_out = (K % 8 == 0) && aligned16(x) && aligned16(perm) && aligned16(signs) &&
             (codes_out == nullptr || aligned16(codes_out)) &&
             (values_out == nullptr || aligned16(values_out));
  *out = a;
  return OQ_OK;
}

int rotate_quantize_dispatch(const void *x, int x_dtype, int64_t M, int64_t K, const int32_t *perm,
                             const int8_t *signs, const float *boundaries, const float *centroids,
                             int levels, int64_t block, float eps, float inv_sqrt_block,
                             void *codes_out, int code_format, void *values_out, int values_mode,
                             float *norms_out, const uint16_t *input_map, const void *plan, hipStream_t stream) {
  // With a rotate plan, launches of more than a few rows take the plan-based kernel (same results);
  // decode-sized launches (and input maps on anything but bf16 rows into codes) stay with the kernel below, which is built for latency.
  // The plan kernel gives every 512-slot unit (or block, if larger) of a row to one wavefront.  With many rows that is
  // all the parallelism it needs; with at most sixteen rows it wins only when a row has several units (K = 14336
  // in blocks of 2048, one token: 7.9 us against 10.1 us; K = 1152: 3.8 against 4.4) and loses when the row is one
  // block (K = 4096 = one block: 9.9 against 5.6 us), which the kernel below spreads over a whole workgroup.
  // A wavefront alone on a block of 2048 or 4096 values takes 7.5 / 10.4 us whatever the number of rows, the
  // workgroup-per-row kernel 6-7 us: up to 512 rows (every row's workgroup has a CU to itself or shares it with
  // one other) rows of one or two such blocks stay with the kernel below too (K = 4096 = one block, 17 to 512
  // rows: 10.3-11.3 against 6.9-9.6 us; from 1024 rows on the plan kernel is level or ahead).
  int64_t fast_min_m = 17;
  const int64_t unit = block > 512 ? block : 512;
  const bool several_units = (K + unit - 1) / unit >= 3;
  if (block >= 2048 && !several_units) fast_min_m = 513;
  if (const char *v = debug_env(ENV_RQ_FAST_MIN_M)) fast_min_m = atoi(v);
  if (plan != nullptr && (input_map == nullptr || x_dtype == OQ_BF16) && (M >= fast_min_m || several_units)) {
    RqArgs checked;
    bool vec_checked = false;
    if (int rc = rotate_quantize_prepare(x, x_dtype, M, K, perm, signs, boundaries, centroids, levels, block, eps,
                                         inv_sqrt_block, codes_out, code_format, values_out, values_mode, norms_out,
                                         input_map, &checked, &vec_checked))
      return rc;
    const int rc = rotate_quantize_fast(x, x_dtype, M, K, plan, levels, block, eps, centroids, codes_out, code_format,
                                        values_out, values_mode, norms_out, input_map, stream);
    if (rc >= 0) return rc;
  }
  RqArgs a;
  bool vec = false;
  const int rc = rotate_quantize_prepare(x, x_dtype, M, K, perm, signs, boundaries, centroids, levels, block, eps,
                                         inv_sqrt_block, codes_out, code_format, values_out, values_mode, norms_out,
                                         input_map, &a, &vec);
  if (rc != OQ_OK || M == 0) return rc;
  switch (x_dtype) {
    case OQ_F32: return vec ? launch_for_block<OQ_F32, true>(a, stream) : launch_for_block<OQ_F32, false>(a, stream);
    case OQ_F16: return vec ? launch_for_block<OQ_F16, true>(a, stream) : launch_for_block<OQ_F16, false>(a, stream);
    default: return vec ? launch_for_block<OQ_BF16, true>(a, stream) : launch_for_block<OQ_BF16, false>(a, stream);
  }
}

}  // namespace oq
