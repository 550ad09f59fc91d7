// The rotate plan: what the rotate+quantize kernel can know about a layer before it sees a
// token, computed once (oq_rotate_plan_build) and kept by the caller next to the layer's other
// constants.  It replaces the work every workgroup of the plain kernel repeats per row:
//   * thresholds: boundary j folded with the 1/sqrt(block) factor.  The specification rounds
//     rot = y * c once and counts the boundaries below rot; RN(y * c) is non-decreasing in y, so
//     for every boundary b there is a largest float t with RN(t * c) <= b, and
//     (b < RN(y * c)) == (t < y) for every y.  The kernel compares y with t and skips the multiply.
//   * cells: the one-read bucketize table over the thresholds (256 uniform cells; cell c holds
//     the number of thresholds in lower cells and the single threshold inside it).
//   * gather entries: permutation and sign of every rotated slot merged into the LDS byte
//     address the kernel reads its input from (16-bit inputs are staged twice, as x and as -x,
//     so a slot with a negative sign simply points into the second copy; fp32 inputs are staged
//     once and carry the sign in bit 31 of the entry).
// Layout of the blob (all offsets in bytes, the blob 16-byte aligned):
//   0     PlanHeader (64 bytes)
//   64    thresholds  float[256]   (+inf beyond levels - 1)
//   1088  cells       uint2[256]   (x: threshold bits or +inf, y: count below)
//   3136  gather16    uint32[K]
//   3136 + 4K  gather32  uint32[K]
#pragma once

#include "oq_common.h"

namespace oq {
namespace plan {

constexpr uint32_t kMagic = 0x4f51504cu;  // "OQPL"
constexpr int kCells = 256;
constexpr int kThresholdsOffset = 64;
constexpr int kCellsOffset = kThresholdsOffset + 256 * 4;
constexpr int kGatherOffset = kCellsOffset + kCells * 8;
constexpr uint32_t kStageAddress = 4160;  // where the kernel stages a row in its LDS; the gather entries are LDS addresses

struct PlanHeader {
  uint32_t magic;
  uint32_t K;
  uint32_t block;
  uint32_t levels;
  uint32_t cells;        // kCells, or 0 when some cell would hold two thresholds (then: binary search)
  float cell_scale;      // cell(v) = sat_u8(v * cell_scale + cell_offset)
  float cell_offset;
  float inv_sqrt_block;  // the factor folded into the thresholds
  uint32_t reserved[8];
};
static_assert(sizeof(PlanHeader) == 64, "the header is 64 bytes");

__host__ __device__ inline size_t plan_bytes(int64_t K) {
  return static_cast<size_t>(kGatherOffset) + 8u * static_cast<size_t>(K);
}

// The cell of a value: one fused multiply-add and one saturating conversion to 0..255.  Any
// monotone map gives exact codes as long as table and lookup use the same one; NaN lands in cell 0.
__device__ __forceinline__ uint32_t cell_of(float v, float scale, float offset) {
  return __builtin_amdgcn_cvt_pk_u8_f32(__builtin_fmaf(v, scale, offset), 0u, 0u);
}

}  // namespace plan

// Host side (rotate_quantize_fast.hip).
int rotate_plan_build(const int32_t *perm, const int8_t *signs, const float *boundaries, int levels, int64_t K,
                      int64_t block, float inv_sqrt_block, void *plan_out, hipStream_t stream);
// -1: this plan / shape has no fast kernel (the caller takes the plain one); else a status.
int rotate_quantize_fast(const void *x, int x_dtype, int64_t M, int64_t K, const void *plan, int levels, int64_t block,
                         float eps, const float *centroids, void *codes_out, int code_format, void *values_out,
                         int values_mode, float *norms_out, const uint16_t *input_map, hipStream_t stream);

// The weight side of a layer on the GPU (rotate_quantize_fast.hip): packed index stream + bf16 row norms.
int quantize_weight_fast(const void *w, int w_dtype, int64_t N, int64_t K, const void *plan, const float *boundaries,
                         int levels, int64_t block, float eps, float inv_sqrt_block, int bits, uint8_t *packed_out,
                         uint16_t *row_norms_out, hipStream_t stream);

}  // namespace oq
