// Small-M (decode-sized, M <= 16) packed-weight linear: a pure stream over the
// packed index bytes.
//
// The token rows are the 16-row side of v_mfma_f32_16x16x32_bf16 (rows beyond M
// are padding), sixteen weight rows are the other side, so the k-reduction
// happens inside the matrix core and the weights are streamed from HBM exactly
// once whatever M is.  A workgroup owns 16*R consecutive weight rows for the
// whole K range; its wavefronts split K between them and add their partial
// tiles through LDS in a fixed order (wave 0, 1, 2, ...), so results do not
// depend on timing.
//
// K is cut like in the tiled GEMM: in a K-step of 128, lane group g (0..3) owns
// the contiguous run k0+32g .. k0+32g+31 of its row and MFMA q (0..3) consumes
// values 8q..8q+7 of every run.
#include "packed_decode.h"

namespace oq {
namespace {

struct GemvArgs {
  const uint8_t *a;          // nibble codes [M, K/2]
  const float *row_scale;    // [M] or NULL
  const float *act_cents;
  int a_levels;
  const uint8_t *w;
  const uint16_t *row_norms;
  const float *w_cents;
  const void *bias;
  int bias_dtype;
  int M;
  int64_t N, K;
  void *out;
  int out_dtype;
};

template <int BITS, int R, int WAVES>
__global__ __launch_bounds__(64 * WAVES) void packed_gemv_kernel(GemvArgs g) {
  extern __shared__ __align__(16) uint32_t lds[];
  uint32_t *wlut = lds;
  uint32_t *alut = lds + WLut<BITS>::kDwords;
  float *partial = reinterpret_cast<float *>(alut + kALutDwords);  // [WAVES][R][64][4]

  fill_lut(wlut, g.w_cents, BITS, 1 << BITS, WLut<BITS>::kPair, false);
  fill_lut(alut, g.act_cents, 4, g.a_levels, true, false);
  __syncthreads();

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int r = lane & 15, grp = lane >> 4;
  const uint32_t wbase = lds_byte_address(wlut) + 4 * (lane & 31);
  const uint32_t abase = lds_byte_address(alut) + 4 * (lane & 31);
  const int64_t n_base = static_cast<int64_t>(blockIdx.x) * (16 * R);

  const int steps = static_cast<int>(g.K / 128);
  const int s_begin = static_cast<int>(static_cast<int64_t>(steps) * wave / WAVES);
  const int s_end = static_cast<int>(static_cast<int64_t>(steps) * (wave + 1) / WAVES);

  const int64_t w_row_bytes = g.K * BITS / 8;
  const uint8_t *ap = g.a + static_cast<int64_t>(min(r, g.M - 1)) * (g.K / 2) + grp * 16;
  const uint8_t *wp[R];
#pragma unroll
  for (int j = 0; j < R; ++j) {
    const int64_t row = min(n_base + 16 * j + r, g.N - 1);
    wp[j] = g.w + row * w_row_bytes + grp * (4 * BITS);
  }

  f32x4 acc[R];
#pragma unroll
  for (int j = 0; j < R; ++j) acc[j] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};

  uint4 a_nxt = make_uint4(0, 0, 0, 0);
  uint32_t w_nxt[R][BITS];
  if (s_begin < s_end) {
    a_nxt = *reinterpret_cast<const uint4 *>(ap + static_cast<int64_t>(s_begin) * 64);
#pragma unroll
    for (int j = 0; j < R; ++j) load_w<BITS>(wp[j] + static_cast<int64_t>(s_begin) * (16 * BITS), w_nxt[j]);
  }
  for (int s = s_begin; s < s_end; ++s) {
    const uint4 a_cur = a_nxt;
    uint32_t w_cur[R][BITS];
#pragma unroll
    for (int j = 0; j < R; ++j)
#pragma unroll
      for (int d = 0; d < BITS; ++d) w_cur[j][d] = w_nxt[j][d];
    if (s + 1 < s_end) {
      a_nxt = *reinterpret_cast<const uint4 *>(ap + static_cast<int64_t>(s + 1) * 64);
#pragma unroll
      for (int j = 0; j < R; ++j) load_w<BITS>(wp[j] + static_cast<int64_t>(s + 1) * (16 * BITS), w_nxt[j]);
    }
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const uint32_t f = q == 0 ? a_cur.x : q == 1 ? a_cur.y : q == 2 ? a_cur.z : a_cur.w;
      const uint4 af = decode_a_nibble(f, abase);
#pragma unroll
      for (int j = 0; j < R; ++j) {
        const uint4 bf = decode_w<BITS>(w_cur[j], q, wbase);
        acc[j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, af), __builtin_bit_cast(bf16x8, bf),
                                                         acc[j], 0, 0, 0);
      }
    }
  }

  // ---- cross-wave sum in LDS, fixed order ----------------------------------------
#pragma unroll
  for (int j = 0; j < R; ++j)
    *reinterpret_cast<float4 *>(partial + ((wave * R + j) * 64 + lane) * 4) =
        make_float4(acc[j][0], acc[j][1], acc[j][2], acc[j][3]);
  __syncthreads();
  // accumulator e of lane l: token row 4*(l/16) + e, weight row l%16
  for (int item = tid; item < R * 64; item += 64 * WAVES) {
    const int j = item >> 6, l = item & 63;
    float4 sum = *reinterpret_cast<const float4 *>(partial + ((0 * R + j) * 64 + l) * 4);
    for (int w = 1; w < WAVES; ++w) {
      const float4 p = *reinterpret_cast<const float4 *>(partial + ((w * R + j) * 64 + l) * 4);
      sum.x += p.x; sum.y += p.y; sum.z += p.z; sum.w += p.w;
    }
    const int64_t n = n_base + 16 * j + (l & 15);
    if (n >= g.N) continue;
    const float rn = bf16_bits_to_f32(g.row_norms[n]);
    const float bv = g.bias != nullptr ? load_dyn_f32(g.bias, g.bias_dtype, n) : 0.0f;
    const float v[4] = {sum.x, sum.y, sum.z, sum.w};
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const int m = 4 * (l >> 4) + e;
      if (m >= g.M) continue;
      const float sc = g.row_scale != nullptr ? g.row_scale[m] : 1.0f;
      const float y = v[e] * sc * rn + bv;
      const int64_t o = static_cast<int64_t>(m) * g.N + n;
      if (g.out_dtype == OQ_BF16) static_cast<uint16_t *>(g.out)[o] = f32_to_bf16_bits(y);
      else if (g.out_dtype == OQ_F16) static_cast<uint16_t *>(g.out)[o] = f32_to_f16_bits(y);
      else static_cast<float *>(g.out)[o] = y;
    }
  }
}

template <int BITS, int R, int WAVES>
int launch(const GemvArgs &g, hipStream_t stream) {
  const int64_t groups = (g.N + 16 * R - 1) / (16 * R);
  if (groups > 0x7fffffffLL) return fail(OQ_ERR_UNSUPPORTED, "packed_gemv: N too large");
  const size_t smem = (WLut<BITS>::kDwords + kALutDwords) * sizeof(uint32_t) + sizeof(float) * WAVES * R * 64 * 4;
  auto kern = packed_gemv_kernel<BITS, R, WAVES>;
  if (smem > 48 * 1024) {
    if (hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                            static_cast<int>(smem)) != hipSuccess)
      return fail(OQ_ERR_LAUNCH, "packed_gemv: cannot reserve %zu bytes of LDS", smem);
  }
  hipLaunchKernelGGL(kern, dim3(static_cast<unsigned>(groups)), dim3(64 * WAVES), smem, stream, g);
  return check_launch("packed_gemv");
}

template <int BITS>
int launch_bits(const GemvArgs &g, hipStream_t stream) {
  // 16 rows per workgroup while that still leaves fewer than ~2 workgroups per CU, else 32
  if (g.N <= 16 * 512) return launch<BITS, 1, 8>(g, stream);
  return launch<BITS, 2, 8>(g, stream);
}

}  // namespace

bool gemv_supported(int64_t M, int64_t K, int bits, int code_format, int a_levels) {
  return M >= 1 && M <= 16 && K % 128 == 0 && code_format == OQ_CODES_NIBBLE && a_levels <= 16 &&
         (bits == 2 || bits == 3 || bits == 4 || bits == 6 || bits == 8);
}

int gemv_dispatch(const void *codes, const float *row_scale, const float *act_cents, int a_levels,
                  const uint8_t *w, int bits, const uint16_t *row_norms, const float *w_cents,
                  const void *bias, int bias_dtype, int64_t M, int64_t N, int64_t K, void *out,
                  int out_dtype, hipStream_t stream) {
  GemvArgs g{};
  g.a = static_cast<const uint8_t *>(codes); g.row_scale = row_scale; g.act_cents = act_cents; g.a_levels = a_levels;
  g.w = w; g.row_norms = row_norms; g.w_cents = w_cents; g.bias = bias; g.bias_dtype = bias_dtype;
  g.M = static_cast<int>(M); g.N = N; g.K = K; g.out = out; g.out_dtype = out_dtype;
  switch (bits) {
    case 2: return launch_bits<2>(g, stream);
    case 3: return launch_bits<3>(g, stream);
    case 4: return launch_bits<4>(g, stream);
    case 6: return launch_bits<6>(g, stream);
    case 8: return launch_bits<8>(g, stream);
    default: return fail(OQ_ERR_UNSUPPORTED, "packed_gemv: weight width %d", bits);
  }
}

}  // namespace oq
