// Packed-weight GEMM on the gfx950 matrix cores.
//
//   out[m,n] = (sum_k A[m,k] * c_w[idx[n,k]]) * scale[m] * r_w[n] + bias[n]
//
// A is either packed 4-bit activation codes (decoded through a codebook table)
// or 16-bit float values; idx is the flat little-endian bit stream of 2/3/4/6/8
// bit weight indices, read from HBM as it is stored.  Nothing is dequantized to
// memory: every wavefront loads the packed dwords of its own rows straight into
// registers, turns them into bf16 MFMA operands through lookup tables held in
// LDS, and feeds v_mfma_f32_32x32x16_bf16.
//
// Operand layout.  One MFMA consumes, per lane, eight k-values of one row
// (lane l: row l%32, k-group l/32).  A dot product does not care in which order
// k is visited as long as both operands agree, so a K-step of 64 is cut as
//   lane group g (0/1) owns k0+32g .. k0+32g+31   (one contiguous run of bits per row)
//   MFMA q (0..3) of the step uses values 8q..8q+7 of that run
// which makes every global load of packed data one contiguous 4*bits-byte run
// per lane (16 bytes for 4-bit), with no cross-lane shuffles and no LDS staging.
//
// Lookup tables: see packed_decode.h (pair tables, replicated per LDS bank).
#include "gemm_epilogue.h"

namespace oq {
namespace {

enum AMode { A_NIBBLE = 0, A_BF16 = 1, A_F16 = 2 };

struct GemmArgs {
  const uint8_t *a;          // [M, K/2] nibble codes or [M, K] 16-bit floats
  const float *row_scale;    // [M] or NULL
  const float *act_cents;    // [16] (nibble mode)
  int a_levels;
  const uint8_t *w;          // packed index stream
  const uint16_t *row_norms; // bf16 [N]
  const float *w_cents;      // [2^bits]
  const void *bias;
  int bias_dtype;
  int64_t M, N, K;
  void *out;
  int out_dtype;
  int tiles_m, tiles_n;
};

template <int AM> struct ARaw { uint4 v[AM == A_NIBBLE ? 1 : 4]; };

template <int AM>
__device__ __forceinline__ void load_a(const uint8_t *p, ARaw<AM> &r) {
  const uint4 *q = reinterpret_cast<const uint4 *>(p);
#pragma unroll
  for (int i = 0; i < (AM == A_NIBBLE ? 1 : 4); ++i) r.v[i] = q[i];
}

template <int AM>
__device__ __forceinline__ f32x16 mfma(uint4 a, uint4 b, f32x16 c) {
  if constexpr (AM == A_F16)
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
  else
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
}

// Workgroup = 4 wavefronts in a 2x2 arrangement; each wavefront owns FM x FN MFMA tiles of 32x32.
template <int AM, int BITS, int FM, int FN>
__global__ __launch_bounds__(256) void packed_gemm_kernel(GemmArgs g) {
  extern __shared__ __align__(16) uint32_t lds[];
  uint32_t *wlut = lds;
  uint32_t *alut = lds + WLut<BITS>::kDwords;

  // Loads of one wavefront return in order, so the handful of centroid values this thread
  // needs for its table entries are requested first, then the packed operands of the first
  // two K-steps; the tables are written while the packed data is still in flight.
  constexpr int kWEntries = WLut<BITS>::kEntries;
  float lut_w0 = 0.0f, lut_w1 = 0.0f, lut_a0 = 0.0f, lut_a1 = 0.0f;
  {
    const int e = threadIdx.x;
    if (e < kWEntries) {
      lut_w0 = g.w_cents[WLut<BITS>::kPair ? (e & ((1 << BITS) - 1)) : e];
      lut_w1 = g.w_cents[WLut<BITS>::kPair ? (e >> BITS) : e];
    }
    if constexpr (AM == A_NIBBLE) {
      const int c0 = e & 15, c1 = e >> 4;
      lut_a0 = c0 < g.a_levels ? g.act_cents[c0] : 0.0f;
      lut_a1 = c1 < g.a_levels ? g.act_cents[c1] : 0.0f;
    }
  }

  constexpr int TM = 2 * FM * 32, TN = 2 * FN * 32;
  // tile order: spread consecutive workgroup ids over the 8 XCDs' private L2s in
  // contiguous chunks, then walk groups of 4 tile-rows column by column
  int bid = blockIdx.x;
  const int total = g.tiles_m * g.tiles_n;
  if ((total & 7) == 0) bid = (bid & 7) * (total >> 3) + (bid >> 3);
  constexpr int GROUP_M = 4;
  const int width = GROUP_M * g.tiles_n;
  const int group = bid / width;
  const int first_m = group * GROUP_M;
  const int gsz = min(g.tiles_m - first_m, GROUP_M);
  const int pid_m = first_m + (bid % width) % gsz;
  const int pid_n = (bid % width) / gsz;

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int r = lane & 31, grp = lane >> 5;
  const uint32_t wbase = lds_byte_address(wlut) + 4 * r;
  const uint32_t abase = lds_byte_address(alut) + 4 * r;
  const int64_t m_base = static_cast<int64_t>(pid_m) * TM + (wave >> 1) * (FM * 32);
  const int64_t n_base = static_cast<int64_t>(pid_n) * TN + (wave & 1) * (FN * 32);

  EpiFactors<FM> epi;
  gemm_epilogue_prefetch<FM>(epi, static_cast<int64_t>(pid_m) * TM, static_cast<int64_t>(pid_n) * TN, (wave >> 1) * (FM * 32), TN, tid, g.M, g.N, g.row_scale, g.row_norms, g.bias, g.bias_dtype);

  constexpr int A_ROW_STEP = AM == A_NIBBLE ? 32 : 128;  // bytes of one row consumed per K-step of 64
  constexpr int A_GRP_OFF = AM == A_NIBBLE ? 16 : 64;
  const int64_t a_row_bytes = AM == A_NIBBLE ? g.K / 2 : g.K * 2;
  const int64_t w_row_bytes = g.K * BITS / 8;

  const uint8_t *ap[FM];
  const uint8_t *wp[FN];
#pragma unroll
  for (int i = 0; i < FM; ++i) {
    const int64_t row = min(m_base + 32 * i + r, g.M - 1);
    ap[i] = g.a + row * a_row_bytes + grp * A_GRP_OFF;
  }
#pragma unroll
  for (int j = 0; j < FN; ++j) {
    const int64_t row = min(n_base + 32 * j + r, g.N - 1);
    wp[j] = g.w + row * w_row_bytes + grp * (4 * BITS);
  }

  f32x16 acc[FM][FN];
#pragma unroll
  for (int i = 0; i < FM; ++i)
#pragma unroll
    for (int j = 0; j < FN; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.0f;

  // ---- main loop: software pipeline over "q-steps" (one MFMA k-slice of 16) -------
  // While the matrix core works on the operands decoded for q-step t, the wavefront
  // issues the table lookups for q-step t+1; packed dwords for K-step ks+1 are in
  // flight from global memory during K-step ks.
  ARaw<AM> a_cur[FM], a_nxt[FM];
  uint32_t w_cur[FN][BITS], w_nxt[FN][BITS];
#pragma unroll
  for (int i = 0; i < FM; ++i) load_a<AM>(ap[i], a_cur[i]);
#pragma unroll
  for (int j = 0; j < FN; ++j) load_w<BITS>(wp[j], w_cur[j]);

  const int steps = static_cast<int>(g.K / 64);
  if (steps > 1) {
#pragma unroll
    for (int i = 0; i < FM; ++i) load_a<AM>(ap[i] + A_ROW_STEP, a_nxt[i]);
#pragma unroll
    for (int j = 0; j < FN; ++j) load_w<BITS>(wp[j] + 8 * BITS, w_nxt[j]);
  }

  {  // table entries: one per thread, 32 copies each
    const int e = threadIdx.x;
    if (e < kWEntries) {
      const uint32_t d = pack16(lut_w0, lut_w1, AM == A_F16);
      uint4 *dst = reinterpret_cast<uint4 *>(wlut + e * 32);
#pragma unroll
      for (int i = 0; i < 8; ++i) dst[i] = make_uint4(d, d, d, d);
    }
    if constexpr (AM == A_NIBBLE) {
      const uint32_t d = pack16(lut_a0, lut_a1, false);
      uint4 *dst = reinterpret_cast<uint4 *>(alut + e * 32);
#pragma unroll
      for (int i = 0; i < 8; ++i) dst[i] = make_uint4(d, d, d, d);
    }
  }
  __syncthreads();

  auto decode = [&](int q, uint4 (&af)[FM], uint4 (&bf)[FN]) {
#pragma unroll
    for (int i = 0; i < FM; ++i) {
      if constexpr (AM == A_NIBBLE) {
        const uint32_t f = q == 0 ? a_cur[i].v[0].x : q == 1 ? a_cur[i].v[0].y : q == 2 ? a_cur[i].v[0].z : a_cur[i].v[0].w;
        af[i] = decode_a_nibble(f, abase);
      } else {
        af[i] = a_cur[i].v[q];
      }
    }
#pragma unroll
    for (int j = 0; j < FN; ++j) bf[j] = decode_w<BITS>(w_cur[j], q, wbase);
  };
  auto multiply = [&](const uint4 (&af)[FM], const uint4 (&bf)[FN]) {
#pragma unroll
    for (int i = 0; i < FM; ++i)
#pragma unroll
      for (int j = 0; j < FN; ++j) acc[i][j] = mfma<AM>(bf[j], af[i], acc[i][j]);  // weights first: transposed tile
  };
  // interleave hint: after each MFMA, the lookups' address arithmetic and LDS reads
  constexpr int kLookupsPerMfma = (AM == A_NIBBLE ? (FM + FN) : FN) * 4 / (FM * FN);
  auto interleave = [&]() {
#if defined(OQ_SCHED_HINTS)
#pragma unroll
    for (int i = 0; i < FM * FN; ++i) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x002, 2 * kLookupsPerMfma, 0);
      __builtin_amdgcn_sched_group_barrier(0x100, kLookupsPerMfma, 0);
    }
#endif
  };

  uint4 af0[FM], bf0[FN], af1[FM], bf1[FN];
  decode(0, af0, bf0);
  for (int ks = 0; ks < steps; ++ks) {
    decode(1, af1, bf1);
    multiply(af0, bf0);
    interleave();
    decode(2, af0, bf0);
    multiply(af1, bf1);
    interleave();
    decode(3, af1, bf1);
    multiply(af0, bf0);
    interleave();
    // rotate: K-step ks+1 becomes current, K-step ks+2 goes in flight
#pragma unroll
    for (int i = 0; i < FM; ++i) a_cur[i] = a_nxt[i];
#pragma unroll
    for (int j = 0; j < FN; ++j)
#pragma unroll
      for (int d = 0; d < BITS; ++d) w_cur[j][d] = w_nxt[j][d];
    if (ks + 2 < steps) {
#pragma unroll
      for (int i = 0; i < FM; ++i) load_a<AM>(ap[i] + static_cast<int64_t>(ks + 2) * A_ROW_STEP, a_nxt[i]);
#pragma unroll
      for (int j = 0; j < FN; ++j) load_w<BITS>(wp[j] + static_cast<int64_t>(ks + 2) * (8 * BITS), w_nxt[j]);
    }
    decode(0, af0, bf0);  // of K-step ks+1 (unused after the last step)
    multiply(af1, bf1);
    interleave();
  }

  __syncthreads();  // every wavefront is done with the lookup tables: LDS is reused by the epilogue
  gemm_epilogue<FM, FN>(acc, static_cast<int64_t>(pid_m) * TM, static_cast<int64_t>(pid_n) * TN, (wave >> 1) * (FM * 32),
                        (wave & 1) * (FN * 32), TN, tid, g.M, g.N, g.row_scale, g.row_norms, g.bias, g.bias_dtype, epi, g.out,
                        g.out_dtype, reinterpret_cast<unsigned char *>(lds));
}

template <int AM, int BITS, int FM, int FN>
int launch_cfg(GemmArgs g, hipStream_t stream) {
  constexpr int TM = 2 * FM * 32, TN = 2 * FN * 32;
  g.tiles_m = static_cast<int>((g.M + TM - 1) / TM);
  g.tiles_n = static_cast<int>((g.N + TN - 1) / TN);
  const int64_t total = static_cast<int64_t>(g.tiles_m) * g.tiles_n;
  if (total > 0x7fffffffLL) return fail(OQ_ERR_UNSUPPORTED, "packed_gemm: too many tiles");
  size_t smem = (WLut<BITS>::kDwords + (AM == A_NIBBLE ? kALutDwords : 0)) * sizeof(uint32_t);
  if (smem < static_cast<size_t>(kEpiLdsBytes)) smem = kEpiLdsBytes;  // the epilogue reuses LDS
  auto kern = packed_gemm_kernel<AM, BITS, FM, FN>;
  if (smem > 48 * 1024) {
    if (hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                            static_cast<int>(smem)) != hipSuccess)
      return fail(OQ_ERR_LAUNCH, "packed_gemm: cannot reserve %zu bytes of LDS", smem);
  }
  hipLaunchKernelGGL(kern, dim3(static_cast<unsigned>(total)), dim3(256), smem, stream, g);
  return check_launch("packed_gemm");
}

template <int AM, int BITS>
int launch_bits(const GemmArgs &g, int tile, hipStream_t stream) {
  if (tile == 2) return launch_cfg<AM, BITS, 4, 4>(g, stream);
  if (tile == 1) return launch_cfg<AM, BITS, 2, 4>(g, stream);
  return launch_cfg<AM, BITS, 2, 2>(g, stream);
}

template <int AM>
int launch_mode(const GemmArgs &g, int bits, int tile, hipStream_t stream) {
  switch (bits) {
    case 2: return launch_bits<AM, 2>(g, tile, stream);
    case 3: return launch_bits<AM, 3>(g, tile, stream);
    case 4: return launch_bits<AM, 4>(g, tile, stream);
    case 6: return launch_bits<AM, 6>(g, tile, stream);
    case 8: return launch_bits<AM, 8>(g, tile, stream);
    default: return fail(OQ_ERR_UNSUPPORTED, "packed_gemm: weight width %d", bits);
  }
}

}  // namespace

// Tile choice: the largest tile that still gives every CU work.
int gemm_choose_tile(int64_t M, int64_t N) {
  const char *force = getenv("OQ_GEMM_TILE");
  if (force != nullptr && force[0] >= '0' && force[0] <= '2') return force[0] - '0';
  auto tiles = [&](int tm, int tn) { return ((M + tm - 1) / tm) * ((N + tn - 1) / tn); };
  if (tiles(256, 256) >= 512) return 2;
  if (tiles(128, 256) >= 384) return 1;
  return 0;
}

bool gemm_supported(int64_t K, int bits) {
  return K % 64 == 0 && (bits == 2 || bits == 3 || bits == 4 || bits == 6 || bits == 8);
}

// a_mode: 0 nibble codes, 1 bf16 values, 2 fp16 values
int gemm_dispatch(int a_mode, const void *a, const float *row_scale, const float *act_cents, int a_levels,
                  const uint8_t *w, int bits, const uint16_t *row_norms, const float *w_cents,
                  const void *bias, int bias_dtype, int64_t M, int64_t N, int64_t K, void *out,
                  int out_dtype, hipStream_t stream) {
  GemmArgs g{};
  g.a = static_cast<const uint8_t *>(a); g.row_scale = row_scale; g.act_cents = act_cents; g.a_levels = a_levels;
  g.w = w; g.row_norms = row_norms; g.w_cents = w_cents; g.bias = bias; g.bias_dtype = bias_dtype;
  g.M = M; g.N = N; g.K = K; g.out = out; g.out_dtype = out_dtype;
  const int tile = gemm_choose_tile(M, N);
  if (a_mode != A_NIBBLE) return fail(OQ_ERR_INVALID, "packed_gemm: a_mode %d", a_mode);
  return launch_mode<A_NIBBLE>(g, bits, tile, stream);
}

}  // namespace oq
