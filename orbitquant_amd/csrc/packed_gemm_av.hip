// Packed-weight GEMM on the gfx950 matrix cores, 16-bit activation values.
//
//   out[m,n] = (sum_k A[m,k] * c_w[idx[n,k]]) * scale[m] * r_w[n] + bias[n]
//
// A is bf16 (or fp16): either the caller's activations, or the unit-norm codebook
// values the fused rotate+quantize kernel emits (then scale[m] is the token norm).
// idx is the flat bit stream of 2/3/4/6/8-bit weight indices, read from HBM as it
// is stored and decoded on the fly; a dequantized weight never exists in memory.
//
// Data flow per workgroup (4 wavefronts, 2x2, each FM x FN MFMA tiles of 32x32):
//   A  global -> registers -> LDS, one [tile rows x 64] slab per K-step, double
//      buffered, 16-byte coalesced loads (8 rows x 128 contiguous bytes per
//      wavefront load); wavefronts read their MFMA operands with ds_read_b128.
//      Rows are padded to 144 bytes so the 16 lanes a ds_read_b128 serves per
//      cycle hit distinct bank groups.
//   W  every wavefront loads the packed dwords of its own rows straight into
//      registers (one K-step ahead) and decodes them through the replicated
//      lookup tables of packed_decode.h.
// K order inside a K-step of 64: lane group g owns k0+32g .. k0+32g+31 of its
// row, MFMA q uses values 8q .. 8q+7 of that run (same cut for A and W).
#include "gemm_epilogue.h"

namespace oq {
namespace {

struct AvArgs {
  const uint8_t *a;          // [M, K] bf16 / fp16
  const float *row_scale;    // [M] or NULL
  const uint8_t *w;
  const uint16_t *row_norms;
  const float *w_cents;
  const void *bias;
  int bias_dtype;
  int64_t M, N, K;
  void *out;
  int out_dtype;
  OutMap out_map;
  int tiles_m, tiles_n;
};

constexpr int kAPitch = 144;  // 128 bytes of one row's 64 values + 16 bytes of padding

template <bool F16>
__device__ __forceinline__ f32x16 mfma16(uint4 a, uint4 b, f32x16 c) {
  if constexpr (F16)
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
  else
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
}

template <bool F16, int BITS, int FM, int FN>
__global__ __launch_bounds__(256) void packed_gemm_av_kernel(AvArgs g) {
  constexpr int TM = 64 * FM, TN = 64 * FN;
  constexpr int A_BUF = TM * kAPitch;
  constexpr int A_PER_T = TM * 8 / 256;  // 16-byte chunks per thread per K-step

  extern __shared__ __align__(16) uint32_t lds[];
  uint32_t *wlut = lds;
  unsigned char *abuf = reinterpret_cast<unsigned char *>(lds + WLut<BITS>::kDwords);  // [2][A_BUF]

  fill_lut(wlut, g.w_cents, BITS, 1 << BITS, WLut<BITS>::kPair, F16);

  // tile order: contiguous chunks of the tile list per XCD (workgroup ids go round-robin
  // over the 8 XCDs), inside a chunk groups of 4 tile-rows walked column by column
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
  const int64_t m0 = static_cast<int64_t>(pid_m) * TM, n0 = static_cast<int64_t>(pid_n) * TN;
  const int wm = (wave >> 1) * (FM * 32), wn = (wave & 1) * (FN * 32);

  EpiRaw<FM> epi_raw;
  gemm_epilogue_request<FM>(epi_raw, m0, n0, wm, tid, g.M, g.N, g.row_scale, g.row_norms, g.bias, g.bias_dtype, g.w_cents);

  // ---- A loader: chunk c = tid + 256*i -> row c/8, 16-byte chunk c%8 of the row's 128-byte slab
  const int64_t a_row_bytes = g.K * 2, w_row_bytes = g.K * BITS / 8;
  const int ld_row = tid >> 3, ld_off = (tid & 7) * 16;
  const int a_dst = ld_row * kAPitch + ld_off;  // + i * 32 * kAPitch
  const uint8_t *wp[FN];
#pragma unroll
  for (int j = 0; j < FN; ++j) wp[j] = g.w + min(n0 + wn + 32 * j + r, g.N - 1) * w_row_bytes + grp * (4 * BITS);

  uint4 sa[A_PER_T];
  auto fetch_a = [&](int ks) {
#pragma unroll
    for (int i = 0; i < A_PER_T; ++i) {
      const int64_t row = min(m0 + ld_row + 32 * i, g.M - 1);
      sa[i] = *reinterpret_cast<const uint4 *>(g.a + row * a_row_bytes + static_cast<int64_t>(ks) * 128 + ld_off);
    }
  };
  auto stash_a = [&](int buf) {
#pragma unroll
    for (int i = 0; i < A_PER_T; ++i)
      *reinterpret_cast<uint4 *>(abuf + buf * A_BUF + a_dst + i * 32 * kAPitch) = sa[i];
  };

  f32x16 acc[FM][FN];
#pragma unroll
  for (int i = 0; i < FM; ++i)
#pragma unroll
    for (int j = 0; j < FN; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.0f;

  // this lane's operand address inside an A buffer: row wm + r (+32 i), chunk 4*grp + q
  const int a_frag_off = (wm + r) * kAPitch + grp * 64;
  auto read_a = [&](int buf, int q, uint4 (&af)[FM]) {
#pragma unroll
    for (int i = 0; i < FM; ++i)
      af[i] = *reinterpret_cast<const uint4 *>(abuf + buf * A_BUF + a_frag_off + i * 32 * kAPitch + q * 16);
  };
  uint32_t w_cur[FN][BITS], w_nxt[FN][BITS];
  auto decode_b = [&](int q, uint4 (&bf)[FN]) {
#pragma unroll
    for (int j = 0; j < FN; ++j) bf[j] = decode_w<BITS>(w_cur[j], q, wbase);
  };
  auto multiply = [&](const uint4 (&af)[FM], const uint4 (&bf)[FN]) {
#pragma unroll
    for (int i = 0; i < FM; ++i)
#pragma unroll
      for (int j = 0; j < FN; ++j) acc[i][j] = mfma16<F16>(bf[j], af[i], acc[i][j]);  // weights first: transposed tile
  };

  // ---- prologue: slabs 0 and 1 into LDS, slab 2 and the weights of K-step 1 in flight ----
  const int steps = static_cast<int>(g.K / 64);
  fetch_a(0);
#pragma unroll
  for (int j = 0; j < FN; ++j) load_w<BITS>(wp[j], w_cur[j]);
  stash_a(0);
  if (steps > 1) {
    fetch_a(1);
#pragma unroll
    for (int j = 0; j < FN; ++j) load_w<BITS>(wp[j] + 8 * BITS, w_nxt[j]);
    stash_a(1);
  }
  if (steps > 2) fetch_a(2);
  uint4 af0[FM], bf0[FN], af1[FM], bf1[FN];
  __syncthreads();  // the lookup table (written by all threads above) and slab 0 are in LDS
  decode_b(0, bf0);
  read_a(0, 0, af0);

  // ---- main loop.  The barrier sits before the last of the four MFMA groups of a K-step, so
  // the matrix core still has that group to chew on while the first operands of the next
  // slab are read from LDS.
  for (int ks = 0; ks < steps; ++ks) {
    const int buf = ks & 1;
    read_a(buf, 1, af1);
    decode_b(1, bf1);
    multiply(af0, bf0);
    read_a(buf, 2, af0);
    decode_b(2, bf0);
    multiply(af1, bf1);
    read_a(buf, 3, af1);
    decode_b(3, bf1);
    multiply(af0, bf0);
    // packed weights of K-step ks+1 become current, K-step ks+2 goes in flight
#pragma unroll
    for (int j = 0; j < FN; ++j)
#pragma unroll
      for (int d = 0; d < BITS; ++d) w_cur[j][d] = w_nxt[j][d];
    if (ks + 2 < steps) {
#pragma unroll
      for (int j = 0; j < FN; ++j) load_w<BITS>(wp[j] + static_cast<int64_t>(ks + 2) * (8 * BITS), w_nxt[j]);
    }
    decode_b(0, bf0);  // of K-step ks+1 (unused after the last step)
    __syncthreads();   // every wavefront holds its last operands of slab ks in registers
    if (ks + 2 < steps) stash_a(buf);   // slab ks+2 (fetched one iteration ago) replaces slab ks
    if (ks + 3 < steps) fetch_a(ks + 3);
    if (ks + 1 < steps) read_a(buf ^ 1, 0, af0);
    multiply(af1, bf1);
  }

  __syncthreads();  // tables and staging buffers are dead: LDS is reused by the epilogue
  EpiFactors<FM> epi;
  gemm_epilogue_factors<FM>(epi, epi_raw, TN, tid, g.row_scale != nullptr, g.bias != nullptr, g.bias_dtype);
  gemm_epilogue<FM, FN>(acc, m0, n0, wm, wn, TN, tid, g.M, g.N, g.row_scale, g.row_norms, g.bias, g.bias_dtype, epi, g.out,
                        g.out_dtype, reinterpret_cast<unsigned char *>(lds), g.out_map);
}

template <bool F16, int BITS, int FM, int FN>
int launch_cfg(AvArgs g, hipStream_t stream) {
  constexpr int TM = 64 * FM, TN = 64 * FN;
  g.tiles_m = static_cast<int>((g.M + TM - 1) / TM);
  g.tiles_n = static_cast<int>((g.N + TN - 1) / TN);
  const int64_t total = static_cast<int64_t>(g.tiles_m) * g.tiles_n;
  if (total > 0x7fffffffLL) return fail(OQ_ERR_UNSUPPORTED, "packed_gemm: too many tiles");
  size_t smem = WLut<BITS>::kDwords * sizeof(uint32_t) + 2 * static_cast<size_t>(TM) * kAPitch;
  if (smem < static_cast<size_t>(kEpiLdsBytes)) smem = kEpiLdsBytes;  // the epilogue reuses LDS
  auto kern = packed_gemm_av_kernel<F16, BITS, FM, FN>;
  if (!reserve_dynamic_lds(reinterpret_cast<const void *>(kern), smem))
    return fail(OQ_ERR_LAUNCH, "packed_gemm: cannot reserve %zu bytes of LDS", smem);
  hipLaunchKernelGGL(kern, dim3(static_cast<unsigned>(total)), dim3(256), smem, stream, g);
  return check_launch("packed_gemm_av");
}

template <bool F16, int BITS>
int launch_bits(const AvArgs &g, int tile, hipStream_t stream) {
  if (tile == 2) return launch_cfg<F16, BITS, 4, 4>(g, stream);
  if (tile == 1) return launch_cfg<F16, BITS, 4, 2>(g, stream);
  return launch_cfg<F16, BITS, 2, 2>(g, stream);
}

template <bool F16>
int launch_mode(const AvArgs &g, int bits, int tile, hipStream_t stream) {
  switch (bits) {
    case 2: return launch_bits<F16, 2>(g, tile, stream);
    case 3: return launch_bits<F16, 3>(g, tile, stream);
    case 4: return launch_bits<F16, 4>(g, tile, stream);
    case 6: return launch_bits<F16, 6>(g, tile, stream);
    case 8: return launch_bits<F16, 8>(g, tile, stream);
    default: return fail(OQ_ERR_UNSUPPORTED, "packed_gemm: weight width %d", bits);
  }
}

}  // namespace

bool gemm_av_supported(int64_t K, int bits) {
  return K % 64 == 0 && (bits == 2 || bits == 3 || bits == 4 || bits == 6 || bits == 8);
}

int gemm_av_dispatch(bool f16, const void *a, const float *row_scale, const uint8_t *w, int bits,
                     const uint16_t *row_norms, const float *w_cents, const void *bias, int bias_dtype,
                     int64_t M, int64_t N, int64_t K, void *out, int out_dtype, int tile, hipStream_t stream) {
  AvArgs g{};
  g.a = static_cast<const uint8_t *>(a); g.row_scale = row_scale; g.w = w; g.row_norms = row_norms;
  g.w_cents = w_cents; g.bias = bias; g.bias_dtype = bias_dtype; g.M = M; g.N = N; g.K = K; g.out = out;
  g.out_dtype = out_dtype;
  g.out_map = OutMap{nullptr, -1};
  return f16 ? launch_mode<true>(g, bits, tile, stream) : launch_mode<false>(g, bits, tile, stream);
}

}  // namespace oq
