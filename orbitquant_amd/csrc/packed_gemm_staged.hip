// Packed-weight GEMM on the gfx950 matrix cores, packed operands staged in LDS.
//
//   out[m,n] = (sum_k c_a[code[m,k]] * c_w[idx[n,k]]) * scale[m] * r_w[n] + bias[n]
//
// Both operands stay packed all the way into the CU: the workgroup copies a
// [tile rows x KS] slab of 4-bit activation codes and of 2/3/4/6/8-bit weight
// indices from global memory into LDS with fully coalesced 16-byte loads
// (register-staged, double-buffered, one barrier per slab), each wavefront then
// reads the runs of its own rows from LDS, decodes them through the replicated
// lookup tables (packed_decode.h) into bf16 operands and issues
// v_mfma_f32_32x32x16_bf16.  A dequantized operand never exists in memory.
//
// K order inside a K-step of 64 is the one described in packed_gemm.hip: lane
// group g owns values k0+32g .. k0+32g+31 of its row, MFMA q uses 8q .. 8q+7.
//
// LDS rows are padded to an odd number of 16-byte units so that the 16 lanes a
// ds_read_b128 serves per cycle fall into distinct bank groups.
#include "gemm_epilogue.h"

namespace oq {
namespace {

struct StagedArgs {
  const uint8_t *a;          // [M, K/2] nibble codes
  const float *row_scale;    // [M] or NULL
  const float *act_cents;
  int a_levels;
  const uint8_t *w;
  const uint16_t *row_norms;
  const float *w_cents;
  const void *bias;
  int bias_dtype;
  int64_t M, N, K;
  void *out;
  int out_dtype;
  int tiles_m, tiles_n;
};

constexpr int odd16(int bytes) { return ((bytes / 16) & 1) ? bytes : bytes + 16; }

template <int BITS>
__device__ __forceinline__ void read_w_run(const unsigned char *p, uint32_t (&w)[BITS]) {
  if constexpr (BITS == 4) {
    const uint4 v = *reinterpret_cast<const uint4 *>(p);
    w[0] = v.x; w[1] = v.y; w[2] = v.z; w[3] = v.w;
  } else if constexpr (BITS == 2) {
    const uint2 v = *reinterpret_cast<const uint2 *>(p);
    w[0] = v.x; w[1] = v.y;
  } else if constexpr (BITS == 8) {
    const uint4 v0 = reinterpret_cast<const uint4 *>(p)[0], v1 = reinterpret_cast<const uint4 *>(p)[1];
    w[0] = v0.x; w[1] = v0.y; w[2] = v0.z; w[3] = v0.w; w[4] = v1.x; w[5] = v1.y; w[6] = v1.z; w[7] = v1.w;
  } else if constexpr (BITS == 6) {
    const uint2 *d = reinterpret_cast<const uint2 *>(p);
#pragma unroll
    for (int i = 0; i < 3; ++i) { const uint2 v = d[i]; w[2 * i] = v.x; w[2 * i + 1] = v.y; }
  } else {
    const uint32_t *d = reinterpret_cast<const uint32_t *>(p);
#pragma unroll
    for (int i = 0; i < BITS; ++i) w[i] = d[i];
  }
}

template <int BITS, int FM, int FN, int KS>
__global__ __launch_bounds__(256) void packed_gemm_staged_kernel(StagedArgs g) {
  constexpr int TM = 64 * FM, TN = 64 * FN;
  constexpr int A_ROW = KS / 2, W_ROW = KS * BITS / 8;        // slab bytes per row
  constexpr int A_PITCH = odd16(A_ROW), W_PITCH = odd16(W_ROW);
  constexpr int A_CH = A_ROW / 16, W_CH = W_ROW / 16;        // 16-byte chunks per row
  constexpr int A_CHUNKS = TM * A_CH, W_CHUNKS = TN * W_CH;
  constexpr int A_PER_T = (A_CHUNKS + 255) / 256, W_PER_T = (W_CHUNKS + 255) / 256;
  constexpr int A_BUF = TM * A_PITCH, W_BUF = TN * W_PITCH;
  constexpr int JSTEPS = KS / 64;

  extern __shared__ __align__(16) uint32_t lds[];
  uint32_t *wlut = lds;
  uint32_t *alut = lds + WLut<BITS>::kDwords;
  unsigned char *abuf = reinterpret_cast<unsigned char *>(alut + kALutDwords);  // [2][A_BUF]
  unsigned char *wbuf = abuf + 2 * A_BUF;                                        // [2][W_BUF]

  fill_lut(wlut, g.w_cents, BITS, 1 << BITS, WLut<BITS>::kPair, false);
  fill_lut(alut, g.act_cents, 4, g.a_levels, true, false);

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
  const uint32_t abase = lds_byte_address(alut) + 4 * r;
  const int64_t m0 = static_cast<int64_t>(pid_m) * TM, n0 = static_cast<int64_t>(pid_n) * TN;
  const int wm = (wave >> 1) * (FM * 32), wn = (wave & 1) * (FN * 32);

  EpiFactors<FM> epi;
  gemm_epilogue_prefetch<FM>(epi, m0, n0, wm, TN, tid, g.M, g.N, g.row_scale, g.row_norms, g.bias, g.bias_dtype);

  // ---- loader assignment: chunk c = tid + 256*i -> (row c / CH, 16-byte chunk c % CH) ----
  const int64_t a_row_bytes = g.K / 2, w_row_bytes = g.K * BITS / 8;
  const uint8_t *a_src[A_PER_T];
  const uint8_t *w_src[W_PER_T];
  int a_dst[A_PER_T], w_dst[W_PER_T];
#pragma unroll
  for (int i = 0; i < A_PER_T; ++i) {
    const int c = tid + 256 * i, row = c / A_CH, ch = c % A_CH;
    a_src[i] = g.a + min(m0 + row, g.M - 1) * a_row_bytes + ch * 16;
    a_dst[i] = (c < A_CHUNKS) ? row * A_PITCH + ch * 16 : -1;
  }
#pragma unroll
  for (int i = 0; i < W_PER_T; ++i) {
    const int c = tid + 256 * i, row = c / W_CH, ch = c % W_CH;
    w_src[i] = g.w + min(n0 + row, g.N - 1) * w_row_bytes + ch * 16;
    w_dst[i] = (c < W_CHUNKS) ? row * W_PITCH + ch * 16 : -1;
  }

  uint4 sa[A_PER_T], sw[W_PER_T];
  auto fetch = [&](int slab) {
#pragma unroll
    for (int i = 0; i < A_PER_T; ++i)
      if (a_dst[i] >= 0) sa[i] = *reinterpret_cast<const uint4 *>(a_src[i] + static_cast<int64_t>(slab) * A_ROW);
#pragma unroll
    for (int i = 0; i < W_PER_T; ++i)
      if (w_dst[i] >= 0) sw[i] = *reinterpret_cast<const uint4 *>(w_src[i] + static_cast<int64_t>(slab) * W_ROW);
  };
  auto stash = [&](int buf) {
#pragma unroll
    for (int i = 0; i < A_PER_T; ++i)
      if (a_dst[i] >= 0) *reinterpret_cast<uint4 *>(abuf + buf * A_BUF + a_dst[i]) = sa[i];
#pragma unroll
    for (int i = 0; i < W_PER_T; ++i)
      if (w_dst[i] >= 0) *reinterpret_cast<uint4 *>(wbuf + buf * W_BUF + w_dst[i]) = sw[i];
  };

  f32x16 acc[FM][FN];
#pragma unroll
  for (int i = 0; i < FM; ++i)
#pragma unroll
    for (int j = 0; j < FN; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.0f;

  const int slabs = static_cast<int>(g.K / KS);
  fetch(0);
  stash(0);
  if (slabs > 1) fetch(1);

  for (int s = 0; s < slabs; ++s) {
    __syncthreads();  // slab s is in buffer s&1 (and the tables, first time round)
    const unsigned char *ab = abuf + (s & 1) * A_BUF + (wm + r) * A_PITCH + grp * 16;
    const unsigned char *wb = wbuf + (s & 1) * W_BUF + (wn + r) * W_PITCH + grp * (4 * BITS);
#pragma unroll
    for (int js = 0; js < JSTEPS; ++js) {
      uint4 a_raw[FM];
      uint32_t w_raw[FN][BITS];
#pragma unroll
      for (int i = 0; i < FM; ++i)
        a_raw[i] = *reinterpret_cast<const uint4 *>(ab + i * 32 * A_PITCH + js * 32);
#pragma unroll
      for (int j = 0; j < FN; ++j) read_w_run<BITS>(wb + j * 32 * W_PITCH + js * (8 * BITS), w_raw[j]);
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        uint4 af[FM], bf[FN];
#pragma unroll
        for (int i = 0; i < FM; ++i) {
          const uint32_t f = q == 0 ? a_raw[i].x : q == 1 ? a_raw[i].y : q == 2 ? a_raw[i].z : a_raw[i].w;
          af[i] = decode_a_nibble(f, abase);
        }
#pragma unroll
        for (int j = 0; j < FN; ++j) bf[j] = decode_w<BITS>(w_raw[j], q, wbase);
#pragma unroll
        for (int i = 0; i < FM; ++i)
#pragma unroll
          for (int j = 0; j < FN; ++j)
            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, bf[j]),
                                                                __builtin_bit_cast(bf16x8, af[i]), acc[i][j], 0, 0, 0);
      }
    }
    if (s + 1 < slabs) {
      stash((s + 1) & 1);  // every wave finished reading that buffer before it passed this slab's barrier
      if (s + 2 < slabs) fetch(s + 2);
    }
  }

  __syncthreads();  // tables and staging buffers are dead: LDS is reused by the epilogue
  gemm_epilogue<FM, FN>(acc, m0, n0, wm, wn, TN, tid, g.M, g.N, g.row_scale, g.row_norms, g.bias, g.bias_dtype, epi, g.out,
                        g.out_dtype, reinterpret_cast<unsigned char *>(lds));
}

template <int BITS, int FM, int FN, int KS>
int launch_cfg(StagedArgs g, hipStream_t stream) {
  constexpr int TM = 64 * FM, TN = 64 * FN;
  g.tiles_m = static_cast<int>((g.M + TM - 1) / TM);
  g.tiles_n = static_cast<int>((g.N + TN - 1) / TN);
  const int64_t total = static_cast<int64_t>(g.tiles_m) * g.tiles_n;
  if (total > 0x7fffffffLL) return fail(OQ_ERR_UNSUPPORTED, "packed_gemm: too many tiles");
  size_t smem = (WLut<BITS>::kDwords + kALutDwords) * sizeof(uint32_t) +
                      2 * (static_cast<size_t>(TM) * odd16(KS / 2) + static_cast<size_t>(TN) * odd16(KS * BITS / 8));
  if (smem < static_cast<size_t>(kEpiLdsBytes)) smem = kEpiLdsBytes;  // the epilogue reuses LDS
  auto kern = packed_gemm_staged_kernel<BITS, FM, FN, KS>;
  if (smem > 160 * 1024) return fail(OQ_ERR_UNSUPPORTED, "packed_gemm: tile needs %zu bytes of LDS", smem);
  if (smem > 48 * 1024) {
    if (hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                            static_cast<int>(smem)) != hipSuccess)
      return fail(OQ_ERR_LAUNCH, "packed_gemm: cannot reserve %zu bytes of LDS", smem);
  }
  hipLaunchKernelGGL(kern, dim3(static_cast<unsigned>(total)), dim3(256), smem, stream, g);
  return check_launch("packed_gemm_staged");
}

template <int BITS>
int launch_bits(const StagedArgs &g, int tile, hipStream_t stream) {
  // 8-bit indices: the 256x256 tile's staging buffers do not fit in 160 KB of LDS
  if (tile == 2 && BITS < 8) return launch_cfg<BITS, 4, 4, 128>(g, stream);
  if (tile >= 1) return launch_cfg<BITS, 2, 4, 128>(g, stream);
  return launch_cfg<BITS, 2, 2, 128>(g, stream);
}

}  // namespace

bool gemm_staged_supported(int64_t K, int bits) {
  return K % 128 == 0 && (bits == 2 || bits == 3 || bits == 4 || bits == 6 || bits == 8);
}

int gemm_staged_dispatch(const void *codes, const float *row_scale, const float *act_cents, int a_levels,
                         const uint8_t *w, int bits, const uint16_t *row_norms, const float *w_cents,
                         const void *bias, int bias_dtype, int64_t M, int64_t N, int64_t K, void *out,
                         int out_dtype, int tile, hipStream_t stream) {
  StagedArgs g{};
  g.a = static_cast<const uint8_t *>(codes); g.row_scale = row_scale; g.act_cents = act_cents; g.a_levels = a_levels;
  g.w = w; g.row_norms = row_norms; g.w_cents = w_cents; g.bias = bias; g.bias_dtype = bias_dtype;
  g.M = M; g.N = N; g.K = K; g.out = out; g.out_dtype = out_dtype;
  switch (bits) {
    case 2: return launch_bits<2>(g, tile, stream);
    case 3: return launch_bits<3>(g, tile, stream);
    case 4: return launch_bits<4>(g, tile, stream);
    case 6: return launch_bits<6>(g, tile, stream);
    case 8: return launch_bits<8>(g, tile, stream);
    default: return fail(OQ_ERR_UNSUPPORTED, "packed_gemm: weight width %d", bits);
  }
}

}  // namespace oq
