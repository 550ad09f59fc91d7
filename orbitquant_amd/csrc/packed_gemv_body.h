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
//
// Lookup tables: the 64 KB block of 256-byte rows the tiled GEMM uses (weight
// entry e 32 times in bytes 0..127 of row e, activation entry e in bytes
// 128..255; lane l reads copy l%32, a byte-indexed lookup is one v_perm_b32 plus
// one ds_read_b32).  The packed stream is requested first thing (right behind the few epilogue
// operands, which are not touched before the epilogue); the tables are
// built meanwhile from centroids fetched with SCALAR loads, which do not queue
// behind the vector loads of the stream, and spread over the lanes so that every lane can pick the two values of its table entry with
// wavefront shuffles.  After the main loop the same LDS holds the partial sums.
//
// The kernel body is a device function here, shared by the plain small-M kernel
// (packed_gemv.hip) and by the one-token linear that quantizes its input in the same launch.
#pragma once

#include <stdio.h>
#include <stdlib.h>

#include <type_traits>

#include "packed_decode.h"

namespace oq {
namespace gemv {

struct GemvArgs {
  const uint8_t *a;          // activation codes: [M, K/2] two per byte, or [M, K] one per byte
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

constexpr int kDepth = 1;  // K-steps of 128 fetched per batch of global loads (two batches in flight: decode of one overlaps the stream of the next)
constexpr int kGemvTableBytes = kRowTableBytes;

// Wavefronts per workgroup (= ways K is split).  When the whole launch is at most one workgroup
// per CU (N <= 4096 with 16 rows each) eight wavefronts leave the CU's memory pipeline half
// empty; sixteen measured 14-17 % faster there (4096x4096: 6.9 -> 5.9 us, 4096x14336:
// 13.6 -> 11.3 us).  Rows shorter than 2048 do not have sixteen K-steps' worth of work.
// The one-token kernel uses the same rule, so that both give the same sums.
inline int gemv_waves(int64_t N, int64_t K) { return N <= 16 * 256 && K >= 2048 ? 16 : 8; }

// Tokens up to which the streaming kernel is taken (beyond: the tile kernel).  OQ_GEMV_MAX_M
// (16, 32 or 64) overrides, for comparisons.
inline int gemv_max_tokens() {
  if (const char *v = debug_env(ENV_GEMV_MAX_M)) {
    const int m = atoi(v);
    if (m == 16 || m == 32 || m == 64) return m;
  }
  return 64;
}

// Whether a launch on nibble codes decodes the activation values once per workgroup (ASTAGE
// below): they must fit the activation half of the table block.  OQ_GEMV_NO_ASTAGE keeps the
// lookups, for comparisons.
inline bool gemv_stages_activations(int64_t M, int64_t K) {
  return M * K <= 16384 && debug_env(ENV_GEMV_NO_ASTAGE) == nullptr;
}

// BYTES: activation codes come one per byte (widths above 4 bits) instead of two per byte.
// LATE: the activation codes and their row scales do not exist yet when the kernel starts;
// `produce(issue_weights)`, called by every thread, writes them and calls `issue_weights()`
// once, at the point from which it no longer waits for loads of its own (a wavefront's loads
// return in order: requested earlier, the weights would hold up everything `produce` reads).
// The lookup tables are built before that, so their construction also overlaps it.
// `lds` is the kernel's table block (OQ_GEMV_TABLE_BLOCK: declared by the kernel, not here, so
// that a kernel holding several instances of this body has one block and not one per instance);
// `group` numbers the workgroup's 16*R rows within the matrix (blockIdx.x in a launch of one
// matrix).
#define OQ_GEMV_TABLE_BLOCK(name) \
  __shared__ __attribute__((aligned(65536))) uint32_t name[::oq::gemv::kGemvTableBytes / 4]

//
// ASTAGE (nibble codes, M*K <= 16384): the activation VALUES are decoded once per workgroup and
// parked in the activation half of the table block (row c, bytes 128..255 = values 64c..64c+63 of
// the [M, K] activations as bf16), which an operand of eight consecutive values reads back with
// ONE 16-byte LDS read (lanes of the same token row read the same address) in place of four
// table lookups and their address arithmetic: a third of the kernel's LDS time at two row blocks
// per wavefront.  The values are the table's (the same conversion of the same centroids), so
// the sums do not change.
constexpr int64_t kStageValues = 16384;  // 256 rows x 64 values

//
// MB: blocks of sixteen token rows (M <= 16*MB).  Every decoded weight operand feeds MB matrix
// instructions, one per block, each with its own activation operand and accumulators; a token
// row's sums are the same whatever MB is.  Launches of 17 to 64 tokens stream the weights once
// this way instead of taking the tile kernel, whose 128-row tiles are mostly padding there and
// whose grid is too small for short-and-long matrices.
template <bool BYTES, int BITS, int R, int WAVES, bool LATE, bool ASTAGE = false, int MB = 1, typename Produce>
__device__ __forceinline__ void packed_gemv_body(const GemvArgs &g, uint32_t *lds, int64_t group, Produce produce) {
  static_assert(!ASTAGE || (!BYTES && !LATE), "staged activation values: nibble codes that exist at launch");
  static_assert(MB == 1 || (!ASTAGE && !LATE), "several row blocks: plain launches with table lookups");
  static_assert(R * MB <= WAVES, "every epilogue item (64 per row block and row step) needs a thread");
  constexpr int kAVec = BYTES ? 2 : 1;      // 16-byte loads of activation codes per lane and K-step
  constexpr int kAStep = 64 * kAVec;        // bytes of one activation row per K-step of 128
  static_assert(WAVES * MB * R * 64 * 16 <= kGemvTableBytes, "partial sums reuse the table block");
  float *partial = reinterpret_cast<float *>(lds);  // [WAVES][MB][R][64][4], after the main loop

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int r = lane & 15, grp = lane >> 4;
  const uint32_t lds_base = lds_byte_address(lds);  // a multiple of 65536 by the alignment
  const uint32_t w_off = lds_base + 4 * (lane & 31), a_off = lds_base + 128 + 4 * (lane & 31);
  const int64_t n_base = group * (16 * R);

  const int steps = static_cast<int>(g.K / 128);
  const int s_begin = static_cast<int>(static_cast<int64_t>(steps) * wave / WAVES);
  const int s_end = static_cast<int>(static_cast<int64_t>(steps) * (wave + 1) / WAVES);

  const int64_t w_row_bytes = g.K * BITS / 8;
  const uint8_t *ap[MB];
#pragma unroll
  for (int mb = 0; mb < MB; ++mb)
    ap[mb] = g.a + static_cast<int64_t>(min(16 * mb + r, g.M - 1)) * (BYTES ? g.K : g.K / 2) + grp * (16 * kAVec);
  const uint8_t *wp[R];
#pragma unroll
  for (int j = 0; j < R; ++j) {
    const int64_t row = min(n_base + 16 * j + r, g.N - 1);
    wp[j] = g.w + row * w_row_bytes + grp * (4 * BITS);
  }

  // a batch = kDepth K-steps: every load of the batch is issued before anything waits on it
  struct Batch {
    uint4 a[kDepth][MB][kAVec];
    uint32_t w[kDepth][R][BITS];
  };
  auto fetch_a = [&](int s0, Batch &bt) {
    if constexpr (ASTAGE) return;
#pragma unroll
    for (int d = 0; d < kDepth; ++d) {
      const int s = max(min(s0 + d, s_end - 1), 0);  // clamped: stays inside the row, result unused
#pragma unroll
      for (int mb = 0; mb < MB; ++mb)
#pragma unroll
        for (int v = 0; v < kAVec; ++v)
          bt.a[d][mb][v] = *reinterpret_cast<const uint4 *>(ap[mb] + static_cast<int64_t>(s) * kAStep + 16 * v);
    }
  };
  auto fetch_w = [&](int s0, Batch &bt) {
#pragma unroll
    for (int d = 0; d < kDepth; ++d) {
      const int s = max(min(s0 + d, s_end - 1), 0);
#pragma unroll
      for (int j = 0; j < R; ++j) load_w<BITS>(wp[j] + static_cast<int64_t>(s) * (16 * BITS), bt.w[d][j]);
    }
  };
  auto fetch = [&](int s0, Batch &bt) {
    fetch_a(s0, bt);
    fetch_w(s0, bt);
  };

  // ASTAGE: the codes this thread decodes (groups of eight values, 4 bytes; requested before
  // everything else so that they are not queued behind the stream), and the address of the lane's
  // operand of K-step 0, MFMA 0: value (row, 32*grp) of the staged activations.
  constexpr int kStageIters = ASTAGE ? static_cast<int>(kStageValues / 8) / (64 * WAVES) : 1;
  uint32_t stage_codes[kStageIters];
  const int stage_groups = ASTAGE ? g.M * static_cast<int>(g.K / 8) : 0;
  uint32_t a_stage = 0;
  // ... and, with them, the centroids this lane's table rows and its decode of the codes need (vector loads,
  // branch-free: requested here they arrive with the codes, ahead of the stream; fetched where the
  // tables are built they were a second memory round trip between the first loads and the first decode)
  constexpr bool kRowsDirect = ASTAGE && BITS <= 4;
  float w_row_lo[8], w_row_hi[8];
  float a_tab_early = 0.0f;
  if constexpr (ASTAGE) {
#pragma unroll
    for (int i = 0; i < kStageIters; ++i)
      stage_codes[i] = reinterpret_cast<const uint32_t *>(g.a)[min(tid + i * 64 * WAVES, stage_groups - 1)];
    a_tab_early = g.act_cents[min(lane & 15, g.a_levels - 1)];
    if constexpr (kRowsDirect) request_w_rows<BITS, WAVES>(w_row_lo, w_row_hi, g.w_cents);
    const uint32_t v0 = static_cast<uint32_t>(min(r, g.M - 1)) * static_cast<uint32_t>(g.K) + 32u * grp;
    a_stage = lds_base + 128u + ((v0 >> 6) << 8) + ((v0 & 63u) << 1);
  }

  f32x4 acc[MB][R];
#pragma unroll
  for (int mb = 0; mb < MB; ++mb)
#pragma unroll
    for (int j = 0; j < R; ++j) acc[mb][j] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
  auto consume = [&](int s0, const Batch &bt, auto guarded) {
#pragma unroll
    for (int d = 0; d < kDepth; ++d) {
      if (!decltype(guarded)::value || s0 + d < s_end) {
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          uint4 af[MB];
#pragma unroll
          for (int mb = 0; mb < MB; ++mb) {
            if constexpr (ASTAGE) {
              af[mb] = lds_read_u128(a_stage + static_cast<uint32_t>(s0 + d) * 512u + q * 16);
            } else if constexpr (!BYTES) {
              const uint4 v = bt.a[d][mb][0];
              af[mb] = decode_bytes(q == 0 ? v.x : q == 1 ? v.y : q == 2 ? v.z : v.w, a_off);
            } else {  // eight single-code lookups (value in both halves), merged two by two
              const uint4 v = bt.a[d][mb][q >> 1];
              const uint4 e0 = decode_bytes((q & 1) ? v.z : v.x, a_off), e1 = decode_bytes((q & 1) ? v.w : v.y, a_off);
              af[mb] = make_uint4(__builtin_amdgcn_perm(e0.y, e0.x, 0x07060100u), __builtin_amdgcn_perm(e0.w, e0.z, 0x07060100u),
                                  __builtin_amdgcn_perm(e1.y, e1.x, 0x07060100u), __builtin_amdgcn_perm(e1.w, e1.z, 0x07060100u));
            }
          }
#pragma unroll
          for (int j = 0; j < R; ++j) {
            uint4 bf;
            if constexpr (BITS == 4) bf = decode_bytes(bt.w[d][j][q], w_off);
            else bf = decode_w<BITS, 6>(bt.w[d][j], q, w_off);
#pragma unroll
            for (int mb = 0; mb < MB; ++mb)
              acc[mb][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, af[mb]),
                                                                   __builtin_bit_cast(bf16x8, bf), acc[mb][j], 0, 0, 0);
          }
        }
      }
    }
  };

  // Epilogue operands of the item this thread will finish (item = tid when tid < 64*R*MB: row
  // block tid / (64*R), row step (tid / 64) % R, accumulator lane tid % 64).  They
  // are requested BEFORE the stream, by every thread, without a branch (clamped indices, a
  // readable stand-in address for an absent operand) and stay untouched, as raw bits, until the
  // epilogue.  A wavefront's loads return in order: a use of one of these values before the main
  // loop - a conversion, or the register copy behind a value that is only loaded on one side of
  // a branch - waits for every weight load issued before it, and did: the wavefronts that own
  // an item used to start their table build only when their first weights had arrived.
  const int ep_mb = (tid >> 6) / R, ep_j = (tid >> 6) % R, ep_l = tid & 63;
  const int64_t ep_n = n_base + 16 * ep_j + (ep_l & 15);
  const int64_t ep_nc = min(ep_n, g.N - 1);
  const bool has_bias = g.bias != nullptr, has_scale = !LATE && g.row_scale != nullptr;
  const int bias_size = has_bias ? dtype_size(g.bias_dtype) : 2;
  const uint8_t *bias_at = (has_bias ? static_cast<const uint8_t *>(g.bias) : reinterpret_cast<const uint8_t *>(g.row_norms)) + ep_nc * bias_size;
  const uint32_t ep_rn_bits = g.row_norms[ep_nc];
  const uint32_t ep_bias_lo = *reinterpret_cast<const uint16_t *>(bias_at);
  const uint32_t ep_bias_hi = *reinterpret_cast<const uint16_t *>(bias_at + (bias_size - 2));
  const float *scale_at = has_scale ? g.row_scale : g.w_cents;
  float ep_sc_raw[4];
#pragma unroll
  for (int e = 0; e < 4; ++e) ep_sc_raw[e] = scale_at[has_scale ? min(16 * ep_mb + 4 * (ep_l >> 4) + e, g.M - 1) : 0];

  // ---- then the packed stream ------------------------------------------------------
  // Batches in flight: two for the plain stream (decode of one overlaps the loads of the next);
  // four when the activations come late, so that more of the weights are on their way while
  // they are being produced (a wavefront's whole share for K up to 4096; with sixteen
  // wavefronts two batches already are).
  constexpr int NB = LATE && WAVES < 16 ? 4 : 2;  // sixteen wavefronts: half the K-steps each, and half the registers
  Batch b[NB];
  auto issue_weights = [&] {
#pragma unroll
    for (int i = 0; i < NB; ++i) fetch_w(s_begin + i * kDepth, b[i]);
  };
  if constexpr (!LATE) {
#pragma unroll
    for (int i = 0; i < NB; ++i) fetch(s_begin + i * kDepth, b[i]);
  }

  // ---- tables (built while the stream is in flight) ---------------------------------------
  if constexpr (kRowsDirect) {
    __builtin_amdgcn_sched_barrier(0);  // nothing that waits for a value above the requests
    write_w_rows<BITS, WAVES>(lds, w_row_lo, w_row_hi);
  } else {
    build_row_tables<BITS, WAVES, BYTES, ASTAGE>(lds, g.w_cents, g.act_cents, g.a_levels);
  }
  if constexpr (ASTAGE) {
    const float a_tab = (lane & 15) < g.a_levels ? a_tab_early : 0.0f;  // centroid l % 16 in lane l (codes past the table read zero)
#pragma unroll
    for (int i = 0; i < kStageIters; ++i) {
      if (i * 64 * WAVES >= stage_groups) break;  // the same for every thread
      const int j = tid + i * 64 * WAVES;
      uint32_t d[4];
#pragma unroll
      for (int b = 0; b < 4; ++b) {  // every lane shuffles (a lane past the end decodes a clamped word and drops it)
        const uint32_t byte = (stage_codes[i] >> (8 * b)) & 0xffu;
        d[b] = pack16(__shfl(a_tab, static_cast<int>(byte & 15u)), __shfl(a_tab, static_cast<int>(byte >> 4)), false);
      }
      if (j < stage_groups) {
        const uint32_t v = 8u * static_cast<uint32_t>(j);
        *reinterpret_cast<uint4 *>(reinterpret_cast<unsigned char *>(lds) + 128u + ((v >> 6) << 8) + ((v & 63u) << 1)) =
            make_uint4(d[0], d[1], d[2], d[3]);
      }
    }
  }
  if constexpr (LATE) {
    produce(issue_weights);
    __syncthreads();
#pragma unroll
    for (int i = 0; i < NB; ++i) fetch_a(s_begin + i * kDepth, b[i]);
  } else {
    __syncthreads();
  }

  // Every fetch is issued unconditionally (past the end of the wavefront's share it re-reads
  // its last K-step, which the caches hold): the number of loads in flight is then the same on
  // every path through the loop, and the wait before a batch is consumed is for that batch
  // only.  With a fetch under a condition the compiler has to wait for every outstanding load
  // at the top of the loop, and the stream stops while a batch is decoded.
  int s = s_begin;
  for (; s + NB * kDepth < s_end; s += NB * kDepth) {
#pragma unroll
    for (int i = 0; i < NB; ++i) {
      consume(s + i * kDepth, b[i], std::false_type{});
      __builtin_amdgcn_sched_barrier(0);  // keep the refill right behind its batch's decode
      fetch(s + (NB + i) * kDepth, b[i]);
      __builtin_amdgcn_sched_barrier(0);
    }
  }
#pragma unroll
  for (int i = 0; i < NB; ++i) consume(s + i * kDepth, b[i], std::true_type{});

  // ---- cross-wave sum in LDS (the tables are dead), fixed order ------------------------
  __syncthreads();
#pragma unroll
  for (int mb = 0; mb < MB; ++mb)
#pragma unroll
    for (int j = 0; j < R; ++j)
      *reinterpret_cast<float4 *>(partial + (((wave * MB + mb) * R + j) * 64 + lane) * 4) =
          make_float4(acc[mb][j][0], acc[mb][j][1], acc[mb][j][2], acc[mb][j][3]);
  __syncthreads();
  // accumulator e of lane l in row block mb: token row 16*mb + 4*(l/16) + e, weight row l%16
  if (tid < 64 * R * MB && ep_n < g.N) {
    const int ep_item = ep_mb * R + ep_j;
    float4 sum = *reinterpret_cast<const float4 *>(partial + (ep_item * 64 + ep_l) * 4);
    for (int w = 1; w < WAVES; ++w) {
      const float4 p = *reinterpret_cast<const float4 *>(partial + ((w * MB * R + ep_item) * 64 + ep_l) * 4);
      sum.x += p.x; sum.y += p.y; sum.z += p.z; sum.w += p.w;
    }
    const float v[4] = {sum.x, sum.y, sum.z, sum.w};
    const float ep_rn = bf16_bits_to_f32(static_cast<uint16_t>(ep_rn_bits));
    const float ep_bv = has_bias ? dyn_bits_to_f32(bias_size == 4 ? (ep_bias_lo | (ep_bias_hi << 16)) : ep_bias_lo, g.bias_dtype) : 0.0f;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const int m = 16 * ep_mb + 4 * (ep_l >> 4) + e;
      if (m >= g.M) continue;
      float sc = has_scale ? ep_sc_raw[e] : 1.0f;
      if constexpr (LATE) {  // produced by this launch: read where it is used
        if (g.row_scale != nullptr) sc = g.row_scale[m];
      }
      const float y = v[e] * sc * ep_rn + ep_bv;
      const int64_t o = static_cast<int64_t>(m) * g.N + ep_n;
      if (g.out_dtype == OQ_BF16) static_cast<uint16_t *>(g.out)[o] = f32_to_bf16_bits(y);
      else if (g.out_dtype == OQ_F16) static_cast<uint16_t *>(g.out)[o] = f32_to_f16_bits(y);
      else static_cast<float *>(g.out)[o] = y;
    }
  }
}

}  // namespace gemv
}  // namespace oq
