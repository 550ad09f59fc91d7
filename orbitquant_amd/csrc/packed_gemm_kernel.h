// Packed-weight GEMM on the gfx950 matrix cores: activation codes x packed weight indices.
// (Kernel template and launchers; packed_gemm.hip instantiates the two-codes-per-byte form,
// packed_gemm_bytes.hip the one-code-per-byte form, so the two compile in parallel.)
//
//   out[m,n] = (sum_k c_a[code[m,k]] * c_w[idx[n,k]]) * scale[m] * r_w[n] + bias[n]
//
// code is the stream of activation codes (two 4-bit codes per byte, or one code per byte), idx the flat little-endian bit
// stream of 2/3/4/6/8-bit weight indices, both read from HBM as they are stored.
// Nothing is dequantized to memory: every wavefront loads the packed dwords of
// its own rows straight into registers, turns them into bf16 MFMA operands
// through lookup tables held in LDS, and feeds v_mfma_f32_32x32x16_bf16.
//
// Operand layout.  One MFMA consumes, per lane, eight k-values of one row
// (lane l: row l%32, k-group l/32).  A dot product does not care in which order
// k is visited as long as both operands agree, so a K-step of 64 is cut as
//   lane group g (0/1) owns k0+32g .. k0+32g+31   (one contiguous run of bits per row)
//   MFMA q (0..3) of the step uses values 8q..8q+7 of that run
// which makes every global load of packed data one contiguous 4*bits-byte run
// per lane (16 bytes for 4-bit), with no cross-lane shuffles and no LDS staging.
//
// Lookup tables.  One 64 KB block of LDS, 256 rows of 256 bytes, placed at LDS
// address 0.  Row e holds, 32 times each, the dword of weight-table entry e
// (bytes 0..127) and of activation-table entry e (bytes 128..255); lane l reads
// copy l%32, so the lanes of a wavefront never collide on a bank whatever codes
// they hold.  The activation table and the 4-bit weight table are indexed by a
// whole byte of the packed stream (two codes) and return both bf16 values in one
// dword, and because a row is 256 bytes the LDS address of a lookup is simply
//   byte 0 = the lane's offset, byte 1 = the code byte
// which one v_perm_b32 assembles: a lookup is one VALU instruction plus one
// ds_read_b32 for two operand values.  Other weight widths index the same rows
// with a bit-field extract (pair tables for 2/3 bits, single-code for 6/8).
//
// The instruction stream of a wavefront is what bounds this kernel (per MFMA of
// 32 cycles it may issue about eight other instructions), hence the tile shapes:
// a wavefront owning FM x FN tiles of 32x32 issues 4*(FM+FN) lookups per FM*FN MFMAs.
#pragma once

#include <type_traits>

#include "gemm_epilogue.h"

namespace oq {

// Activations: codes two per byte, codes one per byte, or 16-bit values (bf16) already in the matrix
// core's operand order: 16-byte piece ((row_tile * K/64 + k_step) * 4 + q) * 64 + lane holds, for lane
// (r = lane % 32, g = lane / 32), the eight values k_step*64 + 32g + 8q .. +7 of row 32*row_tile + r
// (tile_activations_kernel writes it).  Then a wavefront's activation load is 1 KB of consecutive
// bytes, the operand needs no lookup, and only the weights go through the tables.
// A_STAGED: 16-bit values (bf16) as the caller has them, [M, K] row-major.  Every wavefront loads the 128-byte
// K-step pieces of its own FM*32 rows line by line (eight rows per load instruction), parks them in a slab of
// LDS that belongs to it alone (row pitch 144 bytes), and reads its operands back with one 16-byte LDS read per
// row tile and MFMA: no workgroup-wide staging, no barrier in the loop, no copy of the activations in memory.
enum AMode { A_NIBBLE = 0, A_U8 = 1, A_TILED = 2, A_STAGED = 3 };

struct GemmArgs {
  const uint8_t *a;          // [M, K/2] nibble codes, [M, K] one code per byte, or the tiled 16-bit values
  const float *row_scale;    // [M] or NULL
  const float *act_cents;    // [a_levels]
  int a_levels;
  const uint8_t *w;          // packed index stream
  const uint16_t *row_norms; // bf16 [N]
  const float *w_cents;      // [2^bits]
  const void *bias;
  int bias_dtype;
  int64_t M, N, K;
  void *out;
  int out_dtype;
  OutMap out_map;            // optional elementwise function of the outputs (gemm_epilogue.h)
  int tiles_m, tiles_n;
  // K shared between workgroups (grid.y = k_splits > 1; code activations, KSPLIT = 1 only): every
  // workgroup writes its raw fp32 partial tile to partials[blockIdx.y][M][N]; packed_gemm_splitk.hip
  // adds them up and applies the epilogue.
  int k_splits;
  float *partials;
  int window_ahead;          // the launch has kWideBytes of dynamic LDS for the output map's window (set by launch_cfg)
  // Builds with -DOQ_GEMM_STAMPS only: every wavefront writes the shader-clock and real-time counter
  // values it read at its phase boundaries to stamps[(workgroup * 4 + wavefront) * 16 ...] (NULL: none).
  uint64_t *stamps;
};


namespace {

constexpr int kTableBytes = kRowTableBytes;
static_assert(kEpiLdsBytes <= kTableBytes, "the epilogue reuses the table block");

// Workgroup = 4 wavefronts; each wavefront owns FM x FN MFMA tiles of 32x32.
//   KSPLIT = 1: the wavefronts sit 2x2 on a [64 FM x 64 FN] output tile, each runs over all of K.
//   KSPLIT = 4: all four work on the SAME [32 FM x 32 FN] output tile, each over a quarter of K
//               (for short-and-wide problems whose output has too few tiles to fill the chip);
//               the partial tiles are then summed through LDS in a fixed order, each wavefront
//               ending up with one 32-row slice of the tile, which it scales and stores.  FM = 4.
// NBUF = K-steps of packed operands held in registers (NBUF-1 of them in flight from memory).
template <int AM, int BITS, int FM, int FN, int KSPLIT = 1, int NBUF = (FM * FN >= 12 ? 2 : 3)>
__global__ __launch_bounds__(256) void packed_gemm_kernel(const float *w_cents, const float *act_cents, const uint8_t *a_codes,
                                                          const uint8_t *w_packed, const uint16_t *map_table, int K32, int M32,
                                                          int N32, int levels_splits, GemmArgs rest) {
  static_assert(KSPLIT == 1 || (KSPLIT == 4 && FM == 4), "K split: four wavefronts, four row slices");
  // What the first loads need comes as leading scalar arguments: the first fourteen dwords of a kernel's
  // arguments are handed over in scalar registers when a wavefront starts (the build asks for that with
  // -mllvm -amdgpu-kernarg-preload-count=16), so centroids and packed operands are requested without
  // waiting for a load of the argument block; the struct behind them is read for the epilogue's operands.
  GemmArgs g = rest;
  g.w_cents = w_cents; g.act_cents = act_cents; g.a = a_codes; g.w = w_packed;
  g.K = K32; g.M = M32; g.N = N32;
  g.a_levels = levels_splits & 0xffff; g.k_splits = (levels_splits >> 16) & 0xff; g.window_ahead = (levels_splits >> 24) & 1;
  g.out_map.table = map_table;
  {  // (tile counts from the sizes: two divisions by constants instead of two more arguments)
    constexpr int kTM = (KSPLIT == 1 ? 2 : 1) * FM * 32, kTN = (KSPLIT == 1 ? 2 : 1) * FN * 32;
    g.tiles_m = (M32 + kTM - 1) / kTM;
    g.tiles_n = (N32 + kTN - 1) / kTN;
  }
  __shared__ __attribute__((aligned(65536))) uint32_t lds[kTableBytes / 4];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int r = lane & 31, grp = lane >> 5;
#ifdef OQ_GEMM_STAMPS
  uint64_t stamp[8], stamp_extra[6] = {0, 0, 0, 0, 0, 0};
  stamp[0] = __builtin_amdgcn_s_memtime();
  stamp[6] = __builtin_amdgcn_s_memrealtime();
#define OQ_STAMP(i) stamp[i] = __builtin_amdgcn_s_memtime()
#else
#define OQ_STAMP(i)
#endif

  // Loads of one wavefront return in order, and the compiler waits for a load where its value is
  // first touched.  So everything the prologue needs from memory is REQUESTED here, branch-free
  // (indices clamped into the tables, nothing loaded on one side of a branch only), in the order
  // centroids, packed operands of the first K-steps, what only the epilogue needs, and nothing is
  // looked at before the last of these requests has been issued: the tables are then written while the
  // packed data is still in flight.  (Converting a centroid where it was loaded put one memory
  // round trip per table operand in front of the first operand load of every workgroup.)
  constexpr bool kPairTables = BITS <= 4 && AM != A_U8;  // built without a lane exchange (packed_decode.h)
  constexpr bool kHasATable = AM == A_NIBBLE || AM == A_U8;
  constexpr int kWLevels = 1 << BITS;
  float seed_lo_w[4], seed_hi_w[8], seed_lo_a[4], seed_hi_a[4];
  float w_c0 = 0.0f, w_c1 = 0.0f, a_c0 = 0.0f, a_c1 = 0.0f;
  bool w_row_used = false, a_ok0 = false, a_ok1 = false;
  if constexpr (kPairTables) {
    request_pair_seed<BITS, kHasATable>(seed_lo_w, seed_hi_w, seed_lo_a, seed_hi_a, g.w_cents, g.act_cents, g.a_levels);
  } else {  // thread t holds the two dwords of row t, handed round by write_row_tables
    const int w_i0 = tid & (kWLevels - 1), w_i1 = BITS <= 4 ? (tid >> BITS) & (kWLevels - 1) : w_i0;
    w_c0 = g.w_cents[w_i0];
    w_c1 = g.w_cents[w_i1];
    w_row_used = BITS <= 4 ? tid < kWLevels * kWLevels : tid < kWLevels;
    if constexpr (AM == A_NIBBLE) {  // row = a byte of the stream = two codes
      const int c0 = tid & 15, c1 = tid >> 4;
      a_ok0 = c0 < g.a_levels;
      a_ok1 = c1 < g.a_levels;
      a_c0 = g.act_cents[min(c0, g.a_levels - 1)];
      a_c1 = g.act_cents[min(c1, g.a_levels - 1)];
    } else if constexpr (AM == A_U8) {  // row = one code, its value in both halves of the dword
      a_ok0 = a_ok1 = tid < g.a_levels;
      a_c0 = a_c1 = g.act_cents[min(tid, g.a_levels - 1)];
    }
  }
  constexpr int TM = (KSPLIT == 1 ? 2 : 1) * FM * 32, TN = (KSPLIT == 1 ? 2 : 1) * FN * 32;
  // tile order: spread consecutive workgroup ids over the 8 XCDs' private L2s in
  // contiguous chunks, then walk groups of 4 tile-rows column by column
  int bid = blockIdx.x;
  const int total = g.tiles_m * g.tiles_n;
#ifdef OQ_GEMM_STAMPS
  __asm__ volatile("" ::"s"(total));
  stamp_extra[0] = __builtin_amdgcn_s_memtime();  // kernel arguments have arrived
#endif
  if ((total & 7) == 0) bid = (bid & 7) * (total >> 3) + (bid >> 3);
  constexpr int GROUP_M = 4;
  const int width = GROUP_M * g.tiles_n;
  const int group = bid / width;
  const int first_m = group * GROUP_M;
  const int gsz = min(g.tiles_m - first_m, GROUP_M);
  const int in_group = bid - group * width;
  // (full groups, the usual case, by shifts: a division by a run-time value is some thirty instructions)
  const int pid_m = first_m + (gsz == GROUP_M ? in_group & (GROUP_M - 1) : in_group % gsz);
  const int pid_n = gsz == GROUP_M ? in_group >> 2 : in_group / gsz;
  static_assert(GROUP_M == 4);

#ifdef OQ_GEMM_STAMPS
  __asm__ volatile("" ::"s"(pid_n), "s"(pid_m));
  stamp_extra[3] = __builtin_amdgcn_s_memtime();  // centroids requested, tile mapped
#endif
  const uint32_t lds_base = lds_byte_address(lds);           // a multiple of 65536 by the alignment
  const uint32_t w_off = lds_base + 4 * r, a_off = lds_base + 128 + 4 * r;  // the lane's copy inside a table row
  const int wm = KSPLIT == 1 ? (wave >> 1) * (FM * 32) : 0, wn = KSPLIT == 1 ? (wave & 1) * (FN * 32) : 0;
  const int64_t m_base = static_cast<int64_t>(pid_m) * TM + wm;
  const int64_t n_base = static_cast<int64_t>(pid_n) * TN + wn;


  constexpr int kAStep = AM == A_NIBBLE ? 32 : AM == A_U8 ? 64 : AM == A_TILED ? 4096 : 128;  // bytes from one K-step of 64 to the next in a lane's activation stream
  constexpr int kAVec = AM == A_NIBBLE ? 1 : AM == A_U8 ? 2 : 4;        // 16-byte loads per lane per K-step
  constexpr int kAVecStride = AM == A_TILED ? 1024 : 16;
  // A_STAGED: load v of row tile e is row 32 e + 8 v + lane / 8, 16-byte chunk lane % 8 of the row's 128-byte K-step piece
  constexpr int kSlabPitch = 144, kSlabBytes = FM * 32 * kSlabPitch;
  __shared__ __attribute__((aligned(16))) unsigned char aslab[AM == A_STAGED ? 4 * kSlabBytes : 16];
  unsigned char *my_slab = aslab + (AM == A_STAGED ? wave * kSlabBytes : 0);
  uint32_t a_off32[AM == A_STAGED ? FM : 1][4];  // byte offsets from g.a (the host checks M * K * 2 < 4 GB)
  const int64_t a_row_bytes = AM == A_NIBBLE ? g.K / 2 : g.K;
  const int64_t w_row_bytes = g.K * BITS / 8;
  // (row index and row length fit 32 bits - the launcher checks the sizes - so a row's byte offset is one
  // 32 x 32 -> 64 bit multiply instead of the four quarter-rate multiplies of a 64-bit product)
  const int m_base32 = pid_m * TM + wm, n_base32 = pid_n * TN + wn;
  const uint32_t a_row_bytes32 = static_cast<uint32_t>(AM == A_NIBBLE ? K32 / 2 : K32);
  const uint32_t w_row_bytes32 = static_cast<uint32_t>(K32) * BITS / 8;
  auto row_offset = [](int row, uint32_t row_bytes) {
    return static_cast<uint64_t>(static_cast<uint32_t>(row)) * static_cast<uint64_t>(row_bytes);
  };
  const uint8_t *ap[FM];
  const uint8_t *wp[FN];
#pragma unroll
  for (int i = 0; i < FM; ++i) {
    if constexpr (AM == A_STAGED) {
      ap[i] = g.a;
#pragma unroll
      for (int v = 0; v < 4; ++v)
        a_off32[i][v] = static_cast<uint32_t>(min(m_base + 32 * i + 8 * v + (lane >> 3), g.M - 1) * (g.K * 2) + (lane & 7) * 16);
    } else if constexpr (AM == A_TILED) ap[i] = g.a + min(m_base / 32 + i, (g.M + 31) / 32 - 1) * (g.K / 64) * kAStep + lane * 16;
    else ap[i] = g.a + row_offset(min(m_base32 + 32 * i + r, M32 - 1), a_row_bytes32) + grp * (kAStep / 2);
  }
#pragma unroll
  for (int j = 0; j < FN; ++j) wp[j] = g.w + row_offset(min(n_base32 + 32 * j + r, N32 - 1), w_row_bytes32) + grp * (4 * BITS);

  // packed operands of NBUF consecutive K-steps
  uint4 pa[NBUF][FM][kAVec];
  uint32_t pw[NBUF][FN][BITS];
  int steps = static_cast<int>(g.K / 64) / KSPLIT;  // K-steps of this wavefront
  if constexpr (KSPLIT == 1 && (AM == A_NIBBLE || AM == A_U8)) {
    if (g.k_splits > 1) {  // this workgroup's share of the K-steps
      const int z = blockIdx.y;
      const int first = static_cast<int>(static_cast<int64_t>(steps) * z / g.k_splits);
      steps = static_cast<int>(static_cast<int64_t>(steps) * (z + 1) / g.k_splits) - first;
#pragma unroll
      for (int i = 0; i < FM; ++i) ap[i] += static_cast<int64_t>(first) * kAStep;
#pragma unroll
      for (int j = 0; j < FN; ++j) wp[j] += static_cast<int64_t>(first) * (8 * BITS);
    }
  }
  if constexpr (KSPLIT > 1) {
#pragma unroll
    for (int i = 0; i < FM; ++i) ap[i] += static_cast<int64_t>(wave) * steps * kAStep;  // (A_STAGED: every ap[i] is the same base)
#pragma unroll
    for (int j = 0; j < FN; ++j) wp[j] += static_cast<int64_t>(wave) * steps * (8 * BITS);
  }
  // operand `e` (A row-tile e < FM, else weight column-tile e-FM) of K-step ks into buffer B
  auto fetch_one = [&](auto buf, int e, int ks) {
    constexpr int B = decltype(buf)::value;
    const int64_t s = min(ks, steps - 1);  // past the end: re-read the last step (never multiplied)
    if (e < FM) {
#pragma unroll
      for (int v = 0; v < kAVec; ++v) {
        if constexpr (AM == A_STAGED) pa[B][e][v] = *reinterpret_cast<const uint4 *>(ap[e] + (a_off32[e][v] + static_cast<uint32_t>(s) * kAStep));
        else pa[B][e][v] = *reinterpret_cast<const uint4 *>(ap[e] + s * kAStep + kAVecStride * v);
      }
    }
    else load_w<BITS>(wp[e - FM] + s * (8 * BITS), pw[B][e - FM]);
  };
  auto fetch = [&](auto buf, int ks) {
#pragma unroll
    for (int e = 0; e < FM + FN; ++e) fetch_one(buf, e, ks);
  };
#ifdef OQ_GEMM_STAMPS
  __asm__ volatile("" ::"v"(wp[FN - 1]), "v"(ap[FM - 1]));
  __builtin_amdgcn_sched_barrier(0);
  stamp_extra[4] = __builtin_amdgcn_s_memtime();  // operand addresses computed
  __builtin_amdgcn_sched_barrier(0);
#endif
  // buffers 0..NBUF-2 <- K-steps 0..NBUF-2; K-step NBUF-1 is requested by the first step of the loop
  fetch(std::integral_constant<int, 0>{}, 0);
  if constexpr (NBUF == 3) fetch(std::integral_constant<int, 1>{}, 1);
#ifdef OQ_GEMM_STAMPS
  __builtin_amdgcn_sched_barrier(0);
  stamp_extra[5] = __builtin_amdgcn_s_memtime();  // first packed operands requested
  __builtin_amdgcn_sched_barrier(0);
#endif

  // behind the operands (a wavefront's loads return in order): what only the epilogue needs
  // The window of an output map (an activation function as a table, gemm_epilogue.h) is requested with
  // the rest and parked in LDS behind the tables (16 KB of dynamic LDS, which mapped launches ask for),
  // so that the epilogue finds it there instead of starting with a memory round trip of its own.
  extern __shared__ __attribute__((aligned(16))) unsigned char map_window[];
  const bool window_ahead = g.window_ahead != 0;  // uniform
  // (requested without a branch - a launch without a map reads the first bytes of the weights - and held as
  // native vectors: an array of the struct type would be pinned in scratch memory)
  lds_u32x4 window_piece0, window_piece1, window_piece2, window_piece3;  // written and read under the same uniform condition only
  if (window_ahead) {
    constexpr int kChunksPerSign = (2 << kWideLog2) / 16;
    const unsigned char *window_from = reinterpret_cast<const unsigned char *>(g.out_map.table + kWideLoBf16);  // (the launcher parks windows of this base only)
    auto piece = [&](int v) {
      const int i = tid + 256 * v, sign = i / kChunksPerSign, j = i % kChunksPerSign;
      return *reinterpret_cast<const lds_u32x4 *>(window_from + (sign << 16) + 16 * j);
    };
    window_piece0 = piece(0);
    window_piece1 = piece(1);
    window_piece2 = piece(2);
    window_piece3 = piece(3);
  }


  __builtin_amdgcn_sched_barrier(0);  // nothing that waits for a value may be scheduled above the requests
  // (first use of the requested values: every request above has been issued)
#ifdef OQ_GEMM_STAMPS
  stamp_extra[1] = __builtin_amdgcn_s_memtime();  // every request issued
  if constexpr (kPairTables) __asm__ volatile("" ::"v"(seed_lo_w[0]), "v"(seed_hi_w[0]), "v"(seed_lo_a[3]), "v"(seed_hi_a[3]));
  else __asm__ volatile("" ::"v"(w_c0), "v"(w_c1), "v"(a_c0), "v"(a_c1));
  stamp_extra[2] = __builtin_amdgcn_s_memtime();  // centroids have arrived
#endif
  if constexpr (kPairTables) {
    write_pair_tables<BITS, kHasATable>(lds, seed_lo_w, seed_hi_w, seed_lo_a, seed_hi_a, g.a_levels);
  } else {
    const uint32_t my_w = w_row_used ? pack16(w_c0, w_c1, false) : 0u;
    const uint32_t my_a = pack16(a_ok0 ? a_c0 : 0.0f, a_ok1 ? a_c1 : 0.0f, false);
    write_row_tables(lds, my_w, my_a);
  }
  // the epilogue's factors: their addresses come from the argument block in memory, which has arrived by now
  // (requested with the rest, they would hold the table build back until it had)
  EpiRaw<FM> epi_raw;
  gemm_epilogue_request<FM>(epi_raw, static_cast<int64_t>(pid_m) * TM, static_cast<int64_t>(pid_n) * TN, wm, tid, g.M, g.N, g.row_scale, g.row_norms, g.bias, g.bias_dtype, g.w_cents);
  if (window_ahead) {
    lds_u32x4 *dst = reinterpret_cast<lds_u32x4 *>(map_window) + tid;
    dst[0] = window_piece0;
    dst[256] = window_piece1;
    dst[512] = window_piece2;
    dst[768] = window_piece3;
  }

  f32x16 acc[FM][FN];
#pragma unroll
  for (int i = 0; i < FM; ++i)
#pragma unroll
    for (int j = 0; j < FN; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.0f;
  OQ_STAMP(1);  // tables written, first operands requested
  __syncthreads();

  // ---- main loop: software pipeline over "phases" (one MFMA k-slice of 16) -------
  // While the matrix core works on the operands looked up in the previous phase, the
  // wavefront issues the table lookups for the next one.  The instruction order is fixed by
  // hand: after every MFMA come kLook lookups (address arithmetic + LDS read), and nothing
  // may be moved across the boundary between two such groups, so the matrix core never
  // waits behind a burst of lookups and the LDS queue never runs dry.  The first phase of a
  // K-step also carries the FM+FN global loads of the K-step NBUF-1 ahead, one per group.
  //
  // One-code-per-byte activations take two lookups per operand dword (single-code table, the
  // value in both halves); the two are merged with one v_perm_b32 when the operand is used.
  constexpr int kRA = AM == A_NIBBLE ? 4 : AM == A_U8 ? 8 : AM == A_STAGED ? 1 : 0;  // LDS reads per activation tile and phase
  constexpr int kRAd = kRA > 0 ? kRA : 1;
  constexpr int kLookups = kRA * FM + 4 * FN, kGroups = FM * FN;  // group m takes lookups [m*L/G, (m+1)*L/G)
  constexpr int kLook = (kLookups + kGroups - 1) / kGroups;
  uint32_t oa[2][FM][kRAd], ob[2][FN][4];
  uint4 oa4[2][AM == A_STAGED ? FM : 1];  // A_STAGED: the whole operand comes with one 16-byte read
  const uint32_t slab_read = lds_byte_address(my_slab) + r * kSlabPitch + grp * 64;  // + 32 i * pitch + 16 q
  // K-step buffer B (its loads have arrived) into the slab; the reads of the previous K-step were issued before
  auto stash = [&](auto buf) {
    constexpr int B = decltype(buf)::value;
    if constexpr (AM == A_STAGED) {
#pragma unroll
      for (int e = 0; e < FM; ++e)
#pragma unroll
        for (int v = 0; v < 4; ++v)
        {  // (element-wise into a vector store: an aggregate copy from the register array would pin it in scratch)
          const uint4 piece = pa[B][e][v];
          *reinterpret_cast<lds_u32x4 *>(my_slab + (32 * e + 8 * v + (lane >> 3)) * kSlabPitch + (lane & 7) * 16) =
              lds_u32x4{piece.x, piece.y, piece.z, piece.w};
        }
    }
  };  // two operand sets: one being multiplied, one being looked up

  // dword d (0..7 for bytes, 0..3 for nibbles) of this lane's activation run in buffer B, tile i
  auto a_word = [&](auto buf, int i, int d) -> uint32_t {
    constexpr int B = decltype(buf)::value;
    const uint4 v = pa[B][i][d >> 2];
    return (d & 3) == 0 ? v.x : (d & 3) == 1 ? v.y : (d & 3) == 2 ? v.z : v.w;
  };
  // Lookup t of a phase, in the order the MFMAs of the next phase want their operands:
  // activation tile 0, every weight tile, then activation tiles 1..FM-1.  Split in two halves
  // so that the address of a lookup is computed one group before its LDS read is issued.
  auto lookup_address = [&](auto buf, int q, int t) -> uint32_t {
    constexpr int B = decltype(buf)::value;
    const bool is_a = t < kRA || t >= kRA + 4 * FN;
    if constexpr (kRA > 0) {
      if (is_a) {
        const int i = t < kRA ? 0 : 1 + (t - kRA - 4 * FN) / kRAd;
        const int sub = t < kRA ? t : (t - kRA - 4 * FN) % kRAd;
        if constexpr (AM == A_STAGED) return slab_read + i * (32 * kSlabPitch) + q * 16;
        else if constexpr (AM == A_NIBBLE) return row_address(a_word(buf, i, q), a_off, sub);
        else return row_address(a_word(buf, i, 2 * q + (sub >> 2)), a_off, sub & 3);  // byte 8q + sub of the run
      }
    }
    const int j = (t - kRA) >> 2, p = (t - kRA) & 3;
    if constexpr (BITS == 4) return row_address(pw[B][j][q], w_off, p);
    else return 0u;
  };
  auto lookup_read = [&](auto buf, int q, int set, int t, uint32_t address) {
    constexpr int B = decltype(buf)::value;
    const bool is_a = kRA > 0 && (t < kRA || t >= kRA + 4 * FN);
    if (is_a) {
      const int i = t < kRA ? 0 : 1 + (t - kRA - 4 * FN) / kRAd;
      const int sub = t < kRA ? t : (t - kRA - 4 * FN) % kRAd;
      if constexpr (AM == A_STAGED) oa4[set][i] = lds_read_u128(address);
      else oa[set][i][sub] = lds_read_u32(address);
    } else {
      const int j = (t - kRA) >> 2, p = (t - kRA) & 3;
      if constexpr (BITS == 4) ob[set][j][p] = lds_read_u32(address);
      else ob[set][j][p] = decode_w_piece<BITS, 6>(pw[B][j], q, p, w_off);
    }
  };
  // the activation operand of tile i out of `set`
  auto a_operand = [&](int set, int i) -> uint4 {
    if constexpr (AM == A_TILED) {
      return make_uint4(0u, 0u, 0u, 0u);  // (the operand comes straight from the load registers, see phase)
    } else if constexpr (AM == A_STAGED) {
      return oa4[set][i];
    } else if constexpr (AM == A_NIBBLE) {
      return make_uint4(oa[set][i][0], oa[set][i][1], oa[set][i][2], oa[set][i][3]);
    } else {
      return make_uint4(__builtin_amdgcn_perm(oa[set][i][1], oa[set][i][0], 0x07060100u),
                        __builtin_amdgcn_perm(oa[set][i][3], oa[set][i][2], 0x07060100u),
                        __builtin_amdgcn_perm(oa[set][i][5], oa[set][i][4], 0x07060100u),
                        __builtin_amdgcn_perm(oa[set][i][7], oa[set][i][6], 0x07060100u));
    }
  };
  // lookups of (buf, q) into `set` interleaved with the MFMAs on the other set
  // (mul_buf, mul_q): the K-step buffer and MFMA index of the operands being multiplied, i.e. of the previous phase
  auto phase = [&](auto buf, int q, int set, auto fetch_buf, int fetch_ks, bool with_fetch, auto mul_buf, auto mul_q) {
    uint32_t addr[2][kLook];
    uint4 av = make_uint4(0u, 0u, 0u, 0u);
#pragma unroll
    for (int t = 0; t < kLookups / kGroups; ++t) addr[0][t] = lookup_address(buf, q, t);
#pragma unroll
    for (int m = 0; m < kGroups; ++m) {
      const int i = m / FN, j = m % FN;
      if (j == 0) {
        if constexpr (AM == A_TILED) av = pa[decltype(mul_buf)::value][i][decltype(mul_q)::value];
        else av = a_operand(set ^ 1, i);
      }
      const int lo = m * kLookups / kGroups, hi = (m + 1) * kLookups / kGroups, hi2 = (m + 2) * kLookups / kGroups;
      if (with_fetch && m < FM + FN) fetch_one(fetch_buf, m, fetch_ks);
      const uint4 bw = make_uint4(ob[set ^ 1][j][0], ob[set ^ 1][j][1], ob[set ^ 1][j][2], ob[set ^ 1][j][3]);
      // weights first: the accumulator tile is the transposed output tile
#ifdef OQ_GEMM_I8_TIMING
      // Timing experiment only (the results are meaningless): what the loop would cost with the int8 matrix
      // instruction - half as many matrix instructions, each over twice the K, fed by the same number of lookups.
      if constexpr ((decltype(mul_q)::value & 1) == 0) {
        typedef int i32x16_t __attribute__((ext_vector_type(16)));
        typedef int i32x4_t __attribute__((ext_vector_type(4)));
        acc[i][j] = __builtin_bit_cast(f32x16, __builtin_amdgcn_mfma_i32_32x32x32_i8(
            __builtin_bit_cast(i32x4_t, bw), __builtin_bit_cast(i32x4_t, av), __builtin_bit_cast(i32x16_t, acc[i][j]), 0, 0, 0));
      } else {
        __asm__ volatile("" ::"v"(bw.x), "v"(bw.y), "v"(bw.z), "v"(bw.w), "v"(av.x), "v"(av.y), "v"(av.z), "v"(av.w));  // the operands stay looked up
      }
#else
      acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, bw), __builtin_bit_cast(bf16x8, av),
                                                          acc[i][j], 0, 0, 0);
#endif
#pragma unroll
      for (int t = lo; t < hi; ++t) lookup_read(buf, q, set, t, addr[m & 1][t - lo]);
      if (m + 1 < kGroups) {
#pragma unroll
        for (int t = hi; t < hi2; ++t) addr[(m + 1) & 1][t - hi] = lookup_address(buf, q, t);
      }
      __builtin_amdgcn_sched_barrier(0);
    }
  };
  // one K-step out of buffer B; its last phase looks up the first operands of buffer B+1
  auto step = [&](auto buf, int ks) {
    constexpr int B = decltype(buf)::value;
    constexpr auto prev = std::integral_constant<int, (B + NBUF - 1) % NBUF>{};
    constexpr auto next = std::integral_constant<int, (B + 1) % NBUF>{};
    phase(buf, 1, 1, prev, ks + NBUF - 1, FM + FN <= FM * FN, buf, std::integral_constant<int, 0>{});
    if constexpr (FM + FN > FM * FN) fetch(prev, ks + NBUF - 1);
    phase(buf, 2, 0, prev, 0, false, buf, std::integral_constant<int, 1>{});
    phase(buf, 3, 1, prev, 0, false, buf, std::integral_constant<int, 2>{});
    stash(next);  // every operand read of this K-step has been issued; the next K-step's pieces take the slab
    phase(next, 0, 0, prev, 0, false, buf, std::integral_constant<int, 3>{});
  };

  stash(std::integral_constant<int, 0>{});
#pragma unroll
  for (int t = 0; t < kLookups; ++t)
    lookup_read(std::integral_constant<int, 0>{}, 0, 0, t, lookup_address(std::integral_constant<int, 0>{}, 0, t));
  OQ_STAMP(2);  // first operands looked up: the loop starts
  int ks = 0;
  for (; ks + NBUF <= steps; ks += NBUF) {
    step(std::integral_constant<int, 0>{}, ks);
    step(std::integral_constant<int, 1>{}, ks + 1);
    if constexpr (NBUF == 3) step(std::integral_constant<int, 2>{}, ks + 2);
  }
  if (ks < steps) {
    step(std::integral_constant<int, 0>{}, ks);
    if (NBUF == 3 && ks + 1 < steps) step(std::integral_constant<int, 1>{}, ks + 1);
  }

  OQ_STAMP(3);  // loop done
  __syncthreads();  // every wavefront is done with the lookup tables: LDS is reused from here on
  OQ_STAMP(4);
  EpiFactors<FM> epi;
  gemm_epilogue_factors<FM>(epi, epi_raw, TN, tid, g.row_scale != nullptr, g.bias != nullptr, g.bias_dtype);
  if constexpr (KSPLIT == 1) {
    void *out = g.out;
    int out_dtype = g.out_dtype;
    OutMap out_map = g.out_map;
    if (g.k_splits > 1) {  // raw partial sums: factors of one, no bias, fp32 (x * 1 * 1 + 0 is x)
      epi.rn = 1.0f;
      epi.bv = 0.0f;
#pragma unroll
      for (int i = 0; i < FM; ++i) epi.sc[i] = 1.0f;
      out = g.partials + static_cast<int64_t>(blockIdx.y) * g.M * g.N;
      out_dtype = OQ_F32;
      out_map = OutMap{nullptr, -1};
    }
    gemm_epilogue<FM, FN>(acc, static_cast<int64_t>(pid_m) * TM, static_cast<int64_t>(pid_n) * TN, wm, wn, TN, tid, g.M, g.N,
                          g.row_scale, g.row_norms, g.bias, g.bias_dtype, epi, out, out_dtype,
                          reinterpret_cast<unsigned char *>(lds), out_map, 64 * FM,
                          window_ahead ? reinterpret_cast<const uint16_t *>(map_window) : nullptr);
  } else {
    // Reduce-scatter over the wavefronts in four rounds, one per row slice: in round s every wavefront parks
    // slice s of its partial tile in LDS (slot = its own number) and wavefront s adds the other three to its
    // own, in the order s-1, s-2, s-3 (mod 4).  The accumulator slices are registers, so which one is sent or
    // summed has to be a compile-time index: this way it is the round's number, the same instructions for all
    // four wavefronts (a scheme in which each wavefront sends a different slice per round needs four copies
    // of every round, each fetched by one wavefront alone, and measured 0.5 us slower a launch).  Every barrier
    // (and the epilogue, which has one of its own) is reached by all four in the same place.
    // Slot of wavefront v: [FN tiles][4 runs][64 lanes] of float4.
    float4 *slots = reinterpret_cast<float4 *>(lds);
    f32x16 slice[1][FN];
    EpiFactors<1> mine;
    mine.rn = epi.rn;
    mine.bv = epi.bv;
    mine.sc[0] = 1.0f;
#pragma unroll
    for (int j = 0; j < FN; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) slice[0][j][e] = 0.0f;
    auto round = [&](auto st) __attribute__((always_inline)) {
      constexpr int S = decltype(st)::value;
      if (wave != S) {
#pragma unroll
        for (int j = 0; j < FN; ++j) {
          const f32x16 t = acc[S][j];  // whole-tile copies keep the accumulators in registers
#pragma unroll
          for (int a4 = 0; a4 < 4; ++a4)
            slots[((wave * FN + j) * 4 + a4) * 64 + lane] = make_float4(t[4 * a4 + 0], t[4 * a4 + 1], t[4 * a4 + 2], t[4 * a4 + 3]);
        }
      }
      __syncthreads();
      if (wave == S) {
        mine.sc[0] = epi.sc[S];
        // the twelve reads of a tile are issued before its first sum (one LDS round trip a tile, not one a read)
#pragma unroll
        for (int j = 0; j < FN; ++j) {
          float4 part[3][4];
#pragma unroll
          for (int d = 1; d < 4; ++d)
#pragma unroll
            for (int a4 = 0; a4 < 4; ++a4)
              part[d - 1][a4] = slots[((((S + 4 - d) & 3) * FN + j) * 4 + a4) * 64 + lane];
          __builtin_amdgcn_sched_barrier(0);
          f32x16 sum = acc[S][j];
#pragma unroll
          for (int d = 0; d < 3; ++d)
#pragma unroll
            for (int a4 = 0; a4 < 4; ++a4) {
              sum[4 * a4 + 0] += part[d][a4].x;
              sum[4 * a4 + 1] += part[d][a4].y;
              sum[4 * a4 + 2] += part[d][a4].z;
              sum[4 * a4 + 3] += part[d][a4].w;
            }
          slice[0][j] = sum;
          __builtin_amdgcn_sched_barrier(0);
        }
      }
      if (S < 3) __syncthreads();  // the slots are written again by the next round
    };
    round(std::integral_constant<int, 0>{});
    round(std::integral_constant<int, 1>{});
    round(std::integral_constant<int, 2>{});
    round(std::integral_constant<int, 3>{});
    gemm_epilogue<1, FN>(slice, static_cast<int64_t>(pid_m) * TM, static_cast<int64_t>(pid_n) * TN, 32 * wave, 0, TN, tid, g.M,
                         g.N, g.row_scale, g.row_norms, g.bias, g.bias_dtype, mine, g.out, g.out_dtype,
                         reinterpret_cast<unsigned char *>(lds), g.out_map, TM,
                         window_ahead ? reinterpret_cast<const uint16_t *>(map_window) : nullptr);
  }
#ifdef OQ_GEMM_STAMPS
  OQ_STAMP(5);  // epilogue issued
  __asm__ volatile("s_waitcnt vmcnt(0)" ::: "memory");
  stamp[7] = __builtin_amdgcn_s_memrealtime();
  const uint64_t done = __builtin_amdgcn_s_memtime();
  if (g.stamps != nullptr && lane == 0) {
    uint64_t *dst = g.stamps + (static_cast<int64_t>(blockIdx.y * gridDim.x + blockIdx.x) * 4 + wave) * 16;
#pragma unroll
    for (int i = 0; i < 8; ++i) dst[i] = stamp[i];
    dst[8] = done;
    uint32_t hw;
    __asm__ volatile("s_getreg_b32 %0, hwreg(HW_REG_HW_ID)" : "=s"(hw));
    uint32_t xcc;
    __asm__ volatile("s_getreg_b32 %0, hwreg(HW_REG_XCC_ID)" : "=s"(xcc));
    dst[9] = (static_cast<uint64_t>(xcc) << 32) | hw;
#pragma unroll
    for (int i = 0; i < 6; ++i) dst[10 + i] = stamp_extra[i];
  }
#endif
#undef OQ_STAMP
}

template <int AM, int BITS, int FM, int FN, int KSPLIT = 1>
int launch_cfg(GemmArgs g, hipStream_t stream) {
  constexpr int TM = (KSPLIT == 1 ? 2 : 1) * FM * 32, TN = (KSPLIT == 1 ? 2 : 1) * FN * 32;
  g.tiles_m = static_cast<int>((g.M + TM - 1) / TM);
  g.tiles_n = static_cast<int>((g.N + TN - 1) / TN);
  const int64_t total = static_cast<int64_t>(g.tiles_m) * g.tiles_n;
  if (total > 0x7fffffffLL) return fail(OQ_ERR_UNSUPPORTED, "packed_gemm: too many tiles");
  auto kern = packed_gemm_kernel<AM, BITS, FM, FN, KSPLIT>;
  const unsigned splits = (KSPLIT == 1 && (AM == A_NIBBLE || AM == A_U8) && g.k_splits > 1) ? static_cast<unsigned>(g.k_splits) : 1u;
  if (splits == 1) g.k_splits = 1;
  // a mapped launch parks the map's window in LDS ahead of its main loop (not for partial tiles: they are not mapped)
  g.window_ahead = (g.out_map.table != nullptr && g.out_map.lo == kWideLoBf16 && g.out_dtype == OQ_BF16 && splits == 1 &&
                    reserve_dynamic_lds(reinterpret_cast<const void *>(kern), kWideBytes)) ? 1 : 0;
  if (g.M > 0x7fff0000LL || g.N > 0x7fff0000LL || g.K > 0x0fffffffLL || g.a_levels > 0xffff)  // (the kernel's 32-bit row and byte counts)
    return fail(OQ_ERR_UNSUPPORTED, "packed_gemm: a dimension beyond 2^31");
  hipLaunchKernelGGL(kern, dim3(static_cast<unsigned>(total), splits), dim3(256), g.window_ahead ? kWideBytes : 0, stream,
                     g.w_cents, g.act_cents, g.a, g.w, g.out_map.table, static_cast<int>(g.K), static_cast<int>(g.M),
                     static_cast<int>(g.N), g.a_levels | (g.k_splits << 16) | (g.window_ahead << 24), g);
  return check_launch("packed_gemm");
}

template <int AM, int BITS>
int launch_bits(const GemmArgs &g, int tile, hipStream_t stream) {
  if (tile == 4) return launch_cfg<AM, BITS, 4, 3, 4>(g, stream);
  if (tile == 3) return launch_cfg<AM, BITS, 4, 3>(g, stream);
  if constexpr (AM == A_NIBBLE) {
    if (tile == 2) return launch_cfg<AM, BITS, 4, 4>(g, stream);
  } else {
    if (tile == 2) return launch_cfg<AM, BITS, 4, 4>(g, stream);
  }
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
}  // namespace oq
