/*
 * CPU restatement (plain C, OpenMP over rows/columns) of the reference's
 * quantized-linear forward.  TEST INFRASTRUCTURE ONLY: the shipped library never
 * links or loads this file; tests, the smoke check and the CPU-baseline leg of
 * the benchmark use it as the checker / the timed CPU port.
 *
 * Build: gcc -O3 -march=x86-64-v3 -ffp-contract=off -fopenmp -shared -fPIC
 * (-ffp-contract=off matters: every fp32 operation below rounds once, no FMA).
 *
 * Reference lines restated (paths relative to the reference checkout):
 *   oqo_rotate_quantize   src/orbitquant/functional.py:16-21,
 *                         src/orbitquant/rotations/rpbh.py:74-84,
 *                         src/orbitquant/rotations/fwht.py:19-25,
 *                         src/orbitquant/codebooks/lloyd_max.py:40-42
 *   oqo_unpack            src/orbitquant/packing/bitpack.py:63-97,
 *                         native-kernels/orbitquant-packed-matmul/
 *                           orbitquant_packed_matmul_cpu/packed_matmul_scalar.cpp:31-43
 *   oqo_matmul_packed_weight   .../packed_matmul_scalar.cpp:45-74
 *   oqo_linear_from_codes      functional.py:21-22 + src/orbitquant/layers.py:1060-1070,1450-1455
 *
 * The token norm uses the fixed "sumsq-v1" order (the reference's torch.norm
 * order is build-defined): rows are zero-padded to a multiple of 2048 and seen
 * as [passes][256 lanes][8]; per (pass, lane) the eight squares are added as
 * ((s0+s1)+(s2+s3))+((s4+s5)+(s6+s7)); each lane adds its passes left to right;
 * the 256 lane sums are reduced by a balanced binary tree in lane order.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

static float sumsq_v1(const float *x, int64_t k) {
  float lane[256];
  for (int t = 0; t < 256; ++t) lane[t] = 0.0f;
  int64_t passes = (k + 2047) / 2048;
  if (passes < 1) passes = 1;
  for (int64_t c = 0; c < passes; ++c) {
    for (int t = 0; t < 256; ++t) {
      float s[8];
      for (int e = 0; e < 8; ++e) {
        int64_t i = c * 2048 + (int64_t)t * 8 + e;
        float v = i < k ? x[i] : 0.0f;
        s[e] = v * v;
      }
      float v8 = ((s[0] + s[1]) + (s[2] + s[3])) + ((s[4] + s[5]) + (s[6] + s[7]));
      lane[t] = c == 0 ? v8 : lane[t] + v8;
    }
  }
  for (int width = 256; width > 1; width /= 2)
    for (int t = 0; t < width / 2; ++t) lane[t] = lane[2 * t] + lane[2 * t + 1];
  return lane[0];
}

static void fwht_block(float *y, int64_t h) {
  for (int64_t d = 1; d < h; d *= 2)
    for (int64_t base = 0; base < h; base += 2 * d)
      for (int64_t j = base; j < base + d; ++j) {
        float l = y[j], r = y[j + d];
        y[j] = l + r;
        y[j + d] = l - r;
      }
}

static inline uint8_t count_below(const float *bounds, int nb, float v) {
  int lo = 0, hi = nb; /* first index with bounds[idx] >= v */
  while (lo < hi) {
    int mid = (lo + hi) / 2;
    if (bounds[mid] < v) lo = mid + 1; else hi = mid;
  }
  return (uint8_t)lo;
}

/* x: fp32 [m,k] (already upcast). codes: u8 [m,k]. norms: raw ||x|| fp32 [m]. */
int oqo_rotate_quantize(const float *x, int64_t m, int64_t k, const int32_t *perm,
                        const int8_t *signs, const float *bounds, int nb, int64_t block,
                        float eps, float inv_sqrt_block, uint8_t *codes, float *norms,
                        int threads) {
  if (block <= 0 || (block & (block - 1)) || k % block) return 1;
#ifdef _OPENMP
  if (threads > 0) omp_set_num_threads(threads);
#endif
#pragma omp parallel
  {
    float *y = (float *)malloc((size_t)k * sizeof(float));
#pragma omp for schedule(static)
    for (int64_t r = 0; r < m; ++r) {
      const float *row = x + r * k;
      float s = sqrtf(sumsq_v1(row, k));
      float denom = s + eps;
      for (int64_t c = 0; c < k; ++c) y[c] = (row[perm[c]] / denom) * (float)signs[c];
      for (int64_t b = 0; b < k; b += block) fwht_block(y + b, block);
      for (int64_t c = 0; c < k; ++c)
        codes[r * k + c] = count_below(bounds, nb, y[c] * inv_sqrt_block);
      norms[r] = s;
    }
    free(y);
  }
  return 0;
}

static inline uint32_t unpack_one(const uint8_t *packed, int64_t i, int bits, int64_t nbytes) {
  int64_t bit = i * bits;
  int64_t byte = bit >> 3;
  unsigned sh = (unsigned)(bit & 7);
  uint32_t w = packed[byte];
  if (sh + (unsigned)bits > 8 && byte + 1 < nbytes) w |= (uint32_t)packed[byte + 1] << 8;
  return (w >> sh) & ((1u << bits) - 1u);
}

int oqo_unpack(const uint8_t *packed, int bits, int64_t count, uint8_t *out) {
  if (bits < 1 || bits > 8) return 1;
  int64_t nbytes = (count * bits + 7) / 8;
  for (int64_t i = 0; i < count; ++i) out[i] = (uint8_t)unpack_one(packed, i, bits, nbytes);
  return 0;
}

/* out[m,n] = (sum_k x[m,k]*c[idx[n,k]]) * r[n] + bias[n]; fp32 accumulation in k
 * order, norm applied after the sum, as the reference's scalar kernel does. */
int oqo_matmul_packed_weight(const float *x, const uint8_t *packed, const float *row_norms,
                             const float *centroids, const float *bias, int bits, int64_t m,
                             int64_t n, int64_t k, float *out, int threads) {
  if (bits < 1 || bits > 8) return 1;
  int64_t nbytes = (n * k * bits + 7) / 8;
#ifdef _OPENMP
  if (threads > 0) omp_set_num_threads(threads);
#endif
#pragma omp parallel
  {
    float *wrow = (float *)malloc((size_t)k * sizeof(float));
#pragma omp for schedule(static)
    for (int64_t col = 0; col < n; ++col) {
      for (int64_t kk = 0; kk < k; ++kk)
        wrow[kk] = centroids[unpack_one(packed, col * k + kk, bits, nbytes)];
      for (int64_t r = 0; r < m; ++r) {
        const float *xr = x + r * k;
        float acc = 0.0f;
        for (int64_t kk = 0; kk < k; ++kk) acc += xr[kk] * wrow[kk];
        acc *= row_norms[col];
        if (bias) acc += bias[col];
        out[r * n + col] = acc;
      }
    }
    free(wrow);
  }
  return 0;
}

/* y[m,n] = (sum_k c_a[codes[m,k]] * c_w[idx[n,k]]) * s[m] * r[n] + bias[n], fp64. */
int oqo_linear_from_codes(const uint8_t *codes, const float *s, const float *c_a,
                          const uint8_t *packed_w, int w_bits, const float *r_w,
                          const float *c_w, const float *bias, int64_t m, int64_t n,
                          int64_t k, double *out, int threads) {
  if (w_bits < 1 || w_bits > 8) return 1;
  int64_t nbytes = (n * k * w_bits + 7) / 8;
#ifdef _OPENMP
  if (threads > 0) omp_set_num_threads(threads);
#endif
#pragma omp parallel
  {
    double *wrow = (double *)malloc((size_t)k * sizeof(double));
#pragma omp for schedule(static)
    for (int64_t col = 0; col < n; ++col) {
      for (int64_t kk = 0; kk < k; ++kk)
        wrow[kk] = (double)c_w[unpack_one(packed_w, col * k + kk, w_bits, nbytes)];
      for (int64_t r = 0; r < m; ++r) {
        const uint8_t *cr = codes + r * k;
        double acc = 0.0;
        for (int64_t kk = 0; kk < k; ++kk) acc += (double)c_a[cr[kk]] * wrow[kk];
        acc = acc * (double)s[r] * (double)r_w[col];
        if (bias) acc += (double)bias[col];
        out[r * n + col] = acc;
      }
    }
    free(wrow);
  }
  return 0;
}

int oqo_max_threads(void) {
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}
