/* CPU oracle for the quantized-matmul path, in C.  TEST INFRASTRUCTURE ONLY.
 *
 * Restates the reference's UNFUSED chain -- unpack the packed codes, rebuild
 * the weight (one fused multiply-add per element for the affine mode, a table
 * value times a power of two for MXFP4), optionally round the weight tile once
 * to bf16, then a float32-accumulate dot against the activations -- so that
 * tests can check the HIP kernels against it and bench.py can time it as the
 * CPU baseline.  The product library never links or loads this file.
 *
 * Reference lines followed (paths relative to the reference tree):
 *   packed layout          src/metaljax/qmm.py:206-232
 *   affine reconstruction  src/metaljax/qmm.py:71-79, :244-254
 *   MXFP4 grid / E8M0      src/metaljax/qmm.py:167-173, :335-357;
 *                          tests/test_qmm_mxfp4.py:77-90
 *   the product            src/metaljax/qmm.py:2491-2499 (f32 accumulate,
 *                          tests/test_qmm.py:14-16)
 *   per-expert rows        src/metaljax/moe.py:1283-1340
 *
 * Pinned by tests/test_oracle.py against the numpy oracle (itself pinned by
 * the reference's known-answer vectors) on seeded inputs, bit for bit for the
 * unpack / dequant functions and to 1e-6 rel-L2 for the products.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#ifdef _OPENMP
#include <omp.h>
#endif

#define ORACLE_MODE_AFFINE 0
#define ORACLE_MODE_MXFP4 1

static const float kE2M1[16] = {0.0f, 0.5f, 1.0f, 1.5f, 2.0f, 3.0f, 4.0f, 6.0f,
                                -0.0f, -0.5f, -1.0f, -1.5f, -2.0f, -3.0f, -4.0f, -6.0f};

static inline float bf16_to_f32(uint16_t b) {
  uint32_t u = (uint32_t)b << 16;
  float f;
  memcpy(&f, &u, 4);
  return f;
}

static inline uint16_t f32_to_bf16(float f) {
  uint32_t u;
  memcpy(&u, &f, 4);
  if ((u & 0x7FFFFFFFu) > 0x7F800000u) return (uint16_t)((u >> 16) | 0x40u);
  u += 0x7FFFu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}

static inline float e8m0_to_f32(uint8_t e) {
  if (e == 255) return NAN;
  return ldexpf(1.0f, (int)e - 127);
}

int oracle_num_threads(void) {
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}

/* codes[r*k + i] = bits [i*bits, (i+1)*bits) of row r's little-endian stream */
void oracle_unpack_codes(const uint32_t* words, int64_t rows, int64_t k, int bits,
                         uint8_t* codes) {
  const int per = 32 / bits;
  const uint32_t mask = (1u << bits) - 1u;
  for (int64_t r = 0; r < rows; ++r)
    for (int64_t i = 0; i < k; ++i) {
      uint32_t w = words[r * (k / per) + i / per];
      codes[r * k + i] = (uint8_t)((w >> ((i % per) * bits)) & mask);
    }
}

/* One row of the weight, as float32.  tables_bf16 != 0: scales/biases are
 * bf16 bit patterns, else float32.  mode MXFP4: scales are E8M0 bytes. */
static void dequant_row(const uint32_t* wrow, const void* scales, const void* biases,
                        int64_t row, int64_t k, int gs, int bits, int mode,
                        int tables_bf16, int round_tile_bf16, float* out) {
  if (mode == ORACLE_MODE_MXFP4) {
    const uint8_t* bytes = (const uint8_t*)wrow;
    const uint8_t* sb = (const uint8_t*)scales + row * (k / 32);
    for (int64_t i = 0; i < k; ++i) {
      uint8_t c = (bytes[i >> 1] >> ((i & 1) * 4)) & 0xF;
      out[i] = kE2M1[c] * e8m0_to_f32(sb[i / 32]);
    }
  } else {
    const int per = 32 / bits;
    const uint32_t mask = (1u << bits) - 1u;
    const int64_t ng = k / gs;
    for (int64_t i = 0; i < k; ++i) {
      uint32_t q = (wrow[i / per] >> ((i % per) * bits)) & mask;
      float s, b;
      if (tables_bf16) {
        s = bf16_to_f32(((const uint16_t*)scales)[row * ng + i / gs]);
        b = bf16_to_f32(((const uint16_t*)biases)[row * ng + i / gs]);
      } else {
        s = ((const float*)scales)[row * ng + i / gs];
        b = ((const float*)biases)[row * ng + i / gs];
      }
      out[i] = fmaf(s, (float)q, b);
    }
  }
  if (round_tile_bf16)
    for (int64_t i = 0; i < k; ++i) out[i] = bf16_to_f32(f32_to_bf16(out[i]));
}

/* Whole weight [n, k] as float32 (bit-exact reference for the dequant kernels). */
void oracle_dequant(const uint32_t* words, const void* scales, const void* biases,
                    int64_t n, int64_t k, int gs, int bits, int mode, int tables_bf16,
                    int round_tile_bf16, float* out) {
  const int64_t wpr = (mode == ORACLE_MODE_MXFP4) ? k / 8 : k * bits / 32;
#pragma omp parallel for schedule(static)
  for (int64_t r = 0; r < n; ++r)
    dequant_row(words + r * wpr, scales, biases, r, k, gs, bits, mode, tables_bf16,
                round_tile_bf16, out + r * k);
}

/* y[m, n] = sum_k x[m, k] * w[n, k]; x is bf16 bit patterns [m, k]; float32
 * accumulate in k order; y float32 [m, n].  Rows of the weight are rebuilt one
 * at a time (the unfused chain, restated without materializing [n, k]). */
void oracle_qmm(const uint16_t* x, const uint32_t* words, const void* scales,
                const void* biases, int64_t m, int64_t n, int64_t k, int gs, int bits,
                int mode, int tables_bf16, int round_tile_bf16, float* y) {
  const int64_t wpr = (mode == ORACLE_MODE_MXFP4) ? k / 8 : k * bits / 32;
  float* xf = (float*)malloc(sizeof(float) * (size_t)(m * k));
  for (int64_t i = 0; i < m * k; ++i) xf[i] = bf16_to_f32(x[i]);
#pragma omp parallel
  {
    float* wrow = (float*)malloc(sizeof(float) * (size_t)k);
#pragma omp for schedule(static)
    for (int64_t r = 0; r < n; ++r) {
      dequant_row(words + r * wpr, scales, biases, r, k, gs, bits, mode, tables_bf16,
                  round_tile_bf16, wrow);
      for (int64_t i = 0; i < m; ++i) {
        const float* xr = xf + i * k;
        float acc = 0.0f;
        for (int64_t j = 0; j < k; ++j) acc += xr[j] * wrow[j];
        y[i * n + r] = acc;
      }
    }
    free(wrow);
  }
  free(xf);
}

/* Rows sorted by expert: rows [row_offsets[e], row_offsets[e+1]) use expert e. */
void oracle_grouped_qmm(const uint16_t* x, const uint32_t* words, const void* scales,
                        const void* biases, const int32_t* row_offsets, int64_t experts,
                        int64_t n, int64_t k, int gs, int bits, int mode, int tables_bf16,
                        int round_tile_bf16, float* y) {
  const int64_t wpr = (mode == ORACLE_MODE_MXFP4) ? k / 8 : k * bits / 32;
  const int64_t tab = (mode == ORACLE_MODE_MXFP4) ? (k / 32) : (k / gs) * (tables_bf16 ? 2 : 4);
  for (int64_t e = 0; e < experts; ++e) {
    int64_t a = row_offsets[e], b = row_offsets[e + 1];
    if (b <= a) continue;
    oracle_qmm(x + a * k, words + e * n * wpr, (const char*)scales + e * n * tab,
               biases ? (const char*)biases + e * n * tab : NULL, b - a, n, k, gs, bits,
               mode, tables_bf16, round_tile_bf16, y + a * n);
  }
}
