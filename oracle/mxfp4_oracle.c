/*
 * CPU oracle for the MXFP4 block-scaled GEMM path, plain C.
 * TEST INFRASTRUCTURE ONLY: linked by the test-suite, the smoke check and the
 * CPU-baseline leg of the benchmark; the HIP library never calls it.
 *
 * Second, loop-and-index statement of the arithmetic the reference defines in
 * wave_lang/kernel/wave/utils/mxfp_utils.py.  Where the numpy oracle uses
 * reshape/permute, this file uses the explicit index formulas of
 * wave_lang/kernel/wave/templates/tagged_mxfp4_gemm.py:465-536, so that the
 * two can be checked against each other.
 *
 * Pins: e2m1 table against the OCP closed form, e8m0 against IEEE-754 bit
 * patterns, shuffles against the numpy permutes and a bijection check, GEMMs
 * against exact-rational brute force on tiny shapes.  Bitwise equality of an
 * f32 GEMM with the reference's torch.mm is parity unpinned by design
 * (summation order is not part of the contract).
 *
 * Build: gcc -O3 -mavx2 -mfma -fopenmp -shared -fPIC mxfp4_oracle.c -o libmxfp4_oracle.so -lm
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

/* e2m1 code -> value, bit 3 = sign, code 8 = -0.0
 * (wave_lang/kernel/wave/utils/mxfp_utils.py:65-82) */
static const float kE2M1[16] = {0.0f,  0.5f,  1.0f,  1.5f,  2.0f,  3.0f,  4.0f,  6.0f,
                                -0.0f, -0.5f, -1.0f, -1.5f, -2.0f, -3.0f, -4.0f, -6.0f};
/* twice the value, as an integer */
static const int8_t kE2M1x2[16] = {0, 1, 2, 3, 4, 6, 8, 12, 0, -1, -2, -3, -4, -6, -8, -12};

/* low nibble = element 2j, high nibble = element 2j+1
 * (wave_lang/kernel/wave/utils/mxfp_utils.py:62-64) */
void orc_mxfp4_to_f32(const uint8_t *q, int64_t rows, int64_t kp, float *out) {
  for (int64_t r = 0; r < rows; ++r)
    for (int64_t j = 0; j < kp; ++j) {
      uint8_t b = q[r * kp + j];
      out[r * kp * 2 + 2 * j] = kE2M1[b & 0xF];
      out[r * kp * 2 + 2 * j + 1] = kE2M1[b >> 4];
    }
}

/* 2^(s-127); 255 -> NaN; 0 -> subnormal 2^-127
 * (wave_lang/kernel/wave/utils/mxfp_utils.py:86-95) */
float orc_e8m0_scalar(uint8_t s) {
  if (s == 255) return NAN;
  return ldexpf(1.0f, (int)s - 127);
}

void orc_e8m0_to_f32(const uint8_t *s, int64_t n, float *out) {
  for (int64_t i = 0; i < n; ++i) out[i] = orc_e8m0_scalar(s[i]);
}

/* value * scale of its 32-group, f32
 * (wave_lang/kernel/wave/utils/mxfp_utils.py:135-143) */
void orc_dequant_f32(const uint8_t *q, const uint8_t *scale, int64_t rows, int64_t k, float *out) {
  int64_t kp = k / 2, ks = k / 32;
#pragma omp parallel for schedule(static)
  for (int64_t r = 0; r < rows; ++r)
    for (int64_t e = 0; e < k; ++e) {
      uint8_t b = q[r * kp + e / 2];
      uint8_t code = (e & 1) ? (b >> 4) : (b & 0xF);
      out[r * k + e] = kE2M1[code] * orc_e8m0_scalar(scale[r * ks + e / 32]);
    }
}

/* The reference GEMM: C = deq(A) . deq(B)^T in f32, B stored [N, K/2]
 * (wave_lang/kernel/wave/utils/mxfp_utils.py:131-143).  Plain k-ordered f32
 * accumulation; the reference's order is whatever its BLAS picks. */
int orc_gemm_f32(const uint8_t *a, const uint8_t *as, const uint8_t *b, const uint8_t *bs, float *c,
                 int64_t m, int64_t n, int64_t k) {
  float *af = (float *)malloc(sizeof(float) * (size_t)m * k);
  float *bf = (float *)malloc(sizeof(float) * (size_t)n * k);
  if (!af || !bf) {
    free(af);
    free(bf);
    return -1;
  }
  orc_dequant_f32(a, as, m, k, af);
  orc_dequant_f32(b, bs, n, k, bf);
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < m; ++i)
    for (int64_t j = 0; j < n; ++j) {
      const float *x = af + i * k, *y = bf + j * k;
      float acc = 0.0f;
      for (int64_t e = 0; e < k; ++e) acc += x[e] * y[e];
      c[i * n + j] = acc;
    }
  free(af);
  free(bf);
  return 0;
}

/* Block-exact GEMM: per 32-group an exact integer dot of (2a)(2b), scaled by
 * 2^(sa+sb-256) and summed in f64.  rows_idx (may be NULL) selects a subset of
 * M rows; out is [n_rows, n] f64. */
int orc_gemm_exact(const uint8_t *a, const uint8_t *as, const uint8_t *b, const uint8_t *bs,
                   double *c, int64_t m, int64_t n, int64_t k, const int64_t *rows_idx,
                   int64_t n_rows) {
  int64_t kp = k / 2, ks = k / 32;
  int8_t *bi = (int8_t *)malloc((size_t)n * k);
  if (!bi) return -1;
#pragma omp parallel for schedule(static)
  for (int64_t j = 0; j < n; ++j)
    for (int64_t e = 0; e < kp; ++e) {
      uint8_t v = b[j * kp + e];
      bi[j * k + 2 * e] = kE2M1x2[v & 0xF];
      bi[j * k + 2 * e + 1] = kE2M1x2[v >> 4];
    }
  if (!rows_idx) n_rows = m;
#pragma omp parallel
  {
    int8_t *ai = (int8_t *)malloc((size_t)k);
#pragma omp for schedule(dynamic, 1)
    for (int64_t ii = 0; ii < n_rows; ++ii) {
      int64_t i = rows_idx ? rows_idx[ii] : ii;
      int a_nan = 0;
      for (int64_t e = 0; e < kp; ++e) {
        uint8_t v = a[i * kp + e];
        ai[2 * e] = kE2M1x2[v & 0xF];
        ai[2 * e + 1] = kE2M1x2[v >> 4];
      }
      for (int64_t g = 0; g < ks; ++g) a_nan |= (as[i * ks + g] == 255);
      for (int64_t j = 0; j < n; ++j) {
        double acc = 0.0;
        int b_nan = 0;
        const int8_t *y = bi + j * k;
        for (int64_t g = 0; g < ks; ++g) {
          int32_t d = 0;
          for (int e = 0; e < 32; ++e) d += (int32_t)ai[g * 32 + e] * (int32_t)y[g * 32 + e];
          uint8_t sb = bs[j * ks + g];
          b_nan |= (sb == 255);
          acc += ldexp((double)d, (int)as[i * ks + g] + (int)sb - 256);
        }
        c[ii * n + j] = (a_nan || b_nan) ? NAN : acc;
      }
    }
    free(ai);
  }
  free(bi);
  return 0;
}

/* Flat offset of scale (r, kg) in the tile-ordered buffer with padded row
 * length ksp (wave_lang/kernel/wave/templates/tagged_mxfp4_gemm.py:520-527) */
int64_t orc_e8m0_shuffle_index(int64_t r, int64_t kg, int64_t ksp) {
  return (r / 32) * ((ksp / 8) * 256) + (kg / 8) * 256 + ((kg % 8) % 4) * 64 + ((r % 32) % 16) * 4 +
         ((kg % 8) / 4) * 2 + (r % 32) / 16;
}

/* scale [m, ks] -> padded tile-ordered buffer of ceil(m/256)*256 x ceil(ks/8)*8
 * bytes, zero filled (wave_lang/kernel/wave/utils/mxfp_utils.py:113-127) */
void orc_e8m0_shuffle_padded(const uint8_t *scale, int64_t m, int64_t ks, uint8_t *out) {
  int64_t sm = (m + 255) / 256 * 256, sn = (ks + 7) / 8 * 8;
  memset(out, 0, (size_t)(sm * sn));
  for (int64_t r = 0; r < m; ++r)
    for (int64_t g = 0; g < ks; ++g) out[orc_e8m0_shuffle_index(r, g, sn)] = scale[r * ks + g];
}

/* Flat offset of byte (n, kb) after b_preshuffle
 * (wave_lang/kernel/wave/templates/tagged_mxfp4_gemm.py:472-483) */
int64_t orc_b_preshuffle_index(int64_t n, int64_t kb, int64_t kp) {
  int64_t within = (kb / 32) * 512 + ((kb / 16) % 2) * 256 + (n % 16) * 16 + kb % 16;
  return (n / 16) * 16 * kp + within;
}

/* (wave_lang/kernel/wave/utils/mxfp_utils.py:98-110) */
void orc_b_preshuffle(const uint8_t *b, int64_t n, int64_t kp, uint8_t *out) {
  for (int64_t r = 0; r < n; ++r)
    for (int64_t e = 0; e < kp; ++e) out[orc_b_preshuffle_index(r, e, kp)] = b[r * kp + e];
}
