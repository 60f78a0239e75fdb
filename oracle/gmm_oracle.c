/*
 * CPU oracle for the grouped quantized matmul path, plain C.  TEST INFRASTRUCTURE ONLY:
 * it is the checker for the HIP backend and is never linked into or called by the product.
 *
 * It restates the arithmetic the reference pins in its system tests
 *   - grouped W8A8 golden ........ tests/st/test_grouped_matmul.py:62-71
 *   - row ranges from group_list . tests/st/test_grouped_matmul.py:44-52
 *   - counts -> running sum ...... tests/st/test_grouped_matmul_v4_cops.py:296
 *   - weight-only a16w8 .......... tests/st/test_grouped_matmul_v4_cops.py:166-174
 * with an exact integer accumulator (no float32 dot), so it is independent of the numpy
 * oracle's chunked-sgemm path and pins it (tests/test_oracle_pins.py compares the two).
 *
 * Build: make -C oracle   ->  oracle/_build/libgmm_oracle.so
 */
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#include <math.h>

#define ORACLE_API __attribute__((visibility("default")))

/* float32 -> bfloat16 bits, round to nearest even; NaN stays a quiet NaN. */
ORACLE_API uint16_t oracle_f32_to_bf16(float f) {
  uint32_t u;
  memcpy(&u, &f, 4);
  if ((u & 0x7F800000u) == 0x7F800000u && (u & 0x007FFFFFu)) return (uint16_t)((u >> 16) | 0x40u);
  u += 0x7FFFu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}

static float bf16_to_f32(uint16_t b) {
  uint32_t u = (uint32_t)b << 16;
  float f;
  memcpy(&f, &u, 4);
  return f;
}

/* Row range of group g.  type 0: cumulative ends; type 1: counts.  Ends are clamped into
 * [previous end, m]. */
static void group_range(const int64_t *gl, int e, int type, int64_t m, int g, int64_t *s, int64_t *t) {
  int64_t start = 0, end = 0;
  for (int i = 0; i <= g; ++i) {
    start = end;
    int64_t v = gl ? gl[i] : (m / e) * (i + 1);
    end = (type == 1) ? start + v : v;
    if (end < start) end = start;
    if (end > m) end = m;
  }
  (void)e;
  *s = start;
  *t = end;
}

/*
 * x int8 [m,k]; w int8 [e,k,n] (or [e,n,k] when transpose_b); group_list int64 [e] (NULL: e equal
 * groups of m/e rows); bias int32 [e,n] or NULL; scale f32 [e,n] or NULL; per_token f32 [m] or NULL.
 * acc_out int32 [m,n] or NULL (accumulator + bias); bf16_out uint16 [m,n] or NULL.
 * Rows at or past the last boundary are written as zero.
 */
ORACLE_API int oracle_gmm_w8a8(const int8_t *x, const int8_t *w, const int64_t *group_list, int group_list_type,
                               int64_t m, int64_t k, int64_t n, int e, int transpose_b, const int32_t *bias,
                               const float *scale, const float *per_token, int32_t *acc_out, uint16_t *bf16_out) {
  if (m < 0 || k <= 0 || n <= 0 || e <= 0) return 1;
  int64_t last = 0;
  for (int g = 0; g < e; ++g) {
    int64_t s, t;
    group_range(group_list, e, group_list_type, m, g, &s, &t);
    last = t;
    const int8_t *wg = w + (int64_t)g * k * n;
#pragma omp parallel for schedule(static)
    for (int64_t r = s; r < t; ++r) {
      int32_t *row = (int32_t *)malloc(sizeof(int32_t) * (size_t)n);
      memset(row, 0, sizeof(int32_t) * (size_t)n);
      const int8_t *xr = x + r * k;
      if (!transpose_b) {
        for (int64_t kk = 0; kk < k; ++kk) {
          const int32_t xv = xr[kk];
          const int8_t *wr = wg + kk * n;
          for (int64_t j = 0; j < n; ++j) row[j] += xv * (int32_t)wr[j];
        }
      } else {
        for (int64_t j = 0; j < n; ++j) {
          const int8_t *wr = wg + j * k;
          int32_t s32 = 0;
          for (int64_t kk = 0; kk < k; ++kk) s32 += (int32_t)xr[kk] * (int32_t)wr[kk];
          row[j] = s32;
        }
      }
      for (int64_t j = 0; j < n; ++j) {
        int32_t c = row[j];
        if (bias) c = (int32_t)((uint32_t)c + (uint32_t)bias[(int64_t)g * n + j]);
        if (acc_out) acc_out[r * n + j] = c;
        if (bf16_out) {
          float f = (float)c;
          if (scale) f = f * scale[(int64_t)g * n + j];
          if (per_token) f = f * per_token[r];
          bf16_out[r * n + j] = oracle_f32_to_bf16(f);
        }
      }
      free(row);
    }
  }
  for (int64_t r = last; r < m; ++r) {
    if (acc_out) memset(acc_out + r * n, 0, sizeof(int32_t) * (size_t)n);
    if (bf16_out) memset(bf16_out + r * n, 0, sizeof(uint16_t) * (size_t)n);
  }
  return 0;
}

/*
 * Weight-only path in double precision on the exact operand values:
 *   out[r, j] = sum_k x[r,k] * (w[g,k,j] + off[g,j]) * scl[g,j]
 * x, scl, off arrive as bfloat16 bit patterns; w int8 [e,k,n]; out double [m,n].
 */
ORACLE_API int oracle_gmm_a16w8_f64(const uint16_t *x_bf16, const int8_t *w, const uint16_t *scl_bf16,
                                    const uint16_t *off_bf16, const int64_t *group_list, int group_list_type,
                                    int64_t m, int64_t k, int64_t n, int e, double *out) {
  if (m < 0 || k <= 0 || n <= 0 || e <= 0) return 1;
  memset(out, 0, sizeof(double) * (size_t)(m * n));
  for (int g = 0; g < e; ++g) {
    int64_t s, t;
    group_range(group_list, e, group_list_type, m, g, &s, &t);
    const int8_t *wg = w + (int64_t)g * k * n;
#pragma omp parallel for schedule(static)
    for (int64_t r = s; r < t; ++r) {
      double *row = out + r * n;
      double xsum = 0.0;
      for (int64_t kk = 0; kk < k; ++kk) {
        const double xv = (double)bf16_to_f32(x_bf16[r * k + kk]);
        xsum += xv;
        const int8_t *wr = wg + kk * n;
        for (int64_t j = 0; j < n; ++j) row[j] += xv * (double)wr[j];
      }
      for (int64_t j = 0; j < n; ++j) {
        const double o = off_bf16 ? (double)bf16_to_f32(off_bf16[(int64_t)g * n + j]) : 0.0;
        const double sc = scl_bf16 ? (double)bf16_to_f32(scl_bf16[(int64_t)g * n + j]) : 1.0;
        /* sum_k x*(w+o)*s == s*(sum_k x*w + o*sum_k x); exact reals, double rounding only */
        row[j] = (row[j] + o * xsum) * sc;
      }
    }
  }
  return 0;
}
