/*
 * TEST INFRASTRUCTURE ONLY -- CPU oracle for the 4-bit group-quantization path.
 *
 * A scalar, plain-C restatement of the arithmetic of
 *   popxl_addons/ops/group_quantize_decompress/group_quantize_decompress.py:95-141 (decompress)
 *   popxl_addons/ops/group_quantize_decompress/group_quantize_decompress.py:144-196 (compress)
 *   popxl_addons/layers/linear_gq.py:99-109 (decompress, then x @ w, then + bias)
 * Nothing in the shipped library links or loads this file; only the tests, the smoke
 * check and the benchmark's CPU-baseline leg use it, and only as the checker.
 *
 * binary16 arithmetic is done by evaluating every single operation exactly in
 * binary64 (products and sums of two binary16 numbers are exact there; a quotient is
 * correctly rounded to 53 bits, which makes the second rounding to 11 bits innocuous)
 * and rounding once to binary16 with round-to-nearest-even.  That is the IEEE-754
 * result of each operation, which is also what numpy's float16 ufuncs deliver.
 *
 * Pinning status:
 *   gq_oracle_decompress  pinned: all 65 536 packed words x (scale,bias) pairs against an
 *                         exact-rational evaluator, the reference's seeded fixture recipe
 *                         (tests/integration/ops/test_group_quantize_decompress.py:15-42),
 *                         and the invariants scale=0 / bias=0,scale=1 / code 0.
 *   gq_oracle_compress_*  pinned: fixture relation compress(t).packed == packed, arg-min ->
 *                         code 0, arg-max -> code 15, pack/unpack inverse, round-trip bound.
 *                         A constant group (scale == 0) is NOT defined by the reference
 *                         (0/0 cast to uint16); this oracle emits code 0 there.
 *   gq_oracle_linear      pinned: textbook y = x W^T + b in binary32 over the decompressed
 *                         weight; cross-checked against numpy's float32 matmul.
 */
#include <math.h>
#include <stdint.h>
#include <string.h>

/* ---- binary16 <-> binary64 ------------------------------------------------------- */

static double h2d(uint16_t h) {
  const int sign = h >> 15, e = (h >> 10) & 31, m = h & 1023;
  double v;
  if (e == 0)
    v = ldexp((double)m, -24);
  else if (e == 31)
    v = m ? NAN : INFINITY;
  else
    v = ldexp((double)(m | 1024), e - 25);
  return sign ? -v : v;
}

/* round-to-nearest-even binary64 -> binary16, subnormals kept, overflow to infinity */
static uint16_t d2h(double d) {
  uint64_t b;
  memcpy(&b, &d, 8);
  const uint16_t sign = (uint16_t)((b >> 48) & 0x8000u);
  if (isnan(d)) return (uint16_t)(sign | 0x7e00u);
  const double a = fabs(d);
  if (a == 0.0) return sign;
  if (isinf(a)) return (uint16_t)(sign | 0x7c00u);
  int ex;
  (void)frexp(a, &ex); /* a = f * 2^ex, f in [0.5, 1) => a in [2^(ex-1), 2^ex) */
  int q = ex - 11;     /* quantum exponent so that a / 2^q lies in [1024, 2048) */
  if (q < -24) q = -24;
  const double scaled = ldexp(a, -q); /* exact: power-of-two scaling */
  double r = nearbyint(scaled);       /* default rounding mode: to nearest, ties to even */
  if (r >= 2048.0) {
    r *= 0.5;
    q += 1;
  }
  if (q > 5) return (uint16_t)(sign | 0x7c00u); /* >= 65520 rounds to infinity */
  const unsigned m = (unsigned)r;
  if (m < 1024) return (uint16_t)(sign | m); /* subnormal (q == -24) or zero */
  return (uint16_t)(sign | ((unsigned)(q + 25) << 10) | (m - 1024));
}

uint16_t gq_oracle_f64_to_f16(double d) { return d2h(d); }
double gq_oracle_f16_to_f64(uint16_t h) { return h2d(h); }

/* ---- decompress: group_quantize_decompress.py:127-135 ------------------------------
 * packed [rows, n_groups, n_ids] uint16, scale/bias [rows, n_groups] binary16 bits,
 * out [rows, n_groups * n_ids * 4] binary16 bits.
 * The four codes of a word come out most-significant nibble first (shifts 12, 8, 4, 0,
 * :130); value = f16( f16(code * scale) + bias ) with two separate roundings (:134). */
void gq_oracle_decompress(const uint16_t *packed, const uint16_t *scale, const uint16_t *bias,
                          uint16_t *out, int64_t rows, int64_t n_groups, int64_t n_ids) {
  for (int64_t rg = 0; rg < rows * n_groups; ++rg) {
    const double s = h2d(scale[rg]), b = h2d(bias[rg]);
    for (int64_t i = 0; i < n_ids; ++i) {
      const uint16_t w = packed[rg * n_ids + i];
      for (int j = 0; j < 4; ++j) {
        const int code = (w >> (12 - 4 * j)) & 15;
        const uint16_t prod = d2h((double)code * s);
        out[(rg * n_ids + i) * 4 + j] = d2h(h2d(prod) + b);
      }
    }
  }
}

/* ---- compress: group_quantize_decompress.py:178-196 --------------------------------
 * t is [rows, n_groups * group_size] with the grouped axis already last (:172-176).
 * Returns 0, or -1 when a value is not finite (:182-183 raises ValueError).
 * f16 input: every operation rounds to binary16 (:186-192 on a float16 array).
 * f32 input: max/min are cast to binary16 first (:186-187), scale is binary16 (:189),
 *            (x - bias) / scale is evaluated in binary32 (:192 promotes). */
static uint16_t pack4(const unsigned c[4]) {
  /* codes @ [4096, 256, 16, 1] in uint16 arithmetic (:193-195): wraps like the reference */
  return (uint16_t)(c[0] * 4096u + c[1] * 256u + c[2] * 16u + c[3]);
}

int gq_oracle_compress_f16(const uint16_t *t, uint16_t *packed, uint16_t *scale, uint16_t *bias,
                           int64_t rows, int64_t n_groups, int64_t group_size) {
  const int64_t total = rows * n_groups * group_size;
  for (int64_t i = 0; i < total; ++i)
    if (((t[i] >> 10) & 31) == 31) return -1;
  const int64_t n_ids = group_size / 4;
  for (int64_t rg = 0; rg < rows * n_groups; ++rg) {
    const uint16_t *g = t + rg * group_size;
    double mx = h2d(g[0]), mn = mx;
    for (int64_t k = 1; k < group_size; ++k) {
      const double v = h2d(g[k]);
      if (v > mx) mx = v;
      if (v < mn) mn = v;
    }
    const uint16_t range = d2h(mx - mn);
    const uint16_t sc = d2h(h2d(range) / 15.0);
    const uint16_t bi = d2h(mn);
    scale[rg] = sc;
    bias[rg] = bi;
    const double s = h2d(sc), b = h2d(bi);
    for (int64_t i = 0; i < n_ids; ++i) {
      unsigned c[4];
      for (int j = 0; j < 4; ++j) {
        if (s == 0.0) { /* constant group: undefined in the reference, 0 here */
          c[j] = 0;
          continue;
        }
        const uint16_t diff = d2h(h2d(g[4 * i + j]) - b);
        const uint16_t quot = d2h(h2d(diff) / s);
        c[j] = (unsigned)(int)nearbyint(h2d(quot)); /* np.round: ties to even */
      }
      packed[rg * n_ids + i] = pack4(c);
    }
  }
  return 0;
}

int gq_oracle_compress_f32(const float *t, uint16_t *packed, uint16_t *scale, uint16_t *bias,
                           int64_t rows, int64_t n_groups, int64_t group_size) {
  const int64_t total = rows * n_groups * group_size;
  for (int64_t i = 0; i < total; ++i)
    if (!isfinite(t[i])) return -1;
  const int64_t n_ids = group_size / 4;
  for (int64_t rg = 0; rg < rows * n_groups; ++rg) {
    const float *g = t + rg * group_size;
    float mx = g[0], mn = g[0];
    for (int64_t k = 1; k < group_size; ++k) {
      if (g[k] > mx) mx = g[k];
      if (g[k] < mn) mn = g[k];
    }
    const uint16_t hmx = d2h((double)mx), hmn = d2h((double)mn);
    const uint16_t range = d2h(h2d(hmx) - h2d(hmn));
    const uint16_t sc = d2h(h2d(range) / 15.0);
    scale[rg] = sc;
    bias[rg] = hmn;
    const float s = (float)h2d(sc), b = (float)h2d(hmn);
    for (int64_t i = 0; i < n_ids; ++i) {
      unsigned c[4];
      for (int j = 0; j < 4; ++j) {
        if (s == 0.0f) {
          c[j] = 0;
          continue;
        }
        const float diff = g[4 * i + j] - b; /* binary32 */
        const float quot = diff / s;         /* binary32 */
        c[j] = (unsigned)(int)nearbyintf(quot);
      }
      packed[rg * n_ids + i] = pack4(c);
    }
  }
  return 0;
}

/* ---- layer: linear_gq.py:99-109 with dim=0 -----------------------------------------
 * y[m, n] = sum_k x[m, k] * W[n, k] (+ out_bias[n]); W is the decompressed weight
 * [n_out, k_in] (groups along k).  binary32 accumulation in k order, binary32 result:
 * the tolerance-bounded reference the fused kernels are compared with. */
void gq_oracle_linear(const uint16_t *x, const uint16_t *w_dec, const uint16_t *out_bias, float *y,
                      int64_t m_rows, int64_t n_out, int64_t k_in) {
  for (int64_t m = 0; m < m_rows; ++m)
    for (int64_t n = 0; n < n_out; ++n) {
      double acc = 0.0; /* binary64 accumulate: stricter than the binary32 the contract asks */
      for (int64_t k = 0; k < k_in; ++k) acc += h2d(x[m * k_in + k]) * h2d(w_dec[n * k_in + k]);
      if (out_bias) acc += h2d(out_bias[n]);
      y[m * n_out + n] = (float)acc;
    }
}
