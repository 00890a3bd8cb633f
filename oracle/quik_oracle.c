/* Scalar C restatement of the QUIK kernels' arithmetic (CPU oracle, second opinion).
 *
 * TEST INFRASTRUCTURE ONLY: loaded by tests/ (through oracle/c_oracle.py) to
 * cross-check the numpy oracle with an independently written implementation.
 * Nothing the library ships links or calls this file.
 *
 * Half and bfloat16 are handled as 16-bit patterns with hand-written conversions,
 * so no compiler half support is needed.  "fp16 op" = compute exactly or in a wider
 * type and round once (ties to even) to binary16.
 *
 * Reference sources followed (paths relative to the reference checkout):
 *   src/asymmetric/asymmetric.cu:340-381  per-row min/max -> (scale, zero)
 *   src/asymmetric/asymmetric.cu:382-446  indexed quantise 8/4 bit, outlier gather
 *   src/asymmetric/asymmetric.cu:119-173  dequantise (fp32)
 *   src/symmetric/symmetric.cu:6-61       symmetric quantise
 *   src/symmetric/symmetric.cu:91-113     symmetric dequantise (fp16 chain)
 *   src/matmul/matmul.cu:17-55,98-136     integer GEMM operand layout
 *   include/int4.h:78-98                  nibble order (element i at bits 4i)
 */
#include <math.h>
#include <stdint.h>
#include <string.h>

/* ---- binary16 <-> float ------------------------------------------------- */
static float h2f(uint16_t h) {
  uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
  uint32_t exp = (h >> 10) & 0x1Fu;
  uint32_t man = h & 0x3FFu;
  uint32_t bits;
  if (exp == 0) {
    if (man == 0) {
      bits = sign;
    } else { /* subnormal: value = man * 2^-24 */
      float v = (float)man * 5.9604644775390625e-8f;
      memcpy(&bits, &v, 4);
      bits |= sign;
    }
  } else if (exp == 31) {
    bits = sign | 0x7F800000u | (man << 13);
  } else {
    bits = sign | ((exp + 112u) << 23) | (man << 13);
  }
  float f;
  memcpy(&f, &bits, 4);
  return f;
}

/* double -> binary16, round to nearest even (one rounding from the double). */
static uint16_t d2h(double d) {
  uint16_t sign = 0;
  if (d != d) return 0x7E00u;
  if (signbit(d)) { sign = 0x8000u; d = -d; }
  if (d == 0.0) return sign;
  if (isinf(d)) return sign | 0x7C00u;
  int e;
  double m = frexp(d, &e); /* d = m * 2^e, m in [0.5, 1) */
  /* binary16: normal exponents for d in [2^-14, 65520) */
  int unb = e - 1;       /* d = (2m) * 2^unb, 2m in [1, 2) */
  if (unb < -14) {
    /* subnormal: quantum 2^-24 */
    double q = nearbyint(ldexp(d, 24)); /* ties-to-even in default mode */
    if (q >= 1024.0) return sign | 0x0400u;
    return sign | (uint16_t)q;
  }
  double scaled = nearbyint(ldexp(m, 11)); /* 2m * 2^10 in [1024, 2048] */
  if (scaled >= 2048.0) { scaled = 1024.0; unb += 1; }
  if (unb > 15) return sign | 0x7C00u;
  return sign | (uint16_t)((unb + 15) << 10) | (uint16_t)((uint32_t)scaled - 1024u);
}

/* ---- bfloat16 <-> float -------------------------------------------------- */
static float b2f(uint16_t b) {
  uint32_t bits = (uint32_t)b << 16;
  float f;
  memcpy(&f, &bits, 4);
  return f;
}
static uint16_t f2b(float f) {
  uint32_t u;
  if (f != f) return 0x7FC0u;
  memcpy(&u, &f, 4);
  u += 0x7FFFu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}

/* generic over the storage type: is_bf16 = 0 -> binary16, 1 -> bfloat16 */
static float s2f(uint16_t v, int is_bf16) { return is_bf16 ? b2f(v) : h2f(v); }
/* Round a double result of ONE arithmetic op on storage-type inputs. For bfloat16 the
 * double -> float -> bfloat16 chain is innocuous (24 >= 2*8+2, 53 >= 2*24+2). */
static uint16_t d2s(double d, int is_bf16) { return is_bf16 ? f2b((float)d) : d2h(d); }

static int rne_to_int(float d) {
  if (d != d) return 0;
  double r = nearbyint((double)d);
  if (r >= 2147483647.0) return 2147483647;
  if (r <= -2147483648.0) return (-2147483647 - 1);
  return (int)r;
}

/* fmax / fmin that skip NaN, as __hmax / __hmin do */
static float max_nn(float a, float b) { return fmaxf(a, b); }
static float min_nn(float a, float b) { return fminf(a, b); }

/* ---- exported helpers for conversion tests ------------------------------ */
float qo_half_to_float(uint16_t h) { return h2f(h); }
uint16_t qo_double_to_half(double d) { return d2h(d); }
uint16_t qo_float_to_bf16(float f) { return f2b(f); }

/* ---- asymmetric quantise -------------------------------------------------
 * x [rows, cols] storage-type bit patterns; dst is rows*num_int/2 bytes (bits=4)
 * or rows*num_int bytes (bits=8); meta [2*rows]; fp_x [rows, num_fp]. */
void qo_asym_quantize(const uint16_t *x, int64_t rows, int64_t cols,
                      const int64_t *int_idx, int64_t num_int,
                      const int64_t *fp_idx, int64_t num_fp, int bits,
                      int is_bf16, uint8_t *dst, uint16_t *meta, uint16_t *fp_x) {
  const int maxq = (1 << bits) - 1, half_range = 1 << (bits - 1);
  for (int64_t r = 0; r < rows; ++r) {
    const uint16_t *row = x + r * cols;
    /* seeded with the first int column, asymmetric.cu:351-352 */
    float mx = s2f(row[int_idx[0]], is_bf16), mn = mx;
    for (int64_t j = 0; j < num_int; ++j) {
      float v = s2f(row[int_idx[j]], is_bf16);
      mx = max_nn(mx, v);
      mn = min_nn(mn, v);
    }
    float sc = fmaxf((mx - mn) / (float)maxq, 1e-6f); /* asymmetric.cu:375-377 */
    uint16_t scale = d2s((double)sc, is_bf16);
    uint16_t zero = d2s((double)mn, is_bf16); /* exact: mn is a storage value */
    meta[2 * r] = scale;
    meta[2 * r + 1] = zero;
    double zf = (double)s2f(zero, is_bf16), sf = (double)s2f(scale, is_bf16);
    for (int64_t j = 0; j < num_int; ++j) {
      double xv = (double)s2f(row[int_idx[j]], is_bf16);
      uint16_t diff = d2s(xv - zf, is_bf16);                 /* __hsub */
      uint16_t quo = d2s((double)s2f(diff, is_bf16) / sf, is_bf16); /* __hdiv */
      int v = rne_to_int(s2f(quo, is_bf16));
      if (v < 0) v = 0;
      if (v > maxq) v = maxq;
      v -= half_range;
      if (bits == 8) {
        dst[r * num_int + j] = (uint8_t)(int8_t)v;
      } else {
        uint8_t *b = dst + r * (num_int / 2) + j / 2;
        if ((j & 1) == 0) *b = (uint8_t)(v & 0xF);
        else *b = (uint8_t)(*b | ((v & 0xF) << 4));
      }
    }
    for (int64_t j = 0; j < num_fp; ++j) fp_x[r * num_fp + j] = row[fp_idx[j]];
  }
}

/* ---- integer GEMM: C[m,n] = sum_k a[m,k] * b[n,k] ------------------------ */
static int nib(const uint8_t *p, int64_t k) {
  int v = (p[k >> 1] >> ((k & 1) * 4)) & 0xF;
  return v >= 8 ? v - 16 : v;
}
void qo_int4_matmul(const uint8_t *a, const uint8_t *b, int32_t *c, int64_t M,
                    int64_t N, int64_t K) {
  for (int64_t m = 0; m < M; ++m)
    for (int64_t n = 0; n < N; ++n) {
      int64_t acc = 0;
      for (int64_t k = 0; k < K; ++k)
        acc += nib(a + m * (K / 2), k) * nib(b + n * (K / 2), k);
      c[m * N + n] = (int32_t)acc;
    }
}
void qo_int8_matmul(const int8_t *a, const int8_t *b, int32_t *c, int64_t M,
                    int64_t N, int64_t K) {
  for (int64_t m = 0; m < M; ++m)
    for (int64_t n = 0; n < N; ++n) {
      int64_t acc = 0;
      for (int64_t k = 0; k < K; ++k) acc += (int)a[m * K + k] * (int)b[n * K + k];
      c[m * N + n] = (int32_t)acc;
    }
}

/* ---- asymmetric dequantise (fp32, reference association order) ---------- */
void qo_asym_dequantize(const int32_t *acc, const uint16_t *meta,
                        const uint16_t *scale_col, const uint16_t *w_red,
                        const uint16_t *y, int64_t rows, int64_t cols, int bits,
                        int is_bf16, uint16_t *out) {
  const float shift_value = bits == 4 ? 8.0f : 128.0f;
  for (int64_t r = 0; r < rows; ++r)
    for (int64_t c = 0; c < cols; ++c) {
      volatile float x = (float)acc[r * cols + c];
      float srow = s2f(meta[2 * r], is_bf16), z = s2f(meta[2 * r + 1], is_bf16);
      float scol = s2f(scale_col[c], is_bf16);
      volatile float t0 = shift_value * srow;
      volatile float t1 = z + t0;
      volatile float shift = t1 * s2f(w_red[c], is_bf16);
      volatile float ss = srow * scol;
      volatile float prod = x * ss;
      volatile float add = shift + s2f(y[r * cols + c], is_bf16);
      volatile float res = prod + add;
      out[r * cols + c] = is_bf16 ? f2b(res) : d2h((double)res);
    }
}

/* ---- symmetric quantise --------------------------------------------------- */
void qo_sym_quantize(const uint16_t *x, const uint16_t *scale, int64_t rows,
                     int64_t cols, int bits, uint8_t *dst) {
  int64_t cols_dst = bits == 4 ? (cols + 1) / 2 : cols;
  if (bits == 4) memset(dst, 0, (size_t)(rows * cols_dst));
  for (int64_t r = 0; r < rows; ++r)
    for (int64_t c = 0; c < cols; ++c) {
      uint16_t q = d2h((double)h2f(x[r * cols + c]) / (double)h2f(scale[r]));
      int v = rne_to_int(h2f(q));
      if (bits == 8) dst[r * cols + c] = (uint8_t)(v & 0xFF);
      else dst[r * cols_dst + c / 2] |= (uint8_t)((v & 0xF) << ((c & 1) * 4));
    }
}

/* ---- symmetric dequantise (fp16 chain); x_kind: 8 int8, 16 half, 32 int32 - */
void qo_sym_dequantize(const void *x, int x_kind, const uint16_t *scale_row,
                       const uint16_t *scale_col, const uint16_t *y,
                       int64_t rows, int64_t cols, uint16_t *out) {
  for (int64_t r = 0; r < rows; ++r)
    for (int64_t c = 0; c < cols; ++c) {
      int64_t i = r * cols + c;
      uint16_t xh;
      if (x_kind == 16) xh = ((const uint16_t *)x)[i];
      else if (x_kind == 8) xh = d2h((double)((const int8_t *)x)[i]);
      else xh = d2h((double)((const int32_t *)x)[i]);
      uint16_t t = d2h((double)h2f(xh) * (double)h2f(scale_row[r]));
      t = d2h((double)h2f(t) * (double)h2f(scale_col[c]));
      out[i] = d2h((double)h2f(t) + (double)h2f(y[i]));
    }
}
