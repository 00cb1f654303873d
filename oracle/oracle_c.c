/*
 * C restatement of MatGPTQ's slice -> dequantize -> linear path.
 * TEST INFRASTRUCTURE ONLY: a checker for the HIP kernels and a CPU baseline
 * for the benchmark.  The shipped library never links or loads this file.
 *
 * Reference anchors (relative to the reference checkout):
 *   matryoshka_slice   src/quant_utils_matgpqt.py:9-17
 *   dequantize         src/quant_utils_matgpqt.py:19-22
 *   forward            src/quant_utils_matgpqt.py:218-224
 *
 * fp16 is handled by explicit bit conversion (round to nearest even), so the
 * file builds with any C99 compiler and does not depend on _Float16 support.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

/* ---- fp16 <-> fp32 ------------------------------------------------------ */

static float half_to_float(uint16_t h) {
  uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
  uint32_t exp = (h >> 10) & 0x1Fu;
  uint32_t man = h & 0x3FFu;
  uint32_t bits;
  if (exp == 0) {
    if (man == 0) {
      bits = sign;
    } else { /* subnormal: normalise */
      int e = -1;
      do { man <<= 1; e++; } while ((man & 0x400u) == 0);
      man &= 0x3FFu;
      bits = sign | ((uint32_t)(127 - 15 - e) << 23) | (man << 13);
    }
  } else if (exp == 31) {
    bits = sign | 0x7F800000u | (man << 13);
  } else {
    bits = sign | ((exp + 127 - 15) << 23) | (man << 13);
  }
  float f;
  memcpy(&f, &bits, 4);
  return f;
}

/* double -> fp16 bits, round to nearest even, with overflow to inf */
static uint16_t double_to_half(double d) {
  uint16_t sign = 0;
  if (signbit(d)) { sign = 0x8000u; d = -d; }
  if (isnan(d)) return (uint16_t)(sign | 0x7E00u);
  if (d >= 65520.0) return (uint16_t)(sign | 0x7C00u); /* rounds to inf */
  if (d == 0.0) return sign;
  int e;
  double m = frexp(d, &e); /* d = m * 2^e, m in [0.5, 1) */
  /* fp16 normal: 1.xxx * 2^(e-1), exponent field = e - 1 + 15 */
  int exp_field = e - 1 + 15;
  double scaled;
  if (exp_field >= 1) {
    /* mantissa has 10 fractional bits relative to 2^(e-1) */
    scaled = ldexp(m, 11); /* in [1024, 2048) */
  } else {
    /* subnormal: value = k * 2^-24 */
    scaled = ldexp(d, 24);
    exp_field = 0;
  }
  double r = nearbyint(scaled); /* default rounding mode is to nearest even */
  uint32_t k = (uint32_t)r;
  if (exp_field >= 1) {
    if (k == 2048u) { k = 1024u; exp_field += 1; }
    if (exp_field >= 31) return (uint16_t)(sign | 0x7C00u);
    return (uint16_t)(sign | ((uint32_t)exp_field << 10) | (k - 1024u));
  }
  /* subnormal result may round up into the smallest normal (k == 1024) */
  return (uint16_t)(sign | k);
}

/* ---- slice (src/quant_utils_matgpqt.py:9-17) ----------------------------- */

uint8_t matgptq_oracle_slice1(uint8_t q, int slice_bits, int master_bits) {
  int drop = 8 - slice_bits; /* always an 8-bit store (:10) */
  int floor_v = q >> drop;
  int top = (1 << slice_bits) - 1;
  if (master_bits == slice_bits) return (uint8_t)(floor_v > top ? top : floor_v);
  int round_bit = (q >> (drop - 1)) & 1;
  int v = floor_v + round_bit;
  return (uint8_t)(v > top ? top : v);
}

void matgptq_oracle_slice(const uint8_t *q, uint8_t *out, int64_t count, int slice_bits,
                          int master_bits) {
  for (int64_t i = 0; i < count; i++) out[i] = matgptq_oracle_slice1(q[i], slice_bits, master_bits);
}

/* ---- dequantize (src/quant_utils_matgpqt.py:19-22) ------------------------ */
/* q: [N,K] u8 master codes; scale, zero: [N, K/g] fp16 bits; w: [N,K] fp16 bits */
void matgptq_oracle_dequantize(const uint8_t *q, const uint16_t *scale, const uint16_t *zero,
                               uint16_t *w, int64_t n, int64_t k, int group_size, int slice_bits,
                               int master_bits) {
  int64_t g = group_size == -1 ? k : group_size;
  int64_t groups = k / g;
  int shift = master_bits - slice_bits;
#pragma omp parallel for schedule(static)
  for (int64_t r = 0; r < n; r++) {
    for (int64_t c = 0; c < k; c++) {
      int s = (int)matgptq_oracle_slice1(q[r * k + c], slice_bits, master_bits) << shift;
      float z = half_to_float(zero[r * groups + c / g]);
      float sc = half_to_float(scale[r * groups + c / g]);
      /* (q_shifted - zero) is one fp16 op, scale * (...) a second one */
      uint16_t diff = double_to_half((double)s - (double)z);
      w[r * k + c] = double_to_half((double)sc * (double)half_to_float(diff));
    }
  }
}

/* ---- linear (F.linear, src/quant_utils_matgpqt.py:223) --------------------- */
/* x: [M,K] fp16 bits, w: [N,K] fp16 bits, y: [M,N] fp16 bits; double accumulate */
void matgptq_oracle_linear(const uint16_t *x, const uint16_t *w, uint16_t *y, int64_t m, int64_t n,
                           int64_t k) {
  float *xf = (float *)malloc(sizeof(float) * (size_t)(m * k));
  for (int64_t i = 0; i < m * k; i++) xf[i] = half_to_float(x[i]);
#pragma omp parallel for schedule(static)
  for (int64_t r = 0; r < n; r++) {
    for (int64_t b = 0; b < m; b++) {
      double acc = 0.0;
      for (int64_t c = 0; c < k; c++) acc += (double)xf[b * k + c] * (double)half_to_float(w[r * k + c]);
      y[b * n + r] = double_to_half(acc);
    }
  }
  free(xf);
}

/* Whole path in one call: what FakeMatryoshkaLinear.forward computes (no perm, no bias). */
void matgptq_oracle_forward(const uint8_t *q, const uint16_t *scale, const uint16_t *zero,
                            const uint16_t *x, uint16_t *y, int64_t m, int64_t n, int64_t k,
                            int group_size, int slice_bits, int master_bits) {
  uint16_t *w = (uint16_t *)malloc(sizeof(uint16_t) * (size_t)(n * k));
  matgptq_oracle_dequantize(q, scale, zero, w, n, k, group_size, slice_bits, master_bits);
  matgptq_oracle_linear(x, w, y, m, n, k);
  free(w);
}

/* exposed for the conversion tests */
uint16_t matgptq_oracle_f64_to_f16(double d) { return double_to_half(d); }
float matgptq_oracle_f16_to_f32(uint16_t h) { return half_to_float(h); }
