/*
 * CPU oracle for the fused-kernel hot path (plain C).  TEST INFRASTRUCTURE ONLY.
 *
 * An independent restatement of the golden computations in afir_oracle.py,
 * used (a) to cross-check the numpy oracle and (b) as the timed CPU baseline
 * ("port") next to the GPU figures.  Only tests, the smoke check and the
 * benchmark's CPU-baseline leg may load it; the shipped library never does.
 *
 * Reference formulas followed (paths relative to the reference tree):
 *   examples/broadcast-add-reduce/gen_data.py:27-33        (f32 accumulate)
 *   examples/relu-broadcast-transpose/gen_inputs.py:28-35  (relu, f32 add, RNE to f16)
 *   examples/gather-elementwise-fusion/gen_data.py:46-67   (gather, f32 math, RNE to f16)
 *   examples/matmul-add-leakyrelu/gen_data.py:28-36        (f32 matmul + bias, leaky relu)
 *   lib/Runtime/Execution/OutputComparator.cpp:16-65,121-125 (decode + tolerance test)
 *
 * Build: gcc -O2 -fopenmp -ffp-contract=off -shared -fPIC (see Makefile).
 * -ffp-contract=off keeps every f32 add and mul a separate IEEE operation.
 *
 * Pins: each function is compared with the numpy oracle on seeded inputs in
 * tests/test_oracle_c.py; the row-sum reproduces numpy's pairwise order bit
 * for bit, the f16/bf16 conversions are checked over all 65536 bit patterns.
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

/* ---------------- storage dtype conversions ---------------- */

static inline float bits_f32(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }
static inline uint32_t f32_bits(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }

float oracle_f16_to_f32(uint16_t h) {
  uint32_t sign = (uint32_t)(h >> 15) << 31;
  uint32_t exp = (h >> 10) & 0x1f;
  uint32_t frac = h & 0x3ff;
  if (exp == 0) {
    if (frac == 0) return bits_f32(sign);
    /* subnormal: value = frac * 2^-24 */
    float v = (float)frac * 5.9604644775390625e-08f;
    return (sign ? -v : v);
  }
  if (exp == 31) return bits_f32(sign | 0x7f800000u | (frac << 13));
  return bits_f32(sign | ((exp + 112) << 23) | (frac << 13));
}

/* round-to-nearest-even float32 -> float16 */
uint16_t oracle_f32_to_f16(float f) {
  uint32_t u = f32_bits(f);
  uint32_t sign = (u >> 16) & 0x8000u;
  uint32_t absu = u & 0x7fffffffu;
  if (absu >= 0x7f800000u) { /* inf / nan */
    if (absu > 0x7f800000u) return (uint16_t)(sign | 0x7e00u | ((absu >> 13) & 0x3ffu));
    return (uint16_t)(sign | 0x7c00u);
  }
  if (absu >= 0x477ff000u) return (uint16_t)(sign | 0x7c00u); /* rounds to inf */
  if (absu < 0x33000001u) return (uint16_t)sign;              /* rounds to zero */
  int32_t e = (int32_t)(absu >> 23) - 127;
  uint32_t mant = (absu & 0x7fffffu) | 0x800000u;
  uint32_t shift, half_bits;
  if (e < -14) { /* subnormal result */
    shift = (uint32_t)(13 + (-14 - e));
    half_bits = 0;
  } else {
    shift = 13;
    half_bits = (uint32_t)(e + 15) << 10;
    mant &= 0x7fffffu;
  }
  uint32_t q = mant >> shift;
  uint32_t rem = mant & ((1u << shift) - 1u);
  uint32_t halfway = 1u << (shift - 1);
  if (rem > halfway || (rem == halfway && (q & 1u))) q++;
  return (uint16_t)(sign | (half_bits + q)); /* carry propagates into exponent */
}

float oracle_bf16_to_f32(uint16_t b) { return bits_f32((uint32_t)b << 16); }

uint16_t oracle_f32_to_bf16(float f) {
  uint32_t u = f32_bits(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40u);
  uint32_t lsb = (u >> 16) & 1u;
  return (uint16_t)((u + 0x7fffu + lsb) >> 16);
}

/* ---------------- C1: out = (a + b) * b ---------------- */

void oracle_add_mul_f32(const float *a, const float *b, float *out, size_t n) {
#pragma omp parallel for schedule(static)
  for (ptrdiff_t i = 0; i < (ptrdiff_t)n; ++i) {
    float s = a[i] + b[i];
    out[i] = s * b[i];
  }
}

/* ---------------- C2: y[i] = sum_j (x[i,j] + bias[j]) ---------------- */

/* numpy's pairwise summation for a contiguous float run: blocks of at most
 * 128 elements summed with 8 interleaved accumulators, halves split at a
 * multiple of 8 above that. */
static float pairwise_sum_f32(const float *a, ptrdiff_t n) {
  if (n < 8) {
    float res = 0.f;
    for (ptrdiff_t i = 0; i < n; ++i) res += a[i];
    return res;
  }
  if (n <= 128) {
    float r[8];
    for (int j = 0; j < 8; ++j) r[j] = a[j];
    ptrdiff_t i;
    for (i = 8; i < n - (n % 8); i += 8)
      for (int j = 0; j < 8; ++j) r[j] += a[i + j];
    float res = ((r[0] + r[1]) + (r[2] + r[3])) + ((r[4] + r[5]) + (r[6] + r[7]));
    for (; i < n; ++i) res += a[i];
    return res;
  }
  ptrdiff_t n2 = n / 2;
  n2 -= n2 % 8;
  return pairwise_sum_f32(a, n2) + pairwise_sum_f32(a + n2, n - n2);
}

/* scratch: caller-provided m*n floats are avoided by summing one row at a
 * time through a per-thread row buffer of n floats (rowbuf: threads*n). */
void oracle_bcast_add_rowsum_f32(const float *x, const float *bias, float *y,
                                 size_t m, size_t n, float *rowbuf, int nthreads_buf) {
  (void)nthreads_buf;
#pragma omp parallel
  {
    int tid = 0;
#ifdef _OPENMP
    tid = omp_get_thread_num();
#endif
    float *t = rowbuf + (size_t)tid * n;
#pragma omp for schedule(static)
    for (ptrdiff_t i = 0; i < (ptrdiff_t)m; ++i) {
      const float *row = x + (size_t)i * n;
      for (size_t j = 0; j < n; ++j) t[j] = row[j] + bias[j];
      y[i] = pairwise_sum_f32(t, (ptrdiff_t)n);
    }
  }
}

int oracle_max_threads(void) {
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}

/* ---------------- C3: out[b,j,i] = f16(relu(x[b,i,j]) + c[j]) ---------------- */

void oracle_relu_bcast_add_transpose_f16(const uint16_t *x, const uint16_t *c,
                                         uint16_t *out, size_t nb, size_t m, size_t n) {
#pragma omp parallel for schedule(static) collapse(2)
  for (ptrdiff_t b = 0; b < (ptrdiff_t)nb; ++b) {
    for (ptrdiff_t j = 0; j < (ptrdiff_t)n; ++j) {
      float cj = oracle_f16_to_f32(c[j]);
      for (size_t i = 0; i < m; ++i) {
        float v = oracle_f16_to_f32(x[((size_t)b * m + i) * n + (size_t)j]);
        float r = v > 0.f ? v : 0.f;
        if (v != v) r = v; /* maximum propagates NaN */
        out[((size_t)b * n + (size_t)j) * m + i] = oracle_f32_to_f16(r + cj);
      }
    }
  }
}

/* ---------------- C4: out[r,:] = f16(table[idx[r],:] * scale + shift) ---------------- */

int oracle_gather_scale_shift_f16(const uint16_t *table, const int32_t *idx,
                                  const uint16_t *scale, const uint16_t *shift,
                                  uint16_t *out, size_t rows, size_t dim, size_t nidx) {
  int bad = 0;
#pragma omp parallel for schedule(static) reduction(| : bad)
  for (ptrdiff_t r = 0; r < (ptrdiff_t)nidx; ++r) {
    int64_t src = idx[r];
    if (src < 0 || (size_t)src >= rows) { bad |= 1; continue; }
    const uint16_t *row = table + (size_t)src * dim;
    uint16_t *o = out + (size_t)r * dim;
    for (size_t j = 0; j < dim; ++j) {
      float p = oracle_f16_to_f32(row[j]) * oracle_f16_to_f32(scale[j]);
      o[j] = oracle_f32_to_f16(p + oracle_f16_to_f32(shift[j]));
    }
  }
  return bad;
}

/* ---------------- C5: out = bf16(leakyrelu(A@B + bias, alpha)) ---------------- */

/* acc[i,:] accumulates over k in increasing order in float32; accbuf holds
 * one float row of n per thread. */
void oracle_matmul_bias_leakyrelu_bf16(const uint16_t *a, const uint16_t *b,
                                       const uint16_t *bias, uint16_t *out,
                                       size_t m, size_t k, size_t n, float alpha,
                                       float *accbuf) {
#pragma omp parallel
  {
    int tid = 0;
#ifdef _OPENMP
    tid = omp_get_thread_num();
#endif
    float *acc = accbuf + (size_t)tid * n;
#pragma omp for schedule(static)
    for (ptrdiff_t i = 0; i < (ptrdiff_t)m; ++i) {
      for (size_t j = 0; j < n; ++j) acc[j] = 0.f;
      for (size_t kk = 0; kk < k; ++kk) {
        float av = oracle_bf16_to_f32(a[(size_t)i * k + kk]);
        const uint16_t *brow = b + kk * n;
        for (size_t j = 0; j < n; ++j) acc[j] += av * oracle_bf16_to_f32(brow[j]);
      }
      for (size_t j = 0; j < n; ++j) {
        float v = acc[j] + oracle_bf16_to_f32(bias[j]);
        float r = (v >= 0.f) ? v : v * alpha;
        out[(size_t)i * n + j] = oracle_f32_to_bf16(r);
      }
    }
  }
}

/* ---------------- comparator ---------------- */

/* dtype codes: 0 f16, 1 bf16, 2 f32, 3 i8, 4 i32, 5 i64 */
static float cmp_decode(const void *base, size_t idx, int dtype) {
  const uint8_t *p = (const uint8_t *)base;
  switch (dtype) {
  case 0: {
    uint16_t h; memcpy(&h, p + idx * 2, 2);
    uint32_t sign = (h >> 15) & 1, exp = (h >> 10) & 0x1f, frac = h & 0x3ff, f;
    if (exp == 0) f = (sign << 31) | (frac << 13);
    else if (exp == 31) f = (sign << 31) | 0x7f800000u | (frac << 13);
    else f = (sign << 31) | ((exp + 112) << 23) | (frac << 13);
    return bits_f32(f);
  }
  case 1: { uint16_t h; memcpy(&h, p + idx * 2, 2); return bits_f32((uint32_t)h << 16); }
  case 2: { float v; memcpy(&v, p + idx * 4, 4); return v; }
  case 3: { int8_t v; memcpy(&v, p + idx, 1); return (float)v; }
  case 4: { int32_t v; memcpy(&v, p + idx * 4, 4); return (float)v; }
  case 5: { int64_t v; memcpy(&v, p + idx * 8, 8); return (float)v; }
  }
  return 0.f;
}

/* returns number of elements with |a-e| > atol + rtol*|e|; fills max/mean */
size_t oracle_compare(const void *actual, const void *expected, size_t n, int dtype,
                      double atol, double rtol, double *max_abs, double *sum_abs) {
  size_t bad = 0;
  double mx = 0.0, tot = 0.0;
  for (size_t i = 0; i < n; ++i) {
    double a = (double)cmp_decode(actual, i, dtype);
    double e = (double)cmp_decode(expected, i, dtype);
    double d = fabs(a - e);
    tot += d;
    if (d > mx) mx = d;
    if (d > atol + rtol * fabs(e)) ++bad;
  }
  *max_abs = mx;
  *sum_abs = tot;
  return bad;
}
