/*
 * CPU oracle for the tcu_scope hot path.  TEST INFRASTRUCTURE ONLY: nothing in the GPU
 * library links or calls this file (see tcu_oracle.h for what pins each function).
 */
#include "tcu_oracle.h"

#include <math.h>
#include <pthread.h>
#include <stdlib.h>
#include <string.h>

/* ------------------------------------------------------------------------------------ */
/* fp16 conversion                                                                      */
/* ------------------------------------------------------------------------------------ */

typedef union {
  uint32_t u;
  float f;
} bits32;

/* Follows the bit recipe of reference src/utils/fp16_conversion.hpp:91-114: shift the
 * 15 magnitude bits into fp32 position, re-bias the exponent, patch Inf/NaN and
 * renormalise subnormals by a magic subtraction. */
float tcu_oracle_f16_to_f32(uint16_t h) {
  const uint32_t shifted_exp = 0x7c00u << 13;
  bits32 o, magic;
  magic.u = 113u << 23;
  o.u = ((uint32_t)h & 0x7fffu) << 13;
  uint32_t e = o.u & shifted_exp;
  o.u += (127u - 15u) << 23;
  if (e == shifted_exp) {
    o.u += (128u - 16u) << 23;
  } else if (e == 0) {
    o.u += 1u << 23;
    o.f -= magic.f;
  }
  o.u |= ((uint32_t)h & 0x8000u) << 16;
  return o.f;
}

/* IEEE binary32 -> binary16, round to nearest, ties to even.  Works on the integer
 * representation so that no host rounding mode is involved. */
uint16_t tcu_oracle_f32_to_f16(float f) {
  bits32 v;
  v.f = f;
  const uint32_t sign = (v.u >> 16) & 0x8000u;
  const uint32_t absu = v.u & 0x7fffffffu;
  if (absu >= 0x7f800000u) { /* Inf or NaN */
    if (absu > 0x7f800000u) return (uint16_t)(sign | 0x7e00u | ((absu >> 13) & 0x3ffu));
    return (uint16_t)(sign | 0x7c00u);
  }
  if (absu >= 0x477ff000u) { /* >= 65520 rounds to infinity */
    return (uint16_t)(sign | 0x7c00u);
  }
  if (absu < 0x33000001u) { /* <= 2^-25 rounds to zero (tie goes to even = 0) */
    return (uint16_t)sign;
  }
  int32_t exp = (int32_t)(absu >> 23) - 127;
  uint32_t man = (absu & 0x7fffffu) | 0x800000u; /* 24-bit significand */
  int shift;                                     /* bits to drop */
  uint32_t base;
  if (exp < -14) { /* subnormal half: value = man * 2^(exp-23), unit = 2^-24 */
    shift = -exp - 1; /* 13 + (-14 - exp) */
    base = 0;
  } else {
    shift = 13;
    base = (uint32_t)(exp + 15) << 10;
    man &= 0x7fffffu;
  }
  uint32_t q = man >> shift;
  uint32_t rem = man & ((1u << shift) - 1u);
  uint32_t half = 1u << (shift - 1);
  if (rem > half || (rem == half && (q & 1u))) q++;
  /* a carry out of the mantissa bumps the exponent, which is the right answer */
  return (uint16_t)(sign | (base + q));
}

uint16_t tcu_oracle_f64_to_f16(double d) {
  if (isnan(d)) return 0x7e00u;
  uint16_t sign = signbit(d) ? 0x8000u : 0u;
  double a = fabs(d);
  if (a >= 65520.0) return (uint16_t)(sign | 0x7c00u);
  if (a == 0.0) return sign;
  int e;
  (void)frexp(a, &e); /* a = m * 2^e, m in [0.5,1) => a in [2^(e-1), 2^e) */
  int ex = e - 1;     /* floor(log2 a) */
  if (ex < -14) ex = -14;
  double unit = ldexp(1.0, ex - 10);
  double q = a / unit; /* exact: division by a power of two */
  double fl = floor(q);
  double rem = q - fl;
  if (rem > 0.5 || (rem == 0.5 && fmod(fl, 2.0) != 0.0)) fl += 1.0;
  /* fl is an integer <= 2048; 2048 means carry into the next binade */
  uint32_t qi = (uint32_t)fl;
  uint32_t bitsv;
  if (ex == -14 && qi < 1024u) {
    bitsv = qi; /* subnormal */
  } else {
    bitsv = ((uint32_t)(ex + 15) << 10) + (qi - 1024u);
  }
  return (uint16_t)(sign | bitsv);
}

double tcu_oracle_ulp_f16(double v) {
  double a = fabs(v);
  if (!(a >= 6.103515625e-05)) return ldexp(1.0, -24); /* below 2^-14 (or NaN) */
  if (a >= 32768.0) return 32.0;
  int e;
  (void)frexp(a, &e);
  return ldexp(1.0, e - 1 - 10);
}

/* ------------------------------------------------------------------------------------ */
/* inputs                                                                               */
/* ------------------------------------------------------------------------------------ */

static inline uint64_t mix64(uint64_t z) {
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
  return z ^ (z >> 31);
}

uint64_t tcu_oracle_splitmix64(uint64_t seed, uint64_t i) {
  return mix64(seed + (i + 1) * 0x9E3779B97F4A7C15ull);
}

static uint16_t gen_one(uint64_t seed, uint64_t i, int dist) {
  uint64_t z = tcu_oracle_splitmix64(seed, i);
  switch (dist) {
    case TCU_ORACLE_DIST_UNIFORM: {
      uint32_t u = (uint32_t)(z >> 40); /* 24 bits */
      float x = (float)u * 0x1p-23f - 1.0f; /* exact in fp32 */
      uint16_t h = tcu_oracle_f32_to_f16(x);
      return h == 0x3c00u ? 0x3bffu : h;
    }
    case TCU_ORACLE_DIST_GRID: {
      int k = (int)(z >> 52) - 2048;
      return tcu_oracle_f32_to_f16((float)k * 0x1p-11f);
    }
    case TCU_ORACLE_DIST_NORMAL: {
      uint64_t z2 = mix64(z + 0x9E3779B97F4A7C15ull);
      double u1 = ((double)(z >> 40) + 1.0) * 0x1p-24; /* (0,1] */
      double u2 = (double)(z2 >> 40) * 0x1p-24;        /* [0,1) */
      double r = sqrt(-2.0 * log(u1)) * cos(6.283185307179586476925286766559 * u2);
      return tcu_oracle_f32_to_f16((float)r);
    }
    case TCU_ORACLE_DIST_SMALLINT: {
      uint32_t k = (uint32_t)((z >> 33) % 3u);
      return tcu_oracle_f32_to_f16((float)k);
    }
    default: return 0;
  }
}

void tcu_oracle_generate_f16_range(uint16_t *out, size_t first, size_t n, uint64_t seed, int dist) {
  for (size_t i = 0; i < n; i++) out[i] = gen_one(seed, (uint64_t)(first + i), dist);
}

void tcu_oracle_generate_f16(uint16_t *out, size_t n, uint64_t seed, int dist) {
  tcu_oracle_generate_f16_range(out, 0, n, seed, dist);
}

void tcu_oracle_fill_f16(uint16_t *out, float value, size_t n) {
  uint16_t h = tcu_oracle_f32_to_f16(value);
  for (size_t i = 0; i < n; i++) out[i] = h;
}

void tcu_oracle_convert_f32_to_f16(uint16_t *out, const float *in, size_t n) {
  for (size_t i = 0; i < n; i++) out[i] = tcu_oracle_f32_to_f16(in[i]);
}

/* ------------------------------------------------------------------------------------ */
/* reference CPU path: fp32 sequential running sum, fp16 out                             */
/* ------------------------------------------------------------------------------------ */

void tcu_oracle_seg_reduce_ref(const uint16_t *in, uint16_t *out, size_t num_segments, size_t segment_size) {
  for (size_t j = 0; j < num_segments; j++) {
    float correct_segment_sum = 0;
    const uint16_t *p = in + j * segment_size;
    for (size_t i = 0; i < segment_size; i++) correct_segment_sum += tcu_oracle_f16_to_f32(p[i]);
    out[j] = tcu_oracle_f32_to_f16(correct_segment_sum);
  }
}

void tcu_oracle_seg_scan_ref(const uint16_t *in, uint16_t *out, size_t num_segments, size_t segment_size) {
  for (size_t j = 0; j < num_segments; j++) {
    float running = 0;
    const uint16_t *p = in + j * segment_size;
    uint16_t *q = out + j * segment_size;
    for (size_t i = 0; i < segment_size; i++) {
      running += tcu_oracle_f16_to_f32(p[i]);
      q[i] = tcu_oracle_f32_to_f16(running);
    }
  }
}

typedef struct {
  const uint16_t *in;
  uint16_t *out;
  size_t seg0, seg1, segment_size;
  int scan;
} mt_job;

static void *mt_worker(void *arg) {
  mt_job *j = (mt_job *)arg;
  size_t n = j->seg1 - j->seg0;
  if (j->scan)
    tcu_oracle_seg_scan_ref(j->in + j->seg0 * j->segment_size, j->out + j->seg0 * j->segment_size, n, j->segment_size);
  else
    tcu_oracle_seg_reduce_ref(j->in + j->seg0 * j->segment_size, j->out + j->seg0, n, j->segment_size);
  return NULL;
}

static void run_mt(const uint16_t *in, uint16_t *out, size_t num_segments, size_t segment_size, int nthreads, int scan) {
  if (nthreads < 1) nthreads = 1;
  if ((size_t)nthreads > num_segments) nthreads = num_segments ? (int)num_segments : 1;
  pthread_t *th = (pthread_t *)malloc(sizeof(pthread_t) * (size_t)nthreads);
  mt_job *jobs = (mt_job *)malloc(sizeof(mt_job) * (size_t)nthreads);
  for (int t = 0; t < nthreads; t++) {
    jobs[t].in = in;
    jobs[t].out = out;
    jobs[t].segment_size = segment_size;
    jobs[t].scan = scan;
    jobs[t].seg0 = num_segments * (size_t)t / (size_t)nthreads;
    jobs[t].seg1 = num_segments * (size_t)(t + 1) / (size_t)nthreads;
    pthread_create(&th[t], NULL, mt_worker, &jobs[t]);
  }
  for (int t = 0; t < nthreads; t++) pthread_join(th[t], NULL);
  free(jobs);
  free(th);
}

void tcu_oracle_seg_reduce_ref_mt(const uint16_t *in, uint16_t *out, size_t num_segments, size_t segment_size, int nthreads) {
  run_mt(in, out, num_segments, segment_size, nthreads, 0);
}

void tcu_oracle_seg_scan_ref_mt(const uint16_t *in, uint16_t *out, size_t num_segments, size_t segment_size, int nthreads) {
  run_mt(in, out, num_segments, segment_size, nthreads, 1);
}

void tcu_oracle_full_reduce_ref(const uint16_t *in, uint16_t *out, size_t n) {
  float correct_sum = 0;
  for (size_t i = 0; i < n; i++) correct_sum += tcu_oracle_f16_to_f32(in[i]);
  out[0] = tcu_oracle_f32_to_f16(correct_sum);
}

void tcu_oracle_full_scan_ref(const uint16_t *in, uint16_t *out, size_t n) {
  float correct_sum = 0;
  for (size_t i = 0; i < n; i++) {
    correct_sum += tcu_oracle_f16_to_f32(in[i]);
    out[i] = tcu_oracle_f32_to_f16(correct_sum);
  }
}

void tcu_oracle_add_partial_sums_ref(uint16_t *out, const uint16_t *partial_sums, size_t num_segments, size_t segment_size) {
  for (size_t s = 0; s < num_segments; s++) {
    float ps = tcu_oracle_f16_to_f32(partial_sums[s]);
    for (size_t i = 0; i < segment_size; i++) {
      size_t idx = s * segment_size + i;
      out[idx] = tcu_oracle_f32_to_f16(tcu_oracle_f16_to_f32(out[idx]) + ps);
    }
  }
}

/* ------------------------------------------------------------------------------------ */
/* definition: fp64                                                                     */
/* ------------------------------------------------------------------------------------ */

void tcu_oracle_seg_reduce_f64(const uint16_t *in, double *out, size_t num_segments, size_t segment_size) {
  for (size_t j = 0; j < num_segments; j++) {
    double s = 0;
    const uint16_t *p = in + j * segment_size;
    for (size_t i = 0; i < segment_size; i++) s += (double)tcu_oracle_f16_to_f32(p[i]);
    out[j] = s;
  }
}

void tcu_oracle_seg_reduce_offsets_ref(const uint16_t *in, uint16_t *out, size_t num_segments, const int64_t *begin, const int64_t *end) {
  for (size_t j = 0; j < num_segments; j++) {
    float s = 0.0f;
    for (int64_t i = begin[j]; i < end[j]; i++) s += tcu_oracle_f16_to_f32(in[i]);
    out[j] = tcu_oracle_f32_to_f16(s);
  }
}

void tcu_oracle_seg_scan_offsets_ref(const uint16_t *in, uint16_t *out, size_t num_segments, const int64_t *begin, const int64_t *end) {
  for (size_t j = 0; j < num_segments; j++) {
    float s = 0.0f;
    for (int64_t i = begin[j]; i < end[j]; i++) {
      s += tcu_oracle_f16_to_f32(in[i]);
      out[i] = tcu_oracle_f32_to_f16(s);
    }
  }
}

void tcu_oracle_seg_scan_offsets_f64(const uint16_t *in, double *out, size_t num_segments, const int64_t *begin, const int64_t *end) {
  for (size_t j = 0; j < num_segments; j++) {
    double s = 0;
    for (int64_t i = begin[j]; i < end[j]; i++) {
      s += (double)tcu_oracle_f16_to_f32(in[i]);
      out[i] = s;
    }
  }
}

void tcu_oracle_seg_reduce_offsets_f64(const uint16_t *in, double *out, size_t num_segments, const int64_t *begin, const int64_t *end) {
  for (size_t j = 0; j < num_segments; j++) {
    double s = 0;
    for (int64_t i = begin[j]; i < end[j]; i++) s += (double)tcu_oracle_f16_to_f32(in[i]);
    out[j] = s;
  }
}

void tcu_oracle_seg_scan_f64(const uint16_t *in, double *out, size_t num_segments, size_t segment_size) {
  for (size_t j = 0; j < num_segments; j++) {
    double s = 0;
    const uint16_t *p = in + j * segment_size;
    double *q = out + j * segment_size;
    for (size_t i = 0; i < segment_size; i++) {
      s += (double)tcu_oracle_f16_to_f32(p[i]);
      q[i] = s;
    }
  }
}

void tcu_oracle_gemv_f64(const uint16_t *A, const uint16_t *x, const float *y0, double *y, size_t M, size_t K, double alpha, double beta) {
  double *xd = (double *)malloc(sizeof(double) * (K ? K : 1));
  for (size_t k = 0; k < K; k++) xd[k] = (double)tcu_oracle_f16_to_f32(x[k]);
  for (size_t m = 0; m < M; m++) {
    double s = 0;
    const uint16_t *row = A + m * K;
    for (size_t k = 0; k < K; k++) s += (double)tcu_oracle_f16_to_f32(row[k]) * xd[k];
    y[m] = alpha * s + (beta != 0.0 && y0 ? beta * (double)y0[m] : 0.0);
  }
  free(xd);
}

void tcu_oracle_gemm_f64(const uint16_t *A, const uint16_t *B, const float *C, double *D, size_t M, size_t N, size_t K, double alpha, double beta, size_t row0, size_t rows) {
  (void)M;
  double *a = (double *)malloc(sizeof(double) * (K ? K : 1));
  for (size_t r = 0; r < rows; r++) {
    size_t m = row0 + r;
    for (size_t k = 0; k < K; k++) a[k] = (double)tcu_oracle_f16_to_f32(A[m * K + k]);
    for (size_t n = 0; n < N; n++) {
      const uint16_t *bcol = B + n * K;
      double s = 0;
      for (size_t k = 0; k < K; k++) s += a[k] * (double)tcu_oracle_f16_to_f32(bcol[k]);
      D[r * N + n] = alpha * s + (beta != 0.0 && C ? beta * (double)C[m * N + n] : 0.0);
    }
  }
  free(a);
}

/* ------------------------------------------------------------------------------------ */
/* tolerance rule                                                                       */
/* ------------------------------------------------------------------------------------ */

size_t tcu_oracle_check_f16(const uint16_t *got, const double *ref, size_t n, double ulps, double abs_per_sqrt, size_t segment_size, double *worst, size_t *first_bad) {
  size_t bad = 0, fb = n;
  double w = -INFINITY;
  const double slack = abs_per_sqrt * sqrt((double)segment_size);
  for (size_t i = 0; i < n; i++) {
    double r = ref[i];
    uint16_t g = got[i];
    int g_inf = (g & 0x7fffu) == 0x7c00u;
    int g_nan = (g & 0x7fffu) > 0x7c00u;
    double excess;
    if (g_nan || isnan(r)) {
      excess = INFINITY;
    } else if (g_inf) {
      /* correct only when the reference itself rounds to that infinity, give or take
       * the allowance */
      double lim = 65520.0 - (ulps * 32.0 + slack);
      int ok = (g & 0x8000u) ? (r <= -lim) : (r >= lim);
      excess = ok ? -1.0 : INFINITY;
    } else {
      double gv = (double)tcu_oracle_f16_to_f32(g);
      double allow = ulps * tcu_oracle_ulp_f16(r) + slack;
      excess = fabs(gv - r) - allow;
    }
    if (excess > w) w = excess;
    if (excess > 0) {
      if (fb == n) fb = i;
      bad++;
    }
  }
  if (worst) *worst = w;
  if (first_bad) *first_bad = fb;
  return bad;
}

size_t tcu_oracle_check_f32_rel(const float *got, const double *ref, size_t n, double rel, double scale, double *worst, size_t *first_bad) {
  size_t bad = 0, fb = n;
  double w = -INFINITY;
  for (size_t i = 0; i < n; i++) {
    double r = ref[i];
    double g = (double)got[i];
    double denom = fabs(r) > scale ? fabs(r) : scale;
    double excess = (isnan(g) || isnan(r)) ? INFINITY : fabs(g - r) - rel * denom;
    if (excess > w) w = excess;
    if (excess > 0) {
      if (fb == n) fb = i;
      bad++;
    }
  }
  if (worst) *worst = w;
  if (first_bad) *first_bad = fb;
  return bad;
}

/* ------------------------------------------------------------------------------------ */
/* segments given by a key array: a segment is a run of equal consecutive keys            */
/* ------------------------------------------------------------------------------------ */

void tcu_oracle_seg_scan_by_key_ref(const int64_t *keys, const uint16_t *in, uint16_t *out, size_t n) {
  float acc = 0.0f;
  for (size_t i = 0; i < n; i++) {
    if (i == 0 || keys[i] != keys[i - 1]) acc = 0.0f;
    acc += tcu_oracle_f16_to_f32(in[i]);
    out[i] = tcu_oracle_f32_to_f16(acc);
  }
}

void tcu_oracle_seg_scan_by_key_f64(const int64_t *keys, const uint16_t *in, double *out, size_t n) {
  double acc = 0.0;
  for (size_t i = 0; i < n; i++) {
    if (i == 0 || keys[i] != keys[i - 1]) acc = 0.0;
    acc += (double)tcu_oracle_f16_to_f32(in[i]);
    out[i] = acc;
  }
}

size_t tcu_oracle_seg_reduce_by_key_ref(const int64_t *keys, const uint16_t *in, int64_t *keys_out, uint16_t *out, size_t n) {
  size_t runs = 0;
  float acc = 0.0f;
  for (size_t i = 0; i < n; i++) {
    acc += tcu_oracle_f16_to_f32(in[i]);
    if (i + 1 == n || keys[i + 1] != keys[i]) {
      keys_out[runs] = keys[i];
      out[runs] = tcu_oracle_f32_to_f16(acc);
      runs++;
      acc = 0.0f;
    }
  }
  return runs;
}

size_t tcu_oracle_seg_reduce_by_key_f64(const int64_t *keys, const uint16_t *in, int64_t *keys_out, double *out, size_t n) {
  size_t runs = 0;
  double acc = 0.0;
  for (size_t i = 0; i < n; i++) {
    acc += (double)tcu_oracle_f16_to_f32(in[i]);
    if (i + 1 == n || keys[i + 1] != keys[i]) {
      keys_out[runs] = keys[i];
      out[runs] = acc;
      runs++;
      acc = 0.0;
    }
  }
  return runs;
}
