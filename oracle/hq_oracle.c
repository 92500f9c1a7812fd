/*
 * hq_oracle.c — CPU restatement of the reference arithmetic.  TEST
 * INFRASTRUCTURE ONLY (see hq_oracle.h): never linked into the product library.
 *
 * Build: gcc -O2 -ffp-contract=off -fopenmp -fPIC -shared hq_oracle.c -o libhq_oracle.so -lm
 * (-ffp-contract=off matters: the fp32 restatements round after every multiply
 * and add, which is what the functions below document).
 */
#include "hq_oracle.h"

#include <math.h>
#ifdef _OPENMP
#include <omp.h>
#endif
#include <stdlib.h>
#include <string.h>

/* ------------------------------------------------------------------ fp16 */

static double round_to_f16_grid(double d) {
  /* Round a double to the nearest binary16 value (ties to even); the result is
   * returned as a double that binary16 represents exactly (or +-inf). */
  if (d != d || isinf(d)) return d;
  double a = fabs(d);
  if (a == 0.0) return d;
  int e;
  (void)frexp(a, &e); /* a = m * 2^e, m in [0.5,1) => floor(log2 a) = e-1 */
  int q = e - 1 - 10; /* exponent of the last kept bit (11-bit significand) */
  if (q < -24) q = -24; /* subnormal quantum */
  double quantum = ldexp(1.0, q);
  double r = rint(a / quantum) * quantum; /* rint: ties-to-even by default */
  if (r >= 65520.0) r = INFINITY;        /* overflow threshold of binary16 */
  return d < 0 ? -r : r;
}

/* Threads the loops over independent outputs use (1 = serial, the default): the timed CPU baseline
 * runs them serially and again over the host cores; results do not depend on it. */
static int g_threads = 1;
void hqo_set_threads(int n) { g_threads = n < 1 ? 1 : n; }
int hqo_max_threads(void) { return omp_get_max_threads(); }

uint16_t hqo_f64_to_f16(double d) {
  if (d != d) return 0x7e00;
  double r = round_to_f16_grid(d);
  uint16_t sign = signbit(r) ? 0x8000 : 0;
  double a = fabs(r);
  if (isinf(a)) return sign | 0x7c00;
  if (a == 0.0) return sign;
  int e;
  double m = frexp(a, &e); /* a = m*2^e, m in [0.5,1) */
  int E = e - 1;           /* unbiased exponent */
  if (E < -14) {           /* subnormal: a = frac * 2^-24 */
    return sign | (uint16_t)(a * 16777216.0);
  }
  uint16_t frac = (uint16_t)((m * 2.0 - 1.0) * 1024.0);
  return sign | (uint16_t)((E + 15) << 10) | frac;
}

uint16_t hqo_f32_to_f16(float f) { return hqo_f64_to_f16((double)f); }

float hqo_f16_to_f32(uint16_t h) {
  int s = h >> 15, e = (h >> 10) & 31, m = h & 1023;
  double v;
  if (e == 31) v = m ? NAN : INFINITY;
  else if (e == 0) v = ldexp((double)m, -24);
  else v = ldexp(1.0 + m / 1024.0, e - 15);
  return (float)(s ? -v : v);
}

/* Sum p + c rounded to odd in double, so that a second rounding to binary16 is
 * the correctly rounded result of the exact sum. */
static double add_round_to_odd(double p, double c) {
  double s = p + c;
  if (s != s || isinf(s)) return s;
  double bb = s - p;
  double err = (p - (s - bb)) + (c - bb); /* TwoSum: p + c = s + err exactly */
  if (err != 0.0) {
    uint64_t bits;
    memcpy(&bits, &s, 8);
    if (!(bits & 1)) s = nextafter(s, err > 0 ? INFINITY : -INFINITY);
  }
  return s;
}

uint16_t hqo_hfma(uint16_t a, uint16_t b, uint16_t c) {
  double p = (double)hqo_f16_to_f32(a) * (double)hqo_f16_to_f32(b); /* exact */
  return hqo_f64_to_f16(add_round_to_odd(p, (double)hqo_f16_to_f32(c)));
}
uint16_t hqo_hadd(uint16_t a, uint16_t b) {
  return hqo_f64_to_f16((double)hqo_f16_to_f32(a) + (double)hqo_f16_to_f32(b));
}
uint16_t hqo_hmul(uint16_t a, uint16_t b) {
  return hqo_f64_to_f16((double)hqo_f16_to_f32(a) * (double)hqo_f16_to_f32(b));
}

/* ------------------------------------------------------------- GPTQ 3bit */

/* Value i (0..31) of a 32-value group lives at bit 3*i of the 96-bit string
 * formed by the group's three words (word 0 lowest); values 10 and 21 straddle
 * word boundaries (src/quant3MatMul-hip/kernels.h:55,71). */
static inline unsigned q3_get(const uint32_t w[3], int i) {
  int bit = 3 * i, wd = bit >> 5, sh = bit & 31;
  uint32_t v = w[wd] >> sh;
  if (sh > 29) v |= w[wd + 1] << (32 - sh);
  return v & 7u;
}

void hqo_q3_pack(const uint8_t* codes, int K, int N, int32_t* mat) {
  int G = K / 32;
  for (int g = 0; g < G; ++g)
    for (int n = 0; n < N; ++n) {
      uint32_t w[3] = {0, 0, 0};
      for (int i = 0; i < 32; ++i) {
        uint32_t q = codes[(size_t)(32 * g + i) * N + n] & 7u;
        int bit = 3 * i, wd = bit >> 5, sh = bit & 31;
        w[wd] |= q << sh;
        if (sh > 29) w[wd + 1] |= q >> (32 - sh);
      }
      for (int j = 0; j < 3; ++j) mat[(size_t)(3 * g + j) * N + n] = (int32_t)w[j];
    }
}

void hqo_q3_unpack(const int32_t* mat, int K, int N, uint8_t* codes) {
  int G = K / 32;
  for (int g = 0; g < G; ++g)
    for (int n = 0; n < N; ++n) {
      uint32_t w[3];
      for (int j = 0; j < 3; ++j) w[j] = (uint32_t)mat[(size_t)(3 * g + j) * N + n];
      for (int i = 0; i < 32; ++i) codes[(size_t)(32 * g + i) * N + n] = (uint8_t)q3_get(w, i);
    }
}

/* Columns [n0, n1) of the fp32 kernel; every column sees exactly the arithmetic of the
 * reference thread that owns it, so any column partition gives identical results. */
static void q3_matvec_f32_cols(const float* x, const int32_t* mat, float* mul, const float* scales,
                               const float* zeros, int K, int N, int n0, int n1) {
  /* One 256-row block (8 groups) at a time, as the reference grid does
   * (BLOCKWIDTH=256, BLOCKHEIGHT=24, kernels.h:5-6,22-23). */
  int W = n1 - n0;
  float* res = (float*)malloc(sizeof(float) * (size_t)(W > 0 ? W : 1));
  int G = K / 32;
  for (int g0 = 0; g0 < G; g0 += 8) {
    for (int n = 0; n < W; ++n) res[n] = 0.f;
    int g1 = g0 + 8 < G ? g0 + 8 : G;
    for (int g = g0; g < g1; ++g) {
      const uint32_t* r0 = (const uint32_t*)mat + (size_t)(3 * g) * N + n0;
      const uint32_t* r1 = r0 + N;
      const uint32_t* r2 = r1 + N;
      for (int i = 0; i < 32; ++i) {
        float xv = x[32 * g + i];
        int bit = 3 * i, wd = bit >> 5, sh = bit & 31;
        const uint32_t* ra = wd == 0 ? r0 : (wd == 1 ? r1 : r2);
        const uint32_t* rb = wd == 0 ? r1 : r2;
        if (sh <= 29) {
          for (int n = 0; n < W; ++n) {
            float q = (float)((ra[n] >> sh) & 7u);
            res[n] += (scales[n0 + n] * q - zeros[n0 + n]) * xv; /* kernels.h:43-84 */
          }
        } else {
          for (int n = 0; n < W; ++n) {
            float q = (float)(((ra[n] >> sh) | (rb[n] << (32 - sh))) & 7u);
            res[n] += (scales[n0 + n] * q - zeros[n0 + n]) * xv;
          }
        }
      }
    }
    for (int n = 0; n < W; ++n) mul[n0 + n] += res[n]; /* atomicAdd, kernels.h:89 */
  }
  free(res);
}

void hqo_q3_matvec_f32(const float* x, const int32_t* mat, float* mul,
                       const float* scales, const float* zeros, int K, int N) {
  q3_matvec_f32_cols(x, mat, mul, scales, zeros, K, N, 0, N);
}

int hqo_q3_matvec_f32_omp(const float* x, const int32_t* mat, float* mul,
                          const float* scales, const float* zeros, int K, int N) {
  int threads = 1;
#ifdef _OPENMP
  threads = omp_get_max_threads();
#endif
  int chunk = 256; /* one reference block of columns per task */
  int nchunks = (N + chunk - 1) / chunk;
#pragma omp parallel for schedule(dynamic)
  for (int c = 0; c < nchunks; ++c) {
    int n0 = c * chunk, n1 = n0 + chunk < N ? n0 + chunk : N;
    q3_matvec_f32_cols(x, mat, mul, scales, zeros, K, N, n0, n1);
  }
  return threads;
}

void hqo_q3_matvec_f64(const double* x, const int32_t* mat, double* y,
                       const float* scales, const float* zeros, int K, int N) {
  int G = K / 32;
  for (int n = 0; n < N; ++n) y[n] = 0.0;
  for (int g = 0; g < G; ++g)
    for (int n = 0; n < N; ++n) {
      uint32_t w[3];
      for (int j = 0; j < 3; ++j) w[j] = (uint32_t)mat[(size_t)(3 * g + j) * N + n];
      double s = scales[n], z = zeros[n], acc = 0.0;
      for (int i = 0; i < 32; ++i) acc += (s * (double)q3_get(w, i) - z) * x[32 * g + i];
      y[n] += acc;
    }
}

void hqo_q3_matvec_f16(const uint16_t* x, const int32_t* mat, float* mul,
                       const float* scales, const float* zeros, int K, int N) {
  int G = K / 32;
  uint16_t qh[8];
  for (int q = 0; q < 8; ++q) qh[q] = hqo_f32_to_f16((float)q); /* deq2, kernels.h:112-119 */
  for (int n = 0; n < N; ++n) {
    uint16_t s16 = hqo_f32_to_f16(scales[n]);  /* kernels.h:121 */
    uint16_t z16 = hqo_f32_to_f16(-zeros[n]);  /* kernels.h:122 */
    for (int g0 = 0; g0 < G; g0 += 8) {
      float res = 0.f;
      int g1 = g0 + 8 < G ? g0 + 8 : G;
      for (int g = g0; g < g1; ++g) {
        uint32_t w[3];
        for (int j = 0; j < 3; ++j) w[j] = (uint32_t)mat[(size_t)(3 * g + j) * N + n];
        uint16_t ax = 0, ay = 0; /* res2 = half2(0), kernels.h:135 */
        for (int p = 0; p < 16; ++p) {
          uint16_t wl = hqo_hfma(qh[q3_get(w, 2 * p)], s16, z16);
          uint16_t wh = hqo_hfma(qh[q3_get(w, 2 * p + 1)], s16, z16);
          ax = hqo_hfma(wl, x[32 * g + 2 * p], ax);
          ay = hqo_hfma(wh, x[32 * g + 2 * p + 1], ay);
        }
        res += hqo_f16_to_f32(ax) + hqo_f16_to_f32(ay); /* kernels.h:165 */
      }
      mul[n] += res; /* kernels.h:168 */
    }
  }
}

void hqo_q3_gemm(const uint16_t* A, const int32_t* mat, double* out,
                 const float* scales, const float* zeros, int M, int K, int N,
                 int mode) {
  int G = K / 32;
  double* Ad = (double*)malloc(sizeof(double) * (size_t)M * K);
  for (size_t i = 0; i < (size_t)M * K; ++i) Ad[i] = hqo_f16_to_f32(A[i]);
#pragma omp parallel for schedule(static) num_threads(g_threads)
  for (int n = 0; n < N; ++n) {
    double* wcol = (double*)malloc(sizeof(double) * (size_t)K);
    for (int g = 0; g < G; ++g) {
      uint32_t w[3];
      for (int j = 0; j < 3; ++j) w[j] = (uint32_t)mat[(size_t)(3 * g + j) * N + n];
      for (int i = 0; i < 32; ++i) {
        unsigned q = q3_get(w, i);
        if (mode == 0) wcol[32 * g + i] = (double)scales[n] * q - (double)zeros[n];
        else wcol[32 * g + i] = hqo_f16_to_f32(hqo_f32_to_f16(scales[n] * (float)q - zeros[n]));
      }
    }
    for (int m = 0; m < M; ++m) {
      const double* a = Ad + (size_t)m * K;
      double acc = 0.0;
      for (int k = 0; k < K; ++k) acc += a[k] * wcol[k];
      out[(size_t)m * N + n] = acc;
    }
    free(wcol);
  }
  free(Ad);
}

/* --------------------------------------------------------------- NF4/FP4 */

/* bitsandbytes NF4 code book (fp32 literals of the upstream library; the
 * reference tree holds no NF4 table). */
const float hqo_nf4_table[16] = {
    -1.0f, -0.6961928009986877f, -0.5250730514526367f, -0.39491748809814453f,
    -0.28444138169288635f, -0.18477343022823334f, -0.09105003625154495f, 0.0f,
    0.07958029955625534f, 0.16093020141124725f, 0.24611230194568634f,
    0.33791524171829224f, 0.44070982933044434f, 0.5626170039176941f,
    0.7229568362236023f, 1.0f};

/* bitsandbytes FP4 decode tree: bit 3 = sign, low three bits select
 * {0, 1/192, 2/3, 1, 1/3, 1/2, 1/6, 1/4}. */
const float hqo_fp4_table[16] = {
    0.0f, 0.005208333333f, 0.66666667f, 1.0f, 0.33333333f, 0.5f, 0.16666667f, 0.25f,
    -0.0f, -0.005208333333f, -0.66666667f, -1.0f, -0.33333333f, -0.5f, -0.16666667f, -0.25f};

void hqo_dequant_4bit(const uint8_t* packed, const float* absmax, uint16_t* out,
                      int64_t n, int blocksize, int table) {
  const float* T = table ? hqo_fp4_table : hqo_nf4_table;
#pragma omp parallel for schedule(static) num_threads(g_threads)
  for (int64_t e = 0; e < n; ++e) {
    uint8_t b = packed[e >> 1];
    unsigned c = (e & 1) ? (b & 15u) : (b >> 4); /* high nibble first */
    float v = T[c] * absmax[e / blocksize];      /* one fp32 multiply */
    out[e] = hqo_f32_to_f16(v);                  /* one rounding to fp16 */
  }
}

/* Blockwise 4-bit quantisation, PARITY UNPINNED (no counterpart in the reference):
 * absmax = max|x| over the block, v = x * (1/absmax) in fp32, NF4 code = number of fp32
 * midpoints (t[c]+t[c+1])*0.5 strictly below v; FP4 code = nearest magnitude (ties to the
 * smaller), sign in bit 3.  x_is_f16: x holds binary16 bit patterns. */
void hqo_quantize_4bit(const void* x, int x_is_f16, uint8_t* packed, float* absmax, int64_t n,
                       int blocksize, int table) {
  static const float mags[8] = {0.0f, 0.005208333333f, 0.16666667f, 0.25f, 0.33333333f, 0.5f, 0.66666667f, 1.0f};
  static const unsigned code_of[8] = {0, 1, 6, 7, 4, 5, 2, 3};
  int64_t nblocks = (n + blocksize - 1) / blocksize;
  for (int64_t e = 0; e < (n + 1) / 2; ++e) packed[e] = 0;
  for (int64_t b = 0; b < nblocks; ++b) {
    int64_t e0 = b * blocksize, e1 = e0 + blocksize < n ? e0 + blocksize : n;
    float amax = 0.f;
    for (int64_t e = e0; e < e1; ++e) {
      float v = x_is_f16 ? hqo_f16_to_f32(((const uint16_t*)x)[e]) : ((const float*)x)[e];
      v = fabsf(v);
      if (v > amax) amax = v;
    }
    absmax[b] = amax;
    float inv = amax > 0.f ? 1.0f / amax : 0.f;
    for (int64_t e = e0; e < e1; ++e) {
      float v = (x_is_f16 ? hqo_f16_to_f32(((const uint16_t*)x)[e]) : ((const float*)x)[e]) * inv;
      unsigned c = 0;
      if (table == 0) {
        for (int i = 0; i < 15; ++i)
          if (v > (hqo_nf4_table[i] + hqo_nf4_table[i + 1]) * 0.5f) c = (unsigned)i + 1;
      } else {
        float a = fabsf(v);
        unsigned idx = 0;
        for (int i = 0; i < 7; ++i)
          if (a > (mags[i] + mags[i + 1]) * 0.5f) idx = (unsigned)i + 1;
        c = code_of[idx] | (v < 0.f ? 8u : 0u);
      }
      packed[e >> 1] |= (uint8_t)((e & 1) ? c : c << 4);
    }
  }
}

/* ------------------------------------------------ dynamic 8-bit quantize */

uint8_t hqo_dquantize(const float* code, float x) {
  /* src/quantBnB-hip/main.cu:17-66 */
  int pivot = 127, upper_pivot = 255, lower_pivot = 0;
  float lower = -1.0f, upper = 1.0f;
  float val = code[pivot];
  for (int i = 64; i > 0; i >>= 1) {
    if (x > val) { lower_pivot = pivot; lower = val; pivot += i; }
    else         { upper_pivot = pivot; upper = val; pivot -= i; }
    val = code[pivot];
  }
  if (upper_pivot == 255) upper = code[upper_pivot];
  if (lower_pivot == 0) lower = code[lower_pivot];
  if (x > val) {
    float midpoint = (upper + val) * 0.5f;
    return (uint8_t)(x > midpoint ? upper_pivot : pivot);
  } else {
    float midpoint = (lower + val) * 0.5f;
    return (uint8_t)(x < midpoint ? lower_pivot : pivot);
  }
}

void hqo_quantize_dynamic8(const float* code, const float* A, uint8_t* out, int64_t n) {
  for (int64_t i = 0; i < n; ++i) out[i] = hqo_dquantize(code, A[i]);
}

static int cmp_float(const void* a, const void* b) {
  float x = *(const float*)a, y = *(const float*)b;
  return (x > y) - (x < y);
}

static void linspace_f32(float start, float end, int steps, float* o) {
  /* symmetric float32 linspace: lower half counts up from start, upper half
   * counts down from end */
  if (steps == 1) { o[0] = start; return; }
  float step = (end - start) / (float)(steps - 1);
  int half = steps / 2;
  for (int i = 0; i < steps; ++i)
    o[i] = i < half ? start + step * (float)i : end - step * (float)(steps - 1 - i);
}

void hqo_dynamic_map(float* code) {
  /* signed dynamic map, 7 exponent bits, 8 total bits */
  int cnt = 0;
  float b[65];
  for (int i = 0; i < 7; ++i) {
    int items = (1 << i) + 1;
    linspace_f32(0.1f, 1.0f, items, b);
    float sc = (float)pow(10.0, -6 + i);
    for (int j = 0; j + 1 < items; ++j) {
      float mean = (b[j] + b[j + 1]) / 2.0f;
      code[cnt++] = sc * mean;
      code[cnt++] = -sc * mean;
    }
  }
  code[cnt++] = 0.0f;
  code[cnt++] = 1.0f;
  qsort(code, 256, sizeof(float), cmp_float);
}

/* ------------------------------------------------ int8 activation quantisation */

static float act_to_f32(const void* x, int dtype, int64_t i) {
  if (dtype == 0) return ((const float*)x)[i];
  if (dtype == 1) return hqo_f16_to_f32(((const uint16_t*)x)[i]);
  uint32_t b = (uint32_t)((const uint16_t*)x)[i] << 16; /* bf16: upper half of an fp32 */
  float f;
  memcpy(&f, &b, 4);
  return f;
}
/* src/quantVLLM-cuda/utils.h:9-61 */
static int8_t f_to_i8_rn(float x) {
  float d = nearbyintf(x);
  d = d < -128.f ? -128.f : (127.f < d ? 127.f : d);
  return (int8_t)d;
}
static int32_t f_to_i32_rn(float x) {
  float d = nearbyintf(x);
  if (d >= 2147483648.f) return INT32_MAX;
  if (d <= -2147483648.f) return INT32_MIN;
  return (int32_t)d;
}
static int8_t i32_to_i8(int32_t x) { return (int8_t)(x < -128 ? -128 : (127 < x ? 127 : x)); }

/* src/quantVLLM-cuda/reference.h:1-31 */
void hqo_int8_quant_static(const void* x, int dtype, int8_t* out, int64_t tokens, int hidden,
                           float scale, int has_azp, int32_t azp) {
  for (int64_t i = 0; i < tokens * hidden; ++i) {
    float v = act_to_f32(x, dtype, i);
    out[i] = has_azp ? i32_to_i8(f_to_i32_rn(v / scale) + azp) : f_to_i8_rn(v / scale);
  }
}

/* src/quantVLLM-cuda/reference.h:33-93 */
void hqo_int8_quant_dynamic(const void* x, int dtype, int8_t* out, float* scales, int32_t* azp,
                            int64_t tokens, int hidden) {
  for (int64_t t = 0; t < tokens; ++t) {
    if (!azp) {
      float absmax = 0.f;
      for (int i = 0; i < hidden; ++i) {
        float v = act_to_f32(x, dtype, t * hidden + i);
        v = v > 0.f ? v : -v;
        absmax = v > absmax ? v : absmax;
      }
      scales[t] = absmax / 127.0f;
      float tmp = 127.0f / absmax;
      for (int i = 0; i < hidden; ++i) out[t * hidden + i] = f_to_i8_rn(act_to_f32(x, dtype, t * hidden + i) * tmp);
    } else {
      float mx = 1.17549435e-38f, mn = 3.40282347e+38f; /* numeric_limits min() / max() */
      for (int i = 0; i < hidden; ++i) {
        float v = act_to_f32(x, dtype, t * hidden + i);
        mx = v > mx ? v : mx;
        mn = v < mn ? v : mn;
      }
      float sc = (mx - mn) / 255.0f;
      int32_t z = (int32_t)nearbyintf(-128.0f - mn / sc);
      scales[t] = sc;
      azp[t] = z;
      for (int i = 0; i < hidden; ++i)
        out[t * hidden + i] = i32_to_i8(f_to_i32_rn(act_to_f32(x, dtype, t * hidden + i) / sc) + z);
    }
  }
}

/* -------------------------------------------------------------- LUT-GEMM */

void hqo_bcq_pack(const int8_t* signs, int K, int N, int nb, uint32_t* bW) {
  for (int k0 = 0; k0 < K; k0 += 32)
    for (int b = 0; b < nb; ++b)
      for (int n = 0; n < N; ++n) {
        uint32_t s = 0;
        for (int t = 0; t < 32; ++t)
          if (signs[((size_t)(k0 + t) * nb + b) * N + n] > 0) s |= 1u << t;
        bW[((size_t)(k0 / 32) * nb + b) * N + n] = s;
      }
}

void hqo_bcq_dequant(const uint32_t* bW, const uint16_t* alpha, const uint16_t* qbias,
                     int K, int N, int nb, int group, double* W) {
  for (int k = 0; k < K; ++k)
    for (int n = 0; n < N; ++n) {
      int g = k / group;
      double w = qbias ? hqo_f16_to_f32(qbias[(size_t)g * N + n]) : 0.0;
      for (int b = 0; b < nb; ++b) {
        uint32_t word = bW[((size_t)(k / 32) * nb + b) * N + n];
        double s = (word >> (k & 31)) & 1u ? 1.0 : -1.0;
        w += hqo_f16_to_f32(alpha[((size_t)g * nb + b) * N + n]) * s;
      }
      W[(size_t)k * N + n] = w;
    }
}

void hqo_lut_gemv_f64(const uint32_t* bW, const uint16_t* alpha, const uint16_t* qbias,
                      const uint16_t* x, double* y, int K, int N, int nb, int group) {
  int NG = K / group;
  double* xs = (double*)malloc(sizeof(double) * (size_t)K);
  for (int k = 0; k < K; ++k) xs[k] = hqo_f16_to_f32(x[k]);
  for (int n = 0; n < N; ++n) y[n] = 0.0;
  for (int g = 0; g < NG; ++g) {
    double xsum = 0.0;
    for (int k = g * group; k < (g + 1) * group; ++k) xsum += xs[k];
    for (int b = 0; b < nb; ++b)
      for (int kw = g * group / 32; kw < (g + 1) * group / 32; ++kw) {
        const uint32_t* row = bW + ((size_t)kw * nb + b) * N;
        const uint16_t* al = alpha + ((size_t)g * nb + b) * N;
#pragma omp parallel for schedule(static) num_threads(g_threads)
        for (int n = 0; n < N; ++n) {
          uint32_t w = row[n];
          double s = 0.0;
          for (int t = 0; t < 32; ++t) s += (w >> t) & 1u ? xs[kw * 32 + t] : -xs[kw * 32 + t];
          y[n] += (double)hqo_f16_to_f32(al[n]) * s;
        }
      }
    if (qbias)
      for (int n = 0; n < N; ++n) y[n] += (double)hqo_f16_to_f32(qbias[(size_t)g * N + n]) * xsum;
  }
  free(xs);
}

void hqo_lut_gemv_f16(const uint32_t* bW, const uint16_t* alpha, const uint16_t* qbias,
                      const uint16_t* x, uint16_t* y, int K, int N, int nb, int group) {
  /* K tile of 32 (the bias path of the reference, mv_fp16.h:252-258) */
  const uint16_t ONE = 0x3c00, MONE = 0xbc00, TWO = 0x4000;
  for (int n = 0; n < N; ++n) y[n] = 0; /* hipMemset in matmul(), kernels.cu:28 */
  uint16_t lut[4][256];
  for (int kt = 0; kt < K / 32; ++kt) {
    for (int t = 0; t < 4; ++t) {
      const uint16_t* inp = x + kt * 32 + t * 8;
      for (int lx = 0; lx < 64; ++lx) { /* mv_fp16.h:144-153 */
        uint16_t acc = hqo_hmul((lx & 1) ? ONE : MONE, inp[0]);
        for (int j = 1; j < 8; ++j)
          acc = hqo_hadd(acc, hqo_hmul(((lx >> j) & 1) ? ONE : MONE, inp[j]));
        lut[t][lx] = acc;
      }
      for (int s = 6; s < 8; ++s) { /* mv_fp16.h:165-170 */
        uint16_t iv = hqo_hmul(TWO, inp[s]);
        for (int i = 1 << s; i < (1 << (s + 1)); ++i) lut[t][i] = hqo_hadd(lut[t][i - (1 << s)], iv);
      }
    }
    int g = (kt * 32) / group;
    for (int n = 0; n < N; ++n) {
      uint16_t o = 0;
      if (qbias) { /* mv_fp16.h:183-201 */
        uint16_t to = 0;
        for (int t = 0; t < 4; ++t) to = hqo_hadd(to, lut[t][255]);
        o = hqo_hadd(o, hqo_hmul(qbias[(size_t)g * N + n], to));
      }
      for (int b = 0; b < nb; ++b) { /* mv_fp16.h:203-224 */
        uint32_t w = bW[((size_t)kt * nb + b) * N + n];
        uint16_t to = 0;
        for (int t = 0; t < 4; ++t) to = hqo_hadd(to, lut[t][(w >> (8 * t)) & 255u]);
        o = hqo_hadd(o, hqo_hmul(alpha[((size_t)g * nb + b) * N + n], to));
      }
      y[n] = hqo_hadd(y[n], o); /* unsafeAtomicAdd, mv_fp16.h:225 */
    }
  }
}

/* ------------------------------------------------------------------ AQLM */

void hqo_aqlm_matvec(const int16_t* codes, const uint16_t* codebooks,
                     const uint16_t* scales, const uint16_t* x, uint16_t* y16,
                     double* y64, int M, int K, const int cb_a_sizes[4],
                     int cb_stride_int4, int mode) {
  int ncodes = K / 8;
#pragma omp parallel for schedule(static) num_threads(g_threads)
  for (int m = 0; m < M; ++m) {
    const uint16_t* cb = codebooks;
    for (int j = 0; j < 4 && m >= cb_a_sizes[j]; ++j)
      cb += (size_t)cb_stride_int4 * 8; /* main.cu:45-50 */
    const int16_t* row = codes + (size_t)m * ncodes;
    double acc = 0.0;
    if (mode == 0) {
      for (int c = 0; c < ncodes; ++c) {
        const uint16_t* e = cb + (size_t)(uint16_t)row[c] * 8; /* main.cu:72 */
        for (int j = 0; j < 8; ++j)
          acc += (double)hqo_f16_to_f32(e[j]) * (double)hqo_f16_to_f32(x[8 * c + j]);
      }
    } else {
      float lane[64];
      for (int l = 0; l < 64; ++l) lane[l] = 0.f;
      /* lane l, trip it: int4 index l + 64*it of the row = codes 8*(l+64*it).. */
      for (int it = 0; it * 512 < ncodes; ++it)
        for (int l = 0; l < 64; ++l) {
          int c0 = 8 * (l + 64 * it);
          if (c0 >= ncodes) continue;
          for (int i = 0; i < 8; ++i) {
            const uint16_t* e = cb + (size_t)(uint16_t)row[c0 + i] * 8;
            const uint16_t* xv = x + 8 * (c0 + i);
            uint16_t rx = 0, ry = 0;
            for (int j = 0; j < 4; ++j) { /* main.cu:84-86 */
              rx = hqo_hfma(e[2 * j], xv[2 * j], rx);
              ry = hqo_hfma(e[2 * j + 1], xv[2 * j + 1], ry);
            }
            lane[l] += hqo_f16_to_f32(rx) + hqo_f16_to_f32(ry); /* main.cu:87 */
          }
        }
      for (int i = 32; i > 0; i /= 2) { /* __shfl_down tree, main.cu:95-97 */
        float nw[64];
        for (int l = 0; l < 64; ++l) nw[l] = lane[l] + (l + i < 64 ? lane[l + i] : lane[l]);
        memcpy(lane, nw, sizeof(nw));
      }
      acc = lane[0];
    }
    if (y64) y64[m] = scales ? acc * (double)hqo_f16_to_f32(scales[m]) : acc;
    if (y16) {
      float r = (float)acc;
      if (scales) r = r * hqo_f16_to_f32(scales[m]); /* fp32 multiply, one rounding */
      y16[m] = hqo_f32_to_f16(r);
    }
  }
}

/* ------------------------------------------------------------------ gemv */

/* src/gemv-hip/kernels.h:66-311 (kernels) and src/gemv-hip/gemv.cu:134-190 (the reference's own
 * statement of the result: sum of (q - zero_point) * scale * vec).  scale and zero_point are
 * rounded to fp16 first (gemv.cu:18-19); the sum is taken in double. */
void hqo_gemv(const void* mat, int mode, const uint16_t* vec, uint16_t* res_f16, double* res_f64,
              int rows, int n, float scale, float zero_point) {
  const double sc = mode ? (double)hqo_f16_to_f32(hqo_f32_to_f16(scale)) : 1.0;
  const double zp = mode ? (double)hqo_f16_to_f32(hqo_f32_to_f16(zero_point)) : 0.0;
  for (int r = 0; r < rows; ++r) {
    double s = 0.0;
    for (int j = 0; j < n; ++j) {
      double q;
      if (mode == 0) q = (double)hqo_f16_to_f32(((const uint16_t*)mat)[(size_t)r * n + j]);
      else if (mode == 1) q = (double)((const int8_t*)mat)[(size_t)r * n + j];
      else {
        const uint8_t b = ((const uint8_t*)mat)[(size_t)r * (n / 2) + j / 2];
        q = (double)((j & 1) ? (b >> 4) : (b & 15)); /* kernels.h:15-21: X = low nibble pairs with vec[2j] */
      }
      s += (q - zp) * (double)hqo_f16_to_f32(vec[j]);
    }
    s *= sc;
    if (res_f64) res_f64[r] = s;
    if (res_f16) res_f16[r] = hqo_f64_to_f16(s);
  }
}

/* ----------------------------------------------------------------- mxfp4 */

static uint16_t f32_to_bf16(float f) { /* round to nearest even */
  uint32_t b;
  memcpy(&b, &f, 4);
  if ((b & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((b >> 16) | 0x40u);
  b += 0x7fffu + ((b >> 16) & 1u);
  return (uint16_t)(b >> 16);
}
static float bf16_to_f32(uint16_t h) {
  uint32_t b = (uint32_t)h << 16;
  float f;
  memcpy(&f, &b, 4);
  return f;
}

/* Nearest e2m1 value (0, .5, 1, 1.5, 2, 3, 4, 6), ties to the even mantissa, saturating at 6:
 * what fp16_to_fp4_simulate (src/mxfp4-hip/main.cu:19-107) produces for finite inputs. */
static float round_to_e2m1(float a) {
  float m = fabsf(a), r;
  if (m < 2.f) r = nearbyintf(m * 2.f) * 0.5f;
  else if (m < 4.f) r = nearbyintf(m);
  else r = fminf(nearbyintf(m * 0.5f) * 2.f, 6.f);
  return copysignf(r, a);
}

/* Microscaling fp4 quantise-dequantise in place of qdq_mxfp4_kernel, src/mxfp4-hip/main.cu:109-142:
 * per group of 32: the largest magnitude, rounded to a power of two with the carry at a mantissa
 * of 0.75 (main.cu:124-126), gives the shared scale 2^(e-2) clamped to the E8M0 range
 * (main.cu:128-132); every element is divided by it, rounded to e2m1 and multiplied back
 * (main.cu:134-141).  Groups whose rounded maximum is zero give zeros (the reference divides by a
 * zero scale there); groups whose rounded maximum leaves the format use the scale 2^14 / 2^126 (the
 * reference writes NaN there).  Both cases: parity unpinned, behaviour defined by this library. */
void hqo_mxfp4_qdq(const uint16_t* in, uint16_t* out, int64_t n, int is_bf16) {
  const int mant = is_bf16 ? 7 : 10;
  for (int64_t g = 0; g + 32 <= n; g += 32) {
    uint16_t mx = 0;
    for (int i = 0; i < 32; ++i) {
      uint16_t a = in[g + i] & 0x7fffu;
      if (a > mx) mx = a; /* magnitudes of one format order like their bit patterns */
    }
    const uint16_t rounded = (uint16_t)((mx + (1u << (mant - 2))) & (0xffffu << mant) & 0x7fffu);
    const float bmax = is_bf16 ? bf16_to_f32(rounded) : hqo_f16_to_f32(rounded);
    if (!(bmax > 0.f)) {
      for (int i = 0; i < 32; ++i) out[g + i] = (uint16_t)(in[g + i] & 0x8000u);
      continue;
    }
    int e;
    if ((rounded >> mant) == (is_bf16 ? 255u : 31u)) {
      /* The rounding carried past the largest power of two of the format (group maximum >= 61440 in
       * fp16, >= 0x7f60 in bf16, or an infinity).  The reference takes log2 of that infinity and writes
       * NaN for the whole group (main.cu:126-141); the library's stated behaviour is the exponent the
       * carry stands for, restated here.  Parity with the reference is deliberately given up. */
      e = is_bf16 ? 128 : 16;
    } else {
      frexpf(bmax, &e); /* bmax = 0.5 * 2^e exactly */
      e -= 1;
    }
    int scale_exp = 127 + (e - 2 < 127 ? e - 2 : 127);
    if (scale_exp < 0) scale_exp = 0;
    float scale = ldexpf(1.f, scale_exp - 127);
    scale = is_bf16 ? bf16_to_f32(f32_to_bf16(scale)) : hqo_f16_to_f32(hqo_f32_to_f16(scale));
    for (int i = 0; i < 32; ++i) {
      const float x = is_bf16 ? bf16_to_f32(in[g + i]) : hqo_f16_to_f32(in[g + i]);
      const float q = x / scale; /* then rounded to the storage type, as __hdiv does */
      const float qs = is_bf16 ? bf16_to_f32(f32_to_bf16(q)) : hqo_f16_to_f32(hqo_f32_to_f16(q));
      const float r = round_to_e2m1(qs) * scale;
      out[g + i] = is_bf16 ? f32_to_bf16(r) : hqo_f32_to_f16(r);
    }
  }
}
