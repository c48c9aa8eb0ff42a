/* CPU oracle, plain C.  TEST INFRASTRUCTURE ONLY: bound by oracle/native.py for tests/, smoke() and the cpu_baseline
 * leg of bench.py; never linked into or called from the shipped library.
 *
 * A second, independent statement of the integer parts of the path (nibble order, bit-by-bit trellis decode) and an
 * OpenMP dequant-then-matmul that serves as the timed CPU baseline.  Each function cites the reference text it
 * restates; paths are relative to the reference tree.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

/* ---- scalar formats ---------------------------------------------------------------------------------------- */

static inline float bf16_to_f32(uint16_t b) {
  uint32_t u = (uint32_t)b << 16;
  float f;
  memcpy(&f, &u, 4);
  return f;
}

static inline uint16_t f32_to_bf16(float f) { /* round to nearest even */
  uint32_t u;
  memcpy(&u, &f, 4);
  u += 0x7FFFu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}

static inline float round_bf16(float f) { return bf16_to_f32(f32_to_bf16(f)); }

static double half_to_double(uint16_t h) {
  const int sign = h >> 15, e = (h >> 10) & 31, m = h & 1023;
  double v;
  if (e == 0) v = ldexp((double)m, -24);
  else if (e == 31) v = m ? NAN : INFINITY;
  else v = ldexp((double)(m + 1024), e - 25);
  return sign ? -v : v;
}

/* double -> fp16 bits, round to nearest even (values here are finite and well inside the fp16 range) */
static uint16_t double_to_half(double v) {
  const uint16_t sign = (uint16_t)(signbit(v) ? 0x8000 : 0);
  double a = fabs(v);
  if (a == 0.0) return sign;
  int e;
  (void)frexp(a, &e); /* a = f * 2^e, f in [0.5, 1) */
  int exp = e - 1;    /* a = 1.x * 2^exp */
  if (exp < -14) exp = -14; /* subnormal spacing */
  const double scaled = ldexp(a, 10 - exp); /* mantissa units */
  double r = nearbyint(scaled);             /* default rounding mode: to nearest even */
  if (exp == -14 && r < 1024.0) return (uint16_t)(sign | (uint16_t)r);
  if (r >= 2048.0) {
    r *= 0.5;
    ++exp;
  }
  if (exp > 15) return (uint16_t)(sign | 0x7C00);
  return (uint16_t)(sign | ((uint16_t)(exp + 15) << 10) | ((uint16_t)r - 1024));
}

int orc_threads(void) {
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}

void orc_set_threads(int n) {
#ifdef _OPENMP
  if (n > 0) omp_set_num_threads(n);
#else
  (void)n;
#endif
}

uint16_t orc_double_to_half(double v) { return double_to_half(v); }
double orc_half_to_double(uint16_t h) { return half_to_double(h); }

/* ---- MLX 4-bit affine (families/qwen3_5/cuda/qmm.py:132-149; tests/cuda/test_qmm.py:22-26) ------------------ */

/* element 8 w + i of a row is bits [4 i, 4 i + 4) of word w */
static inline int code_at(const uint32_t* row, int k) { return (int)((row[k >> 3] >> (4 * (k & 7))) & 15u); }

void orc_affine_dequant(const uint32_t* words, const uint16_t* scales, const uint16_t* biases, int64_t n, int k,
                        int gs, float* out) {
  const int kg = k / gs;
#pragma omp parallel for schedule(static)
  for (int64_t r = 0; r < n; ++r) {
    const uint32_t* row = words + r * (k / 8);
    for (int c = 0; c < k; ++c) {
      const float s = bf16_to_f32(scales[r * kg + c / gs]), b = bf16_to_f32(biases[r * kg + c / gs]);
      const float prod = (float)code_at(row, c) * s;
      out[r * k + c] = prod + b;
    }
  }
}

/* one weight row, dequantized; prefill rounds each weight once: the reference to bf16 (cuda/kernels/qmm_prefill.cu:1),
 * this build's kernels 256 w to fp16, which is what is restated here */
static void dequant_row(const uint32_t* row, const uint16_t* s, const uint16_t* b, int k, int gs, int prefill,
                        float* w) {
  for (int g = 0; g < k / gs; ++g) {
    const float sv = bf16_to_f32(s[g]), bv = bf16_to_f32(b[g]);
    for (int c = g * gs; c < (g + 1) * gs; ++c) {
      const float prod = (float)code_at(row, c) * sv;
      const float v = prod + bv;
      /* prefill 1: this build's fp16 form; 2: the reference's bf16(fmaf(q, s, b)) (cuda/kernels/qmm_prefill.cu:116-117) */
      if (prefill == 2) w[c] = round_bf16(fmaf((float)code_at(row, c), sv, bv));
      else w[c] = prefill ? (float)(half_to_double(double_to_half((double)v * 256.0)) / 256.0) : v;
    }
  }
}

static float dot_f32(const float* a, const float* b, int k) {
  float p[8] = {0, 0, 0, 0, 0, 0, 0, 0};
  int i = 0;
  for (; i + 8 <= k; i += 8)
    for (int j = 0; j < 8; ++j) p[j] += a[i + j] * b[i + j];
  float t = 0.f;
  for (; i < k; ++i) t += a[i] * b[i];
  return ((p[0] + p[4]) + (p[1] + p[5])) + ((p[2] + p[6]) + (p[3] + p[7])) + t;
}

/* y[m, n] = x[m, :] . W[n, :], W dequantized to fp32 first (families/qwen3_5/cuda/reference.py:11-15);
 * x bf16 bits [m, k]; y fp32 [m, n] (the caller rounds to bf16 when it wants the bf16 result) */
void orc_affine_linear(const uint16_t* x, int m, const uint32_t* words, const uint16_t* scales,
                       const uint16_t* biases, int n, int k, int gs, int prefill, float* y) {
  float* xf = (float*)malloc(sizeof(float) * (size_t)m * k);
  for (int64_t i = 0; i < (int64_t)m * k; ++i) xf[i] = bf16_to_f32(x[i]);
  const int kg = k / gs;
#pragma omp parallel
  {
    float* w = (float*)malloc(sizeof(float) * (size_t)k);
#pragma omp for schedule(static)
    for (int c = 0; c < n; ++c) {
      dequant_row(words + (int64_t)c * (k / 8), scales + (int64_t)c * kg, biases + (int64_t)c * kg, k, gs, prefill, w);
      for (int r = 0; r < m; ++r) y[(int64_t)r * n + c] = dot_f32(xf + (int64_t)r * k, w, k);
    }
    free(w);
  }
  free(xf);
}

/* ---- routed experts: every (row, slot) pair through its expert, then the weighted combine --------------------
 * cuda/experts.cuh:53-103 (rounding points), cuda/moe.py:131-142 (combine), families/nemotron_h/cuda/reference.py:43-59 */

static inline float relu2_f(float a) {
  const float u = fmaxf(round_bf16(a), 0.f);
  return round_bf16(u * u);
}

static inline float swiglu_f(float g, float u, float limit) {
  float gv = round_bf16(g), uv = round_bf16(u);
  if (limit > 0.f) {
    gv = fminf(gv, limit);
    uv = fminf(fmaxf(uv, -limit), limit);
  }
  return round_bf16(round_bf16(gv / (1.f + expf(-gv))) * uv);
}

/* x bf16 [rows, d]; picks int32 [rows, slots]; wts fp32 [rows, slots]; tables in MLX layout: gate (may be NULL) and
 * up [E, ni, d/8] words with [E, ni, d/gs] scales/biases, down [E, d, ni/8] with [E, d, ni/gs];
 * act_out (may be NULL) bf16 bits [rows*slots, ni]; y_out (may be NULL) fp32 [rows*slots, d]; out bf16 bits [rows, d] */
void orc_moe_layer(const uint16_t* x, int rows, int d, const int32_t* picks, const float* wts, int slots,
                   const uint32_t* gate_w, const uint16_t* gate_s, const uint16_t* gate_b, const uint32_t* up_w,
                   const uint16_t* up_s, const uint16_t* up_b, const uint32_t* down_w, const uint16_t* down_s,
                   const uint16_t* down_b, int ni, int gs, float limit, int prefill, uint16_t* act_out, float* y_out,
                   uint16_t* out) {
  float* acc = (float*)calloc((size_t)rows * d, sizeof(float));
  float* xf = (float*)malloc(sizeof(float) * (size_t)d);
  float* act = (float*)malloc(sizeof(float) * (size_t)ni);
  float* yv = (float*)malloc(sizeof(float) * (size_t)d);
  const int64_t up_words = (int64_t)ni * (d / 8), up_sb = (int64_t)ni * (d / gs);
  const int64_t dn_words = (int64_t)d * (ni / 8), dn_sb = (int64_t)d * (ni / gs);
  for (int r = 0; r < rows; ++r) {
    for (int i = 0; i < d; ++i) xf[i] = bf16_to_f32(x[(int64_t)r * d + i]);
    for (int s = 0; s < slots; ++s) {
      const int64_t e = picks[r * slots + s];
      const float wt = wts[r * slots + s];
#pragma omp parallel
      {
        float* w = (float*)malloc(sizeof(float) * (size_t)(d > ni ? d : ni));
#pragma omp for schedule(static)
        for (int c = 0; c < ni; ++c) {
          dequant_row(up_w + e * up_words + (int64_t)c * (d / 8), up_s + e * up_sb + (int64_t)c * (d / gs),
                      up_b + e * up_sb + (int64_t)c * (d / gs), d, gs, prefill, w);
          const float u = dot_f32(xf, w, d);
          if (gate_w) {
            dequant_row(gate_w + e * up_words + (int64_t)c * (d / 8), gate_s + e * up_sb + (int64_t)c * (d / gs),
                        gate_b + e * up_sb + (int64_t)c * (d / gs), d, gs, prefill, w);
            act[c] = swiglu_f(dot_f32(xf, w, d), u, limit);
          } else {
            act[c] = relu2_f(u);
          }
        }
#pragma omp for schedule(static)
        for (int c = 0; c < d; ++c) {
          dequant_row(down_w + e * dn_words + (int64_t)c * (ni / 8), down_s + e * dn_sb + (int64_t)c * (ni / gs),
                      down_b + e * dn_sb + (int64_t)c * (ni / gs), ni, gs, prefill, w);
          yv[c] = dot_f32(act, w, ni);
        }
        free(w);
      }
      const int64_t p = (int64_t)r * slots + s;
      if (act_out)
        for (int c = 0; c < ni; ++c) act_out[p * ni + c] = f32_to_bf16(act[c]);
      if (y_out) memcpy(y_out + p * d, yv, sizeof(float) * (size_t)d);
      for (int c = 0; c < d; ++c) {
        const float term = wt * yv[c];
        acc[(int64_t)r * d + c] += term; /* slot order, fp32 */
      }
    }
  }
  for (int64_t i = 0; i < (int64_t)rows * d; ++i) out[i] = f32_to_bf16(acc[i]);
  free(acc);
  free(xf);
  free(act);
  free(yv);
}

/* ---- EXL3 (docs/recipes/exl3.md:43-74; cuda/exl3/format.py:31-110) ------------------------------------------- */

static uint16_t exl3_value(uint32_t s, int cb) {
  if (cb == 2) { /* mul1 */
    const uint32_t x = s * 0x83DCD12Du;
    const uint32_t h = 1024u + (x & 255u) + ((x >> 8) & 255u) + ((x >> 16) & 255u) + (x >> 24);
    return double_to_half((double)h * half_to_double(0x1EEE) + half_to_double(0xC931));
  }
  uint32_t x = cb == 1 ? s * 0xCBAC1FEDu : s * 89226354u + 64248484u;
  x = (x & 0x8FFF8FFFu) ^ 0x3B603B60u;
  return double_to_half(half_to_double((uint16_t)(x & 0xFFFFu)) + half_to_double((uint16_t)(x >> 16)));
}

void orc_exl3_codebook(int cb, uint16_t* table /* [65536] fp16 bits */) {
  for (uint32_t s = 0; s < 65536u; ++s) table[s] = exl3_value(s, cb);
}

/* One tile, bit by bit: k2 = 2 * bits; tile = 8 * k2 int16 words; vals[256] fp16 bits in stream order. */
static void exl3_tile(const int16_t* tile, int k2, int cb, uint16_t* vals) {
  const int nbits = 128 * k2;
  uint8_t stream[2048];
  for (int j = 0; j < 8 * k2; j += 2) {
    const uint32_t word = (uint32_t)(uint16_t)tile[j] | ((uint32_t)(uint16_t)tile[j + 1] << 16);
    for (int b = 0; b < 32; ++b) stream[16 * j + b] = (uint8_t)((word >> (31 - b)) & 1u);
  }
  int end = 0;
  for (int p = 0; p < 256; ++p) {
    end += k2 / 2 + ((k2 & 1) && (p & 1) ? 1 : 0);
    uint32_t s = 0;
    for (int b = end - 16; b < end; ++b) s = (s << 1) | stream[((b % nbits) + nbits) % nbits];
    vals[p] = exl3_value(s, cb);
  }
}

/* trellis int16 [kt, nt, 8*k2] -> W_q fp16 bits [16 kt, 16 nt] */
void orc_exl3_unpack(const int16_t* trellis, int kt, int nt, int k2, int cb, uint16_t* w) {
  const int n = 16 * nt;
#pragma omp parallel for schedule(static)
  for (int64_t t = 0; t < (int64_t)kt * nt; ++t) {
    uint16_t vals[256];
    exl3_tile(trellis + t * 8 * k2, k2, cb, vals);
    const int k0 = (int)(t / nt) * 16, n0 = (int)(t % nt) * 16;
    for (int p = 0; p < 256; ++p) {
      const int l = p >> 3, j = p & 7;
      const int row = 2 * (l & 3) + (j & 1) + 8 * ((j >> 1) & 1), col = (l >> 2) + 8 * (j >> 2);
      w[(int64_t)(k0 + row) * n + n0 + col] = vals[p];
    }
  }
}

static void fwht128_d(double* v) {
  for (int h = 1; h < 128; h <<= 1)
    for (int i = 0; i < 128; i += 2 * h)
      for (int j = i; j < i + h; ++j) {
        const double a = v[j], b = v[j + h];
        v[j] = a + b;
        v[j + h] = a - b;
      }
  for (int i = 0; i < 128; ++i) v[i] *= 0.08838834764831845; /* 1 / sqrt(128) */
}

/* y fp32 [m, n] = ((((x * suh) H) W_q) H) * svh (+ bias); x fp16 bits [m, k]; the rotated input is rounded to fp16
 * as the kernels do (cuda/exl3/linear.cu:110-124); sums in double. */
void orc_exl3_linear(const uint16_t* x, int m, const int16_t* trellis, const uint16_t* suh, const uint16_t* svh,
                     const uint16_t* bias, int k, int n, int k2, int cb, float* y) {
  double* xh = (double*)malloc(sizeof(double) * (size_t)m * k);
  for (int r = 0; r < m; ++r)
    for (int b = 0; b < k / 128; ++b) {
      double v[128];
      for (int i = 0; i < 128; ++i)
        v[i] = half_to_double(x[(int64_t)r * k + 128 * b + i]) * half_to_double(suh[128 * b + i]);
      fwht128_d(v);
      for (int i = 0; i < 128; ++i) xh[(int64_t)r * k + 128 * b + i] = half_to_double(double_to_half(v[i]));
    }
  const int kt = k / 16, nt = n / 16;
#pragma omp parallel
  {
    double* acc = (double*)malloc(sizeof(double) * (size_t)m * 128);
    uint16_t vals[256];
    double wt[256];
#pragma omp for schedule(static)
    for (int nb = 0; nb < n / 128; ++nb) {
      memset(acc, 0, sizeof(double) * (size_t)m * 128);
      for (int t = 0; t < kt; ++t)
        for (int j = 0; j < 8; ++j) {
          exl3_tile(trellis + ((int64_t)t * nt + nb * 8 + j) * 8 * k2, k2, cb, vals);
          for (int p = 0; p < 256; ++p) {
            const int l = p >> 3, q = p & 7;
            const int row = 2 * (l & 3) + (q & 1) + 8 * ((q >> 1) & 1), col = (l >> 2) + 8 * (q >> 2);
            wt[row * 16 + col] = half_to_double(vals[p]);
          }
          for (int r = 0; r < m; ++r)
            for (int row = 0; row < 16; ++row) {
              const double xv = xh[(int64_t)r * k + 16 * t + row];
              for (int col = 0; col < 16; ++col) acc[r * 128 + 16 * j + col] += xv * wt[row * 16 + col];
            }
        }
      for (int r = 0; r < m; ++r) {
        fwht128_d(acc + r * 128);
        for (int i = 0; i < 128; ++i) {
          double v = acc[r * 128 + i] * half_to_double(svh[128 * nb + i]);
          if (bias) v += half_to_double(bias[128 * nb + i]);
          y[(int64_t)r * n + 128 * nb + i] = (float)v;
        }
      }
    }
    free(acc);
  }
  free(xh);
}
