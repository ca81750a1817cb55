/*
 * arcq_oracle.c -- CPU restatement of ARCQuant's fake-quant arithmetic for the
 * quantized-linear path.  TEST INFRASTRUCTURE ONLY: nothing that ships (the HIP
 * library, the Python op surface) may link, import or call this file.  It is the
 * checker the GPU kernels are compared with, and the thing bench.py times as the
 * host-CPU baseline.
 *
 * Each function names the reference lines it restates (paths relative to the
 * reference checkout):
 *   model/quantize.py:14-22    quantize_e2m1       -> oq_e2m1
 *   model/quantize.py:40-49    quantize_ue4m3      -> oq_ue4m3
 *   model/quantize.py:54-59    quantize_ue8m0      -> oq_ue8m0
 *   model/quantize.py:145-201  quantize_{nv,mx}fp4_tensor -> oq_block
 *   model/quantize.py:314-343  fake_reorder_quantize_x    -> arcq_oracle_quantize_x
 *   model/quantize.py:287-312  fake_reorder_quantize_w    -> arcq_oracle_quantize_w
 *   benchmarks/modeling_arc.py:237-242 (HF RMSNorm formula) followed by
 *   fake_reorder_quantize_x                        -> arcq_oracle_rmsnorm_quantize_x
 *
 * The reference returns dequantised VALUES only.  Codes and scale bytes are read
 * off the same intermediates: a code is the index of the chosen grid value, a
 * scale byte is an exact re-encoding of the fp32 scale the reference computes.
 *
 * All arithmetic is IEEE binary32 with one rounding per operation, as torch's
 * CPU kernels do it: build with -ffp-contract=off -mfpmath=sse (see Makefile).
 *
 * Pinning status (see tests/test_oracle_*.py):
 *   oq_e2m1   : literal 15-way argmin; pinned by the tie table the reference's
 *               argmin implies and by brute force against the torch restatement.
 *   oq_ue4m3  : pinned by closed form (RNE to 3 mantissa bits, no subnormals)
 *               on a dense sweep and against golden vectors of the reference.
 *   oq_ue8m0  : pinned by closed form around every power of two and golden vectors.
 *   quantize_x/w : pinned by structure (main = blockwise Q, tail = Q(err) / copy),
 *               by an end-to-end golden vector, and against the torch restatement.
 *   rmsnorm_quantize_x : the reference has no fake-quant path for the fused op;
 *               the normalisation step is this build's own statement of the HF
 *               formula with a correctly rounded mean of squares -> "parity
 *               unpinned" for that step (match-rate checked against torch fp32).
 */
#include <math.h>
#include <stdint.h>
#include <string.h>
#include <stdlib.h>

#define ARCQ_FMT_NVFP4 0
#define ARCQ_FMT_MXFP4 1

static inline float bf16_to_f32(uint16_t h) {
  uint32_t u = (uint32_t)h << 16;
  float f;
  memcpy(&f, &u, 4);
  return f;
}

/* round-to-nearest-even float -> bf16, as torch's .to(torch.bfloat16) does */
static inline uint16_t f32_to_bf16(float f) {
  uint32_t u;
  memcpy(&u, &f, 4);
  if ((u & 0x7fffffffu) > 0x7f800000u) return 0x7fc0; /* NaN */
  u += 0x7fffu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}

static const float kGrid[15] = {-6.0f, -4.0f, -3.0f, -2.0f, -1.5f, -1.0f, -0.5f, 0.0f,
                                0.5f,  1.0f,  1.5f,  2.0f,  3.0f,  4.0f,  6.0f};
/* grid index -> 4-bit e2m1 code (sign<<3 | magnitude index); zero is always 0x0 */
static const uint8_t kGridCode[15] = {0xF, 0xE, 0xD, 0xC, 0xB, 0xA, 0x9, 0x0,
                                      0x1, 0x2, 0x3, 0x4, 0x5, 0x6, 0x7};
static const float kCodeValue[16] = {0.0f, 0.5f,  1.0f,  1.5f,  2.0f,  3.0f,  4.0f,  6.0f,
                                     0.0f, -0.5f, -1.0f, -1.5f, -2.0f, -3.0f, -4.0f, -6.0f};

/* quantize.py:14-22 : |n - v_j| over the ascending 15-value grid, first minimum wins */
float oq_e2m1(float n, uint8_t *code) {
  int best = 0;
  float bestd = fabsf(n - kGrid[0]);
  for (int j = 1; j < 15; ++j) {
    float d = fabsf(n - kGrid[j]);
    if (d < bestd) { bestd = d; best = j; }
  }
  if (code) *code = kGridCode[best];
  return kGrid[best];
}

/* log2 rounded once to binary32 (double log2 is accurate far below half an fp32 ulp) */
static inline float log2_f32(float u) { return (float)log2((double)u); }

/*
 * quantize.py:40-49.  Scale byte: ((e+9)<<3)|m8 for the value (1+m8/8)*2^e,
 * e in [-9,8].  For values >= 2^-6 this is the standard E4M3 byte plus 16; the
 * three extra binades exist because the reference's emulation has no subnormals
 * and therefore produces (1+k/8)*2^e for e in {-9,-8,-7}, most of which no real
 * E4M3 byte can hold.
 */
float oq_ue4m3(float t, uint8_t *byte) {
  if (t < 2e-3f) t = 2e-3f;
  if (t > 448.0f) t = 448.0f;
  float e = floorf(log2_f32(t + 1e-9f));
  float p = exp2f(e);               /* exact power of two */
  float m = t / p - 1.0f;
  float qm = rintf(m * 8.0f) / 8.0f; /* torch.round: half to even */
  float v = (1.0f + qm) * p;
  if (byte) {
    int ee;
    float fr = frexpf(v, &ee);      /* v = fr * 2^ee, fr in [0.5,1) */
    int e2 = ee - 1;                /* v = (2*fr) * 2^e2 */
    int m8 = (int)((2.0f * fr - 1.0f) * 8.0f);
    *byte = (uint8_t)(((e2 + 9) << 3) | m8);
  }
  return v;
}

/* quantize.py:54-59.  Scale byte: e + 127 (standard E8M0). */
float oq_ue8m0(float t, uint8_t *byte) {
  float e = ceilf(log2_f32(t + 1e-9f));
  if (e < -127.0f) e = -127.0f;
  if (e > 127.0f) e = 127.0f;
  if (byte) *byte = (uint8_t)((int)e + 127);
  return exp2f(e);
}

float oq_scale_value(int fmt, uint8_t byte) {
  if (fmt == ARCQ_FMT_NVFP4)
    return ldexpf(1.0f + (float)(byte & 7) / 8.0f, (int)(byte >> 3) - 9);
  return ldexpf(1.0f, (int)byte - 127);
}

float oq_code_value(uint8_t code) { return kCodeValue[code & 15]; }

/*
 * quantize.py:145-172 (G=16) / 174-201 (G=32), one block:
 * amax -> /6 -> (0 -> 1e-9) -> scale format -> true divide -> e2m1 -> q*s.
 */
static void oq_block(int fmt, const float *x, int G, uint8_t *codes /*G*/, uint8_t *sbyte, float *dq /*G*/) {
  float amax = 0.0f;
  for (int i = 0; i < G; ++i) {
    float a = fabsf(x[i]);
    if (a > amax) amax = a;
  }
  float t = amax / 6.0f;
  if (t == 0.0f) t = 1e-9f;
  float s = (fmt == ARCQ_FMT_NVFP4) ? oq_ue4m3(t, sbyte) : oq_ue8m0(t, sbyte);
  for (int i = 0; i < G; ++i) {
    float n = x[i] / s;
    float q = oq_e2m1(n, &codes[i]);
    dq[i] = q * s;
  }
}

static inline int fmt_group(int fmt) { return fmt == ARCQ_FMT_NVFP4 ? 16 : 32; }

static void pack_codes(const uint8_t *c, int n, uint8_t *out) {
  for (int j = 0; j < n / 2; ++j) out[j] = (uint8_t)(c[2 * j] | (c[2 * j + 1] << 4));
}

/*
 * One row of fake_reorder_quantize_x (quantize.py:330-343) on already-gathered
 * fp32 values r[K] (= x.float()/scale): main blocks, then the residual of the
 * last S channels re-quantised as S/G more blocks.  Writes K+S codes (packed),
 * (K+S)/G scale bytes and, when dq != NULL, the K+S dequantised values q*s.
 */
static void oq_row_x(int fmt, const float *r, int K, int S, uint8_t *codes_packed, uint8_t *scales, float *dq,
                     uint8_t *cbuf, float *vbuf, float *ebuf) {
  const int G = fmt_group(fmt);
  for (int b = 0; b < K / G; ++b) oq_block(fmt, r + b * G, G, cbuf + b * G, scales + b, vbuf + b * G);
  for (int k = 0; k < S; ++k) ebuf[k] = r[K - S + k] - vbuf[K - S + k]; /* quantize.py:339, fp32 */
  for (int b = 0; b < S / G; ++b)
    oq_block(fmt, ebuf + b * G, G, cbuf + K + b * G, scales + K / G + b, vbuf + K + b * G);
  pack_codes(cbuf, K + S, codes_packed);
  if (dq) memcpy(dq, vbuf, sizeof(float) * (size_t)(K + S));
}

/*
 * fake_reorder_quantize_x, with the caller's index_select folded in
 * (model/qLlamaLayer.py:84-86 gathers x[:, reorder_index] first).
 *   x      bf16 [M,K] row-major           idx  int16 [K] (NULL = identity)
 *   gscale the fp32 tensor scale the values are divided by (quantize.py:330)
 *   codes  u8 [M,(K+S)/2], element 2j in the low nibble
 *   scales u8 [M,(K+S)/G]
 *   dq     optional fp32 [M,K+S]: q*s (NOT multiplied back by gscale)
 * Returns 0, or -1 on a shape the path does not define.
 */
int arcq_oracle_quantize_x(const uint16_t *x, int M, int K, const int16_t *idx, int S, int fmt, float gscale,
                           uint8_t *codes, uint8_t *scales, float *dq) {
  const int G = fmt_group(fmt);
  if (K <= 0 || K % G || S < 0 || S % G || S > K) return -1;
  const int Kp = K + S;
  int rc = 0;
#pragma omp parallel
  {
    float *r = (float *)malloc(sizeof(float) * (size_t)K);
    float *v = (float *)malloc(sizeof(float) * (size_t)Kp);
    float *e = (float *)malloc(sizeof(float) * (size_t)(S ? S : 1));
    uint8_t *c = (uint8_t *)malloc((size_t)Kp);
#pragma omp for schedule(static)
    for (int m = 0; m < M; ++m) {
      const uint16_t *xr = x + (size_t)m * K;
      for (int k = 0; k < K; ++k) {
        int src = idx ? (int)idx[k] : k;
        if (src < 0 || src >= K) { rc = -2; src = 0; }
        r[k] = bf16_to_f32(xr[src]) / gscale;
      }
      oq_row_x(fmt, r, K, S, codes + (size_t)m * (Kp / 2), scales + (size_t)m * (Kp / G),
               dq ? dq + (size_t)m * Kp : NULL, c, v, e);
    }
    free(r); free(v); free(e); free(c);
  }
  return rc;
}

/*
 * fake_reorder_quantize_w (quantize.py:287-312): main blocks of w.float()/scale,
 * then the last S channels quantised again -- the same values, hence the same
 * codes and scales, so the tail is a verbatim copy of the last S/G blocks.
 * The reference does not multiply back by scale (quantize.py:311-312); dq here
 * is q*s as well.
 */
int arcq_oracle_quantize_w(const uint16_t *w, int N, int K, const int16_t *idx, int S, int fmt, float gscale,
                           uint8_t *codes, uint8_t *scales, float *dq) {
  const int G = fmt_group(fmt);
  if (K <= 0 || K % G || S < 0 || S % G || S > K) return -1;
  const int Kp = K + S;
  int rc = 0;
#pragma omp parallel
  {
    float *r = (float *)malloc(sizeof(float) * (size_t)Kp);
    float *v = (float *)malloc(sizeof(float) * (size_t)Kp);
    uint8_t *c = (uint8_t *)malloc((size_t)Kp);
#pragma omp for schedule(static)
    for (int n = 0; n < N; ++n) {
      const uint16_t *wr = w + (size_t)n * K;
      for (int k = 0; k < K; ++k) {
        int src = idx ? (int)idx[k] : k;
        if (src < 0 || src >= K) { rc = -2; src = 0; }
        r[k] = bf16_to_f32(wr[src]) / gscale;
      }
      for (int k = 0; k < S; ++k) r[K + k] = r[K - S + k]; /* cat([w, w[:, -S:]]) */
      uint8_t *srow = scales + (size_t)n * (Kp / G);
      for (int b = 0; b < Kp / G; ++b) oq_block(fmt, r + b * G, G, c + b * G, srow + b, v + b * G);
      pack_codes(c, Kp, codes + (size_t)n * (Kp / 2));
      if (dq) memcpy(dq + (size_t)n * Kp, v, sizeof(float) * (size_t)Kp);
    }
    free(r); free(v); free(c);
  }
  return rc;
}

/*
 * RMSNorm (benchmarks/modeling_arc.py:237-242: fp32 x*rsqrt(mean(x^2)+eps) -> bf16,
 * then gamma * that in bf16) followed by fake_reorder_quantize_x.  mean(x^2) is
 * the correctly rounded one: squares of bf16 values are exact in fp32, the sum is
 * taken in fp64 and rounded once.  rsqrt is 1/sqrt with both steps correctly
 * rounded, which is what torch's CPU kernel computes.
 *   normed (optional) bf16 [M,K]: the un-reordered RMSNorm output, for match-rate
 *   checks against torch's own fp32 reduction.
 */
int arcq_oracle_rmsnorm_quantize_x(const uint16_t *x, const uint16_t *gamma, float eps, int M, int K,
                                   const int16_t *idx, int S, int fmt, float gscale, uint8_t *codes,
                                   uint8_t *scales, float *dq, uint16_t *normed) {
  const int G = fmt_group(fmt);
  if (K <= 0 || K % G || S < 0 || S % G || S > K) return -1;
  const int Kp = K + S;
  int rc = 0;
#pragma omp parallel
  {
    float *y = (float *)malloc(sizeof(float) * (size_t)K);
    float *r = (float *)malloc(sizeof(float) * (size_t)K);
    float *v = (float *)malloc(sizeof(float) * (size_t)Kp);
    float *e = (float *)malloc(sizeof(float) * (size_t)(S ? S : 1));
    uint8_t *c = (uint8_t *)malloc((size_t)Kp);
#pragma omp for schedule(static)
    for (int m = 0; m < M; ++m) {
      const uint16_t *xr = x + (size_t)m * K;
      double ss = 0.0;
      for (int k = 0; k < K; ++k) {
        float f = bf16_to_f32(xr[k]);
        ss += (double)(f * f);
      }
      float var = (float)(ss / (double)K);
      float rstd = 1.0f / sqrtf(var + eps);
      for (int k = 0; k < K; ++k) {
        uint16_t h = f32_to_bf16(bf16_to_f32(xr[k]) * rstd);
        uint16_t o = f32_to_bf16(bf16_to_f32(gamma[k]) * bf16_to_f32(h));
        if (normed) normed[(size_t)m * K + k] = o;
        y[k] = bf16_to_f32(o);
      }
      for (int k = 0; k < K; ++k) {
        int src = idx ? (int)idx[k] : k;
        if (src < 0 || src >= K) { rc = -2; src = 0; }
        r[k] = y[src] / gscale;
      }
      oq_row_x(fmt, r, K, S, codes + (size_t)m * (Kp / 2), scales + (size_t)m * (Kp / G),
               dq ? dq + (size_t)m * Kp : NULL, c, v, e);
    }
    free(y); free(r); free(v); free(e); free(c);
  }
  return rc;
}

/* codes+scales -> fp32 values q*s, rows x Kp (what F.linear sees before the tensor scales) */
int arcq_oracle_dequantize(const uint8_t *codes, const uint8_t *scales, int rows, int Kp, int fmt, float *out) {
  const int G = fmt_group(fmt);
  if (Kp % G) return -1;
#pragma omp parallel for schedule(static)
  for (int r = 0; r < rows; ++r) {
    const uint8_t *cr = codes + (size_t)r * (Kp / 2);
    const uint8_t *sr = scales + (size_t)r * (Kp / G);
    float *o = out + (size_t)r * Kp;
    for (int k = 0; k < Kp; ++k) {
      uint8_t byte = cr[k >> 1];
      uint8_t code = (k & 1) ? (byte >> 4) : (byte & 15);
      o[k] = kCodeValue[code] * oq_scale_value(fmt, sr[k / G]);
    }
  }
  return 0;
}

/*
 * F.linear on the fake-quantised values (model/qLinearLayer.py:71), restated on
 * codes: Y[m,n] = alpha * sum_k dq(A)[m,k]*dq(B)[n,k], accumulated in fp64 (the
 * tolerance test compares the GPU's fp32-accumulated bf16 output with this).
 */
int arcq_oracle_matmul(const uint8_t *ca, const uint8_t *sa, const uint8_t *cb, const uint8_t *sb, int M, int N,
                       int Kp, int fmt, float alpha, float *Y) {
  const int G = fmt_group(fmt);
  if (Kp % G) return -1;
  float *A = (float *)malloc(sizeof(float) * (size_t)M * Kp);
  float *B = (float *)malloc(sizeof(float) * (size_t)N * Kp);
  arcq_oracle_dequantize(ca, sa, M, Kp, fmt, A);
  arcq_oracle_dequantize(cb, sb, N, Kp, fmt, B);
#pragma omp parallel for schedule(static)
  for (int m = 0; m < M; ++m)
    for (int n = 0; n < N; ++n) {
      double acc = 0.0;
      const float *a = A + (size_t)m * Kp, *b = B + (size_t)n * Kp;
      for (int k = 0; k < Kp; ++k) acc += (double)a[k] * (double)b[k];
      Y[(size_t)m * N + n] = (float)(acc * (double)alpha);
    }
  free(A); free(B);
  return 0;
}

/* elementwise entry points for the sweep tests */
void arcq_oracle_e2m1_many(const float *n, int cnt, float *val, uint8_t *code) {
  for (int i = 0; i < cnt; ++i) val[i] = oq_e2m1(n[i], &code[i]);
}
void arcq_oracle_ue4m3_many(const float *t, int cnt, float *val, uint8_t *byte) {
  for (int i = 0; i < cnt; ++i) val[i] = oq_ue4m3(t[i], &byte[i]);
}
void arcq_oracle_ue8m0_many(const float *t, int cnt, float *val, uint8_t *byte) {
  for (int i = 0; i < cnt; ++i) val[i] = oq_ue8m0(t[i], &byte[i]);
}
