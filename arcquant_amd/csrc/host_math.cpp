// host_math.cpp -- g++ build of the kernels' scalar arithmetic (arcq_math.h) so that CPU tests
// can sweep it exhaustively.  Not part of the shipped GPU path; exports array wrappers only.
#include <stdint.h>

#include "arcq_math.h"

extern "C" {

void arcq_host_ue4m3(const float *t, int n, float *val, uint8_t *byte) {
  for (int i = 0; i < n; ++i) byte[i] = (uint8_t)arcq::ue4m3_scale(t[i], &val[i]);
}

void arcq_host_ue8m0(const float *t, int n, float *val, uint8_t *byte) {
  for (int i = 0; i < n; ++i) byte[i] = (uint8_t)arcq::ue8m0_scale(t[i], &val[i]);
}

void arcq_host_e2m1(const float *x, int n, float *val, uint8_t *code) {
  for (int i = 0; i < n; ++i) {
    code[i] = (uint8_t)arcq::e2m1_code(x[i]);
    val[i] = arcq::e2m1_value(code[i]);
  }
}

void arcq_host_scale_values(const uint8_t *b, int n, int fmt, float *val) {
  for (int i = 0; i < n; ++i) val[i] = fmt == 0 ? arcq::nvfp4_scale_value(b[i]) : arcq::mxfp4_scale_value(b[i]);
}

// ---- exhaustive check of the coarse fast path -------------------------------------------------
// For every block scale s of the format, every bf16 value y with |y| <= 8s (beyond that the code
// saturates either way; a few such values are included), and reciprocals r = (1/s)(1 + d),
// d in {0, +-2^-21}: the fast code must equal the exact one.  With residual != 0 the ARC residual
// e = y - q*s is pushed through the same comparison against every scale s2 that a block
// containing e could get (|e| <= 6.5 s2) and that can still resolve it (|e| >= s2/8).
// Returns the number of disagreements; *checked receives the number of comparisons.
static inline uint32_t fast_code(float y, float r) {
  const float w = __builtin_fmaf(y, r, -arcq::kCoarseNudge);
  return arcq::drop_negative_zeros(arcq::e2m1_rne_hw_model(w)) & 15u;
}

long long arcq_host_check_coarse(int fmt, int residual, long long *checked) {
  const int nscale = fmt == 0 ? 143 : 60;
  long long bad = 0, cnt = 0;
#pragma omp parallel for schedule(dynamic, 1) reduction(+ : bad, cnt)
  for (int si = 0; si < nscale; ++si) {
    const uint32_t sb = fmt == 0 ? (uint32_t)si : (uint32_t)(127 - 40 + si);
    const float s = fmt == 0 ? arcq::nvfp4_scale_value(sb) : arcq::mxfp4_scale_value(sb);
    const float perturb[3] = {1.0f, 1.0f + 0x1p-21f, 1.0f - 0x1p-21f};
    for (uint32_t hb = 0; hb < 0x10000u; ++hb) {
      if ((hb & 0x7f80u) == 0x7f80u) continue;  // inf / nan
      const float y = arcq::bf16_bits_to_f32(hb);
      const float ay = y < 0 ? -y : y;
      if (ay > 8.0f * s && (hb & 0x7fu) != 0x15u) continue;  // keep a sample of the saturating range
      for (int pi = 0; pi < 3; ++pi) {
        const float r = (fmt == 0 ? 1.0f / s : arcq::u2f((254u << 23) - arcq::f2u(s))) * perturb[pi];
        if (fmt == 1 && pi) break;  // a power-of-two scale has an exact reciprocal
        const uint32_t exact = arcq::e2m1_code(y / s);
        ++cnt;
        if (fast_code(y, r) != exact) ++bad;
        if (!residual || pi) continue;
        const float e = y - arcq::e2m1_value(exact) * s;
        const float ae = e < 0 ? -e : e;
        if (ae == 0.0f) continue;
        const int n2 = fmt == 0 ? 143 : 60;
        for (int s2i = 0; s2i < n2; ++s2i) {
          const uint32_t sb2 = fmt == 0 ? (uint32_t)s2i : (uint32_t)(127 - 40 + s2i);
          const float s2 = fmt == 0 ? arcq::nvfp4_scale_value(sb2) : arcq::mxfp4_scale_value(sb2);
          if (ae > 6.5f * s2 || ae < 0.125f * s2) continue;
          for (int pj = 0; pj < (fmt == 0 ? 3 : 1); ++pj) {
            const float r2 = (fmt == 0 ? 1.0f / s2 : arcq::u2f((254u << 23) - arcq::f2u(s2))) * perturb[pj];
            ++cnt;
            if (fast_code(e, r2) != arcq::e2m1_code(e / s2)) ++bad;
          }
        }
      }
    }
  }
  *checked = cnt;
  return bad;
}

// amax/6 through div6_coarse for every positive finite bf16 value vs the IEEE quotient
int arcq_host_check_div6(void) {
  int bad = 0;
  for (uint32_t hb = 0x0080u; hb < 0x7f00u; ++hb) {
    const float a = arcq::bf16_bits_to_f32(hb);
    if (arcq::f2u(arcq::div6_coarse(a)) != arcq::f2u(a / 6.0f)) ++bad;
  }
  return bad;
}

}  // extern "C"
