// host_math.cpp -- g++ build of the kernels' scalar arithmetic (arcq_math.h) so that CPU tests
// can sweep it exhaustively.  Not part of the shipped GPU path; exports array wrappers only.
#include <math.h>
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

// a/6 through div6_any for every fp32 significand at three exponents vs the IEEE quotient
long arcq_host_check_div6_any(void) {
  long bad = 0;
  const uint32_t expo[3] = {37u, 127u, 240u};
#pragma omp parallel for reduction(+ : bad)
  for (int64_t m = 0; m < (1 << 23); ++m) {
    for (int e = 0; e < 3; ++e) {
      const float a = arcq::u2f((expo[e] << 23) | (uint32_t)m);
      if (arcq::f2u(arcq::div6_any(a)) != arcq::f2u(a / 6.0f)) ++bad;
    }
  }
  return bad;
}

// x/g through div_bf16_by for every bf16 significand of x and every `stride`-th fp32 significand
// of g (stride 1 = all of them), both signs of g, vs the IEEE quotient
long arcq_host_check_div_bf16(int stride) {
  long bad = 0;
#pragma omp parallel for schedule(static) reduction(+ : bad)
  for (int64_t m = 0; m < (1 << 23); m += stride) {
    const float g = arcq::u2f(0x3f800000u | (uint32_t)m);
    const float rg = 1.0f / g;
    for (uint32_t xm = 0; xm < 128u; ++xm) {
      const float x = arcq::u2f(0x40000000u | (xm << 16));
      if (arcq::f2u(arcq::div_bf16_by(x, g, rg)) != arcq::f2u(x / g)) ++bad;
      if (arcq::f2u(arcq::div_bf16_by(-x, g, rg)) != arcq::f2u(-x / g)) ++bad;
      if (arcq::f2u(arcq::div_bf16_by(x, -g, -rg)) != arcq::f2u(x / -g)) ++bad;
    }
  }
  return bad;
}

// The two-sided encode of the quantizer kernels (y*r*(1+2^-20) and y*r*(1-2^-20) through the RNE
// convert; where the two codes agree that is the code, where they differ e2m1_resolve decides)
// against e2m1_code(y / s), for n pseudo-random fp32 y per scale plus a dense band of y around
// every decision point, every scale of the format and r = 1/s moved by -1, 0, +1 ulp.  Returns the
// number of wrong codes; *accepted / *checked report how often the two conversions agreed.
long long arcq_host_check_two_sided(int fmt, long n, long long *accepted, long long *checked) {
  const int nscale = fmt == 0 ? 143 : 60;
  long long bad = 0, acc = 0, cnt = 0;
  static const float mids[7] = {0.25f, 0.75f, 1.25f, 1.75f, 2.5f, 3.5f, 5.0f};
#pragma omp parallel for schedule(dynamic, 1) reduction(+ : bad, acc, cnt)
  for (int si = 0; si < nscale; ++si) {
    const uint32_t sb = fmt == 0 ? (uint32_t)si : (uint32_t)(127 - 40 + si);
    const float s = fmt == 0 ? arcq::nvfp4_scale_value(sb) : arcq::mxfp4_scale_value(sb);
    const float r_exact = 1.0f / s;
    uint64_t st = 0x243f6a8885a308d3ull + (uint64_t)si;
    const long band = 200;
    const long total = n + 7 * (2 * band + 1) * 2;
    for (long i = 0; i < total; ++i) {
      float y;
      if (i < n) {
        st = st * 6364136223846793005ull + 1442695040888963407ull;
        const uint32_t mant = (uint32_t)(st >> 40) & 0x7fffffu;
        const uint32_t ex = 121u + (uint32_t)((st >> 20) % 10u);          // |y/s| in [2^-6, 2^4)
        y = arcq::u2f(((uint32_t)(st >> 63) << 31) | (ex << 23) | mant) * s;
      } else {
        const long j = i - n;
        const int sign = (int)(j & 1);
        const long k = (j >> 1) % (2 * band + 1) - band;
        const int mi = (int)((j >> 1) / (2 * band + 1));
        const float c = mids[mi] * s;                                      // exact: few significant bits
        y = arcq::u2f(arcq::f2u(c) + (uint32_t)k);
        if (sign) y = -y;
      }
      const uint32_t exact = arcq::e2m1_code(y / s);
      for (int d = -1; d <= 1; ++d) {
        const float r = arcq::u2f(arcq::f2u(r_exact) + (uint32_t)d);
        const float ra = r * 0x1.00001p+0f, rb = r * 0x1.ffffep-1f;
        uint32_t ca = arcq::e2m1_rne_hw_model(y * ra), cb = arcq::e2m1_rne_hw_model(y * rb);
        ++cnt;
        uint32_t got;
        if (ca != cb) {
          got = arcq::e2m1_resolve(y, s, ca, cb);
        } else {
          ++acc;
          got = (ca & 7u) == 0u ? 0u : ca;  // drop_negative_zeros
        }
        if (got != exact) ++bad;
      }
    }
  }
  *accepted = acc;
  *checked = cnt;
  return bad;
}

// The quantizer's encode for a tensor scale g that is not a power of two, without forming y = x/g per element:
// the block scale comes from RN(max|x| / g) (RN(x/g) is monotone in |x|, so that is max|y|), the codes from
// x * R * (1 +- 2^-20) with R = RN(rg * r), rg = RN(1/g), r within an ulp of 1/s, through the RNE convert; where
// the two codes differ, y = RN(x/g) is formed for that element and e2m1_resolve decides.  Checked against the
// reference's e2m1_code(RN(RN(x/g) / s)) for every finite bf16 x with |x/g| <= 8s (and a sample beyond), every
// block scale s, r off by -1, 0, +1 ulp, and tensor scales g = m / 2688 for every bf16 significand m (what
// max|x| / 2688 can be) at several exponents plus n_random pseudo-random fp32 g.  Returns the number of wrong
// codes; *accepted / *checked report how often the two conversions agreed.
long long arcq_host_check_scaled_direct(int fmt, int n_random, long long *accepted, long long *checked) {
  const int nscale = fmt == 0 ? 143 : 60;
  const int n_struct = 128 * 3;
  long long bad = 0, acc = 0, cnt = 0;
#pragma omp parallel for schedule(dynamic, 4) reduction(+ : bad, acc, cnt)
  for (int gi = 0; gi < n_struct + n_random; ++gi) {
    float g;
    if (gi < n_struct) {
      const float mx = arcq::u2f(((uint32_t)(127 - 3 + 4 * (gi / 128)) << 23) | ((uint32_t)(gi % 128) << 16));
      g = mx / 2688.0f;
    } else {
      uint64_t st = 0x9e3779b97f4a7c15ull * (uint64_t)(gi + 1);
      st = st * 6364136223846793005ull + 1442695040888963407ull;
      g = arcq::u2f(((uint32_t)(115 + (st >> 59) % 12) << 23) | ((uint32_t)(st >> 20) & 0x7fffffu));
    }
    const float rg = 1.0f / g;
    for (int si = 0; si < nscale; ++si) {
      const uint32_t sb = fmt == 0 ? (uint32_t)si : (uint32_t)(127 - 40 + si);
      const float s = fmt == 0 ? arcq::nvfp4_scale_value(sb) : arcq::mxfp4_scale_value(sb);
      const float r_exact = fmt == 0 ? 1.0f / s : arcq::u2f((254u << 23) - arcq::f2u(s));
      for (uint32_t hb = 0; hb < 0x10000u; ++hb) {
        if ((hb & 0x7f80u) == 0x7f80u) continue;  // inf / nan
        const float x = arcq::bf16_bits_to_f32(hb);
        const float y = x / g;                     // the reference's x32 (quantize.py:330)
        const float ay = y < 0 ? -y : y;
        if (!(ay <= 8.0f * s) && (hb & 0x7fu) != 0x2bu) continue;        // a sample of the saturating range
        if (ay < 0x1p-8f * s && (hb & 0x7fu) != 0x2bu) continue;          // far below the first decision point
        if (!(ay < 0x1p+100f) || (ay != 0.0f && ay < 0x1p-100f)) continue;  // such units are redone with IEEE divisions
        const uint32_t exact = arcq::e2m1_code(y / s);
        for (int d = (fmt == 0 ? -1 : 0); d <= (fmt == 0 ? 1 : 0); ++d) {
          const float r = arcq::u2f(arcq::f2u(r_exact) + (uint32_t)d);
          const float R = rg * r;
          const float Ra = R * 0x1.00001p+0f, Rb = R * 0x1.ffffep-1f;
          const uint32_t ca = arcq::e2m1_rne_hw_model(x * Ra), cb = arcq::e2m1_rne_hw_model(x * Rb);
          ++cnt;
          uint32_t got;
          if (ca != cb) {
            got = arcq::e2m1_resolve(arcq::div_bf16_by(x, g, rg), s, ca, cb);
          } else {
            ++acc;
            got = (ca & 7u) == 0u ? 0u : ca;  // drop_negative_zeros
          }
          if (got != exact) ++bad;
        }
      }
    }
  }
  *accepted = acc;
  *checked = cnt;
  return bad;
}

// 1/sqrt(a) as the RMSNorm kernel forms it (sqrt_from_estimate, rcp_from_estimate) against
// 1.0f / sqrtf(a), with the hardware estimates modelled as the correctly rounded value moved by
// -1, 0, +1 ulp.  a runs over n values spread across [2^-90, 2^100] plus a dense stretch.
long arcq_host_check_rstd(long n) {
  long bad = 0;
  uint64_t st = 0x9e3779b97f4a7c15ull;
  for (long i = 0; i < n; ++i) {
    st = st * 6364136223846793005ull + 1442695040888963407ull;
    uint32_t bits;
    if (i & 1) {
      bits = (uint32_t)(st >> 33) % ((227u - 37u) << 23) + (37u << 23);   // exponents -90 .. 100
    } else {
      bits = 0x3f000000u + (uint32_t)(i >> 1);                             // dense from 0.5 upward
    }
    const float a = arcq::u2f(bits);
    const float s_ref = sqrtf(a);
    const float want = 1.0f / s_ref;
    for (int ds = -1; ds <= 1; ++ds) {
      const float s = arcq::sqrt_from_estimate(a, arcq::u2f(arcq::f2u(s_ref) + (uint32_t)ds));
      if (arcq::f2u(s) != arcq::f2u(s_ref)) { ++bad; continue; }
      for (int dr = -1; dr <= 1; ++dr) {
        const float r = arcq::rcp_from_estimate(s, arcq::u2f(arcq::f2u(want) + (uint32_t)dr));
        if (arcq::f2u(r) != arcq::f2u(want)) ++bad;
      }
    }
  }
  return bad;
}

}  // extern "C"
