// arcq_math.h -- the scalar arithmetic of the quantizers, written once for device and host.
//
// Every routine here is a closed form of one step of the reference's PyTorch fake quantizer
// (model/quantize.py); the same source is compiled by hipcc into the kernels and by g++ into
// a host library (csrc/host_math.cpp) so that CPU tests can sweep it exhaustively.
#ifndef ARCQ_MATH_H_
#define ARCQ_MATH_H_

#include <stdint.h>

#if defined(__HIPCC__)
#define ARCQ_HD __host__ __device__ __forceinline__
#else
#define ARCQ_HD inline
#endif

namespace arcq {

ARCQ_HD uint32_t f2u(float f) { return __builtin_bit_cast(uint32_t, f); }
ARCQ_HD float u2f(uint32_t u) { return __builtin_bit_cast(float, u); }
ARCQ_HD float bf16_bits_to_f32(uint32_t h) { return u2f(h << 16); }

// float -> bf16 bits, round to nearest even (finite inputs)
ARCQ_HD uint32_t f32_to_bf16_bits(float f) {
  uint32_t u = f2u(f);
  return (u + 0x7fffu + ((u >> 16) & 1u)) >> 16;
}

// quantize_ue4m3 (model/quantize.py:40-49) of t = amax/6 >= 0: clamp to [2e-3, 448], round to
// nearest even on a 1+3-bit significand, no subnormals (the floor 2e-3 rounds to 2^-9).
// Returns the scale byte ((e+9)<<3 | m); *s receives the scale value.
// A zero block needs no special case: 0 -> 1e-9 -> clamp -> 2e-3 in the reference as well.
ARCQ_HD uint32_t ue4m3_scale(float t, float *s) {
  t = t < 2e-3f ? 2e-3f : t;
  t = t > 448.0f ? 448.0f : t;
  uint32_t b = f2u(t);
  b += 0x7ffffu + ((b >> 20) & 1u);
  b &= 0xfff00000u;
  *s = u2f(b);
  return (b >> 20) - ((127u - 9u) << 3);
}

// quantize_ue8m0 (model/quantize.py:54-59) of t = amax/6 >= 0 (0 is replaced by 1e-9 first,
// quantize.py:185): 2^ceil(fl(log2(fl(t + 1e-9)))), clamped to 2^+-127.
// With u = fl(t+1e-9) = 2^k (1 + j 2^-23), fl(log2 u) equals k exactly when j = 0 or when
// log2(1 + j 2^-23) is below half an ulp of the floats just above k, i.e. j <= jmax(p) with
// 2^p the binade of those floats: jmax = floor(2^(p-1) ln 2) = 0,0,1,2,5,11,22 for p = 0..6.
// Otherwise the ceiling is k+1.
ARCQ_HD uint32_t ue8m0_scale(float t, float *s) {
  if (t == 0.0f) t = 1e-9f;
  const uint32_t b = f2u(t + 1e-9f);
  const int k = (int)(b >> 23) - 127;
  const uint32_t j = b & 0x7fffffu;
  const int mag = k > 0 ? k : -k - 1;              // floats just above k lie in the binade of mag
  const int p = mag > 0 ? 31 - __builtin_clz((unsigned)mag) : -1;
  const uint32_t jmax = p < 2 ? 0u : ((0x160b050201ull >> (8 * (p - 2))) & 0xffu);
  int e = k + (j > jmax ? 1 : 0);
  e = e < -127 ? -127 : (e > 127 ? 127 : e);
  *s = u2f((uint32_t)(e + 127) << 23);             // e = -127 would be a subnormal; unreachable (u >= 1e-9)
  return (uint32_t)(e + 127);
}

// quantize_e2m1 (model/quantize.py:14-22) of the exact quotient n: nearest of
// {0,.5,1,1.5,2,3,4,6} in magnitude; a tie goes to the lower VALUE (argmin keeps the first
// minimum on the ascending grid): toward zero for n > 0, away from zero for n < 0.
// Returns sign<<3 | magnitude index, zero always 0.
ARCQ_HD uint32_t e2m1_code(float n) {
  const uint32_t b = f2u(n);
  const uint32_t neg = b >> 31;
  const uint32_t u = (b & 0x7fffffffu) + neg;      // "u > bits(mid)"  <=>  |n| > mid, or == mid and n < 0
  uint32_t i = (u > 0x3e800000u) + (u > 0x3f400000u) + (u > 0x3fa00000u) + (u > 0x3fe00000u) +
               (u > 0x40200000u) + (u > 0x40600000u) + (u > 0x40a00000u);
  return i ? (i | (neg << 3)) : 0u;
}

ARCQ_HD float e2m1_value(uint32_t code) {
  // 0,.5,1,1.5,2,3,4,6: index i >= 2 is 2^((i>>1)-1) * (1 + (i&1)/2); 1 is the subnormal 0.5
  const uint32_t i = code & 7u;
  float v = i ? 0.5f : 0.0f;
  if (i >= 2u) v = u2f(((126u + (i >> 1)) << 23) | ((i & 1u) << 22));
  return (code & 8u) ? -v : v;
}

// ---------------------------------------------------------------------------------------------
// Fast encode for COARSE operands.
//
// When the value to encode has few significant bits (a bf16 activation with tensor scale 1: 8
// bits; its ARC residual y - q*s: the same grid), it is either exactly on a rounding boundary
// s*mid (a 7-bit number) or at least 2^-10 away from it in units of the block scale.  Then an
// approximate quotient is enough: w = y*r - 2^-13 with r within 2^-21 (relative) of 1/s lands
//   * strictly below the boundary for an exact tie  -> the lower value, as the reference's argmin,
//   * on the correct side of it for everything else,
// and w is never itself a tie, so the hardware's round-to-nearest-even FP4 conversion
// (v_cvt_scalef32_pk_fp4_f32) returns the reference's code.  Only "-0" needs cleaning up.
// tests/test_hostmath.py checks this exhaustively over every bf16 value, block scale and
// perturbed reciprocal, for main blocks and for residual blocks.
// ---------------------------------------------------------------------------------------------
constexpr float kCoarseNudge = 1.220703125e-4f;  // 2^-13

// Model of v_cvt_scalef32_pk_fp4_f32 with scale 1 for one element: round to nearest even,
// saturate at 6, keep the sign bit even on zero.
ARCQ_HD uint32_t e2m1_rne_hw_model(float w) {
  const uint32_t b = f2u(w);
  const uint32_t a = b & 0x7fffffffu;
  const uint32_t i = (a > 0x3e800000u) + (a >= 0x3f400000u) + (a > 0x3fa00000u) + (a >= 0x3fe00000u) +
                     (a > 0x40200000u) + (a >= 0x40600000u) + (a > 0x40a00000u);
  return i | ((b >> 31) << 3);
}

// 8 packed codes: a nibble 0x8 (negative zero) becomes 0x0, everything else is unchanged
ARCQ_HD uint32_t drop_negative_zeros(uint32_t x) {
  const uint32_t t = (x & 0x77777777u) + 0x77777777u;  // bit 3 of a nibble set iff its magnitude != 0
  return x & (t | 0x77777777u);
}

// amax/6 for a coarse amax (bf16-valued): correctly rounded quotient from the rounded reciprocal
// and one exact remainder (checked for all 128 significands in tests/test_hostmath.py)
ARCQ_HD float div6_coarse(float a) {
  const float r6 = 0x1.555556p-3f;
  const float q = a * r6;
  const float rem = __builtin_fmaf(-6.0f, q, a);
  return __builtin_fmaf(rem, r6, q);
}

// Correctly rounded sqrt(a) from an estimate s0 within 1 ulp of it (the hardware's v_sqrt_f32):
// the two neighbours' exact residuals decide.  a must be normal and finite (no rescaling here).
ARCQ_HD float sqrt_from_estimate(float a, float s0) {
  const float lo = u2f(f2u(s0) - 1u), hi = u2f(f2u(s0) + 1u);
  const float rlo = __builtin_fmaf(-lo, s0, a), rhi = __builtin_fmaf(-hi, s0, a);
  float s = rlo <= 0.0f ? lo : s0;
  s = rhi > 0.0f ? hi : s;
  return s;
}

// Correctly rounded 1/s from an estimate r0 within 1 ulp of it (v_rcp_f32): the fused
// Newton/remainder sequence of an IEEE fp32 division with numerator 1, without the range
// scaling -- s must lie well inside the normal range (2^-60 < s < 2^60).
ARCQ_HD float rcp_from_estimate(float s, float r0) {
  const float e = __builtin_fmaf(-s, r0, 1.0f);
  const float r = __builtin_fmaf(e, r0, r0);
  float q = r;
  q = __builtin_fmaf(__builtin_fmaf(-s, q, 1.0f), r, q);
  q = __builtin_fmaf(__builtin_fmaf(-s, q, 1.0f), r, q);
  // a significand of all ones is the one case where the iteration can settle one ulp low
  // (1/s lies just above a rounding midpoint); its reciprocal is 2^-(e+1) * (1 + 2^-23)
  if ((f2u(s) & 0x7fffffu) == 0x7fffffu) q = u2f(0x7f000000u - f2u(s));
  return q;
}

// Midpoint between grid magnitudes m and m+1 (m = 0..6): 0.25 0.75 1.25 1.75 2.5 3.5 5
ARCQ_HD float e2m1_midpoint(uint32_t m) {
  // as bits, without a branch: 0.25 and 0.75 are 0xc00000 apart, from 1.25 on the steps are 0x400000
  return u2f(m < 2u ? 0x3e800000u + m * 0x00c00000u : 0x3f200000u + m * 0x00400000u);
}

// The reference's code for y/s when two conversions of approximate quotients just below and just
// above it disagree (ca, cb: sign | magnitude, magnitudes one apart, midpoint t between them).
// With n = RN(y/s) the reference picks the larger magnitude iff n > t (y > 0) or n <= -t (y < 0):
// nearest value, ties toward the lower value (quantize.py:14-22).  B = t*s is exact in fp32 (3 x 4
// significant bits), and n > t <=> |y| > B, n <= -t <=> |y| >= B: the half-ulp of slack that the
// rounding of y/s allows around t is, scaled by s, less than the distance from B to its fp32
// neighbours, so no fp32 |y| other than B itself can fall inside it.
ARCQ_HD uint32_t e2m1_resolve(float y, float s, uint32_t ca, uint32_t cb) {
  const uint32_t ma = ca & 7u, mb = cb & 7u;
  const uint32_t m = ma < mb ? ma : mb;
  const float B = e2m1_midpoint(m) * s;
  const uint32_t neg = f2u(y) >> 31;
  const uint32_t au = (f2u(y) & 0x7fffffffu) + neg;  // negative y: |y| >= B  <=>  bits(|y|) + 1 > bits(B)
  const uint32_t mag = m + (au > f2u(B) ? 1u : 0u);
  return mag ? ((neg << 3) | mag) : 0u;
}

// a/6 for any a: the same three operations; exact for every significand while a and a*2^-25 are
// normal (checked exhaustively in tests/test_hostmath.py).  Below that the result may be off by an
// ulp, which no block scale can see: both scale formats map everything under 2^-40 to one value.
ARCQ_HD float div6_any(float a) { return div6_coarse(a); }

// x/g for a bf16-valued x: q + (x - g*q)*rg with q = x*rg and rg = RN(1/g)
ARCQ_HD float div_bf16_by(float x, float g, float rg) {
  const float q = x * rg;
  return __builtin_fmaf(__builtin_fmaf(-g, q, x), rg, q);
}

ARCQ_HD float nvfp4_scale_value(uint32_t byte) { return u2f((byte << 20) + ((127u - 9u) << 23)); }
ARCQ_HD float mxfp4_scale_value(uint32_t byte) { return u2f(byte << 23); }

}  // namespace arcq
#endif  // ARCQ_MATH_H_
