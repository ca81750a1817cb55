// arcq_quantize.hip -- reorder + block-FP4 quantize (+ ARC residual channels, + fused RMSNorm)
// for gfx950.  HBM-bound: one pass over the bf16 rows, coalesced 128-bit loads into LDS, the
// channel gather done out of LDS, 64-bit packed-code stores.
//
// One workgroup walks rows r = blockIdx.x, blockIdx.x + gridDim.x, ...; reorder_index (and
// gamma for the fused op) are staged in LDS once per workgroup.  A thread owns 16 consecutive
// reordered channels ("unit"): a whole NVFP4 block, or half an MXFP4 block whose other half
// sits in the neighbouring lane (one cross-lane max).
#include <hip/hip_runtime.h>
#include <type_traits>

#include "arcq_internal.h"
#include "arcq_math.h"
#include "arcq_swiglu.h"

namespace arcq {
namespace {

enum { MODE_X = 0, MODE_W = 1, MODE_NORM = 2, MODE_SWIGLU = 3 };

// Workgroup barrier that orders LDS traffic only.  __syncthreads() also drains outstanding
// global loads and stores (s_waitcnt vmcnt(0)), which would serialise the next row's prefetch
// and this row's stores with every barrier.
__device__ __forceinline__ void lds_barrier() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
  __builtin_amdgcn_s_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}
constexpr int kThreads = 256;

struct QuantParams {
  const uint16_t *x;      // bf16 [rows, K]
  const uint16_t *gamma;  // bf16 [K] (MODE_NORM)
  const uint16_t *up;     // bf16 rows of the "up" operand (MODE_SWIGLU; x holds the "gate" rows)
  int ldx;                // row stride of x (and up) in elements; K except for MODE_SWIGLU
  const int16_t *idx;     // [K]
  uint8_t *codes;         // [rows, (K+S)/2]
  uint8_t *scales;        // [rows, (K+S)/G]
  const float *d_gscale;  // optional device scalar
  float gscale;
  float eps;
  int rows, K, S;
  double inv_k;           // 1/K (MODE_NORM)
  // grouped launches (rows sorted by segment, e.g. tokens by expert): rows seg[e] .. seg[e+1]-1 take
  // reorder_index row e of idx [n_seg, K] and tensor scale d_gscale[e]
  const int *seg = nullptr;
  int n_seg = 0;
};

// Block scale from the block's amax: t = amax/6 (quantize.py:155 / :184), then the format's rounding.
template <int FMT>
__device__ __forceinline__ uint32_t block_scale(float amax, float *s) {
  const float t = amax / 6.0f;
  return FMT == ARCQ_FMT_NVFP4 ? ue4m3_scale(t, s) : ue8m0_scale(t, s);
}

// Quantizes the 16 values of one unit with block scale s.  Returns the packed codes (element 2j
// in the low nibble of byte j); if RESID, v[] is overwritten with the fp32 residual v - q*s
// (quantize.py:339).
template <int FMT, bool RESID>
__device__ __forceinline__ uint2 encode_unit(float (&v)[16], float s) {
  uint32_t w[2] = {0u, 0u};
  // MXFP4: s is a power of two, v * 2^-e is the exact quotient.  NVFP4: correctly rounded divide.
  const float inv = FMT == ARCQ_FMT_MXFP4 ? u2f((254u << 23) - f2u(s)) : 0.0f;
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    const float n = FMT == ARCQ_FMT_MXFP4 ? v[i] * inv : v[i] / s;
    const uint32_t c = e2m1_code(n);
    w[i >> 3] |= c << (4 * (i & 7));
    if (RESID) v[i] = v[i] - e2m1_value(c) * s;
  }
  return make_uint2(w[0], w[1]);
}

template <int FMT>
__device__ __forceinline__ float unit_amax(const float (&v)[16]) {
  float a = 0.0f;
#pragma unroll
  for (int i = 0; i < 16; ++i) a = fmaxf(a, fabsf(v[i]));
  if (FMT == ARCQ_FMT_MXFP4) a = fmaxf(a, __shfl_xor(a, 1));  // the other half of the 32-block
  return a;
}

// Codes and scale bytes are written once and not read again by these kernels: non-temporal stores keep
// them from displacing the rows still to be read (about a microsecond per 4096 x 4096 launch).  The scale
// bytes of a wave are 64-byte pieces of rows that are not multiples of 64 bytes long; written non-temporally
// they reach memory as more write requests than L2 would have merged them into (WRITE_SIZE +12 % on the
// fused-norm launch), and the launch is still 0.2 us faster than with ordinary scale stores.
typedef uint32_t v2u32 __attribute__((ext_vector_type(2)));
template <int FMT>
__device__ __forceinline__ void store_unit(uint8_t *crow, uint8_t *srow, int unit, uint2 packed, uint32_t sbyte) {
  const v2u32 pv = {packed.x, packed.y};
  __builtin_nontemporal_store(pv, reinterpret_cast<v2u32 *>(crow + unit * 8));
  if (FMT == ARCQ_FMT_NVFP4) {
    __builtin_nontemporal_store((uint8_t)sbyte, srow + unit);
  } else if ((unit & 1) == 0) {
    __builtin_nontemporal_store((uint8_t)sbyte, srow + (unit >> 1));
  }
}

template <int FMT, int MODE>
__global__ __launch_bounds__(kThreads) void quantize_rows_kernel(QuantParams p) {
  extern __shared__ uint4 smem[];
  const int K = p.K, S = p.S, Kp = K + S;
  constexpr int G = FMT == ARCQ_FMT_NVFP4 ? 16 : 32;
  uint16_t *row = reinterpret_cast<uint16_t *>(smem);
  const int16_t *lidx = reinterpret_cast<const int16_t *>(row + K);
  const uint16_t *lgam = row + 2 * K;
  double *red = reinterpret_cast<double *>(row + 3 * K);  // MODE_NORM: kThreads/64 partial sums

  const int tid = threadIdx.x;
  const int nvec = K >> 3;  // 16-byte chunks per row
  for (int c = tid; c < nvec; c += kThreads) {
    reinterpret_cast<uint4 *>(row + K)[c] = reinterpret_cast<const uint4 *>(p.idx)[c];
    if (MODE == MODE_NORM) reinterpret_cast<uint4 *>(row + 2 * K)[c] = reinterpret_cast<const uint4 *>(p.gamma)[c];
  }
  const float g = p.d_gscale ? *p.d_gscale : p.gscale;
  const bool unit_scale = g == 1.0f;
  const int nunits = K >> 4;
  const int tail0 = (K - S) >> 4;  // first unit whose channels are among the select_num outliers

  for (int r = blockIdx.x; r < p.rows; r += gridDim.x) {
    lds_barrier();  // the previous row has been consumed (first pass: nothing pending)
    const uint4 *src = reinterpret_cast<const uint4 *>(p.x + (size_t)r * K);
    double ss = 0.0;
    for (int c = tid; c < nvec; c += kThreads) {
      const uint4 q = src[c];
      reinterpret_cast<uint4 *>(row)[c] = q;
      if (MODE == MODE_NORM) {
        const uint32_t w[4] = {q.x, q.y, q.z, q.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const float lo = u2f(w[i] << 16), hi = u2f(w[i] & 0xffff0000u);
          ss += (double)(lo * lo);  // a bf16 square is exact in fp32
          ss += (double)(hi * hi);
        }
      }
    }
    float rstd = 1.0f;
    if (MODE == MODE_NORM) {
#pragma unroll
      for (int o = 32; o > 0; o >>= 1) ss += __shfl_xor(ss, o);
      if ((tid & 63) == 0) red[tid >> 6] = ss;
      lds_barrier();
      double tot = 0.0;
#pragma unroll
      for (int w = 0; w < kThreads / 64; ++w) tot += red[w];
      const float var = (float)(tot / (double)K);
      rstd = 1.0f / sqrtf(var + p.eps);
    } else {
      lds_barrier();
    }

    uint8_t *crow = p.codes + (size_t)r * (Kp >> 1);
    uint8_t *srow = p.scales + (size_t)r * (Kp / G);
    for (int u = tid; u < nunits; u += kThreads) {
      const uint4 i0 = reinterpret_cast<const uint4 *>(lidx)[2 * u];
      const uint4 i1 = reinterpret_cast<const uint4 *>(lidx)[2 * u + 1];
      const uint32_t iw[8] = {i0.x, i0.y, i0.z, i0.w, i1.x, i1.y, i1.z, i1.w};
      float v[16];
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const uint32_t ch = (iw[i >> 1] >> (16 * (i & 1))) & 0xffffu;
        float f = bf16_bits_to_f32(row[ch]);
        if (MODE == MODE_NORM) {
          const float h = bf16_bits_to_f32(f32_to_bf16_bits(f * rstd));
          f = bf16_bits_to_f32(f32_to_bf16_bits(bf16_bits_to_f32(lgam[ch]) * h));
        }
        v[i] = unit_scale ? f : f / g;
      }
      float s;
      uint32_t sb = block_scale<FMT>(unit_amax<FMT>(v), &s);
      if (MODE == MODE_W || u < tail0) {
        const uint2 pk = encode_unit<FMT, false>(v, s);
        store_unit<FMT>(crow, srow, u, pk, sb);
        if (MODE == MODE_W && u >= tail0) store_unit<FMT>(crow, srow, nunits + (u - tail0), pk, sb);
      } else {
        uint2 pk = encode_unit<FMT, true>(v, s);
        store_unit<FMT>(crow, srow, u, pk, sb);
        sb = block_scale<FMT>(unit_amax<FMT>(v), &s);
        pk = encode_unit<FMT, false>(v, s);
        store_unit<FMT>(crow, srow, nunits + (u - tail0), pk, sb);
      }
    }
  }
}

// ---------------------------------------------------------------------------------------------
// Fast kernels for tensor scale 1 (the fused RMSNorm op, MXFP4, and NVFP4 callers that pass
// global_scale = 1): every operand of the encoder is then exactly a bf16 value or the residual
// of one, and the coarse encode of arcq_math.h applies -- one fma and half a hardware FP4
// conversion per element instead of an IEEE division and seven compares.
//
// One workgroup per row at a time, one thread per 16-channel unit (blockDim = K/16 rounded up
// to whole waves), so everything that depends only on the channel -- gather addresses, gamma --
// lives in registers across rows:
//   pass 1 (natural order)  global 2 x 128-bit per thread (next row prefetched), [sum of squares
//                           in fp64, normalise, gamma] -> packed bf16 into the LDS row
//   pass 2 (reordered)      16 ds_read_u16_d16_hi into registers whose low halves stay zero
//                           (a bf16 in the high half IS the fp32), amax, scale, encode, 64-bit store
// ---------------------------------------------------------------------------------------------
// 16 coarse values -> 16 codes with block scale s (r ~ 1/s)
__device__ __forceinline__ uint2 encode_unit_coarse(const float (&y)[16], float r) {
  float w[16];
#pragma unroll
  for (int i = 0; i < 16; ++i) w[i] = __builtin_fmaf(y[i], r, -kCoarseNudge);
  uint32_t a = 0u, b = 0u;
  a = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(a, w[0], w[1], 1.0f, 0);
  a = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(a, w[2], w[3], 1.0f, 1);
  a = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(a, w[4], w[5], 1.0f, 2);
  a = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(a, w[6], w[7], 1.0f, 3);
  b = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(b, w[8], w[9], 1.0f, 0);
  b = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(b, w[10], w[11], 1.0f, 1);
  b = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(b, w[12], w[13], 1.0f, 2);
  b = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(b, w[14], w[15], 1.0f, 3);
  return make_uint2(drop_negative_zeros(a), drop_negative_zeros(b));
}

// 16 codes -> their e2m1 values (hardware FP4 -> fp32 convert, exact)
__device__ __forceinline__ void decode_unit(uint2 pk, float (&q)[16]) {
  typedef float v2f __attribute__((ext_vector_type(2)));
#define ARCQ_DEC(j, word, sel)                                                      \
  {                                                                                 \
    const v2f t = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(word, 1.0f, sel);        \
    q[2 * (j)] = t.x;                                                               \
    q[2 * (j) + 1] = t.y;                                                           \
  }
  ARCQ_DEC(0, pk.x, 0) ARCQ_DEC(1, pk.x, 1) ARCQ_DEC(2, pk.x, 2) ARCQ_DEC(3, pk.x, 3)
  ARCQ_DEC(4, pk.y, 0) ARCQ_DEC(5, pk.y, 1) ARCQ_DEC(6, pk.y, 2) ARCQ_DEC(7, pk.y, 3)
#undef ARCQ_DEC
}

template <int FMT>
__device__ __forceinline__ float unit_amax3(const float (&v)[16]) {
  float a = fmaxf(fabsf(v[0]), fabsf(v[1]));
#pragma unroll
  for (int i = 2; i < 16; i += 2) a = fmaxf(fmaxf(a, fabsf(v[i])), fabsf(v[i + 1]));  // v_max3_f32
  if (FMT == ARCQ_FMT_MXFP4) a = fmaxf(a, __shfl_xor(a, 1));
  return a;
}

// reciprocal of a block scale, within 1 ulp (NVFP4: v_rcp_f32) or exact (MXFP4: power of two)
template <int FMT>
__device__ __forceinline__ float scale_rcp(float s) {
  return FMT == ARCQ_FMT_NVFP4 ? __builtin_amdgcn_rcpf(s) : u2f((254u << 23) - f2u(s));
}

// pack_bf16_rne(h_even * gamma_even, h_odd * gamma_odd) for four registers of bf16 pairs.  Written as
// one block because the compiler only reaches the two-operand v_dot2c_f32_bf16 (a zeroed accumulator
// register per product, then wait states in front of every conversion).  A dot instruction's result
// may be read by another kind of VALU instruction only three issue slots later: each conversion
// below has at least three instructions between it and the later of its two products, and nothing
// outside the block can come closer than that to a product either.  The compiler does not know what
// the block's instructions are, so the block also opens with the two wait states that cover every
// forwarding hazard between a VALU instruction in front of it and a dot reading that result.
__device__ __forceinline__ void gamma_mul_pack4(const uint32_t *h, const uint32_t *glo, const uint32_t *ghi, uint32_t *out) {
  float a0, a1, a2, a3, b0, b1, b2, b3;
  asm("s_nop 1\n\t"
      "v_dot2_f32_bf16 %4, %12, %16, 0\n\t"
      "v_dot2_f32_bf16 %8, %12, %20, 0\n\t"
      "v_dot2_f32_bf16 %5, %13, %17, 0\n\t"
      "v_dot2_f32_bf16 %9, %13, %21, 0\n\t"
      "v_dot2_f32_bf16 %6, %14, %18, 0\n\t"
      "v_dot2_f32_bf16 %10, %14, %22, 0\n\t"
      "v_dot2_f32_bf16 %7, %15, %19, 0\n\t"
      "v_dot2_f32_bf16 %11, %15, %23, 0\n\t"
      "v_cvt_pk_bf16_f32 %0, %4, %8\n\t"
      "v_cvt_pk_bf16_f32 %1, %5, %9\n\t"
      "v_cvt_pk_bf16_f32 %2, %6, %10\n\t"
      "v_cvt_pk_bf16_f32 %3, %7, %11"
      : "=&v"(out[0]), "=&v"(out[1]), "=&v"(out[2]), "=&v"(out[3]), "=&v"(a0), "=&v"(a1), "=&v"(a2), "=&v"(a3),
        "=&v"(b0), "=&v"(b1), "=&v"(b2), "=&v"(b3)
      : "v"(h[0]), "v"(h[1]), "v"(h[2]), "v"(h[3]), "v"(glo[0]), "v"(glo[1]), "v"(glo[2]), "v"(glo[3]), "v"(ghi[0]),
        "v"(ghi[1]), "v"(ghi[2]), "v"(ghi[3]));
}

// Sum of one double per lane over the 64 lanes of a wave, in DPP register moves (no LDS round
// trips): prefix sums inside each row of 16 lanes, then the row totals are passed along.
// The total ends up in lane 63.
__device__ __forceinline__ double wave_sum_to_lane63(double v) {
#define ARCQ_DPP_STEP_BC(ctrl)                                                                \
  {                                                                                           \
    const uint64_t b = __builtin_bit_cast(uint64_t, v);                                       \
    const uint32_t lo = __builtin_amdgcn_update_dpp(0u, (uint32_t)b, ctrl, 0xf, 0xf, true);   \
    const uint32_t hi = __builtin_amdgcn_update_dpp(0u, (uint32_t)(b >> 32), ctrl, 0xf, 0xf, true); \
    v += __builtin_bit_cast(double, ((uint64_t)hi << 32) | lo);                               \
  }
#define ARCQ_DPP_STEP(ctrl, row_mask)                                                                     \
  {                                                                                                        \
    const uint64_t b = __builtin_bit_cast(uint64_t, v);                                                   \
    const uint32_t lo = __builtin_amdgcn_update_dpp(0u, (uint32_t)b, ctrl, row_mask, 0xf, false);         \
    const uint32_t hi = __builtin_amdgcn_update_dpp(0u, (uint32_t)(b >> 32), ctrl, row_mask, 0xf, false); \
    v += __builtin_bit_cast(double, ((uint64_t)hi << 32) | lo);                                           \
  }
  ARCQ_DPP_STEP_BC(0x111)    // row_shr:1  (lanes shifted in from outside the row read as 0)
  ARCQ_DPP_STEP_BC(0x112)    // row_shr:2
  ARCQ_DPP_STEP_BC(0x114)    // row_shr:4
  ARCQ_DPP_STEP_BC(0x118)    // row_shr:8  -> lane 15 of each row holds the row total
  ARCQ_DPP_STEP(0x142, 0xa)  // row_bcast:15 into rows 1 and 3
  ARCQ_DPP_STEP(0x143, 0xc)  // row_bcast:31 into rows 2 and 3 -> lane 63 holds the wave total
#undef ARCQ_DPP_STEP
#undef ARCQ_DPP_STEP_BC
  return v;
}

// Two-sided encode for operands that are not coarse (tensor scale not a power of two): the block
// is converted twice with the hardware RNE convert, from y*r*(1+2^-20) and y*r*(1-2^-20) with
// r ~ 1/s.  The true quotient y/s, its fp32 rounding and every point where the reference's decision
// changes differ by far less than 2^-20 relatively, so where the two conversions agree no decision
// point lies between them and both equal the reference's code.  Where they differ (a few elements
// in 10^4; exact ties are built into the NVFP4 tensor scale max/2688 = max/(2^7*3*7)) e2m1_resolve
// decides that element from one exact product.
__device__ __forceinline__ uint32_t resolve_word(float v0, float v1, float v2, float v3, float v4, float v5, float v6,
                                                 float v7, float s, uint32_t a, uint32_t b) {
  uint32_t out = drop_negative_zeros(a);
  uint32_t d = a ^ b;
  while (d) {  // one pass per differing element of this lane
    const int nib = __builtin_ctz(d) >> 2;
    const float a0 = (nib & 1) ? v1 : v0, a1 = (nib & 1) ? v3 : v2;  // the values are passed one by one
    const float a2 = (nib & 1) ? v5 : v4, a3 = (nib & 1) ? v7 : v6;  // so that they stay in registers
    const float b0 = (nib & 2) ? a1 : a0, b1 = (nib & 2) ? a3 : a2;
    const float yi = (nib & 4) ? b1 : b0;
    const uint32_t sh = 4u * (uint32_t)nib;
    const uint32_t c = e2m1_resolve(yi, s, (a >> sh) & 15u, (b >> sh) & 15u);
    out = (out & ~(15u << sh)) | (c << sh);
    d &= ~(15u << sh);
  }
  return out;
}

__device__ __forceinline__ uint2 encode_unit_two_sided(const float (&y)[16], float s, float r) {
  const float ra = r * 0x1.00001p+0f, rb = r * 0x1.ffffep-1f;
  uint32_t a0 = 0u, a1 = 0u, b0 = 0u, b1 = 0u;
#define ARCQ_ENC2(dst, rr, i, sel) \
  dst = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(dst, y[i] * rr, y[i + 1] * rr, 1.0f, sel);
  ARCQ_ENC2(a0, ra, 0, 0) ARCQ_ENC2(a0, ra, 2, 1) ARCQ_ENC2(a0, ra, 4, 2) ARCQ_ENC2(a0, ra, 6, 3)
  ARCQ_ENC2(a1, ra, 8, 0) ARCQ_ENC2(a1, ra, 10, 1) ARCQ_ENC2(a1, ra, 12, 2) ARCQ_ENC2(a1, ra, 14, 3)
  ARCQ_ENC2(b0, rb, 0, 0) ARCQ_ENC2(b0, rb, 2, 1) ARCQ_ENC2(b0, rb, 4, 2) ARCQ_ENC2(b0, rb, 6, 3)
  ARCQ_ENC2(b1, rb, 8, 0) ARCQ_ENC2(b1, rb, 10, 1) ARCQ_ENC2(b1, rb, 12, 2) ARCQ_ENC2(b1, rb, 14, 3)
#undef ARCQ_ENC2
  return make_uint2(resolve_word(y[0], y[1], y[2], y[3], y[4], y[5], y[6], y[7], s, a0, b0),
                    resolve_word(y[8], y[9], y[10], y[11], y[12], y[13], y[14], y[15], s, a1, b1));
}

// The same for a unit under a tensor scale g whose values y = x / g have not been formed: the two conversions start
// from the raw bf16 x with R ~ 1 / (g * s) (R = RN(rg * r)); an element on which they differ gets its exact
// y = RN(x / g) and goes through e2m1_resolve as above.  (tests/test_hostmath.py sweeps this against the reference's
// code of RN(RN(x/g) / s) for every bf16 x, block scale, reciprocal within an ulp and tensor scale max / 2688.)
__device__ __forceinline__ uint32_t resolve_word_x(float v0, float v1, float v2, float v3, float v4, float v5, float v6,
                                                   float v7, float g, float rg, float s, uint32_t a, uint32_t b) {
  uint32_t out = drop_negative_zeros(a);
  uint32_t d = a ^ b;
  while (d) {
    const int nib = __builtin_ctz(d) >> 2;
    const float a0 = (nib & 1) ? v1 : v0, a1 = (nib & 1) ? v3 : v2;
    const float a2 = (nib & 1) ? v5 : v4, a3 = (nib & 1) ? v7 : v6;
    const float b0 = (nib & 2) ? a1 : a0, b1 = (nib & 2) ? a3 : a2;
    const float xi = (nib & 4) ? b1 : b0;
    const uint32_t sh = 4u * (uint32_t)nib;
    const uint32_t c = e2m1_resolve(div_bf16_by(xi, g, rg), s, (a >> sh) & 15u, (b >> sh) & 15u);
    out = (out & ~(15u << sh)) | (c << sh);
    d &= ~(15u << sh);
  }
  return out;
}

__device__ __forceinline__ uint2 encode_unit_two_sided_x(const float (&x)[16], float g, float rg, float s, float R) {
  const float ra = R * 0x1.00001p+0f, rb = R * 0x1.ffffep-1f;
  uint32_t a0 = 0u, a1 = 0u, b0 = 0u, b1 = 0u;
#define ARCQ_ENC2(dst, rr, i, sel) \
  dst = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(dst, x[i] * rr, x[i + 1] * rr, 1.0f, sel);
  ARCQ_ENC2(a0, ra, 0, 0) ARCQ_ENC2(a0, ra, 2, 1) ARCQ_ENC2(a0, ra, 4, 2) ARCQ_ENC2(a0, ra, 6, 3)
  ARCQ_ENC2(a1, ra, 8, 0) ARCQ_ENC2(a1, ra, 10, 1) ARCQ_ENC2(a1, ra, 12, 2) ARCQ_ENC2(a1, ra, 14, 3)
  ARCQ_ENC2(b0, rb, 0, 0) ARCQ_ENC2(b0, rb, 2, 1) ARCQ_ENC2(b0, rb, 4, 2) ARCQ_ENC2(b0, rb, 6, 3)
  ARCQ_ENC2(b1, rb, 8, 0) ARCQ_ENC2(b1, rb, 10, 1) ARCQ_ENC2(b1, rb, 12, 2) ARCQ_ENC2(b1, rb, 14, 3)
#undef ARCQ_ENC2
  return make_uint2(resolve_word_x(x[0], x[1], x[2], x[3], x[4], x[5], x[6], x[7], g, rg, s, a0, b0),
                    resolve_word_x(x[8], x[9], x[10], x[11], x[12], x[13], x[14], x[15], g, rg, s, a1, b1));
}

// amax values for which the division-free arithmetic above is not trusted (results that
// underflow or overflow on the way): everything but zero and the comfortable normal range
__device__ __forceinline__ bool amax_needs_exact(float a) {
  return !(a == 0.0f || (a >= 0x1p-100f && a <= 0x1p+120f));
}

// One unit with IEEE divisions throughout, from the raw bf16 operands: what the reference's
// arithmetic prescribes literally (quantize.py:154-161, 330, 337-340).
template <int FMT, bool WITH_RESID>
__device__ __forceinline__ void unit_exact(const uint32_t (&yv)[16], float g, uint2 *pk, uint32_t *sb, uint2 *pk2,
                                           uint32_t *sb2) {
  float v[16];
#pragma unroll
  for (int i = 0; i < 16; ++i) v[i] = u2f(yv[i]) / g;
  float s;
  *sb = block_scale<FMT>(unit_amax<FMT>(v), &s);
  if (!WITH_RESID) {
    *pk = encode_unit<FMT, false>(v, s);
  } else {
    *pk = encode_unit<FMT, true>(v, s);
    *sb2 = block_scale<FMT>(unit_amax<FMT>(v), &s);
    *pk2 = encode_unit<FMT, false>(v, s);
  }
}

// One unit's arithmetic, shared by the row kernels below: yv holds the unit's 16 gathered bf16 values as fp32
// bits (all zero in a lane without a unit).  Returns codes and scale byte of the unit (pk, sb) and, for a unit
// among the last select_num channels of an activation (tail), those of its residual block (pk2, sb2; for
// weights and elsewhere a copy of pk, sb).  Every lane of the wave must call it (MXFP4 exchanges the maxima
// of the two halves of a 32-block between neighbouring lanes).
template <int FMT, int MODE, bool SCALED>
__device__ __forceinline__ void quantize_unit(const uint32_t (&yv)[16], bool active, bool tail, float g, float rg, bool g_odd,
                                              bool coarse, uint2 &pk, uint32_t &sb, uint2 &pk2, uint32_t &sb2) {
  float y[16];
#pragma unroll
  for (int i = 0; i < 16; ++i) y[i] = u2f(yv[i]);
  if (SCALED) {
    // A tensor scale that is not a power of two: one division per unit for the main block.  RN(x / g) is monotone in
    // |x|, so the block maximum of y is the quotient of the block maximum of x; the codes come straight from x
    // (encode_unit_two_sided_x).  Only a wave that holds residual units forms y = x / g itself, for the residual.
    if (!coarse) {
      float s;
      const float amax = div_bf16_by(unit_amax3<FMT>(y), g, rg);
      const float t = div6_any(amax);
      sb = FMT == ARCQ_FMT_NVFP4 ? ue4m3_scale(t, &s) : ue8m0_scale(t, &s);
      pk = encode_unit_two_sided_x(y, g, rg, s, rg * scale_rcp<FMT>(s));
      bool redo = amax_needs_exact(amax) || g_odd;
      pk2 = pk;
      sb2 = sb;
      const bool wave_has_tail = MODE != MODE_W && __builtin_amdgcn_ballot_w64(tail) != 0ull;
      if (wave_has_tail) {
        float e[16];
        decode_unit(pk, e);
#pragma unroll
        for (int i = 0; i < 16; ++i) e[i] = __builtin_fmaf(-e[i], s, div_bf16_by(y[i], g, rg));  // the fp32 residual y - q*s
        float s2;
        const float amax2 = unit_amax3<FMT>(e);
        const float t2 = div6_any(amax2);
        const uint32_t sbr = FMT == ARCQ_FMT_NVFP4 ? ue4m3_scale(t2, &s2) : ue8m0_scale(t2, &s2);
        const uint2 pkr = encode_unit_two_sided(e, s2, scale_rcp<FMT>(s2));
        if (tail) {
          pk2 = pkr;
          sb2 = sbr;
          redo = amax_needs_exact(amax2) || redo;
        }
      }
      if (FMT == ARCQ_FMT_MXFP4) redo = __shfl_xor((int)redo, 1) != 0 || redo;  // both halves of a 32-block
      if (redo && active) {
        if (MODE != MODE_W && tail) {
          unit_exact<FMT, true>(yv, g, &pk, &sb, &pk2, &sb2);
        } else {
          unit_exact<FMT, false>(yv, g, &pk, &sb, &pk2, &sb2);
          pk2 = pk;
          sb2 = sb;
        }
      }
      return;
    }
#pragma unroll
    for (int i = 0; i < 16; ++i) y[i] = div_bf16_by(y[i], g, rg);
  }
  float s;
  const float amax = unit_amax3<FMT>(y);
  const float t = div6_any(amax);
  sb = FMT == ARCQ_FMT_NVFP4 ? ue4m3_scale(t, &s) : ue8m0_scale(t, &s);
  bool redo = false;  // SCALED only: this unit needs unit_exact
  if (coarse) {
    pk = encode_unit_coarse(y, scale_rcp<FMT>(s));
    if (SCALED) redo = amax_needs_exact(amax) || g_odd;
  } else {
    pk = encode_unit_two_sided(y, s, scale_rcp<FMT>(s));
    redo = amax_needs_exact(amax) || g_odd;
  }
  pk2 = pk;
  sb2 = sb;
  if (MODE != MODE_W && tail) {
    float e[16];
    decode_unit(pk, e);
#pragma unroll
    for (int i = 0; i < 16; ++i) e[i] = __builtin_fmaf(-e[i], s, y[i]);  // q*s is exact: the fp32 residual y - q*s
    float s2;
    const float amax2 = unit_amax3<FMT>(e);
    const float t2 = div6_any(amax2);
    sb2 = FMT == ARCQ_FMT_NVFP4 ? ue4m3_scale(t2, &s2) : ue8m0_scale(t2, &s2);
    if (coarse) {
      pk2 = encode_unit_coarse(e, scale_rcp<FMT>(s2));
      if (SCALED) redo = amax_needs_exact(amax2) || redo;
    } else {
      pk2 = encode_unit_two_sided(e, s2, scale_rcp<FMT>(s2));
      redo = amax_needs_exact(amax2) || redo;
    }
  }
  if (SCALED && FMT == ARCQ_FMT_MXFP4) redo = __shfl_xor((int)redo, 1) != 0 || redo;  // both halves of a 32-block
  if (SCALED && redo && active) {
    if (MODE != MODE_W && tail) {
      unit_exact<FMT, true>(yv, g, &pk, &sb, &pk2, &sb2);
    } else {
      unit_exact<FMT, false>(yv, g, &pk, &sb, &pk2, &sb2);
      pk2 = pk;
      sb2 = sb;
    }
  }
}

template <int FMT, int MODE, bool SCALED, bool GROUPED = false>
__global__ __launch_bounds__(1024) void quantize_rows_unit_kernel(QuantParams p) {
  extern __shared__ uint4 smem[];
  constexpr int G = FMT == ARCQ_FMT_NVFP4 ? 16 : 32;
  const int K = p.K, S = p.S, Kp = K + S;
  uint16_t *row = reinterpret_cast<uint16_t *>(smem);
  double *red = reinterpret_cast<double *>(row + K);  // one partial sum per wave
  const int nwaves = (blockDim.x + 63) >> 6;
  // Thread -> unit mapping rotated by whole waves per workgroup.  The waves that own the last
  // select_num channels also encode the residual; a workgroup's wave i always lands on SIMD i, so
  // without the rotation one SIMD of every CU would carry all of that extra work.
  int tid = threadIdx.x + 64 * (int)(blockIdx.x % (unsigned)nwaves);
  if (tid >= (int)blockDim.x) tid -= blockDim.x;
  const int nunits = K >> 4;                           // == number of working threads
  const bool active = tid < nunits;
  const int tail0 = (K - S) >> 4;
  const bool k_pow2 = (K & (K - 1)) == 0;
  const double inv_k = p.inv_k;
  // SCALED: x32 = x / g (quantize.py:330) as q + (x - g*q)*rg with q = x*rg, rg = RN(1/g): the
  // correctly rounded quotient for every bf16 x (checked exhaustively on the host).  A tensor scale
  // outside 2^-60..2^60 in magnitude sends every unit through unit_exact.
  // GROUPED: the scale (and the channel order below) belong to the segment of the row and are
  // replaced when the workgroup's rows enter another segment
  float g = SCALED ? (p.d_gscale ? *p.d_gscale : p.gscale) : 1.0f;
  float rg = SCALED ? 1.0f / g : 1.0f;
  bool g_odd = SCALED && !(fabsf(g) >= 0x1p-60f && fabsf(g) <= 0x1p+60f);
  // a power-of-two tensor scale leaves bf16 operands bf16-valued: the coarse encode applies (and
  // such operands sit on the grid's ties far too often for the two-sided test to pay)
  bool coarse = !SCALED || (f2u(g) & 0x7fffffu) == 0u;
  // var + eps >= eps: with eps comfortably normal the square root needs no range scaling
  const bool eps_normal = p.eps >= 0x1p-90f;

  int r = blockIdx.x;
  const size_t ldx = MODE == MODE_SWIGLU ? (size_t)p.ldx : (size_t)K;
  uint4 q0 = make_uint4(0, 0, 0, 0), q1 = q0, u0 = q0, u1 = q0;
  if (r < p.rows && active) {  // first row in flight before anything that has to wait for memory
    const uint4 *src = reinterpret_cast<const uint4 *>(p.x + (size_t)r * ldx);
    q0 = src[tid];
    q1 = src[tid + nunits];
    if (MODE == MODE_SWIGLU) {
      const uint4 *usrc = reinterpret_cast<const uint4 *>(p.up + (size_t)r * ldx);
      u0 = usrc[tid];
      u1 = usrc[tid + nunits];
    }
  }

  // channel-only state, loaded once
  uint32_t addr[16];
  uint32_t glo[8], ghi[8];
  auto gather_addresses = [&](const int16_t *idx) {
    const uint32_t base = (uint32_t)reinterpret_cast<uintptr_t>(row);
    uint4 i0 = make_uint4(0, 0, 0, 0), i1 = i0;
    if (active) {
      i0 = reinterpret_cast<const uint4 *>(idx)[2 * tid];
      i1 = reinterpret_cast<const uint4 *>(idx)[2 * tid + 1];
    }
    const uint32_t iw[8] = {i0.x, i0.y, i0.z, i0.w, i1.x, i1.y, i1.z, i1.w};
#pragma unroll
    for (int i = 0; i < 16; ++i) addr[i] = base + 2u * ((iw[i >> 1] >> (16 * (i & 1))) & 0xffffu);
  };
  if (!GROUPED) gather_addresses(p.idx);
  int seg_cur = -1, seg_end = 0;  // GROUPED: rows below seg_end belong to segment seg_cur (or to an earlier one)
  {
    if (MODE == MODE_NORM) {
      uint4 g0 = make_uint4(0, 0, 0, 0), g1 = g0;
      if (active) {
        g0 = reinterpret_cast<const uint4 *>(p.gamma)[tid];
        g1 = reinterpret_cast<const uint4 *>(p.gamma)[tid + nunits];
      }
      const uint32_t gw[8] = {g0.x, g0.y, g0.z, g0.w, g1.x, g1.y, g1.z, g1.w};
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        glo[j] = gw[j] & 0xffffu;       // (gamma_even, 0): v_dot2_f32_bf16 with it = gamma_even * h_even, exact
        ghi[j] = gw[j] & 0xffff0000u;   // (0, gamma_odd)
      }
    }
  }
  uint32_t yv[16];
#pragma unroll
  for (int i = 0; i < 16; ++i) yv[i] = 0u;  // low halves stay zero: only d16_hi loads write these

  for (; r < p.rows; r += gridDim.x) {
    if (GROUPED && r >= seg_end) {  // workgroup-uniform: the rows are sorted, so this happens once per segment at most
      while (seg_cur + 1 < p.n_seg && r >= seg_end) {
        ++seg_cur;
        seg_end = p.seg[seg_cur + 1];
      }
      if (r >= seg_end) break;  // rows behind the last segment belong to nobody
      gather_addresses(p.idx + (size_t)seg_cur * K);
      if (SCALED) {
        g = p.d_gscale[seg_cur];
        rg = 1.0f / g;
        g_odd = !(fabsf(g) >= 0x1p-60f && fabsf(g) <= 0x1p+60f);
        coarse = (f2u(g) & 0x7fffffu) == 0u;
      }
    }
    uint4 n0, n1, un0, un1;  // left undefined past the last row: nothing reads them then
    if (r + (int)gridDim.x < p.rows && active) {  // prefetch the next row of this workgroup
      const uint4 *src = reinterpret_cast<const uint4 *>(p.x + (size_t)(r + gridDim.x) * ldx);
      n0 = src[tid];
      n1 = src[tid + nunits];
      if (MODE == MODE_SWIGLU) {
        const uint4 *usrc = reinterpret_cast<const uint4 *>(p.up + (size_t)(r + gridDim.x) * ldx);
        un0 = usrc[tid];
        un1 = usrc[tid + nunits];
      }
    }
    if (MODE == MODE_NORM) {
      const uint32_t xw[8] = {q0.x, q0.y, q0.z, q0.w, q1.x, q1.y, q1.z, q1.w};
      float f[16];
      double ss = 0.0;
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        f[2 * j] = u2f(xw[j] << 16);
        f[2 * j + 1] = u2f(xw[j] & 0xffff0000u);
        const double d0 = (double)f[2 * j], d1 = (double)f[2 * j + 1];
        ss = __builtin_fma(d0, d0, ss);  // exact squares, fp64 accumulation
        ss = __builtin_fma(d1, d1, ss);
      }
      ss = wave_sum_to_lane63(ss);
      if ((tid & 63) == 63) red[tid >> 6] = ss;
      lds_barrier();  // partial sums visible; the previous row's gathers are over
      double tot = 0.0, tot1 = 0.0;
      int w = 0;
      for (; w + 4 <= nwaves; w += 4) {  // two independent chains, 16-byte LDS reads
        const double2 a = *reinterpret_cast<const double2 *>(red + w);
        const double2 b = *reinterpret_cast<const double2 *>(red + w + 2);
        tot += a.x;
        tot1 += a.y;
        tot += b.x;
        tot1 += b.y;
      }
      for (; w < nwaves; ++w) tot += red[w];
      tot += tot1;
      // mean = tot / K, exactly: a power-of-two K is a scaling, anything else an IEEE division
      const float var = k_pow2 ? (float)(tot * inv_k) : (float)(tot / (double)K);
      const float a = var + p.eps;
      float rstd;
      if (eps_normal) {
        // 1.0f / sqrtf(a) with both roundings, from the hardware estimates
        const float sq = sqrt_from_estimate(a, __builtin_amdgcn_sqrtf(a));
        rstd = rcp_from_estimate(sq, __builtin_amdgcn_rcpf(sq));
        if (!(a < __builtin_inff())) rstd = a != a ? a : 0.0f;  // 1/sqrt(inf) = 0, NaN stays NaN
      } else {
        rstd = 1.0f / sqrtf(a);
      }
      uint32_t hw[8], yw[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) hw[j] = pack_bf16_rne(f[2 * j] * rstd, f[2 * j + 1] * rstd);
      gamma_mul_pack4(hw, glo, ghi, yw);
      gamma_mul_pack4(hw + 4, glo + 4, ghi + 4, yw + 4);
      if (active) {
        reinterpret_cast<uint4 *>(row)[tid] = make_uint4(yw[0], yw[1], yw[2], yw[3]);
        reinterpret_cast<uint4 *>(row)[tid + nunits] = make_uint4(yw[4], yw[5], yw[6], yw[7]);
      }
    } else if (MODE == MODE_SWIGLU) {
      const uint4 t0 = make_uint4(swiglu_pair(q0.x, u0.x), swiglu_pair(q0.y, u0.y), swiglu_pair(q0.z, u0.z),
                                  swiglu_pair(q0.w, u0.w));
      const uint4 t1 = make_uint4(swiglu_pair(q1.x, u1.x), swiglu_pair(q1.y, u1.y), swiglu_pair(q1.z, u1.z),
                                  swiglu_pair(q1.w, u1.w));
      lds_barrier();  // the previous row's gathers are over
      if (active) {
        reinterpret_cast<uint4 *>(row)[tid] = t0;
        reinterpret_cast<uint4 *>(row)[tid + nunits] = t1;
      }
    } else {
      lds_barrier();  // the previous row's gathers are over
      if (active) {
        reinterpret_cast<uint4 *>(row)[tid] = q0;
        reinterpret_cast<uint4 *>(row)[tid + nunits] = q1;
      }
    }
    lds_barrier();

    if (active) {
#pragma unroll
      for (int i = 0; i < 16; ++i) asm volatile("ds_read_u16_d16_hi %0, %1" : "+v"(yv[i]) : "v"(addr[i]) : "memory");
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    }
    uint8_t *crow = p.codes + (size_t)r * (Kp >> 1);
    uint8_t *srow = p.scales + (size_t)r * (Kp / G);
    const bool tail = active && tid >= tail0;
    uint2 pk, pk2;
    uint32_t sb, sb2;
    quantize_unit<FMT, MODE, SCALED>(yv, active, tail, g, rg, g_odd, coarse, pk, sb, pk2, sb2);
    // The next row's registers are taken over before this row's stores are issued: the wait for
    // the prefetch (in flight since the top of the iteration) then stands in front of the stores, and
    // the top of the next iteration has no memory operation of this one left to wait for.
    q0 = n0;
    q1 = n1;
    asm volatile("" : "+v"(q0.x), "+v"(q0.y), "+v"(q0.z), "+v"(q0.w), "+v"(q1.x), "+v"(q1.y), "+v"(q1.z), "+v"(q1.w));
    if (MODE == MODE_SWIGLU) {
      u0 = un0;
      u1 = un1;
      asm volatile("" : "+v"(u0.x), "+v"(u0.y), "+v"(u0.z), "+v"(u0.w), "+v"(u1.x), "+v"(u1.y), "+v"(u1.z), "+v"(u1.w));
    }
    if (active) {
      store_unit<FMT>(crow, srow, tid, pk, sb);
      if (tail) store_unit<FMT>(crow, srow, nunits + (tid - tail0), pk2, sb2);
    }
  }
}

// ---------------------------------------------------------------------------------------------
// Rows of more than 16384 channels (the reference's dedicated shapes: 18944, 27648, 28672;
// kernels/src/bindings.cpp:141-160, down.cu:71-233, reorder.cu:380-555), every mode but the fused norm.
// A thread per unit would need more than 1024 threads and a row of up to 64 KB leaves room for one such
// workgroup per CU, which would then load, gather and store in turns.  Here a thread owns FOUR units
// (u = tid + h * blockDim, so that a wave's code stores stay contiguous), a workgroup is K/64 threads
// (at most 512) and two of them fit a CU: one loads its next row while the other encodes.  The channel
// order stays in registers as the 16-bit indices themselves (eight registers per unit); a gather address
// is one multiply-add away.  The arithmetic per unit is quantize_unit, as in the kernel above.
// ---------------------------------------------------------------------------------------------
// slot address of channel `half` (0 / 1) of an index pair: base + 2 * index, one instruction
template <int HALF>
__device__ __forceinline__ uint32_t gather_addr(uint32_t pair, uint32_t base) {
  uint32_t a;
  if (HALF == 0)
    asm("v_mad_u32_u16 %0, %1, 2, %2" : "=v"(a) : "v"(pair), "v"(base));
  else
    asm("v_mad_u32_u16 %0, %1, 2, %2 op_sel:[1,0,0,0]" : "=v"(a) : "v"(pair), "v"(base));
  return a;
}

constexpr int kWideUnits = 4;

template <int FMT, int MODE, bool SCALED, bool GROUPED = false>
__global__ __launch_bounds__(512, 4) void quantize_rows_wide_kernel(QuantParams p) {
  extern __shared__ uint4 smem[];
  static_assert(MODE != MODE_NORM, "the fused norm has no rows this long");
  constexpr int G = FMT == ARCQ_FMT_NVFP4 ? 16 : 32;
  const int K = p.K, S = p.S, Kp = K + S;
  uint16_t *row = reinterpret_cast<uint16_t *>(smem);
  const uint32_t row_addr = (uint32_t)reinterpret_cast<uintptr_t>(row);
  const int T = blockDim.x, nwaves = T >> 6;
  int tid = threadIdx.x + 64 * (int)(blockIdx.x % (unsigned)nwaves);  // the waves with residual units rotate over the SIMDs
  if (tid >= T) tid -= T;
  const int nunits = K >> 4, nchunks = K >> 3, tail0 = (K - S) >> 4;
  const size_t ldx = MODE == MODE_SWIGLU ? (size_t)p.ldx : (size_t)K;

  float g = SCALED ? (p.d_gscale && !GROUPED ? *p.d_gscale : p.gscale) : 1.0f;
  float rg = SCALED ? 1.0f / g : 1.0f;
  bool g_odd = SCALED && !(fabsf(g) >= 0x1p-60f && fabsf(g) <= 0x1p+60f);
  bool coarse = !SCALED || (f2u(g) & 0x7fffffu) == 0u;

  uint32_t iw[kWideUnits][8];
  auto load_order = [&](const int16_t *idx) {
#pragma unroll
    for (int h = 0; h < kWideUnits; ++h) {
      const int u = tid + h * T;
      uint4 i0 = make_uint4(0, 0, 0, 0), i1 = i0;
      if (u < nunits) {
        i0 = reinterpret_cast<const uint4 *>(idx)[2 * u];
        i1 = reinterpret_cast<const uint4 *>(idx)[2 * u + 1];
      }
      iw[h][0] = i0.x, iw[h][1] = i0.y, iw[h][2] = i0.z, iw[h][3] = i0.w;
      iw[h][4] = i1.x, iw[h][5] = i1.y, iw[h][6] = i1.z, iw[h][7] = i1.w;
    }
  };
  if (!GROUPED) load_order(p.idx);
  int seg_cur = -1, seg_end = 0;
  uint32_t yv[16];
#pragma unroll
  for (int i = 0; i < 16; ++i) yv[i] = 0u;  // low halves stay zero: only d16_hi loads write these

  for (int r = blockIdx.x; r < p.rows; r += gridDim.x) {
    if (GROUPED && r >= seg_end) {  // workgroup-uniform; once per segment at most (rows are sorted)
      while (seg_cur + 1 < p.n_seg && r >= seg_end) {
        ++seg_cur;
        seg_end = p.seg[seg_cur + 1];
      }
      if (r >= seg_end) break;
      load_order(p.idx + (size_t)seg_cur * K);
      if (SCALED) {
        g = p.d_gscale[seg_cur];
        rg = 1.0f / g;
        g_odd = !(fabsf(g) >= 0x1p-60f && fabsf(g) <= 0x1p+60f);
        coarse = (f2u(g) & 0x7fffffu) == 0u;
      }
    }
    // the row, natural order: 2 * kWideUnits 16-byte chunks per thread, all in flight at once (SwiGLU, which
    // reads two rows: in two halves)
    const uint4 *src = reinterpret_cast<const uint4 *>(p.x + (size_t)r * ldx);
    const uint4 *usrc = MODE == MODE_SWIGLU ? reinterpret_cast<const uint4 *>(p.up + (size_t)r * ldx) : nullptr;
    constexpr int kParts = MODE == MODE_SWIGLU ? 2 : 1, kPer = 2 * kWideUnits / kParts;
    // Everything derived from the thread number below (chunk and unit offsets, their bounds checks) is the same
    // for every row; hoisted out of the row loop it would stay in some forty registers across the encode.
    // The thread number is therefore made opaque once per row and once per unit.
    int tid_r = tid;
    asm volatile("" : "+v"(tid_r));
#pragma unroll
    for (int part = 0; part < kParts; ++part) {
      uint4 q[kPer], uq[kPer];
#pragma unroll
      for (int j = 0; j < kPer; ++j) {
        const int c = tid_r + (part * kPer + j) * T;
        q[j] = make_uint4(0, 0, 0, 0);
        uq[j] = q[j];
        if (c < nchunks) {
          q[j] = src[c];
          if (MODE == MODE_SWIGLU) uq[j] = usrc[c];
        }
      }
      if (part == 0) lds_barrier();  // the previous row's gathers are over (the loads above are already on their way)
#pragma unroll
      for (int j = 0; j < kPer; ++j) {
        const int c = tid_r + (part * kPer + j) * T;
        if (MODE == MODE_SWIGLU)
          q[j] = make_uint4(swiglu_pair(q[j].x, uq[j].x), swiglu_pair(q[j].y, uq[j].y), swiglu_pair(q[j].z, uq[j].z),
                            swiglu_pair(q[j].w, uq[j].w));
        if (c < nchunks) reinterpret_cast<uint4 *>(row)[c] = q[j];
      }
    }
    lds_barrier();

    uint8_t *crow = p.codes + (size_t)r * (Kp >> 1);
    uint8_t *srow = p.scales + (size_t)r * (Kp / G);
#pragma unroll
    for (int h = 0; h < kWideUnits; ++h) {
      if (h * T >= nunits) break;  // workgroup-uniform: nobody has a unit in this round
      int u = tid + h * T;
      asm volatile("" : "+v"(u));
      const bool active = u < nunits;  // a lane without a unit keeps the previous unit's values: nothing of it is stored
      if (active) {
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          // (volatile: the addresses do not depend on the row, and hoisted out of the row loop they would
          // occupy 64 registers)
          uint32_t a0, a1;
          asm volatile("v_mad_u32_u16 %0, %1, 2, %2" : "=v"(a0) : "v"(iw[h][j]), "v"(row_addr));
          asm volatile("v_mad_u32_u16 %0, %1, 2, %2 op_sel:[1,0,0,0]" : "=v"(a1) : "v"(iw[h][j]), "v"(row_addr));
          asm volatile("ds_read_u16_d16_hi %0, %1" : "+v"(yv[2 * j]) : "v"(a0) : "memory");
          asm volatile("ds_read_u16_d16_hi %0, %1" : "+v"(yv[2 * j + 1]) : "v"(a1) : "memory");
        }
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
      }
#pragma unroll
      for (int i = 0; i < 16; ++i) asm volatile("" : "+v"(yv[i]));  // read after the wait above
      const bool tail = active && u >= tail0;
      uint2 pk, pk2;
      uint32_t sb, sb2;
      quantize_unit<FMT, MODE, SCALED>(yv, active, tail, g, rg, g_odd, coarse, pk, sb, pk2, sb2);
      if (active) {
        store_unit<FMT>(crow, srow, u, pk, sb);
        if (tail) store_unit<FMT>(crow, srow, nunits + (u - tail0), pk2, sb2);
      }
    }
  }
}

// ---------------------------------------------------------------------------------------------
// Wave-per-row kernel for many rows of K = 1024 * KU <= 4096 channels with tensor scale 1 (plain
// reorder + quantize, and the fused RMSNorm).  A wave owns a whole row, so nothing after the set-up
// is shared between waves: no workgroup barrier per row, and everything that happens once per row
// (the reduction of the sum of squares, 1/sqrt) is paid once per KU units of a lane instead of
// once per unit.  Sixteen waves per workgroup, one workgroup per CU: every SIMD holds four rows in
// different phases (load, normalise, gather, encode), which is what hides their latencies.
//   * the row travels global -> LDS by LDS-direct loads (no staging registers) into the wave's slot;
//   * fused norm: the lane reads its 16 * KU natural-order values back from the slot twice (sum of
//     squares, then normalise) and writes the bf16 results over them; gamma sits in LDS once per
//     workgroup, already split into the (gamma_even, 0) / (0, gamma_odd) operands of the dot instruction;
//   * a lane owns the KU units u * 64 + lane (a wave's code stores are contiguous); their gather
//     addresses are rebuilt per unit from a copy of reorder_index in LDS (one multiply-add each),
//     which keeps the kernel at 128 registers, i.e. four waves per SIMD.
// With more rows than waves in flight a wave walks rows with stride (waves in flight).
// ---------------------------------------------------------------------------------------------
constexpr int kRowWaves = 16;  // waves per workgroup = rows in progress per CU (four per SIMD)

// Comment-only markers in the compiler's assembly output (-DARCQ_PHASE_MARKERS), for counting the instructions of
// each phase of the wave-per-row kernel; nothing in a normal build.
#ifdef ARCQ_PHASE_MARKERS
#define ARCQ_PHASE(name) asm volatile("; ARCQ_PHASE " name)
#else
#define ARCQ_PHASE(name)
#endif

template <int OFF>
__device__ __forceinline__ void row_dma16(const void *g, uint32_t lds_base) {
  // writes M0 (reserved: cannot be listed as clobbered); nothing else in this kernel reads M0
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off offset:%2"
               :
               : "s"(lds_base), "v"(g), "n"(OFF)
               : "memory");
}

// NCH chunks of 1024 bytes -> LDS at lds_base; lane l of chunk c fetches bytes c*1024 + 16*l
template <int NCH>
__device__ __forceinline__ void row_dma(const void *row, int lane, uint32_t lds_base) {
  const uint8_t *g = reinterpret_cast<const uint8_t *>(row) + 16 * lane;
#pragma unroll
  for (int h = 0; h < (NCH + 3) / 4; ++h) {
    const uint8_t *gh = g + 4096 * h;
    const uint32_t lb = lds_base + 4096 * h;
    row_dma16<0>(gh, lb);
    if (4 * h + 1 < NCH) row_dma16<1024>(gh, lb);
    if (4 * h + 2 < NCH) row_dma16<2048>(gh, lb);
    if (4 * h + 3 < NCH) row_dma16<3072>(gh, lb);
  }
}

__device__ __forceinline__ void gather16(uint32_t (&yv)[16], const uint32_t (&addr)[16]) {
#pragma unroll
  for (int i = 0; i < 16; ++i) asm volatile("ds_read_u16_d16_hi %0, %1" : "+v"(yv[i]) : "v"(addr[i]) : "memory");
}

template <int N>
__device__ __forceinline__ void wait_vm() {
  asm volatile("s_waitcnt vmcnt(%0)" : : "n"(N) : "memory");
}

template <int FMT, int MODE, int KU>
__global__ __launch_bounds__(64 * kRowWaves) void quantize_rows_wave_kernel(QuantParams p) {
  extern __shared__ uint4 smem[];
  constexpr int G = FMT == ARCQ_FMT_NVFP4 ? 16 : 32;
  constexpr int K = 1024 * KU, NCH = 2 * KU, SLOT = 2 * K;   // NCH: 16-byte chunks per lane and row
  constexpr int TABLES = MODE == MODE_NORM ? 3 * SLOT : SLOT;  // reorder_index [+ the two gamma tables]
  static_assert(MODE == MODE_X || MODE == MODE_NORM, "the wave-per-row kernel quantizes activations");
  static_assert(KU >= 1 && KU <= 4, "gather offsets are 16-bit");
  const int S = p.S, Kp = K + S;
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  uint8_t *lds = reinterpret_cast<uint8_t *>(smem);
  const uint32_t lds0 = (uint32_t)reinterpret_cast<uintptr_t>(lds);
  const uint32_t slot_addr = lds0 + TABLES + wave * SLOT;  // this wave's row
  uint4 *slot = reinterpret_cast<uint4 *>(lds + TABLES + wave * SLOT);
  const int nunits = K >> 4, tail0 = (K - S) >> 4;
  const int stride = gridDim.x * kRowWaves;
  int row = blockIdx.x * kRowWaves + wave;

  // A few waves request their rows at once, then the tables are fetched and the workgroup meets, then the
  // other waves request theirs.  Measured on 4096 x 4096 rows: all sixteen rows requested up front (tables
  // first, the waves told of their arrival through a counter in LDS instead of a barrier) is 1.3 us slower
  // than this, no row requested before the barrier 0.5 us slower: a CU takes its sixteen 8 KB rows at about
  // 20 KB per microsecond, the four early rows keep its queue busy while the tables make their round trip,
  // and requests queued behind many rows (the tables, every wave's later instructions) wait for all of them.
  constexpr int kEarlyWaves = 4;  // 2: +0.9 us, 6 or 8: +0.3 us on the 4096 x 4096 fused norm
  const bool early = wave >= kRowWaves - kEarlyWaves && row < p.rows;
  if (early) row_dma<NCH>(p.x + (size_t)row * K, lane, slot_addr);
  if (wave < NCH) {  // reorder_index: 2K bytes = NCH wave-loads of 1024 bytes, straight into LDS
    const uint8_t *g = reinterpret_cast<const uint8_t *>(p.idx) + 1024 * wave + 16 * lane;
    row_dma16<0>(g, lds0 + 1024 * wave);
  }
  if (MODE == MODE_NORM && (int)threadIdx.x < (K >> 3)) {  // gamma, split for the dot instruction
    const uint4 g = reinterpret_cast<const uint4 *>(p.gamma)[threadIdx.x];
    uint4 *glo_t = reinterpret_cast<uint4 *>(lds + SLOT), *ghi_t = reinterpret_cast<uint4 *>(lds + 2 * SLOT);
    glo_t[threadIdx.x] = make_uint4(g.x & 0xffffu, g.y & 0xffffu, g.z & 0xffffu, g.w & 0xffffu);
    ghi_t[threadIdx.x] = make_uint4(g.x & 0xffff0000u, g.y & 0xffff0000u, g.z & 0xffff0000u, g.w & 0xffff0000u);
  }
  if (early) wait_vm<NCH>();  // loads return in order: NCH outstanding means only the row is still on its way
  else wait_vm<0>();
  lds_barrier();  // everybody's table chunks are in LDS
  if (row >= p.rows) return;
  if (!early) row_dma<NCH>(p.x + (size_t)row * K, lane, slot_addr);

  const float eps = p.eps;
  const bool eps_normal = eps >= 0x1p-90f;
  const double inv_k = p.inv_k;
  const uint4 *idx_t = reinterpret_cast<const uint4 *>(lds);
  uint32_t yvA[16], yvB[16];
#pragma unroll
  for (int i = 0; i < 16; ++i) yvA[i] = yvB[i] = 0u;  // low halves stay zero: only d16_hi loads write these

  auto unit_addresses = [&](int u, uint32_t (&addr)[16]) {
    const uint4 i0 = idx_t[2 * (u * 64 + lane)], i1 = idx_t[2 * (u * 64 + lane) + 1];
    const uint32_t iw[8] = {i0.x, i0.y, i0.z, i0.w, i1.x, i1.y, i1.z, i1.w};
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      addr[2 * j] = gather_addr<0>(iw[j], slot_addr);
      addr[2 * j + 1] = gather_addr<1>(iw[j], slot_addr);
    }
  };

  for (;;) {
    wait_vm<0>();  // the row has landed (past the first row this also waits for the previous row's stores;
                   // the SIMD's other waves fill the gap)
    if (MODE == MODE_NORM) {
      ARCQ_PHASE("pass1 sum of squares");
      // pass 1 over the lane's natural-order values: sum of squares (exact squares, fp64 accumulation)
      double ss0 = 0.0, ss1 = 0.0;
#pragma unroll
      for (int c = 0; c < NCH; ++c) {
        const uint4 q = slot[c * 64 + lane];
        const uint32_t w[4] = {q.x, q.y, q.z, q.w};
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const double d0 = (double)u2f(w[j] << 16), d1 = (double)u2f(w[j] & 0xffff0000u);
          ss0 = __builtin_fma(d0, d0, ss0);
          ss1 = __builtin_fma(d1, d1, ss1);
        }
      }
      ARCQ_PHASE("wave reduction and 1/sqrt");
      double tot = wave_sum_to_lane63(ss0 + ss1);
      {
        const uint64_t b = __builtin_bit_cast(uint64_t, tot);
        const uint32_t lo = __builtin_amdgcn_readlane((uint32_t)b, 63);
        const uint32_t hi = __builtin_amdgcn_readlane((uint32_t)(b >> 32), 63);
        tot = __builtin_bit_cast(double, ((uint64_t)hi << 32) | lo);
      }
      // mean = tot / K exactly: a power-of-two K is a scaling, 3072 an IEEE division
      const float var = KU == 3 ? (float)(tot / (double)K) : (float)(tot * inv_k);
      const float a = var + eps;
      float rstd;
      if (eps_normal) {
        const float sq = sqrt_from_estimate(a, __builtin_amdgcn_sqrtf(a));
        rstd = rcp_from_estimate(sq, __builtin_amdgcn_rcpf(sq));
        if (!(a < __builtin_inff())) rstd = a != a ? a : 0.0f;  // 1/sqrt(inf) = 0, NaN stays NaN
      } else {
        rstd = 1.0f / sqrtf(a);
      }
      ARCQ_PHASE("pass2 normalise and gamma");
      // pass 2: normalise, multiply by gamma, write the bf16 results over the raw values this lane read
      const uint4 *glo_t = reinterpret_cast<const uint4 *>(lds + SLOT), *ghi_t = reinterpret_cast<const uint4 *>(lds + 2 * SLOT);
#pragma unroll
      for (int c = 0; c < NCH; ++c) {
        const uint4 q = slot[c * 64 + lane];  // (kept in registers across the passes the kernel would spill)
        const uint4 gl = glo_t[c * 64 + lane], gh = ghi_t[c * 64 + lane];
        const uint32_t w[4] = {q.x, q.y, q.z, q.w};
        const uint32_t glo[4] = {gl.x, gl.y, gl.z, gl.w}, ghi[4] = {gh.x, gh.y, gh.z, gh.w};
        uint32_t hw[4], yw[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) hw[j] = pack_bf16_rne(u2f(w[j] << 16) * rstd, u2f(w[j] & 0xffff0000u) * rstd);
        gamma_mul_pack4(hw, glo, ghi, yw);
        slot[c * 64 + lane] = make_uint4(yw[0], yw[1], yw[2], yw[3]);
      }
      // the gather below reads what other lanes wrote: LDS operations of one wave execute in order
    }

    ARCQ_PHASE("units: gather addresses, encode, stores");
    uint8_t *crow = p.codes + (size_t)row * (Kp >> 1), *srow = p.scales + (size_t)row * (Kp / G);
    const int next_row = row + stride;
    {
      uint32_t addr[16];
      unit_addresses(0, addr);
      gather16(yvA, addr);
    }
#pragma unroll
    for (int u = 0; u < KU; ++u) {
      uint32_t(&cur)[16] = (u & 1) ? yvB : yvA;
      uint32_t(&nxt)[16] = (u & 1) ? yvA : yvB;
      uint32_t addr[16];
      if (u + 1 < KU) unit_addresses(u + 1, addr);
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
      float y[16];
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        asm volatile("" : "+v"(cur[i]));  // read after the wait above
        y[i] = u2f(cur[i]);
      }
      if (u + 1 < KU) {
        gather16(nxt, addr);  // the next unit's values fly while this one is encoded
      } else if (next_row < p.rows) {
        // every read of the slot is over: the next row of this wave may land in it
        row_dma<NCH>(p.x + (size_t)next_row * K, lane, slot_addr);
      }
      float s;
      const float amax = unit_amax3<FMT>(y);
      const float t = div6_any(amax);
      const uint32_t sb = FMT == ARCQ_FMT_NVFP4 ? ue4m3_scale(t, &s) : ue8m0_scale(t, &s);
      const uint2 pk = encode_unit_coarse(y, scale_rcp<FMT>(s));
      const int n = u * 64 + lane;
      store_unit<FMT>(crow, srow, n, pk, sb);
      if (u * 64 + 63 >= tail0) {  // wave-uniform: some lane's unit of this round is among the last select_num channels
        ARCQ_PHASE("residual block");
        float e[16];
        decode_unit(pk, e);
#pragma unroll
        for (int i = 0; i < 16; ++i) e[i] = __builtin_fmaf(-e[i], s, y[i]);  // q*s is exact: the fp32 residual y - q*s
        float s2;
        const float t2 = div6_any(unit_amax3<FMT>(e));
        const uint32_t sb2 = FMT == ARCQ_FMT_NVFP4 ? ue4m3_scale(t2, &s2) : ue8m0_scale(t2, &s2);
        const uint2 pk2 = encode_unit_coarse(e, scale_rcp<FMT>(s2));
        if (n >= tail0) store_unit<FMT>(crow, srow, nunits + (n - tail0), pk2, sb2);
        ARCQ_PHASE("units (continued)");
      }
    }
    ARCQ_PHASE("row loop end");
    if (next_row >= p.rows) break;
    row = next_row;
  }
}

// ---------------------------------------------------------------------------------------------
// Tensor scale and quantizer in one launch, for activations that fit the chip's LDS (sixteen rows of up to 4096
// channels per CU: 4096 rows on 256 CUs).  The reference's callers form max|x| / 2688 with torch ahead of the
// quantizer (model/qLlamaLayer.py:73-77): two passes over x.  Here a wave loads its row into LDS once, takes its
// maximum and gathers its units into registers in the channel order; the workgroups exchange their maxima; then
// the units are encoded under the scale.
//
// Exchange: workgroup b stores (tag, maximum) as one 64-bit word into slot b (48 bits of tag; the maximum is a bf16
// value, its upper 16 bits say everything); wave 0 of every workgroup reads all slots until each carries the
// launch's tag.  The tag is one more than the value of an epoch word read at the
// start; on its way out every workgroup raises the epoch word to its tag (atomic maximum), so the next launch on
// the stream -- which starts after this one has ended -- takes a tag above every tag ever stored.  No counter to
// reset, no read-modify-write on the way in, nothing the host has to pass: a captured launch replays correctly.
//
// The workgroups can only meet if all of them are on the chip at once, which nothing guarantees (another kernel
// may hold CUs).  So the wait is bounded: when it runs out the workgroup takes the maximum over the whole tensor
// by itself, from global memory, and goes on.  Every workgroup therefore finishes whatever the others do; the
// result is the same either way (a maximum), the bounded wait only decides how it was obtained.
// ---------------------------------------------------------------------------------------------
constexpr int kResidentSlots = 256;        // workgroups per launch at most (512 of half the size: 2 us slower at 2048 rows)
constexpr int kResidentSlotWord = 256;     // slots start at this 64-bit word of the tensor-scale scratch (byte 2048)
constexpr int kResidentEpochWord = 480;   // 32-bit word index of the 64-bit epoch, on a 128-byte line of its own behind the
                                          // (maximum, counter) pairs of tensor_scale_kernel

typedef uint16_t v2u16 __attribute__((ext_vector_type(2)));

__device__ __forceinline__ uint32_t absmax_bf16_pairs(uint32_t m, uint32_t w) {
  const v2u16 a = __builtin_bit_cast(v2u16, m), b = __builtin_bit_cast(v2u16, w & 0x7fff7fffu);
  return __builtin_bit_cast(uint32_t, __builtin_elementwise_max(a, b));  // v_pk_max_u16
}

// Compile-time loop over 0 .. N-1 and a choice among four arrays by a compile-time index: the units' values live in
// four separate arrays of sixteen registers (one array of 64 stays in scratch memory: the compiler does not split it).
template <int N, typename F>
__device__ __forceinline__ void static_for(F &&f) {
  if constexpr (N > 0) {
    static_for<N - 1>(f);
    f(std::integral_constant<int, N - 1>{});
  }
}
template <int U>
__device__ __forceinline__ uint32_t (&pick16(uint32_t (&a)[16], uint32_t (&b)[16], uint32_t (&c)[16], uint32_t (&d)[16]))[16] {
  if constexpr (U == 0) return a;
  else if constexpr (U == 1) return b;
  else if constexpr (U == 2) return c;
  else return d;
}

// WPR waves share a row (1, 2 or 4: a row's units are dealt out to them by whole rounds of 64), so that a launch of
// few rows still spreads over the chip: a workgroup holds 16 / WPR rows, and a wave's share of the arithmetic that
// follows the exchange -- where nothing else can hide it -- is 1 / WPR of a row.
template <int FMT, int KU, int WPR>
__global__ __launch_bounds__(64 * kRowWaves) __attribute__((amdgpu_waves_per_eu(4, 4))) void quantize_rows_resident_kernel(QuantParams p, float divisor, uint32_t spin_ticks,
                                                                                 uint32_t *ws, float *scale_out) {
  extern __shared__ uint4 smem[];
  constexpr int G = FMT == ARCQ_FMT_NVFP4 ? 16 : 32;
  constexpr int K = 1024 * KU, NCH = 2 * KU, SLOT = 2 * K;
  constexpr int TABLES = SLOT;  // reorder_index
  constexpr int RPW = kRowWaves / WPR;  // rows per workgroup
  constexpr int UPL = KU / WPR;         // units per lane
  constexpr int CPW = NCH / WPR;        // 1024-byte chunks of the row that a wave fetches
  static_assert(KU % WPR == 0 && kRowWaves % WPR == 0, "a row's rounds of 64 units are dealt out whole");
  const int S = p.S, Kp = K + S;
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int r_in = wave / WPR;
  // which part of the row: rotated from row to row, so that the waves that own the last select_num channels (and
  // encode the residual on top) fall on different SIMDs (wave i of a workgroup runs on SIMD i mod 4)
  const int sub = WPR == 1 ? 0 : (wave + r_in) % WPR;
  uint8_t *lds = reinterpret_cast<uint8_t *>(smem);
  const uint32_t lds0 = (uint32_t)reinterpret_cast<uintptr_t>(lds);
  const uint32_t slot_addr = lds0 + TABLES + r_in * SLOT;  // this wave's row
  const uint4 *part = reinterpret_cast<const uint4 *>(lds + TABLES + r_in * SLOT + sub * CPW * 1024);
  uint32_t *meet = reinterpret_cast<uint32_t *>(lds + TABLES + RPW * SLOT);  // [0..15] wave maxima, [16] maximum, [17] timed out
  const int nunits = K >> 4, tail0 = (K - S) >> 4;
  const int row = blockIdx.x * RPW + r_in;
  const bool has_row = row < p.rows;
  unsigned long long *slots = reinterpret_cast<unsigned long long *>(ws) + kResidentSlotWord;
  unsigned long long *epoch = reinterpret_cast<unsigned long long *>(ws + kResidentEpochWord);
  const uint16_t *src = p.x + (size_t)row * K + sub * CPW * 512;
  const uint32_t dst = slot_addr + sub * CPW * 1024;

  // rows and table as in the wave-per-row kernel above: four waves request their rows ahead of the table
  constexpr int kEarlyWaves = 4;
  const bool early = wave >= kRowWaves - kEarlyWaves && has_row;
  if (early) row_dma<CPW>(src, lane, dst);
  if (wave < NCH) {
    const uint8_t *g = reinterpret_cast<const uint8_t *>(p.idx) + 1024 * wave + 16 * lane;
    row_dma16<0>(g, lds0 + 1024 * wave);
  }
  unsigned long long tag = 0ull;
  if (wave == 0) tag = __hip_atomic_load(epoch, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) + 1ull;  // every lane: uniform
  if (early) wait_vm<CPW>();
  else wait_vm<0>();
  lds_barrier();
  if (!early && has_row) row_dma<CPW>(src, lane, dst);
  wait_vm<0>();

  // what does not depend on the scale: the maximum, and the units' values in the channel order
  uint32_t m = 0u;
  uint32_t ya[16], yb[16], yc[16], yd[16];  // fp32 bits: a bf16 loaded into the upper half of a zeroed register IS the fp32
#pragma unroll
  for (int k = 0; k < 16; ++k) ya[k] = yb[k] = yc[k] = yd[k] = 0u;
  if (has_row) {
#pragma unroll
    for (int c = 0; c < CPW; ++c) {
      const uint4 q = part[c * 64 + lane];
      m = absmax_bf16_pairs(absmax_bf16_pairs(absmax_bf16_pairs(absmax_bf16_pairs(m, q.x), q.y), q.z), q.w);
    }
  }
  auto gather_units = [&]() {
    if (!has_row) return;
    const uint4 *idx_t = reinterpret_cast<const uint4 *>(lds);
    static_for<UPL>([&](auto U) {
      constexpr int u = decltype(U)::value;
      const int n = (sub * UPL + u) * 64 + lane;
      const uint4 i0 = idx_t[2 * n], i1 = idx_t[2 * n + 1];
      const uint32_t iw[8] = {i0.x, i0.y, i0.z, i0.w, i1.x, i1.y, i1.z, i1.w};
      uint32_t addr[16];
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        addr[2 * j] = gather_addr<0>(iw[j], slot_addr);
        addr[2 * j + 1] = gather_addr<1>(iw[j], slot_addr);
      }
      gather16(pick16<u>(ya, yb, yc, yd), addr);
    });
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    static_for<UPL>([&](auto U) {
      uint32_t(&v)[16] = pick16<decltype(U)::value>(ya, yb, yc, yd);
#pragma unroll
      for (int k = 0; k < 16; ++k) asm volatile("" : "+v"(v[k]));  // read after the wait above
    });
  };
  if (WPR == 1) gather_units();  // the row is this wave's own: no need to wait for anybody
  m = (m & 0xffffu) > (m >> 16) ? (m << 16) : (m & 0xffff0000u);  // the larger half, as the bits of an fp32
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    const uint32_t v = (uint32_t)__shfl_xor((int)m, o);
    m = v > m ? v : m;
  }
  if (lane == 0) meet[wave] = m;
  lds_barrier();  // the maxima are in LDS; every part of every row has landed

  if (wave == 0) {
    uint32_t wg = lane < kRowWaves ? meet[lane] : 0u;
#pragma unroll
    for (int o = 8; o > 0; o >>= 1) {
      const uint32_t v = (uint32_t)__shfl_xor((int)wg, o);
      wg = v > wg ? v : wg;
    }
    wg = __builtin_amdgcn_readfirstlane(wg);
    if (lane == 0)
      __hip_atomic_store(slots + blockIdx.x, (tag << 16) | (wg >> 16), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
  if (WPR != 1) gather_units();  // while the slot is on its way
  if (wave == 0) {
    // lane l watches slots l, l + 64, l + 128, ...
    const int nslots = (int)gridDim.x;
    uint32_t all = 0u;
    unsigned pending = 0u;
#pragma unroll
    for (int j = 0; j < kResidentSlots / 64; ++j)
      if (lane + 64 * j < nslots) pending |= 1u << j;
    const unsigned long long t0 = wall_clock64();
    bool timed_out = false;
    for (;;) {
#pragma unroll
      for (int j = 0; j < kResidentSlots / 64; ++j) {
        if (pending & (1u << j)) {
          const unsigned long long v = __hip_atomic_load(slots + lane + 64 * j, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          if ((v >> 16) == tag) {
            const uint32_t mv = ((uint32_t)v & 0xffffu) << 16;
            all = mv > all ? mv : all;
            pending &= ~(1u << j);
          }
        }
      }
      if (__builtin_amdgcn_ballot_w64(pending != 0u) == 0ull) break;
      if (wall_clock64() - t0 >= (unsigned long long)spin_ticks) {  // the clock is read once per wave
        timed_out = true;
        break;
      }
      __builtin_amdgcn_s_sleep(2);
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
      const uint32_t v = (uint32_t)__shfl_xor((int)all, o);
      all = v > all ? v : all;
    }
    if (lane == 0) {
      meet[16] = all;
      meet[17] = timed_out ? 1u : 0u;
    }
  }
  lds_barrier();
  uint32_t all = meet[16];
  if (meet[17] != 0u) {
    // the others did not show up in time: this workgroup takes the maximum over the whole tensor by itself
    const size_t total = (size_t)p.rows * (K >> 3);
    uint32_t mm = 0u;
    for (size_t c = threadIdx.x; c < total; c += 64 * kRowWaves) {
      const uint4 q = reinterpret_cast<const uint4 *>(p.x)[c];
      mm = absmax_bf16_pairs(absmax_bf16_pairs(absmax_bf16_pairs(absmax_bf16_pairs(mm, q.x), q.y), q.z), q.w);
    }
    mm = (mm & 0xffffu) > (mm >> 16) ? (mm << 16) : (mm & 0xffff0000u);
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
      const uint32_t v = (uint32_t)__shfl_xor((int)mm, o);
      mm = v > mm ? v : mm;
    }
    lds_barrier();  // meet[16], meet[17] have been read by everybody
    if (lane == 0) meet[wave] = mm;
    lds_barrier();
    all = 0u;
    for (int w = 0; w < kRowWaves; ++w) all = meet[w] > all ? meet[w] : all;
  }
  if (threadIdx.x == 0) atomicMax(epoch, tag);  // nobody waits for it: the next launch on the stream reads it
  const float quot = u2f(all) / divisor;
  const float g = quot == 0.0f ? 1.0f : quot;
  if (blockIdx.x == 0 && threadIdx.x == 0) *scale_out = g;
  if (!has_row) return;

  const float rg = 1.0f / g;
  const bool g_odd = !(fabsf(g) >= 0x1p-60f && fabsf(g) <= 0x1p+60f);
  const bool coarse = (f2u(g) & 0x7fffffu) == 0u;
  uint8_t *crow = p.codes + (size_t)row * (Kp >> 1), *srow = p.scales + (size_t)row * (Kp / G);
  static_for<UPL>([&](auto U) {
    constexpr int u = decltype(U)::value;
    const int n = (sub * UPL + u) * 64 + lane;
    const bool tail = n >= tail0;
    uint2 pk, pk2;
    uint32_t sb, sb2;
    quantize_unit<FMT, MODE_X, true>(pick16<u>(ya, yb, yc, yd), true, tail, g, rg, g_odd, coarse, pk, sb, pk2, sb2);
    store_unit<FMT>(crow, srow, n, pk, sb);
    if (tail) store_unit<FMT>(crow, srow, nunits + (n - tail0), pk2, sb2);
  });
}

// max |act_fn(gate) * up| over the whole tensor (the NVFP4 tensor scale's numerator,
// model/qLlamaLayer.py:74), as the fp32 bits of a non-negative value: atomicMax on them is a max
__global__ __launch_bounds__(256) void swiglu_absmax_kernel(const uint16_t *gate, const uint16_t *up, size_t ld, int rows,
                                                            int K, uint32_t *out) {
  const int cpr = K >> 3;  // 16-byte chunks per row
  const size_t total = (size_t)rows * cpr;
  uint32_t m = 0u;
  for (size_t c = (size_t)blockIdx.x * blockDim.x + threadIdx.x; c < total; c += (size_t)gridDim.x * blockDim.x) {
    const size_t r = c / cpr, k = (c % cpr) << 3;
    const uint4 g = *reinterpret_cast<const uint4 *>(gate + r * ld + k);
    const uint4 u = *reinterpret_cast<const uint4 *>(up + r * ld + k);
    const uint32_t t[4] = {swiglu_pair(g.x, u.x), swiglu_pair(g.y, u.y), swiglu_pair(g.z, u.z), swiglu_pair(g.w, u.w)};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const uint32_t lo = (t[i] << 16) & 0x7fffffffu, hi = t[i] & 0x7fff0000u;
      m = lo > m ? lo : m;
      m = hi > m ? hi : m;
    }
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    const uint32_t v = (uint32_t)__shfl_xor((int)m, o);
    m = v > m ? v : m;
  }
  if ((threadIdx.x & 63) == 0 && m) atomicMax(out, m);
}

// NVFP4 tensor scale of an activation tensor in one launch: max |x| / divisor (model/qLlamaLayer.py:74),
// 1 for an all-zero tensor, as an fp32 scalar on the device.  SWIGLU: x = act_fn(gate) * up formed on the fly.
//
// A read-only stream: at most one workgroup of 512 or 1024 threads per CU, every thread with eight (SwiGLU: four per
// operand) independent 16-byte loads in flight per trip.  The workgroups then meet through a persistent
// workspace touched only by device-scope atomics.  Atomics on one word are served one after the other (10-30 ns
// each: with a thousand workgroups arriving on one counter the launch spent 30 us there), so they meet in two
// levels: a workgroup arrives at the (maximum, counter) pair of its group -- blockIdx mod kScaleGroups, each pair
// on a cache line of its own -- and the
// last arrival of a group arrives at the top counter; the last arrival there reads the groups' maxima, divides,
// writes the scale and leaves every word zero.  A workgroup's arrival is issued after its maximum has returned,
// so whoever sees a counter complete reads the maxima of all that were counted.
constexpr int kScaleThreads = 1024;  // at most; launches that one trip of 512 threads per CU covers take 512
constexpr unsigned kScaleGroups = 8;
constexpr int kScaleLine = 32;  // words between the pairs: 128 bytes
constexpr unsigned kScaleSingle = 32;  // launches of up to this many workgroups meet on one pair

template <bool SWIGLU>
__global__ __launch_bounds__(kScaleThreads) void tensor_scale_kernel(const uint16_t *x, const uint16_t *up, size_t ld, int rows,
                                                                      int K, float divisor, uint32_t *ws, float *out) {
  __shared__ uint32_t wave_max[kScaleThreads / 64];
  const int cpr = K >> 3;  // 16-byte chunks per row
  const size_t total = (size_t)rows * cpr;
  const bool dense = ld == (size_t)K;  // chunk c sits at x + 8 * c: no division per chunk
  constexpr int U = SWIGLU ? 4 : 8;
  uint32_t m = 0u;
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  for (size_t c0 = (size_t)blockIdx.x * blockDim.x + threadIdx.x; c0 < total; c0 += U * stride) {
    uint4 g[U], u[U];
#pragma unroll
    for (int j = 0; j < U; ++j) {
      const size_t c = c0 + j * stride;
      g[j] = make_uint4(0, 0, 0, 0);
      u[j] = g[j];
      if (c < total) {
        size_t off = c << 3;
        if (!dense) {
          const size_t r = c / cpr;
          off = r * ld + ((c - r * cpr) << 3);
        }
        g[j] = *reinterpret_cast<const uint4 *>(x + off);
        if (SWIGLU) u[j] = *reinterpret_cast<const uint4 *>(up + off);
      }
    }
#pragma unroll
    for (int j = 0; j < U; ++j) {  // an absent chunk is zeros: act_fn(0) * 0 = 0 leaves the maximum alone
      uint32_t t[4] = {g[j].x, g[j].y, g[j].z, g[j].w};
      if (SWIGLU) {
        t[0] = swiglu_pair(g[j].x, u[j].x), t[1] = swiglu_pair(g[j].y, u[j].y);
        t[2] = swiglu_pair(g[j].z, u[j].z), t[3] = swiglu_pair(g[j].w, u[j].w);
      }
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const uint32_t lo = (t[i] << 16) & 0x7fffffffu, hi = t[i] & 0x7fff0000u;
        m = lo > m ? lo : m;
        m = hi > m ? hi : m;
      }
    }
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    const uint32_t v = (uint32_t)__shfl_xor((int)m, o);
    m = v > m ? v : m;
  }
  if ((threadIdx.x & 63) == 0) wave_max[threadIdx.x >> 6] = m;
  __syncthreads();
  if (threadIdx.x != 0) return;
  for (int w = 1; w < (int)(blockDim.x >> 6); ++w) m = wave_max[w] > m ? wave_max[w] : m;
  // Every step below waits for the one before it to return (about half a microsecond each), so there are as few
  // as the protocol allows: maximum, arrival; the last arrival of a group arrives at the top; the last arrival
  // there reads the groups' maxima.  Up to kScaleSingle workgroups meet on the top pair alone.
  uint32_t *top = ws;
  if (gridDim.x > kScaleSingle) {
    const int grp = (int)blockIdx.x % kScaleGroups;
    const uint32_t members = ((uint32_t)gridDim.x - (uint32_t)grp + kScaleGroups - 1u) / kScaleGroups;
    uint32_t *gw = ws + (1 + grp) * kScaleLine;  // this group's (maximum, counter)
    const uint32_t old = atomicMax(gw, m);
    if (atomicAdd(gw + 1, 1u + (old >> 31)) != members - 1u) return;  // old < 2^31: the add waits for the maximum
    if (atomicAdd(top + 1, 1u) != kScaleGroups - 1u) return;
    // every group's last arrival has been counted, each after all of its group's maxima: read them, zero them
    for (int q = 0; q < kScaleGroups; ++q) {
      const uint32_t v = atomicExch(ws + (1 + q) * kScaleLine, 0u);
      m = q == 0 ? v : (v > m ? v : m);
      __hip_atomic_store(ws + (1 + q) * kScaleLine + 1, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
  } else {
    const uint32_t old = atomicMax(top, m);
    if (atomicAdd(top + 1, 1u + (old >> 31)) != gridDim.x - 1u) return;
    m = atomicExch(top, 0u);
  }
  __hip_atomic_store(top + 1, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  const float scale = u2f(m) / divisor;
  *out = scale == 0.0f ? 1.0f : scale;
}

// Per-segment maxima for grouped launches (rows sorted by segment): max |x|, or max |act_fn(gate) * up|,
// over the rows of each segment, accumulated as the bits of a non-negative float in bits[segment] (zeroed
// by the caller's launch in front).  A workgroup takes a contiguous run of rows and flushes its running
// maximum with one atomicMax when its rows enter another segment, and at the end: atomics on one word are
// served one after the other (about 10 ns each), so there must be few of them -- with rows dealt out
// round-robin every row of every workgroup ended in one (8192 rows over 8 segments: 86 us, all of it waiting).
template <bool SWIGLU>
__global__ __launch_bounds__(256) void grouped_absmax_kernel(const uint16_t *x, const uint16_t *up, size_t ld, int rows,
                                                             int K, const int *seg, int n_seg, uint32_t *bits) {
  __shared__ uint32_t wave_max[4];
  const int cpr = K >> 3;  // 16-byte chunks per row
  int seg_cur = -1, seg_end = 0;
  uint32_t m = 0u;
  auto flush = [&]() {  // workgroup-uniform
    if (seg_cur < 0) return;
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
      const uint32_t v = (uint32_t)__shfl_xor((int)m, o);
      m = v > m ? v : m;
    }
    __syncthreads();  // the previous flush's readers are done with wave_max
    if ((threadIdx.x & 63) == 0) wave_max[threadIdx.x >> 6] = m;
    __syncthreads();
    if (threadIdx.x == 0) {
      for (int w = 1; w < 4; ++w) m = wave_max[w] > m ? wave_max[w] : m;
      if (m) atomicMax(bits + seg_cur, m);
    }
    m = 0u;
  };
  const int per_wg = (rows + (int)gridDim.x - 1) / (int)gridDim.x;
  const int r_end = min(rows, ((int)blockIdx.x + 1) * per_wg);
  for (int r = (int)blockIdx.x * per_wg; r < r_end; ++r) {
    if (r >= seg_end) {
      flush();
      while (seg_cur + 1 < n_seg && r >= seg_end) {
        ++seg_cur;
        seg_end = seg[seg_cur + 1];
      }
      if (r >= seg_end) {  // behind the last segment
        seg_cur = -1;
        break;
      }
    }
    // four rows of the workgroup at a time while they stay inside the segment: all their loads are issued
    // before the first maximum is taken (a row of a few thousand channels is only two loads per thread)
    const int nr = (!SWIGLU && r + 3 < min(seg_end, r_end)) ? 4 : 1;
    for (int c = threadIdx.x; c < cpr; c += 256) {
      uint4 gq[4];
#pragma unroll
      for (int j = 0; j < 4; ++j)
        if (j < nr) gq[j] = *reinterpret_cast<const uint4 *>(x + (size_t)(r + j) * ld + 8 * c);
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        if (j >= nr) break;
        uint32_t t[4] = {gq[j].x, gq[j].y, gq[j].z, gq[j].w};
        if (SWIGLU) {
          const uint4 uq = *reinterpret_cast<const uint4 *>(up + (size_t)r * ld + 8 * c);
          t[0] = swiglu_pair(gq[j].x, uq.x), t[1] = swiglu_pair(gq[j].y, uq.y);
          t[2] = swiglu_pair(gq[j].z, uq.z), t[3] = swiglu_pair(gq[j].w, uq.w);
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const uint32_t lo = (t[i] << 16) & 0x7fffffffu, hi = t[i] & 0x7fff0000u;
          m = lo > m ? lo : m;
          m = hi > m ? hi : m;
        }
      }
    }
    r += nr - 1;
  }
  flush();
}

__global__ void zero_words_kernel(uint32_t *w, int n) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) w[i] = 0u;
}

// bits of the maxima -> tensor scales max / divisor in place (IEEE division; an all-zero or empty segment gets 1)
__global__ void grouped_scale_finish_kernel(uint32_t *bits, int n, float divisor) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  const float scale = u2f(bits[i]) / divisor;
  reinterpret_cast<float *>(bits)[i] = scale == 0.0f ? 1.0f : scale;
}

template <int FMT, int MODE, bool SCALED, bool GROUPED = false>
int launch_quantize_unit(const QuantParams &p, hipStream_t stream) {
  const int threads = (((p.K >> 4) + 63) / 64) * 64;
  const size_t lds = (size_t)p.K * 2 + 16 * sizeof(double);
  const int waves_per_wg = threads / 64;
  // the kernel's register count lets 4 waves per SIMD (16 per CU) be resident: launch exactly the
  // resident workgroups so that each amortises its set-up over as many rows as possible
  int grid = 256 * (16 / waves_per_wg > 0 ? 16 / waves_per_wg : 1);
  if (tuning().quant_grid > 0) grid = tuning().quant_grid;
  if (grid > p.rows) grid = p.rows;
  hipLaunchKernelGGL((quantize_rows_unit_kernel<FMT, MODE, SCALED, GROUPED>), dim3(grid), dim3(threads), lds, stream, p);
  ARCQ_HIP_TRY(hipGetLastError());
  return ARCQ_OK;
}

template <int FMT, int MODE, bool SCALED, bool GROUPED = false>
int launch_quantize_wide(const QuantParams &p, hipStream_t stream) {
  const int threads = (((p.K >> 4) + 4 * 64 - 1) / (4 * 64)) * 64;  // four units per thread, whole waves
  const size_t lds = (size_t)p.K * 2;
  auto kern = quantize_rows_wide_kernel<FMT, MODE, SCALED, GROUPED>;
  if (lds > 64 * 1024 - 512)
    ARCQ_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
  // as many workgroups as the chip holds at once: four waves per SIMD by registers, 160 KB of LDS per CU
  const int by_waves = 16 / (threads / 64), by_lds = (int)((160 * 1024) / (lds + 256));
  int grid = 256 * std::max(1, std::min(by_waves, by_lds));
  if (tuning().quant_grid > 0) grid = tuning().quant_grid;
  if (grid > p.rows) grid = p.rows;
  hipLaunchKernelGGL(kern, dim3(grid), dim3(threads), lds, stream, p);
  ARCQ_HIP_TRY(hipGetLastError());
  return ARCQ_OK;
}

template <int FMT, int MODE, int KU>
int launch_quantize_wave(const QuantParams &p, hipStream_t stream) {
  constexpr int K = 1024 * KU;
  const size_t lds = (size_t)(MODE == MODE_NORM ? 3 : 1) * 2 * K + (size_t)kRowWaves * 2 * K;  // tables, row slots
  auto kern = quantize_rows_wave_kernel<FMT, MODE, KU>;
  if (lds > 64 * 1024) {
    ARCQ_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                     (int)lds));
  }
  // one workgroup of sixteen waves per CU; with more rows than that, waves walk rows with stride (waves in flight)
  int grid = (p.rows + kRowWaves - 1) / kRowWaves;
  if (grid > 256) grid = 256;
  if (tuning().quant_grid > 0) grid = tuning().quant_grid;
  hipLaunchKernelGGL(kern, dim3(grid), dim3(64 * kRowWaves), lds, stream, p);
  ARCQ_HIP_TRY(hipGetLastError());
  return ARCQ_OK;
}

// the wave-per-row kernel for (format, mode, K); -1 when it has no instance for them
int launch_quantize_wave_for(int fmt, int mode, const QuantParams &p, hipStream_t st) {
#define ARCQ_WAVE_CASE(KU)                                                                                       \
  if (p.K == 1024 * KU) {                                                                                        \
    if (fmt == ARCQ_FMT_NVFP4)                                                                                   \
      return mode == MODE_X ? launch_quantize_wave<ARCQ_FMT_NVFP4, MODE_X, KU>(p, st)                            \
                            : launch_quantize_wave<ARCQ_FMT_NVFP4, MODE_NORM, KU>(p, st);                        \
    return mode == MODE_X ? launch_quantize_wave<ARCQ_FMT_MXFP4, MODE_X, KU>(p, st)                              \
                          : launch_quantize_wave<ARCQ_FMT_MXFP4, MODE_NORM, KU>(p, st);                          \
  }
  if (mode != MODE_X && mode != MODE_NORM) return -1;
  ARCQ_WAVE_CASE(1)
  ARCQ_WAVE_CASE(2)
  ARCQ_WAVE_CASE(3)
  ARCQ_WAVE_CASE(4)
#undef ARCQ_WAVE_CASE
  return -1;
}

// tensor scale and quantizer in one launch (quantize_rows_resident_kernel); -1 when the tensor does not fit it
template <int KU, int WPR>
int launch_quantize_resident_as(const QuantParams &p, float divisor, float *d_scale, uint32_t *ws, hipStream_t st) {
  constexpr int RPW = kRowWaves / WPR;
  const size_t lds = (size_t)p.K * 2 * (1 + RPW) + 128;
  const int grid = (p.rows + RPW - 1) / RPW;
  const int spin_us = tuning().resident_spin_us;
  const uint32_t ticks = (uint32_t)(spin_us < 0 ? 0 : spin_us) * 100u;  // the wall clock counts at 100 MHz
  auto kern = quantize_rows_resident_kernel<ARCQ_FMT_NVFP4, KU, WPR>;
  if (lds > 64 * 1024)
    ARCQ_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
  hipLaunchKernelGGL(kern, dim3(grid), dim3(64 * kRowWaves), lds, st, p, divisor, ticks, ws, d_scale);
  ARCQ_HIP_TRY(hipGetLastError());
  return ARCQ_OK;
}

int launch_quantize_resident(const QuantParams &p, float divisor, float *d_scale, hipStream_t st) {
  if (p.K % 1024 != 0 || p.K > 4096) return -1;
  // As many waves per row as the rows leave room for: the workgroups must fit the chip all at once (160 KB of LDS
  // per CU, 256 CUs) and the slots they meet on.
  auto fits = [&](int wpr) {
    const int rpw = kRowWaves / wpr;
    const size_t lds = (size_t)p.K * 2 * (1 + rpw) + 128;
    const int grid = (p.rows + rpw - 1) / rpw;
    return grid <= kResidentSlots && grid <= 256 * (int)((160 * 1024) / lds);
  };
  const int ku = p.K >> 10;
  int wpr = 0;
  for (int w : {4, 2, 1})
    if (wpr == 0 && ku % w == 0 && fits(w)) wpr = w;
  if (wpr == 0) return -1;
  int status = ARCQ_OK;
  uint32_t *ws = static_cast<uint32_t *>(stream_workspace(kWsTensorScale, st, &status));
  if (!ws) return status;
  switch (ku * 10 + wpr) {
    case 11: return launch_quantize_resident_as<1, 1>(p, divisor, d_scale, ws, st);
    case 21: return launch_quantize_resident_as<2, 1>(p, divisor, d_scale, ws, st);
    case 22: return launch_quantize_resident_as<2, 2>(p, divisor, d_scale, ws, st);
    case 31: return launch_quantize_resident_as<3, 1>(p, divisor, d_scale, ws, st);
    case 41: return launch_quantize_resident_as<4, 1>(p, divisor, d_scale, ws, st);
    case 42: return launch_quantize_resident_as<4, 2>(p, divisor, d_scale, ws, st);
    case 44: return launch_quantize_resident_as<4, 4>(p, divisor, d_scale, ws, st);
  }
  return -1;
}

__global__ void check_index_kernel(const int16_t *idx, int K, int *bad) {
  extern __shared__ uint4 smem[];
  uint32_t *seen = reinterpret_cast<uint32_t *>(smem);
  for (int i = threadIdx.x; i < (K + 31) / 32; i += blockDim.x) seen[i] = 0u;
  lds_barrier();
  for (int i = threadIdx.x; i < K; i += blockDim.x) {
    const int v = idx[i];
    if (v < 0 || v >= K) {
      atomicAdd(bad, 1);
    } else {
      const uint32_t old = atomicOr(&seen[v >> 5], 1u << (v & 31));
      if (old & (1u << (v & 31))) atomicAdd(bad, 1);
    }
  }
}

template <int FMT>
__global__ __launch_bounds__(256) void dequantize_kernel(const uint8_t *codes, const uint8_t *scales, int rows, int Kp,
                                                         float *out) {
  constexpr int G = FMT == ARCQ_FMT_NVFP4 ? 16 : 32;
  const size_t total = (size_t)rows * (Kp >> 1);
  for (size_t b = (size_t)blockIdx.x * blockDim.x + threadIdx.x; b < total; b += (size_t)gridDim.x * blockDim.x) {
    const size_t r = b / (Kp >> 1);
    const int kb = (int)(b - r * (Kp >> 1));
    const uint32_t byte = codes[b];
    const uint32_t sb = scales[r * (Kp / G) + (2 * kb) / G];
    const float s = FMT == ARCQ_FMT_NVFP4 ? nvfp4_scale_value(sb) : mxfp4_scale_value(sb);
    out[r * Kp + 2 * kb] = e2m1_value(byte & 15u) * s;
    out[r * Kp + 2 * kb + 1] = e2m1_value(byte >> 4) * s;
  }
}

size_t quant_lds_bytes(int K, int mode) { return (size_t)K * 2 * (mode == MODE_NORM ? 3 : 2) + 64; }

template <int FMT, int MODE>
int launch_quantize(const QuantParams &p, hipStream_t stream) {
  const size_t lds = quant_lds_bytes(p.K, MODE);
  auto kern = quantize_rows_kernel<FMT, MODE>;
  if (lds > 64 * 1024) {
    ARCQ_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                     (int)lds));
  }
  // enough workgroups to fill 256 CUs several times over; each then streams rows/grid rows
  const int grid = p.rows < 2048 ? p.rows : 2048;
  hipLaunchKernelGGL(kern, dim3(grid), dim3(kThreads), lds, stream, p);
  ARCQ_HIP_TRY(hipGetLastError());
  return ARCQ_OK;
}

int quantize_entry(int mode, const void *x, const void *gamma, float eps, int rows, int K, const int16_t *idx, int S,
                   int fmt, float gscale, const float *d_gscale, void *codes, void *scales, void *stream) {
  if (fmt != ARCQ_FMT_NVFP4 && fmt != ARCQ_FMT_MXFP4) return ARCQ_ERR_FORMAT;
  const int G = arcq_group_size(fmt);
  if (rows < 0 || K < 32 || K % 32 != 0 || K > 32736 || S < 0 || S > K || S % G != 0) return ARCQ_ERR_SHAPE;
  if (quant_lds_bytes(K, mode) > 160 * 1024) return ARCQ_ERR_SHAPE;
  if (rows == 0) return ARCQ_OK;
  if (!x || !idx || !codes || !scales || (mode == MODE_NORM && !gamma)) return ARCQ_ERR_NULL;
  if (!aligned16(x) || !aligned16(idx) || !aligned16(codes) || (mode == MODE_NORM && !aligned16(gamma)))
    return ARCQ_ERR_ALIGN;
  QuantParams p;
  p.x = static_cast<const uint16_t *>(x);
  p.gamma = static_cast<const uint16_t *>(gamma);
  p.idx = idx;
  p.codes = static_cast<uint8_t *>(codes);
  p.scales = static_cast<uint8_t *>(scales);
  p.d_gscale = d_gscale;
  p.gscale = gscale;
  p.eps = eps;
  p.rows = rows;
  p.K = K;
  p.S = S;
  p.inv_k = 1.0 / (double)K;
  p.up = nullptr;
  p.ldx = K;
  hipStream_t st = static_cast<hipStream_t>(stream);
  // rows beyond what a thread per unit covers: four units per thread, two workgroups per CU
  if (mode != MODE_NORM && (K > 16384 || (tuning().quant_kernel == 3 && K >= 1024))) {
    const bool unit = !d_gscale && gscale == 1.0f;
#define ARCQ_WIDE(F)                                                                                         \
    if (mode == MODE_X) return unit ? launch_quantize_wide<F, MODE_X, false>(p, st) : launch_quantize_wide<F, MODE_X, true>(p, st); \
    return unit ? launch_quantize_wide<F, MODE_W, false>(p, st) : launch_quantize_wide<F, MODE_W, true>(p, st);
    if (fmt == ARCQ_FMT_NVFP4) { ARCQ_WIDE(ARCQ_FMT_NVFP4) }
    ARCQ_WIDE(ARCQ_FMT_MXFP4)
#undef ARCQ_WIDE
  }
  // tensor scale known on the host to be 1: operands are exactly bf16 -> fast kernels
  if (!d_gscale && gscale == 1.0f && K <= 16384) {
    // fused norm over many rows of a hidden size up to 4096: a wave per row, sixteen rows per CU at a time (4096
    // rows fill 256 CUs; 12.8 against 14.4 us there).  With fewer rows the workgroup-per-row kernel below keeps
    // more of the machine busy, and the plain quantizer is faster with it at any row count (9.9 against 10.5 us).
    const int qk = tuning().quant_kernel;
    if (qk != 1 && ((rows >= 3072 && mode == MODE_NORM) || qk == 2)) {
      const int rc = launch_quantize_wave_for(fmt, mode, p, st);
      if (rc >= 0) return rc;
    }
    if (fmt == ARCQ_FMT_NVFP4) {
      if (mode == MODE_X) return launch_quantize_unit<ARCQ_FMT_NVFP4, MODE_X, false>(p, st);
      if (mode == MODE_W) return launch_quantize_unit<ARCQ_FMT_NVFP4, MODE_W, false>(p, st);
      return launch_quantize_unit<ARCQ_FMT_NVFP4, MODE_NORM, false>(p, st);
    }
    if (mode == MODE_X) return launch_quantize_unit<ARCQ_FMT_MXFP4, MODE_X, false>(p, st);
    if (mode == MODE_W) return launch_quantize_unit<ARCQ_FMT_MXFP4, MODE_W, false>(p, st);
    return launch_quantize_unit<ARCQ_FMT_MXFP4, MODE_NORM, false>(p, st);
  }
  // any other tensor scale, on the host or on the device: same kernel with the two-sided encode
  if (mode != MODE_NORM && K <= 16384) {
    if (fmt == ARCQ_FMT_NVFP4) {
      if (mode == MODE_X) return launch_quantize_unit<ARCQ_FMT_NVFP4, MODE_X, true>(p, st);
      return launch_quantize_unit<ARCQ_FMT_NVFP4, MODE_W, true>(p, st);
    }
    if (mode == MODE_X) return launch_quantize_unit<ARCQ_FMT_MXFP4, MODE_X, true>(p, st);
    return launch_quantize_unit<ARCQ_FMT_MXFP4, MODE_W, true>(p, st);
  }
  if (fmt == ARCQ_FMT_NVFP4) {
    if (mode == MODE_X) return launch_quantize<ARCQ_FMT_NVFP4, MODE_X>(p, st);
    if (mode == MODE_W) return launch_quantize<ARCQ_FMT_NVFP4, MODE_W>(p, st);
    return launch_quantize<ARCQ_FMT_NVFP4, MODE_NORM>(p, st);
  }
  if (mode == MODE_X) return launch_quantize<ARCQ_FMT_MXFP4, MODE_X>(p, st);
  if (mode == MODE_W) return launch_quantize<ARCQ_FMT_MXFP4, MODE_W>(p, st);
  return launch_quantize<ARCQ_FMT_MXFP4, MODE_NORM>(p, st);
}

int swiglu_entry(const void *gate, const void *up, int ld, int rows, int K, const int16_t *idx, int S, int fmt,
                 float gscale, const float *d_gscale, void *codes, void *scales, void *stream) {
  if (fmt != ARCQ_FMT_NVFP4 && fmt != ARCQ_FMT_MXFP4) return ARCQ_ERR_FORMAT;
  const int G = arcq_group_size(fmt);
  if (rows < 0 || K < 32 || K % 32 != 0 || K > 32736 || S < 0 || S > K || S % G != 0 || ld < K || ld % 8 != 0)
    return ARCQ_ERR_SHAPE;
  if (rows == 0) return ARCQ_OK;
  if (!gate || !up || !idx || !codes || !scales) return ARCQ_ERR_NULL;
  if (!aligned16(gate) || !aligned16(up) || !aligned16(idx) || !aligned16(codes)) return ARCQ_ERR_ALIGN;
  QuantParams p;
  p.x = static_cast<const uint16_t *>(gate);
  p.up = static_cast<const uint16_t *>(up);
  p.ldx = ld;
  p.gamma = nullptr;
  p.idx = idx;
  p.codes = static_cast<uint8_t *>(codes);
  p.scales = static_cast<uint8_t *>(scales);
  p.d_gscale = d_gscale;
  p.gscale = gscale;
  p.eps = 0.0f;
  p.rows = rows;
  p.K = K;
  p.S = S;
  p.inv_k = 0.0;
  hipStream_t st = static_cast<hipStream_t>(stream);
  const bool unit = !d_gscale && gscale == 1.0f;
  if (K > 16384 || (tuning().quant_kernel == 3 && K >= 1024)) {
    if (fmt == ARCQ_FMT_NVFP4)
      return unit ? launch_quantize_wide<ARCQ_FMT_NVFP4, MODE_SWIGLU, false>(p, st)
                  : launch_quantize_wide<ARCQ_FMT_NVFP4, MODE_SWIGLU, true>(p, st);
    return unit ? launch_quantize_wide<ARCQ_FMT_MXFP4, MODE_SWIGLU, false>(p, st)
                : launch_quantize_wide<ARCQ_FMT_MXFP4, MODE_SWIGLU, true>(p, st);
  }
  if (fmt == ARCQ_FMT_NVFP4)
    return unit ? launch_quantize_unit<ARCQ_FMT_NVFP4, MODE_SWIGLU, false>(p, st)
                : launch_quantize_unit<ARCQ_FMT_NVFP4, MODE_SWIGLU, true>(p, st);
  return unit ? launch_quantize_unit<ARCQ_FMT_MXFP4, MODE_SWIGLU, false>(p, st)
              : launch_quantize_unit<ARCQ_FMT_MXFP4, MODE_SWIGLU, true>(p, st);
}

// grouped forms of reorder_quantize_x / swiglu_quantize_x: rows sorted by segment, segment offsets on the device
int grouped_quantize_entry(int mode, const void *x, const void *up, int ld, int rows, int K, const int *seg, int n_seg,
                           const int16_t *idx, int S, int fmt, const float *d_gscales, void *codes, void *scales,
                           void *stream) {
  if (fmt != ARCQ_FMT_NVFP4 && fmt != ARCQ_FMT_MXFP4) return ARCQ_ERR_FORMAT;
  const int G = arcq_group_size(fmt);
  if (rows < 0 || n_seg < 1 || K < 32 || K % 32 != 0 || K > 32736 || S < 0 || S > K || S % G != 0 || ld < K || ld % 8 != 0)
    return ARCQ_ERR_SHAPE;
  if (rows == 0) return ARCQ_OK;
  if (!x || !seg || !idx || !codes || !scales || (mode == MODE_SWIGLU && !up)) return ARCQ_ERR_NULL;
  if (!aligned16(x) || !aligned16(idx) || !aligned16(codes) || (mode == MODE_SWIGLU && !aligned16(up))) return ARCQ_ERR_ALIGN;
  QuantParams p;
  p.x = static_cast<const uint16_t *>(x);
  p.up = static_cast<const uint16_t *>(up);
  p.ldx = ld;
  p.gamma = nullptr;
  p.idx = idx;
  p.codes = static_cast<uint8_t *>(codes);
  p.scales = static_cast<uint8_t *>(scales);
  p.d_gscale = d_gscales;
  p.gscale = 1.0f;
  p.eps = 0.0f;
  p.rows = rows;
  p.K = K;
  p.S = S;
  p.inv_k = 0.0;
  p.seg = seg;
  p.n_seg = n_seg;
  hipStream_t st = static_cast<hipStream_t>(stream);
  const bool unit = d_gscales == nullptr;
  if (K > 16384) {
    if (mode == MODE_X && ld != K) return ARCQ_ERR_SHAPE;
#define ARCQ_WIDE_G(F, MD) return unit ? launch_quantize_wide<F, MD, false, true>(p, st) : launch_quantize_wide<F, MD, true, true>(p, st);
    if (mode == MODE_X) {
      if (fmt == ARCQ_FMT_NVFP4) { ARCQ_WIDE_G(ARCQ_FMT_NVFP4, MODE_X) }
      ARCQ_WIDE_G(ARCQ_FMT_MXFP4, MODE_X)
    }
    if (fmt == ARCQ_FMT_NVFP4) { ARCQ_WIDE_G(ARCQ_FMT_NVFP4, MODE_SWIGLU) }
    ARCQ_WIDE_G(ARCQ_FMT_MXFP4, MODE_SWIGLU)
#undef ARCQ_WIDE_G
  }
  if (mode == MODE_X) {
    if (ld != K) return ARCQ_ERR_SHAPE;
    if (fmt == ARCQ_FMT_NVFP4)
      return unit ? launch_quantize_unit<ARCQ_FMT_NVFP4, MODE_X, false, true>(p, st)
                  : launch_quantize_unit<ARCQ_FMT_NVFP4, MODE_X, true, true>(p, st);
    return unit ? launch_quantize_unit<ARCQ_FMT_MXFP4, MODE_X, false, true>(p, st)
                : launch_quantize_unit<ARCQ_FMT_MXFP4, MODE_X, true, true>(p, st);
  }
  if (fmt == ARCQ_FMT_NVFP4)
    return unit ? launch_quantize_unit<ARCQ_FMT_NVFP4, MODE_SWIGLU, false, true>(p, st)
                : launch_quantize_unit<ARCQ_FMT_NVFP4, MODE_SWIGLU, true, true>(p, st);
  return unit ? launch_quantize_unit<ARCQ_FMT_MXFP4, MODE_SWIGLU, false, true>(p, st)
              : launch_quantize_unit<ARCQ_FMT_MXFP4, MODE_SWIGLU, true, true>(p, st);
}

}  // namespace
}  // namespace arcq

extern "C" {

int arcq_group_size(int fmt) { return fmt == ARCQ_FMT_NVFP4 ? 16 : (fmt == ARCQ_FMT_MXFP4 ? 32 : 0); }

size_t arcq_codes_bytes(int rows, int K, int select_num) { return (size_t)rows * (size_t)((K + select_num) / 2); }

size_t arcq_scales_bytes(int rows, int K, int select_num, int fmt) {
  const int G = arcq_group_size(fmt);
  return G ? (size_t)rows * (size_t)((K + select_num) / G) : 0;
}

int arcq_reorder_quantize_x(const void *x, int M, int K, const int16_t *reorder_index, int select_num, int fmt,
                            float global_scale, const float *d_global_scale, void *codes, void *scales,
                            void *stream) {
  return arcq::quantize_entry(arcq::MODE_X, x, nullptr, 0.0f, M, K, reorder_index, select_num, fmt, global_scale,
                              d_global_scale, codes, scales, stream);
}

int arcq_reorder_quantize_w(const void *w, int N, int K, const int16_t *reorder_index, int select_num, int fmt,
                            float global_scale, const float *d_global_scale, void *codes, void *scales,
                            void *stream) {
  return arcq::quantize_entry(arcq::MODE_W, w, nullptr, 0.0f, N, K, reorder_index, select_num, fmt, global_scale,
                              d_global_scale, codes, scales, stream);
}

int arcq_rmsnorm_quantize_x(const void *x, const void *gamma, float eps, int M, int K,
                            const int16_t *reorder_index, int select_num, int fmt, float global_scale,
                            const float *d_global_scale, void *codes, void *scales, void *stream) {
  return arcq::quantize_entry(arcq::MODE_NORM, x, gamma, eps, M, K, reorder_index, select_num, fmt, global_scale,
                              d_global_scale, codes, scales, stream);
}

int arcq_check_index(const int16_t *reorder_index, int K, void *stream) {
  if (!reorder_index) return ARCQ_ERR_NULL;
  if (K <= 0 || K > 32767) return ARCQ_ERR_SHAPE;
  hipStream_t st = static_cast<hipStream_t>(stream);
  int *d_bad = nullptr;
  ARCQ_HIP_TRY(hipMalloc(&d_bad, sizeof(int)));
  int bad = 0;
  hipError_t e = hipMemcpyAsync(d_bad, &bad, sizeof(int), hipMemcpyHostToDevice, st);
  if (e == hipSuccess) {
    hipLaunchKernelGGL(arcq::check_index_kernel, dim3(1), dim3(256), ((K + 31) / 32) * 4 + 16, st, reorder_index, K,
                       d_bad);
    e = hipGetLastError();
  }
  if (e == hipSuccess) e = hipMemcpyAsync(&bad, d_bad, sizeof(int), hipMemcpyDeviceToHost, st);
  if (e == hipSuccess) e = hipStreamSynchronize(st);
  (void)hipFree(d_bad);
  if (e != hipSuccess) return arcq::note_hip_error(e);
  return bad ? ARCQ_ERR_INDEX : ARCQ_OK;
}

int arcq_swiglu_quantize_x(const void *gate, const void *up, int ld, int M, int K, const int16_t *reorder_index,
                           int select_num, int fmt, float global_scale, const float *d_global_scale, void *codes,
                           void *scales, void *stream) {
  return arcq::swiglu_entry(gate, up, ld, M, K, reorder_index, select_num, fmt, global_scale, d_global_scale, codes,
                            scales, stream);
}

int arcq_swiglu_absmax(const void *gate, const void *up, int ld, int M, int K, float *d_absmax, void *stream) {
  if (M < 0 || K < 8 || K % 8 != 0 || ld < K || ld % 8 != 0) return ARCQ_ERR_SHAPE;
  if (M == 0) return ARCQ_OK;
  if (!gate || !up || !d_absmax) return ARCQ_ERR_NULL;
  if (!arcq::aligned16(gate) || !arcq::aligned16(up)) return ARCQ_ERR_ALIGN;
  const size_t chunks = (size_t)M * (K >> 3);
  const int grid = (int)((chunks + 255) / 256 < 4096 ? (chunks + 255) / 256 : 4096);
  hipLaunchKernelGGL(arcq::swiglu_absmax_kernel, dim3(grid), dim3(256), 0, static_cast<hipStream_t>(stream),
                     static_cast<const uint16_t *>(gate), static_cast<const uint16_t *>(up), (size_t)ld, M, K,
                     reinterpret_cast<uint32_t *>(d_absmax));
  ARCQ_HIP_TRY(hipGetLastError());
  return ARCQ_OK;
}

int arcq_tensor_scale(const void *x, const void *up, int ld, int M, int K, float divisor, float *d_scale, void *stream) {
  if (M < 0 || K < 8 || K % 8 != 0 || ld < K || ld % 8 != 0 || !(divisor > 0.0f)) return ARCQ_ERR_SHAPE;
  if (!x || !d_scale) return ARCQ_ERR_NULL;
  if (!arcq::aligned16(x) || (up && !arcq::aligned16(up))) return ARCQ_ERR_ALIGN;
  hipStream_t st = static_cast<hipStream_t>(stream);
  int status = ARCQ_OK;
  uint32_t *ws = static_cast<uint32_t *>(arcq::stream_workspace(arcq::kWsTensorScale, st, &status));
  if (!ws) return status;
  const size_t chunks = (size_t)M * (K >> 3);
  // at most one workgroup per CU; 512 threads x 8 chunks each while one trip of that covers the tensor (small
  // tensors: fewer waves to meet at the end), 1024 threads beyond
  const int threads = chunks <= (size_t)256 * 512 * 8 ? 512 : arcq::kScaleThreads;
  const size_t per_wg = (size_t)threads * 8;
  int grid = (int)std::min<size_t>(256, (chunks + per_wg - 1) / per_wg);
  if (grid < 1) grid = 1;  // M == 0: one block writes the scale of an empty tensor, 1
  if (up)
    hipLaunchKernelGGL(arcq::tensor_scale_kernel<true>, dim3(grid), dim3(threads), 0, st,
                       static_cast<const uint16_t *>(x), static_cast<const uint16_t *>(up), (size_t)ld, M, K, divisor, ws, d_scale);
  else
    hipLaunchKernelGGL(arcq::tensor_scale_kernel<false>, dim3(grid), dim3(threads), 0, st,
                       static_cast<const uint16_t *>(x), static_cast<const uint16_t *>(nullptr), (size_t)ld, M, K, divisor, ws,
                       d_scale);
  ARCQ_HIP_TRY(hipGetLastError());
  return ARCQ_OK;
}

int arcq_reorder_quantize_x_absmax(const void *x, int M, int K, const int16_t *reorder_index, int select_num, int fmt,
                                   float divisor, float *d_scale, void *codes, void *scales, void *stream) {
  if (fmt != ARCQ_FMT_NVFP4 && fmt != ARCQ_FMT_MXFP4) return ARCQ_ERR_FORMAT;
  const int G = arcq_group_size(fmt);
  if (M < 0 || K < 32 || K % 32 != 0 || K > 32736 || select_num < 0 || select_num > K || select_num % G != 0 || !(divisor > 0.0f))
    return ARCQ_ERR_SHAPE;
  if (!d_scale || (M > 0 && (!x || !reorder_index || !codes || !scales))) return ARCQ_ERR_NULL;
  if (M > 0 && (!arcq::aligned16(x) || !arcq::aligned16(reorder_index) || !arcq::aligned16(codes))) return ARCQ_ERR_ALIGN;
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (M == 0) {  // an empty tensor: nothing to quantize, scale 1 (one workgroup of the scale kernel over no rows)
    int status = ARCQ_OK;
    uint32_t *ws = static_cast<uint32_t *>(arcq::stream_workspace(arcq::kWsTensorScale, st, &status));
    if (!ws) return status;
    hipLaunchKernelGGL(arcq::tensor_scale_kernel<false>, dim3(1), dim3(512), 0, st, static_cast<const uint16_t *>(nullptr),
                       static_cast<const uint16_t *>(nullptr), (size_t)K, 0, K, divisor, ws, d_scale);
    ARCQ_HIP_TRY(hipGetLastError());
    return ARCQ_OK;
  }
  if (fmt == ARCQ_FMT_NVFP4 && arcq::tuning().resident_spin_us >= 0) {
    arcq::QuantParams p;
    p.x = static_cast<const uint16_t *>(x);
    p.gamma = nullptr;
    p.up = nullptr;
    p.ldx = K;
    p.idx = reorder_index;
    p.codes = static_cast<uint8_t *>(codes);
    p.scales = static_cast<uint8_t *>(scales);
    p.d_gscale = nullptr;
    p.gscale = 1.0f;
    p.eps = 0.0f;
    p.rows = M;
    p.K = K;
    p.S = select_num;
    p.inv_k = 1.0 / (double)K;
    const int rc = arcq::launch_quantize_resident(p, divisor, d_scale, st);
    if (rc >= 0) return rc;
  }
  // tensors beyond the chip's LDS, other row lengths, MXFP4: the scale, then the quantizer under it
  const int rc = arcq_tensor_scale(x, nullptr, K, M, K, divisor, d_scale, stream);
  if (rc != ARCQ_OK) return rc;
  return arcq::quantize_entry(arcq::MODE_X, x, nullptr, 0.0f, M, K, reorder_index, select_num, fmt, 1.0f, d_scale, codes, scales,
                              stream);
}

int arcq_grouped_reorder_quantize_x(const void *x, int M, int K, const int *seg_offsets, int n_seg,
                                    const int16_t *reorder_index, int select_num, int fmt, const float *d_global_scales,
                                    void *codes, void *scales, void *stream) {
  return arcq::grouped_quantize_entry(arcq::MODE_X, x, nullptr, K, M, K, seg_offsets, n_seg, reorder_index, select_num, fmt,
                                      d_global_scales, codes, scales, stream);
}

int arcq_grouped_swiglu_quantize_x(const void *gate, const void *up, int ld, int M, int K, const int *seg_offsets, int n_seg,
                                   const int16_t *reorder_index, int select_num, int fmt, const float *d_global_scales,
                                   void *codes, void *scales, void *stream) {
  return arcq::grouped_quantize_entry(arcq::MODE_SWIGLU, gate, up, ld, M, K, seg_offsets, n_seg, reorder_index, select_num,
                                      fmt, d_global_scales, codes, scales, stream);
}

int arcq_grouped_tensor_scale(const void *x, const void *up, int ld, int M, int K, const int *seg_offsets, int n_seg,
                              float divisor, float *d_scales, void *stream) {
  if (M < 0 || n_seg < 1 || K < 8 || K % 8 != 0 || ld < K || ld % 8 != 0 || !(divisor > 0.0f)) return ARCQ_ERR_SHAPE;
  if (!d_scales || !seg_offsets || (M > 0 && !x)) return ARCQ_ERR_NULL;
  if (M > 0 && (!arcq::aligned16(x) || (up && !arcq::aligned16(up)))) return ARCQ_ERR_ALIGN;
  hipStream_t st = static_cast<hipStream_t>(stream);
  uint32_t *bits = reinterpret_cast<uint32_t *>(d_scales);
  const int fin = (n_seg + 255) / 256;
  hipLaunchKernelGGL(arcq::zero_words_kernel, dim3(fin), dim3(256), 0, st, bits, n_seg);
  if (M > 0) {
    const int grid = std::min(1024, (M + 7) / 8);  // eight or more contiguous rows per workgroup
    if (up)
      hipLaunchKernelGGL(arcq::grouped_absmax_kernel<true>, dim3(grid), dim3(256), 0, st, static_cast<const uint16_t *>(x),
                         static_cast<const uint16_t *>(up), (size_t)ld, M, K, seg_offsets, n_seg, bits);
    else
      hipLaunchKernelGGL(arcq::grouped_absmax_kernel<false>, dim3(grid), dim3(256), 0, st, static_cast<const uint16_t *>(x),
                         static_cast<const uint16_t *>(nullptr), (size_t)ld, M, K, seg_offsets, n_seg, bits);
  }
  hipLaunchKernelGGL(arcq::grouped_scale_finish_kernel, dim3(fin), dim3(256), 0, st, bits, n_seg, divisor);
  ARCQ_HIP_TRY(hipGetLastError());
  return ARCQ_OK;
}

int arcq_dequantize(const void *codes, const void *scales, int rows, int Kp, int fmt, float *out, void *stream) {
  const int G = arcq_group_size(fmt);
  if (!G) return ARCQ_ERR_FORMAT;
  if (rows < 0 || Kp <= 0 || Kp % G) return ARCQ_ERR_SHAPE;
  if (rows == 0) return ARCQ_OK;
  if (!codes || !scales || !out) return ARCQ_ERR_NULL;
  hipStream_t st = static_cast<hipStream_t>(stream);
  const size_t total = (size_t)rows * (Kp / 2);
  const int grid = (int)((total + 255) / 256 < 4096 ? (total + 255) / 256 : 4096);
  if (fmt == ARCQ_FMT_NVFP4)
    hipLaunchKernelGGL(arcq::dequantize_kernel<ARCQ_FMT_NVFP4>, dim3(grid), dim3(256), 0, st,
                       static_cast<const uint8_t *>(codes), static_cast<const uint8_t *>(scales), rows, Kp, out);
  else
    hipLaunchKernelGGL(arcq::dequantize_kernel<ARCQ_FMT_MXFP4>, dim3(grid), dim3(256), 0, st,
                       static_cast<const uint8_t *>(codes), static_cast<const uint8_t *>(scales), rows, Kp, out);
  ARCQ_HIP_TRY(hipGetLastError());
  return ARCQ_OK;
}

}  // extern "C"
