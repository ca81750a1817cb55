// arcq_swiglu.h -- device helpers shared by the quantizers and the GEMM epilogue: bf16 packing, the exact
// bf16 x bf16 product through the dot instruction, and act_fn(gate) * up as the reference's layers form it.
#ifndef ARCQ_SWIGLU_H_
#define ARCQ_SWIGLU_H_
#include <hip/hip_runtime.h>

#include "arcq_math.h"

namespace arcq {

typedef __bf16 v2bf __attribute__((ext_vector_type(2)));
typedef float v2f __attribute__((ext_vector_type(2)));

__device__ __forceinline__ uint32_t pack_bf16_rne(float lo, float hi) {
  const v2f v = {lo, hi};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, v2bf));  // v_cvt_pk_bf16_f32
}

// gamma * h for the two bf16 halves of one register: v_dot2_f32_bf16 with the other half of the
// gamma operand zeroed gives the exact fp32 product without unpacking h
__device__ __forceinline__ float dot2_bf16(uint32_t a, uint32_t b) {
  // the builtin, not a bare inline-asm instruction: the compiler then sees a dot instruction and
  // keeps the wait states its result needs before another kind of instruction may read it
  return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(v2bf, a), __builtin_bit_cast(v2bf, b), 0.0f, false);
}

// act_fn(gate) * up as the reference's layers form it in bf16 (model/qLlamaLayer.py:432,
// model/qMixtralLayer.py:531): SiLU evaluated in fp32 as x / (1 + exp(-x)) and rounded to bf16,
// then a bf16 multiply (fp32 product, one rounding).  Two elements per call, packed.
// The SiLU of a bf16 value has only 65536 possible inputs: the hardware estimates
// x * rcp(1 + exp2(-x * log2 e)) round to the same bf16 as the library expression for every one of them
// except 5.9375 and -87.5, -88, -88.5 (all 65536 inputs compared on the GPU; a test repeats it).  Waves
// that hold one of those, anything of magnitude >= 87, or a NaN take the library expression.
__device__ __forceinline__ uint32_t silu_pair_bf16(uint32_t gw) {
  const float g0 = u2f(gw << 16), g1 = u2f(gw & 0xffff0000u);
  const uint32_t m0 = gw & 0x7fffu, m1 = (gw >> 16) & 0x7fffu;
  const bool special = m0 >= 0x42aeu || m1 >= 0x42aeu || (gw & 0xffffu) == 0x40beu || (gw >> 16) == 0x40beu;
  if (__builtin_amdgcn_ballot_w64(special) != 0)
    return pack_bf16_rne(g0 / (1.0f + expf(-g0)), g1 / (1.0f + expf(-g1)));
  const float e0 = __builtin_amdgcn_exp2f(g0 * -1.4426950408889634f), e1 = __builtin_amdgcn_exp2f(g1 * -1.4426950408889634f);
  return pack_bf16_rne(g0 * __builtin_amdgcn_rcpf(1.0f + e0), g1 * __builtin_amdgcn_rcpf(1.0f + e1));
}

__device__ __forceinline__ uint32_t swiglu_pair(uint32_t gw, uint32_t uw) {
  const uint32_t a = silu_pair_bf16(gw);
  // The dot instruction adds (other half) * 0 to each product: an infinite or NaN activation in one half would
  // turn its neighbour's product into NaN where torch's elementwise multiply leaves it alone.  Waves that hold
  // one (a vote, as for the special values above) multiply the unpacked halves instead: the same bits otherwise.
  const bool nonfinite = (a & 0x7f80u) == 0x7f80u || (a & 0x7f800000u) == 0x7f800000u;
  if (__builtin_amdgcn_ballot_w64(nonfinite) != 0)
    return pack_bf16_rne(u2f(a << 16) * u2f(uw << 16), u2f(a & 0xffff0000u) * u2f(uw & 0xffff0000u));
  return pack_bf16_rne(dot2_bf16(a, uw & 0xffffu), dot2_bf16(a, uw & 0xffff0000u));
}

}  // namespace arcq
#endif  // ARCQ_SWIGLU_H_
