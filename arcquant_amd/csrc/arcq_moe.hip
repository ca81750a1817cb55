// arcq_moe.hip -- the last step of a mixture-of-experts block for gfx950: every token's expert outputs,
// weighted by the router and summed (model/qMixtralLayer.py:466-471: `expert(x) * routing_weights`, then
// final_hidden_states.index_add_ per expert).  HBM-bound: each expert-output row is read once, each token
// row written once, 16 bytes per lane.
#include <hip/hip_runtime.h>

#include "arcq_internal.h"
#include "arcq_math.h"

namespace arcq {
namespace {

constexpr int kMaxTopK = 8;

// y [pairs, H]: expert outputs in expert-sorted order; position[t * top_k + j]: row of y that holds token t's
// j-th expert; weight [pairs]: router weights in the same sorted order.  The reference adds expert after
// expert, in ascending expert number, into a bf16 tensor of zeros: out = bf16(bf16(0 + p_a) + p_b) ... with
// p = bf16(y * w).  Ascending expert number is ascending sorted position, so a token's positions are sorted
// first; every partial sum is rounded to bf16 as the reference's in-place adds are.
__global__ __launch_bounds__(256) void moe_combine_kernel(const uint16_t *y, const int64_t *position, const uint16_t *weight,
                                                          int tokens, int H, int top_k, int pairs, uint16_t *out) {
  const int t = blockIdx.x;
  int pos[kMaxTopK];
  float w[kMaxTopK];
#pragma unroll
  for (int j = 0; j < kMaxTopK; ++j) {
    pos[j] = 0x7fffffff;
    if (j < top_k) {
      const int64_t p = position[(size_t)t * top_k + j];
      pos[j] = (p >= 0 && p < pairs) ? (int)p : 0x7fffffff;  // a position outside y contributes nothing
    }
  }
#pragma unroll
  for (int a = 0; a < kMaxTopK; ++a)  // sort ascending (fixed network of compare-exchanges; absent slots stay last)
#pragma unroll
    for (int b = 0; b + 1 < kMaxTopK - a; ++b)
      if (pos[b + 1] < pos[b]) {
        const int s = pos[b];
        pos[b] = pos[b + 1];
        pos[b + 1] = s;
      }
#pragma unroll
  for (int j = 0; j < kMaxTopK; ++j) w[j] = pos[j] != 0x7fffffff ? bf16_bits_to_f32(weight[pos[j]]) : 0.0f;
  for (int c = threadIdx.x; c < (H >> 3); c += 256) {
    uint4 v[kMaxTopK];
#pragma unroll
    for (int j = 0; j < kMaxTopK; ++j)
      if (j < top_k && pos[j] != 0x7fffffff) v[j] = *reinterpret_cast<const uint4 *>(y + (size_t)pos[j] * H + 8 * c);
    float acc[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) acc[i] = 0.0f;
#pragma unroll
    for (int j = 0; j < kMaxTopK; ++j) {
      if (j >= top_k || pos[j] == 0x7fffffff) continue;
      const uint32_t q[4] = {v[j].x, v[j].y, v[j].z, v[j].w};
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float p0 = bf16_bits_to_f32(f32_to_bf16_bits(bf16_bits_to_f32(q[i] & 0xffffu) * w[j]));
        const float p1 = bf16_bits_to_f32(f32_to_bf16_bits(bf16_bits_to_f32(q[i] >> 16) * w[j]));
        acc[2 * i] = bf16_bits_to_f32(f32_to_bf16_bits(acc[2 * i] + p0));
        acc[2 * i + 1] = bf16_bits_to_f32(f32_to_bf16_bits(acc[2 * i + 1] + p1));
      }
    }
    uint4 o;
    o.x = f32_to_bf16_bits(acc[0]) | (f32_to_bf16_bits(acc[1]) << 16);
    o.y = f32_to_bf16_bits(acc[2]) | (f32_to_bf16_bits(acc[3]) << 16);
    o.z = f32_to_bf16_bits(acc[4]) | (f32_to_bf16_bits(acc[5]) << 16);
    o.w = f32_to_bf16_bits(acc[6]) | (f32_to_bf16_bits(acc[7]) << 16);
    *reinterpret_cast<uint4 *>(out + (size_t)t * H + 8 * c) = o;
  }
}

}  // namespace
}  // namespace arcq

extern "C" int arcq_moe_combine(const void *y, const int64_t *position, const void *weight, int tokens, int H, int top_k,
                                int pairs, void *out, void *stream) {
  using namespace arcq;
  if (tokens < 0 || H < 8 || H % 8 != 0 || top_k < 1 || top_k > kMaxTopK || pairs < 0) return ARCQ_ERR_SHAPE;
  if (tokens == 0) return ARCQ_OK;
  if (!y || !position || !weight || !out) return ARCQ_ERR_NULL;
  if (!aligned16(y) || !aligned16(out)) return ARCQ_ERR_ALIGN;
  hipLaunchKernelGGL(moe_combine_kernel, dim3(tokens), dim3(256), 0, static_cast<hipStream_t>(stream),
                     static_cast<const uint16_t *>(y), position, static_cast<const uint16_t *>(weight), tokens, H, top_k, pairs,
                     static_cast<uint16_t *>(out));
  ARCQ_HIP_TRY(hipGetLastError());
  return ARCQ_OK;
}
