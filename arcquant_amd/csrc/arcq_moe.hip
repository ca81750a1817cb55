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

// ---------------------------------------------------------------------------------------------
// Routing (model/qMixtralLayer.py:441-452: softmax over the experts in fp32, top-k, the k weights divided by
// their sum and cast to the activations' type; :456-471 then walks the experts and the tokens routed to each).
// Two launches (three beyond 16384 tokens) replace a dozen of torch's: per token the choice and its weights, per (token, slot) pair its row
// in the expert-sorted order (pairs of one expert in ascending pair number, as a stable sort by expert gives),
// the expert segments, and the sorted views of token number and weight the grouped launches read.
//
// Arithmetic follows torch's on this device so that the weights come out as the same bits: maximum and sum of
// exp(l - max) as the butterfly over the next power of two that its warp softmax forms (padding adds zeros),
// exp(l - max) / sum, top-k weights divided by their sum left to right (exact for k = 2, the Mixtral case).
// Equal probabilities: the lower expert number wins (torch.topk leaves the choice among equals unspecified).
// Non-finite logits (a NaN, a +inf, or a row of -inf) make every probability of the row NaN, as in torch; the
// choice stays total -- NaN ranks above every number, as torch.topk orders it, and equals again go to the lower
// expert -- so every pair names an expert in [0, E), is counted in the histograms and gets a row; only that
// token's weights, and through them its output, are NaN.
// ---------------------------------------------------------------------------------------------
constexpr int kMaxExperts = 64;
constexpr int kRouteThreads = 64;

template <bool F32, int P>  // P: the power of two the experts are padded to
__global__ __launch_bounds__(kRouteThreads) void moe_route_choose_kernel(const void *logits, int T, int E, int top_k, int *sel,
                                                                         uint16_t *w, int64_t *position, int *hist) {
  __shared__ int cnt[kRouteThreads / 64][kMaxExperts];
  const int t = blockIdx.x * kRouteThreads + threadIdx.x;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const bool live = t < T;
  float prob[P];
  int my[kMaxTopK];
  float mw[kMaxTopK];
#pragma unroll
  for (int j = 0; j < kMaxTopK; ++j) { my[j] = -1; mw[j] = 0.0f; }
  if (live) {
    float v[P];
#pragma unroll
    for (int e = 0; e < P; ++e) {
      float x = -__builtin_inff();
      if (e < E)
        x = F32 ? static_cast<const float *>(logits)[(size_t)t * E + e]
                : bf16_bits_to_f32(static_cast<const uint16_t *>(logits)[(size_t)t * E + e]);
      v[e] = x;
    }
    float mx = v[0];
#pragma unroll
    for (int e = 1; e < P; ++e) mx = fmaxf(mx, v[e]);  // the padding is -inf
    float red[P];
#pragma unroll
    for (int e = 0; e < P; ++e) {
      prob[e] = e < E ? expf(v[e] - mx) : 0.0f;
      red[e] = prob[e];
    }
#pragma unroll
    for (int off = P >> 1; off > 0; off >>= 1) {  // lane i of the butterfly: red[i] + red[i ^ off]
      float nxt[P];
#pragma unroll
      for (int e = 0; e < P; ++e) nxt[e] = red[e] + red[e ^ off];
#pragma unroll
      for (int e = 0; e < P; ++e) red[e] = nxt[e];
    }
    const float sum = red[0];
#pragma unroll
    for (int e = 0; e < P; ++e) prob[e] = e < E ? prob[e] / sum : -1.0f;
    // top-k: k passes over the probabilities, the largest not yet taken, ties to the lower expert number
    float tot = 0.0f;
    for (int j = 0; j < top_k; ++j) {
      int best = -1;
      float bv = -1.0f;
#pragma unroll
      for (int e = 0; e < P; ++e) {
        bool taken = false;
#pragma unroll
        for (int q = 0; q < kMaxTopK; ++q) taken |= q < j && my[q] == e;
        const bool above = prob[e] != prob[e] ? bv == bv : prob[e] > bv;  // NaN above every number, not above NaN
        if (e < E && !taken && (best < 0 || above)) { bv = prob[e]; best = e; }
      }
      my[j] = best;
      mw[j] = bv;
      tot = j == 0 ? bv : tot + bv;
    }
    for (int j = 0; j < top_k; ++j) {
      sel[(size_t)t * top_k + j] = my[j];
      w[(size_t)t * top_k + j] = (uint16_t)f32_to_bf16_bits(mw[j] / tot);
    }
  }
  // rank of every pair among the pairs of its expert inside this workgroup, in pair order
  int rank[kMaxTopK];
#pragma unroll
  for (int j = 0; j < kMaxTopK; ++j) rank[j] = 0;
  const unsigned long long below = lane == 0 ? 0ull : (~0ull >> (64 - lane));
  for (int e = 0; e < E; ++e) {
    int wave_cnt = 0, before_me = 0;
    for (int j = 0; j < top_k; ++j) {
      const unsigned long long m = __builtin_amdgcn_ballot_w64(live && my[j] == e);
      wave_cnt += __builtin_popcountll(m);
      before_me += __builtin_popcountll(m & below);
    }
    for (int j = 0; j < top_k; ++j)
      if (my[j] == e) rank[j] = before_me;  // a token takes an expert once: no earlier slot of its own to count
    if (lane == 0) cnt[wave][e] = wave_cnt;
  }
  __syncthreads();
  if (live)
    for (int j = 0; j < top_k; ++j) {
      int base = 0;
      for (int q = 0; q < wave; ++q) base += cnt[q][my[j]];
      position[(size_t)t * top_k + j] = base + rank[j];  // finished by the second launch
    }
  if (threadIdx.x < E) {
    int tot = 0;
    for (int q = 0; q < kRouteThreads / 64; ++q) tot += cnt[q][threadIdx.x];
    hist[(size_t)blockIdx.x * E + threadIdx.x] = tot;
  }
}

// Many tokens (more than kScanFromBlocks workgroups of the first launch): every workgroup of the placing launch
// summing the whole histogram would be quadratic in the token count.  One workgroup turns the histograms
// [blocks][E] into running sums over the earlier workgroups, expert by expert (a thread adds up a contiguous
// run of workgroups, the runs' sums are scanned in LDS, the thread writes its run's prefixes back), and writes
// the segments; the placing launch then reads E words per workgroup.
constexpr int kScanThreads = 256;
constexpr int kScanFromBlocks = 256;

__global__ __launch_bounds__(kScanThreads) void moe_route_scan_kernel(int blocks, int E, int *hist, int *seg) {
  __shared__ int part[kScanThreads];
  __shared__ int total[kMaxExperts];
  const int run = (blocks + kScanThreads - 1) / kScanThreads;
  const int b0 = (int)threadIdx.x * run, b1 = min(blocks, b0 + run);
  for (int e = 0; e < E; ++e) {
    int sum = 0;
    for (int b = b0; b < b1; ++b) sum += hist[(size_t)b * E + e];
    part[threadIdx.x] = sum;
    __syncthreads();
    for (int off = 1; off < kScanThreads; off <<= 1) {  // inclusive scan of the runs' sums
      const int add = (int)threadIdx.x >= off ? part[threadIdx.x - off] : 0;
      __syncthreads();
      part[threadIdx.x] += add;
      __syncthreads();
    }
    int before = part[threadIdx.x] - sum;
    for (int b = b0; b < b1; ++b) {
      const int v = hist[(size_t)b * E + e];
      hist[(size_t)b * E + e] = before;
      before += v;
    }
    if (threadIdx.x == kScanThreads - 1) total[e] = part[threadIdx.x];
    __syncthreads();
  }
  if (threadIdx.x == 0) {
    int at = 0;
    for (int e = 0; e < E; ++e) {
      seg[e] = at;
      at += total[e];
    }
    seg[E] = at;
  }
}

template <bool SCANNED>
__global__ __launch_bounds__(kRouteThreads) void moe_route_place_kernel(int T, int E, int top_k, const int *sel, const uint16_t *w,
                                                                        const int *hist, int64_t *position, int *seg, int *tok,
                                                                        uint16_t *ws) {
  __shared__ int start[kMaxExperts];  // first sorted row of this workgroup's pairs of expert e
  __shared__ int total[kMaxExperts], earlier[kMaxExperts];
  if (SCANNED) {  // hist holds the sums over the earlier workgroups, seg is final
    if ((int)threadIdx.x < E) start[threadIdx.x] = seg[threadIdx.x] + hist[(size_t)blockIdx.x * E + threadIdx.x];
    __syncthreads();
    const int t = blockIdx.x * kRouteThreads + threadIdx.x;
    if (t >= T) return;
    for (int j = 0; j < top_k; ++j) {
      const size_t pair = (size_t)t * top_k + j;
      if ((unsigned)sel[pair] >= (unsigned)E) continue;
      const int64_t pos = start[sel[pair]] + position[pair];
      position[pair] = pos;
      tok[pos] = t;
      ws[pos] = w[pair];
    }
    return;
  }
  if (threadIdx.x < kMaxExperts) total[threadIdx.x] = earlier[threadIdx.x] = 0;
  __syncthreads();
  // The histograms [workgroups][E] were written on other XCDs and come from memory: a lane takes eight of
  // their words at a time, all eight loads in flight together, and adds them to the experts' sums in LDS.
  const int words = (int)gridDim.x * E, mine = (int)blockIdx.x * E;  // words below `mine` belong to earlier workgroups
  for (int f0 = 0; f0 < words; f0 += 8 * kRouteThreads) {
    int v[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const int fl = f0 + u * kRouteThreads + (int)threadIdx.x;
      v[u] = fl < words ? hist[fl] : 0;
    }
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const int fl = f0 + u * kRouteThreads + (int)threadIdx.x;
      if (fl < words && v[u]) {
        atomicAdd(&total[fl % E], v[u]);
        if (fl < mine) atomicAdd(&earlier[fl % E], v[u]);
      }
    }
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    int run = 0;
    for (int e = 0; e < E; ++e) {
      start[e] = run + earlier[e];
      if (blockIdx.x == 0) seg[e] = run;
      run += total[e];
    }
    if (blockIdx.x == 0) seg[E] = run;
  }
  __syncthreads();
  const int t = blockIdx.x * kRouteThreads + threadIdx.x;
  if (t >= T) return;
  for (int j = 0; j < top_k; ++j) {
    const size_t pair = (size_t)t * top_k + j;
    if ((unsigned)sel[pair] >= (unsigned)E) continue;  // cannot happen with the choice above; never index LDS with it
    const int64_t pos = start[sel[pair]] + position[pair];
    position[pair] = pos;
    tok[pos] = t;
    ws[pos] = w[pair];
  }
}

}  // namespace
}  // namespace arcq

extern "C" size_t arcq_moe_route_workspace_bytes(int tokens, int experts) {
  if (tokens < 0 || experts < 1) return 0;
  const int blocks = tokens == 0 ? 1 : (tokens + arcq::kRouteThreads - 1) / arcq::kRouteThreads;
  return (size_t)blocks * (size_t)experts * sizeof(int);
}

extern "C" int arcq_moe_route(const void *logits, int logits_f32, int tokens, int experts, int top_k, int *sel, void *weight,
                              int *seg_offsets, int64_t *position, int *token_of_row, void *weight_of_row, void *workspace,
                              size_t workspace_bytes, void *stream) {
  using namespace arcq;
  if (tokens < 0 || experts < 1 || experts > kMaxExperts || top_k < 1 || top_k > kMaxTopK || top_k > experts)
    return ARCQ_ERR_SHAPE;
  if (!seg_offsets) return ARCQ_ERR_NULL;
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (!workspace) return ARCQ_ERR_NULL;
  if (tokens > 0 && (!logits || !sel || !weight || !position || !token_of_row || !weight_of_row)) return ARCQ_ERR_NULL;
  const int blocks = tokens == 0 ? 1 : (tokens + kRouteThreads - 1) / kRouteThreads;
  if (workspace_bytes < (size_t)blocks * experts * sizeof(int)) return ARCQ_ERR_WORKSPACE;
  int *hist = static_cast<int *>(workspace);
#define ARCQ_ROUTE(PP)                                                                                                      \
  if (logits_f32)                                                                                                          \
    hipLaunchKernelGGL((moe_route_choose_kernel<true, PP>), dim3(blocks), dim3(kRouteThreads), 0, st, logits, tokens, experts, \
                       top_k, sel, static_cast<uint16_t *>(weight), position, hist);                                      \
  else                                                                                                                     \
    hipLaunchKernelGGL((moe_route_choose_kernel<false, PP>), dim3(blocks), dim3(kRouteThreads), 0, st, logits, tokens, experts, \
                       top_k, sel, static_cast<uint16_t *>(weight), position, hist);
  if (experts <= 2) { ARCQ_ROUTE(2) }
  else if (experts <= 4) { ARCQ_ROUTE(4) }
  else if (experts <= 8) { ARCQ_ROUTE(8) }
  else if (experts <= 16) { ARCQ_ROUTE(16) }
  else if (experts <= 32) { ARCQ_ROUTE(32) }
  else { ARCQ_ROUTE(64) }
#undef ARCQ_ROUTE
  ARCQ_HIP_TRY(hipGetLastError());
  if (blocks > kScanFromBlocks) {
    hipLaunchKernelGGL(moe_route_scan_kernel, dim3(1), dim3(kScanThreads), 0, st, blocks, experts, hist, seg_offsets);
    ARCQ_HIP_TRY(hipGetLastError());
    hipLaunchKernelGGL(moe_route_place_kernel<true>, dim3(blocks), dim3(kRouteThreads), 0, st, tokens, experts, top_k, sel,
                       static_cast<const uint16_t *>(weight), hist, position, seg_offsets, token_of_row,
                       static_cast<uint16_t *>(weight_of_row));
  } else {
    hipLaunchKernelGGL(moe_route_place_kernel<false>, dim3(blocks), dim3(kRouteThreads), 0, st, tokens, experts, top_k, sel,
                       static_cast<const uint16_t *>(weight), hist, position, seg_offsets, token_of_row,
                       static_cast<uint16_t *>(weight_of_row));
  }
  ARCQ_HIP_TRY(hipGetLastError());
  return ARCQ_OK;
}

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
