// INT4 paged KV cache: quantize + append, and batched decode attention over the quantized pages.
//
// Replaces the reference's agemm.init_kv_i4 / append_kv_i4 / batch_decode_i4
// (kernels/src/bindings.cpp:287-413 -> kernels/src/flashinfer.cu:9-112, a thin wrapper around a
// patched FlashInfer that is not part of the reference tree) together with the torch-side quantizer
// asym_quantize_and_pack_i4 (model/kv_cache.py:23-37), which is fused into the append here.
//
// Container layout = the reference's (model/kv_cache.py:148-160):
//   kv_data   u8  [pages, n_layers, 2 (k, v), kv_heads, page_size, head_dim / 2]   element 2j in the low nibble
//   kv_param  T2  [pages, n_layers, 2,        kv_heads, page_size, 2]              (scale, zero) in the model dtype T
//   kv_indptr int32 [batch + 1], kv_indices int32 [kv_indptr[batch]], last_page_offset int32 [batch]:
//   sequence b owns pages kv_indices[kv_indptr[b] .. kv_indptr[b+1]) in order and holds
//   (pages_b - 1) * page_size + last_page_offset[b] tokens.
// A stored value n (0..15) of a (token, head) row stands for n * scale - zero (kv_cache.py:39-43).
//
// head_dim is 128 (the only instantiation of the reference, flashinfer.cu:212-223).
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdlib.h>

#include <algorithm>
#include <type_traits>

#include "../../include/arcq.h"
#include "arcq_internal.h"
#include "arcq_math.h"

namespace arcq {
namespace {

constexpr int kHeadDim = 128;
constexpr int kRowBytes = kHeadDim / 2;  // one (token, head) row of codes

struct KvLayout {
  uint8_t *data;
  uint32_t *param;  // two T values per row
  const int32_t *indptr, *indices, *last_page_offset;
  int n_layers, layer, heads, page_size;
};

// row index of (page, k_or_v, head, slot) in units of one (token, head) row
__device__ __forceinline__ size_t kv_row(const KvLayout &c, int page, int kv, int head, int slot) {
  return ((((size_t)page * c.n_layers + c.layer) * 2 + kv) * c.heads + head) * c.page_size + slot;
}

__device__ __forceinline__ float half_bits_to_f32(uint32_t h) {
  return (float)__builtin_bit_cast(_Float16, (uint16_t)h);
}
__device__ __forceinline__ uint32_t f32_to_half_bits(float f) {
  return (uint32_t)__builtin_bit_cast(uint16_t, (_Float16)f);  // round to nearest even
}
template <bool BF16>
__device__ __forceinline__ float rn(float f) {  // one torch elementwise op's result in the tensor dtype
  return BF16 ? bf16_bits_to_f32(f32_to_bf16_bits(f)) : half_bits_to_f32(f32_to_half_bits(f));
}
template <bool BF16>
__device__ __forceinline__ float from_bits(uint32_t b) {
  return BF16 ? bf16_bits_to_f32(b & 0xffffu) : half_bits_to_f32(b & 0xffffu);
}
template <bool BF16>
__device__ __forceinline__ uint32_t to_bits(float f) {
  return BF16 ? f32_to_bf16_bits(f) : f32_to_half_bits(f);
}

// all-reduce over the 16 lanes of a DPP row
#define ARCQ_ROW_XCHG(x, ctrl) __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), ctrl, 0xf, 0xf, true))
__device__ __forceinline__ float row16_sum(float v) {
  v += ARCQ_ROW_XCHG(v, 0xb1);   // quad_perm [1,0,3,2]
  v += ARCQ_ROW_XCHG(v, 0x4e);   // quad_perm [2,3,0,1]
  v += ARCQ_ROW_XCHG(v, 0x141);  // row_half_mirror
  v += ARCQ_ROW_XCHG(v, 0x140);  // row_mirror
  return v;
}
__device__ __forceinline__ float row16_max(float v) {
  v = fmaxf(v, ARCQ_ROW_XCHG(v, 0xb1));
  v = fmaxf(v, ARCQ_ROW_XCHG(v, 0x4e));
  v = fmaxf(v, ARCQ_ROW_XCHG(v, 0x141));
  v = fmaxf(v, ARCQ_ROW_XCHG(v, 0x140));
  return v;
}

// ---------------------------------------------------------------------------------------------
// append: quantize new (token, head) rows of K and V and scatter them into their pages.
// asym_quantize_and_pack_i4 (model/kv_cache.py:23-37), every torch op rounded to the tensor dtype:
//   scale = (max - min).clamp(min=1e-5) / 15 ; zero = -min ; q = clamp(round((x + zero) / scale), 0, 15)
// 16 lanes per row (8 values each), one wave = 4 rows.
// ---------------------------------------------------------------------------------------------
template <bool BF16>
__device__ __forceinline__ void unpack8(const uint4 raw, float (&x)[8]) {
  const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    x[2 * i] = from_bits<BF16>(w[i]);
    x[2 * i + 1] = from_bits<BF16>(w[i] >> 16);
  }
}

// x: this lane's 8 values of the row (values of the tensor dtype)
template <bool BF16>
__device__ __forceinline__ void quantize_values_store(const float (&x)[8], const KvLayout &c, size_t row, int lane16) {
  float mx = x[0], mn = x[0];
#pragma unroll
  for (int i = 1; i < 8; ++i) {
    mx = fmaxf(mx, x[i]);
    mn = fminf(mn, x[i]);
  }
  mx = row16_max(mx);
  mn = -row16_max(-mn);
  float d = rn<BF16>(mx - mn);
  d = d < 1e-5f ? rn<BF16>(1e-5f) : d;
  const float scale = rn<BF16>(d / 15.0f);
  const float zero = -mn;
  uint32_t packed = 0u;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const float t = rn<BF16>(rn<BF16>(x[i] + zero) / scale);
    const float r = fminf(fmaxf(rintf(t), 0.0f), 15.0f);  // torch.round: half to even
    packed |= (uint32_t)r << (4 * i);
  }
  reinterpret_cast<uint32_t *>(c.data + row * kRowBytes)[lane16] = packed;
  if (lane16 == 0) c.param[row] = to_bits<BF16>(scale) | (to_bits<BF16>(zero) << 16);
}

template <bool BF16>
__device__ __forceinline__ void quantize_row_store(const uint16_t *src, const KvLayout &c, size_t row, int lane16) {
  float x[8];
  unpack8<BF16>(reinterpret_cast<const uint4 *>(src)[lane16], x);
  quantize_values_store<BF16>(x, c, row, lane16);
}

// ---------------------------------------------------------------------------------------------
// decode step: rotary embedding of the new token's query and key heads and the append of its key
// and value heads in one launch.  qkv [batch, ld]: per sequence the query heads, then the key
// heads, then the value heads, 128 values each (the output row of a fused qkv projection).
// Rotary embedding as torch evaluates q * cos + rotate_half(q) * sin on tensors of the model dtype
// (model/qLlamaLayer.py:30-64, 316-321): each product and the sum rounded to that dtype, with
// rotate_half(x) = (-x[64:], x[:64]).  cos / sin come from tables [positions, 64] in the model dtype
// (both halves of the 128 share them).  The rotated keys and the values are quantized and stored as
// in kv_append_i4_kernel; the rotated queries go to q_out [batch, query heads, 128].
// 16 lanes per head row, 8 values each: the partner of value e is value e +- 64, in lane +- 8.
// ---------------------------------------------------------------------------------------------
template <bool BF16>
__global__ __launch_bounds__(256) void rope_kv_append_i4_kernel(const uint16_t *qkv, int ld, const uint16_t *cos_t,
                                                                const uint16_t *sin_t, int max_positions,
                                                                const int32_t *positions, uint16_t *q_out,
                                                                int num_qo_heads, KvLayout c) {
  const int b = blockIdx.x;
  const int lane16 = threadIdx.x & 15;
  const int rows = num_qo_heads + 2 * c.heads;
  const int p0 = c.indptr[b], np = c.indptr[b + 1] - p0;
  const int len = (np - 1) * c.page_size + c.last_page_offset[b];  // length after the append
  const bool has_slot = np > 0 && len > 0;                          // a table without room for the new token: no append
  const int page = has_slot ? c.indices[p0 + (len - 1) / c.page_size] : 0, slot = has_slot ? (len - 1) % c.page_size : 0;
  const int pos = min(max(positions[b], 0), max_positions - 1);
  for (int r = blockIdx.y * 16 + (threadIdx.x >> 4); r < rows; r += gridDim.y * 16) {
    const uint4 raw = reinterpret_cast<const uint4 *>(qkv + (size_t)b * ld + (size_t)r * kHeadDim)[lane16];
    float x[8];
    unpack8<BF16>(raw, x);
    if (r < num_qo_heads + c.heads) {  // a query or key head: rotate
      float xp[8], cs[8], sn[8];
      uint4 praw;
      praw.x = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)raw.x, 0x128, 0xf, 0xf, true);  // row_ror:8 = lane ^ 8
      praw.y = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)raw.y, 0x128, 0xf, 0xf, true);
      praw.z = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)raw.z, 0x128, 0xf, 0xf, true);
      praw.w = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)raw.w, 0x128, 0xf, 0xf, true);
      unpack8<BF16>(praw, xp);
      const size_t t = (size_t)pos * (kHeadDim / 2) + 8 * (lane16 & 7);
      unpack8<BF16>(*reinterpret_cast<const uint4 *>(cos_t + t), cs);
      unpack8<BF16>(*reinterpret_cast<const uint4 *>(sin_t + t), sn);
      const float sgn = lane16 < 8 ? -1.0f : 1.0f;
#pragma unroll
      for (int i = 0; i < 8; ++i) x[i] = rn<BF16>(rn<BF16>(x[i] * cs[i]) + rn<BF16>((sgn * xp[i]) * sn[i]));
    }
    if (r < num_qo_heads) {
      uint4 o;
      o.x = to_bits<BF16>(x[0]) | (to_bits<BF16>(x[1]) << 16);
      o.y = to_bits<BF16>(x[2]) | (to_bits<BF16>(x[3]) << 16);
      o.z = to_bits<BF16>(x[4]) | (to_bits<BF16>(x[5]) << 16);
      o.w = to_bits<BF16>(x[6]) | (to_bits<BF16>(x[7]) << 16);
      reinterpret_cast<uint4 *>(q_out + ((size_t)b * num_qo_heads + r) * kHeadDim)[lane16] = o;
    } else if (has_slot) {
      const int kv = r >= num_qo_heads + c.heads ? 1 : 0;
      const int head = r - num_qo_heads - kv * c.heads;
      quantize_values_store<BF16>(x, c, kv_row(c, page, kv, head, slot), lane16);
    }
  }
}

// the rotary embedding alone, for whole prompts: token t of the flattened [sequences x q_len] batch sits
// at position pos0 + t % q_len; rotated query heads go to q_out [tokens, query heads, 128], rotated key
// heads to k_out [tokens, kv heads, 128] (the value heads stay where they are)
template <bool BF16>
__global__ __launch_bounds__(256) void rope_rows_kernel(const uint16_t *qkv, int ld, const uint16_t *cos_t,
                                                        const uint16_t *sin_t, int max_positions, int q_len, int pos0,
                                                        long rows_total, int num_qo_heads, int num_kv_heads,
                                                        uint16_t *q_out, uint16_t *k_out) {
  const int lane16 = threadIdx.x & 15;
  const int heads = num_qo_heads + num_kv_heads;
  for (long row = (long)blockIdx.x * 16 + (threadIdx.x >> 4); row < rows_total; row += (long)gridDim.x * 16) {
    const long tok = row / heads;
    const int head = (int)(row - tok * heads);
    const int pos = min(max(pos0 + (int)(tok % q_len), 0), max_positions - 1);
    const uint4 raw = reinterpret_cast<const uint4 *>(qkv + (size_t)tok * ld + (size_t)head * kHeadDim)[lane16];
    float x[8], xp[8], cs[8], sn[8];
    unpack8<BF16>(raw, x);
    uint4 praw;
    praw.x = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)raw.x, 0x128, 0xf, 0xf, true);  // row_ror:8 = lane ^ 8
    praw.y = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)raw.y, 0x128, 0xf, 0xf, true);
    praw.z = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)raw.z, 0x128, 0xf, 0xf, true);
    praw.w = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)raw.w, 0x128, 0xf, 0xf, true);
    unpack8<BF16>(praw, xp);
    const size_t t = (size_t)pos * (kHeadDim / 2) + 8 * (lane16 & 7);
    unpack8<BF16>(*reinterpret_cast<const uint4 *>(cos_t + t), cs);
    unpack8<BF16>(*reinterpret_cast<const uint4 *>(sin_t + t), sn);
    const float sgn = lane16 < 8 ? -1.0f : 1.0f;
#pragma unroll
    for (int i = 0; i < 8; ++i) x[i] = rn<BF16>(rn<BF16>(x[i] * cs[i]) + rn<BF16>((sgn * xp[i]) * sn[i]));
    uint4 o;
    o.x = to_bits<BF16>(x[0]) | (to_bits<BF16>(x[1]) << 16);
    o.y = to_bits<BF16>(x[2]) | (to_bits<BF16>(x[3]) << 16);
    o.z = to_bits<BF16>(x[4]) | (to_bits<BF16>(x[5]) << 16);
    o.w = to_bits<BF16>(x[6]) | (to_bits<BF16>(x[7]) << 16);
    uint16_t *dst = head < num_qo_heads ? q_out + ((size_t)tok * num_qo_heads + head) * kHeadDim
                                        : k_out + ((size_t)tok * num_kv_heads + (head - num_qo_heads)) * kHeadDim;
    reinterpret_cast<uint4 *>(dst)[lane16] = o;
  }
}

template <bool BF16>
__global__ __launch_bounds__(256) void kv_append_i4_kernel(const uint16_t *k, const uint16_t *v, const int32_t *seq_indptr,
                                                           KvLayout c) {
  const int b = blockIdx.x;
  const int tok0 = seq_indptr ? seq_indptr[b] : b;                 // first new token of this sequence in k / v
  const int n_new = seq_indptr ? seq_indptr[b + 1] - tok0 : 1;
  const int p0 = c.indptr[b], np = c.indptr[b + 1] - p0;
  const int len = (np - 1) * c.page_size + c.last_page_offset[b];  // length after the append
  const int lane16 = threadIdx.x & 15;
  const int rows = n_new * c.heads;
  for (int r = blockIdx.y * 16 + (threadIdx.x >> 4); r < rows; r += gridDim.y * 16) {
    const int i = r / c.heads, head = r - i * c.heads;
    const int pos = len - n_new + i;
    if (np <= 0 || pos < 0 || pos >= np * c.page_size) continue;  // a table without room for this token: no store
    const int page = c.indices[p0 + pos / c.page_size], slot = pos % c.page_size;
    const size_t src = ((size_t)(tok0 + i) * c.heads + head) * kHeadDim;
    quantize_row_store<BF16>(k + src, c, kv_row(c, page, 0, head, slot), lane16);
    quantize_row_store<BF16>(v + src, c, kv_row(c, page, 1, head, slot), lane16);
  }
}

// the same scatter for rows a caller has quantized already (what the reference's init_kv_i4 /
// append_kv_i4 take: codes [tokens, heads, 64] and (scale, zero) pairs [tokens, heads, 2])
__global__ __launch_bounds__(256) void kv_store_i4_kernel(const uint32_t *kq, const uint32_t *vq, const uint32_t *kpar,
                                                          const uint32_t *vpar, const int32_t *seq_indptr, KvLayout c) {
  const int b = blockIdx.x;
  const int tok0 = seq_indptr ? seq_indptr[b] : b;
  const int n_new = seq_indptr ? seq_indptr[b + 1] - tok0 : 1;
  const int p0 = c.indptr[b], np = c.indptr[b + 1] - p0;
  const int len = (np - 1) * c.page_size + c.last_page_offset[b];
  const int lane16 = threadIdx.x & 15;
  const int rows = n_new * c.heads;
  for (int r = blockIdx.y * 16 + (threadIdx.x >> 4); r < rows; r += gridDim.y * 16) {
    const int i = r / c.heads, head = r - i * c.heads;
    const int pos = len - n_new + i;
    if (np <= 0 || pos < 0 || pos >= np * c.page_size) continue;  // a table without room for this token: no store
    const int page = c.indices[p0 + pos / c.page_size], slot = pos % c.page_size;
    const size_t src = (size_t)(tok0 + i) * c.heads + head;
    const size_t krow = kv_row(c, page, 0, head, slot), vrow = kv_row(c, page, 1, head, slot);
    reinterpret_cast<uint32_t *>(c.data + krow * kRowBytes)[lane16] = kq[src * 16 + lane16];
    reinterpret_cast<uint32_t *>(c.data + vrow * kRowBytes)[lane16] = vq[src * 16 + lane16];
    if (lane16 == 0) {
      c.param[krow] = kpar[src];
      c.param[vrow] = vpar[src];
    }
  }
}

// ---------------------------------------------------------------------------------------------
// decode: o[b, h] = softmax(q[b, h] . K[b]^T * sm_scale) V[b] for one new token per sequence.
// One workgroup per (sequence, kv head); the G query heads of the group share every K / V read.
// A row of 16 lanes covers the 128 dims of one token (4 code bytes = 8 dims per lane), so a wave
// takes 4 tokens at a time and the workgroup 16.  With a stored value n standing for n*s - z,
//   q . k = s * (q . n) - z * sum(q)     and     sum_t p_t v_t = sum_t (p_t s_t) n_t - sum_t p_t z_t,
// so the codes are only converted to fp32, never dequantized element by element.
// Each (wave, token slot) runs its own online softmax (base 2, sm_scale * log2(e) folded into q);
// the 16 partial results are merged through LDS at the end.
// ---------------------------------------------------------------------------------------------
template <bool BF16, int G>
__global__ __launch_bounds__(256) void kv_decode_i4_kernel(uint16_t *o, const uint16_t *q, KvLayout c, int num_qo_heads,
                                                           float sm_scale_log2) {
  __shared__ float part_o[16][G][kHeadDim];
  __shared__ float part_ml[16][G][2];
  const int b = blockIdx.x, h = blockIdx.y;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int dg = lane & 15, ts = lane >> 4;
  const int p0 = c.indptr[b], np = c.indptr[b + 1] - p0;
  const int len = np > 0 ? (np - 1) * c.page_size + c.last_page_offset[b] : 0;

  float qv[G][8], qsum[G];
#pragma unroll
  for (int g = 0; g < G; ++g) {
    const uint4 raw = reinterpret_cast<const uint4 *>(q + ((size_t)b * num_qo_heads + h * G + g) * kHeadDim)[dg];
    const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
    float s = 0.0f;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      qv[g][2 * i] = from_bits<BF16>(w[i]) * sm_scale_log2;
      qv[g][2 * i + 1] = from_bits<BF16>(w[i] >> 16) * sm_scale_log2;
      s += qv[g][2 * i] + qv[g][2 * i + 1];
    }
    qsum[g] = row16_sum(s);
  }

  constexpr float kNegBig = -1e30f;
  float m[G], l[G], zacc[G], acc[G][8];
#pragma unroll
  for (int g = 0; g < G; ++g) {
    m[g] = kNegBig;
    l[g] = 0.0f;
    zacc[g] = 0.0f;
#pragma unroll
    for (int i = 0; i < 8; ++i) acc[g][i] = 0.0f;
  }

  for (int t0 = 0; t0 < len; t0 += 16) {
    const int t = t0 + 4 * wave + ts;
    const bool valid = t < len;
    const int tc = valid ? t : len - 1;
    const int page = c.indices[p0 + tc / c.page_size], slot = tc % c.page_size;
    const size_t krow = kv_row(c, page, 0, h, slot), vrow = kv_row(c, page, 1, h, slot);
    const uint32_t kd = reinterpret_cast<const uint32_t *>(c.data + krow * kRowBytes)[dg];
    const uint32_t vd = reinterpret_cast<const uint32_t *>(c.data + vrow * kRowBytes)[dg];
    const uint32_t kp = c.param[krow], vp = c.param[vrow];
    const float ks = from_bits<BF16>(kp), kz = from_bits<BF16>(kp >> 16);
    const float vs = from_bits<BF16>(vp), vz = from_bits<BF16>(vp >> 16);
    float kn[8], vn[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      kn[i] = (float)((kd >> (4 * i)) & 15u);
      vn[i] = (float)((vd >> (4 * i)) & 15u);
    }
#pragma unroll
    for (int g = 0; g < G; ++g) {
      float dot = 0.0f;
#pragma unroll
      for (int i = 0; i < 8; ++i) dot = __builtin_fmaf(qv[g][i], kn[i], dot);
      dot = row16_sum(dot);
      const float s = valid ? ks * dot - kz * qsum[g] : kNegBig;
      const float mn = fmaxf(m[g], s);
      const float corr = __builtin_amdgcn_exp2f(m[g] - mn);
      const float p = __builtin_amdgcn_exp2f(s - mn);
      m[g] = mn;
      l[g] = l[g] * corr + p;
      zacc[g] = zacc[g] * corr + p * vz;
      const float pv = p * vs;
#pragma unroll
      for (int i = 0; i < 8; ++i) acc[g][i] = __builtin_fmaf(pv, vn[i], acc[g][i] * corr);
    }
  }

  // merge the 16 partial softmaxes: part index = 4*wave + ts
  const int pi = 4 * wave + ts;
#pragma unroll
  for (int g = 0; g < G; ++g) {
#pragma unroll
    for (int i = 0; i < 8; ++i) part_o[pi][g][8 * dg + i] = acc[g][i] - zacc[g];
    if (dg == 0) {
      part_ml[pi][g][0] = m[g];
      part_ml[pi][g][1] = l[g];
    }
  }
  __syncthreads();
  // thread -> (g, dim): G * 128 outputs over 256 threads
  for (int idx = threadIdx.x; idx < G * kHeadDim; idx += 256) {
    const int g = idx / kHeadDim, dim = idx - g * kHeadDim;
    float M = kNegBig;
#pragma unroll
    for (int p = 0; p < 16; ++p) M = fmaxf(M, part_ml[p][g][0]);
    float num = 0.0f, den = 0.0f;
#pragma unroll
    for (int p = 0; p < 16; ++p) {
      const float wgt = __builtin_amdgcn_exp2f(part_ml[p][g][0] - M);
      num = __builtin_fmaf(wgt, part_o[p][g][dim], num);
      den = __builtin_fmaf(wgt, part_ml[p][g][1], den);
    }
    const float out = den > 0.0f ? num / den : 0.0f;
    o[((size_t)b * num_qo_heads + h * G + g) * kHeadDim + dim] = (uint16_t)to_bits<BF16>(out);
  }
}

// ---------------------------------------------------------------------------------------------
// The same decode on the matrix cores, for page sizes that are multiples of 16.  A wave takes chunks
// of 16 tokens (always inside one page):
//   S^T[token, head] = Kn[token, dim] . Q^T[dim, head]      4 x v_mfma_f32_16x16x32_f16
//   O[head, dim]    += P[head, token] . Vn[token, dim]      8 x v_mfma_f32_16x16x16_f16
// Kn, Vn are the stored codes 0..15 as fp16; scale and zero of the rows enter through the identities
// above (s * dot - z * sum(q), and p * s_v folded into P), so no element is dequantized.
// Codes become fp16 by or-ing them into the mantissa of 1024 (0x6400 | n = 1024 + n; the high nibble
// of a byte lands four bits up and reads 1024 + 16 n): for K the factor 16 is divided out of the
// matching q elements and the 1024 terms leave the scores as one number per head; for V both are
// removed from the accumulated sums at the end (sum_t p_t * 1024 is tracked beside the softmax
// denominator).
// Layouts make every operand a plain load: the K operand row of a lane is its token's 16 bytes
// (the MFMA's K index is a permutation of the dims, applied to Q^T as well), S^T comes out with a
// lane holding 4 tokens of one head, which is exactly the A operand of the second product, and the
// V operand of a lane is one dword (8 dims) of each of its 4 tokens, output column j of MFMA j being
// dim 8 * (lane % 16) + j.
// ---------------------------------------------------------------------------------------------
typedef _Float16 v2h __attribute__((ext_vector_type(2)));
typedef _Float16 v4h __attribute__((ext_vector_type(4)));
typedef _Float16 v8h __attribute__((ext_vector_type(8)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef uint32_t v2u __attribute__((ext_vector_type(2)));
typedef uint32_t v4u __attribute__((ext_vector_type(4)));

// 8 codes of a dword -> 8 fp16 values with the 1024 left in: bytes b0..b3 hold dims (0,1) (2,3) (4,5) (6,7) as
// (low, high) nibbles; the result is (1024 + n0, 1024 + n4, 1024 + 16 n1, 1024 + 16 n5, 1024 + n2, 1024 + n6,
// 1024 + 16 n3, 1024 + 16 n7): five instructions.  Q^T is laid out in the same order with the
// elements that meet a 16 n divided by 16, and the 1024 terms are subtracted from the scores as one
// number per head (1024 * sum of q over the low-nibble dims + 64 * sum over the high-nibble dims).
constexpr int kDimOfElem[8] = {0, 4, 1, 5, 2, 6, 3, 7};
// The three constants (0x64006400 = fp16 1024 twice, and the two nibble masks) are held in registers
// the compiler knows nothing about: this chip's three-operand encoding takes no literal, so with
// literals (x & mask) | 0x64006400 is two instructions, with registers it is one v_and_or_b32.
struct NibbleConsts {
  uint32_t one_k, lo, hi;
};
__device__ __forceinline__ v8h k_operand(uint32_t x, const NibbleConsts &k) {
  v4u d;
  const uint32_t y = x >> 8;
  d[0] = (x & k.lo) | k.one_k;
  d[1] = (x & k.hi) | k.one_k;
  d[2] = (y & k.lo) | k.one_k;
  d[3] = (y & k.hi) | k.one_k;
  return __builtin_bit_cast(v8h, d);
}

// kDecodeWaves waves per workgroup share the chunks of one (sequence, KV head): a chunk is a chain of
// dependent steps (loads, four MFMAs on one accumulator, cross-lane maxima, exponentials, eight more
// MFMAs), so the kernel lives on waves per SIMD, and batch x KV heads workgroups of four waves give
// only two.
// maximum over the four lanes L, L^16, L^32, L^48 in every one of them, on the VALU: the lane-swap
// instructions exchange rows (of 16 lanes) and halves between two registers; with both registers
// holding m, the two results hold a lane's own value and its partner's
__device__ __forceinline__ float max_over_lane_groups(float m) {
  const uint32_t b = __builtin_bit_cast(uint32_t, m);
  const auto r = __builtin_amdgcn_permlane16_swap(b, b, false, false);
  const float m16 = fmaxf(__builtin_bit_cast(float, r[0]), __builtin_bit_cast(float, r[1]));
  const uint32_t c = __builtin_bit_cast(uint32_t, m16);
  const auto q = __builtin_amdgcn_permlane32_swap(c, c, false, false);
  return fmaxf(__builtin_bit_cast(float, q[0]), __builtin_bit_cast(float, q[1]));
}

constexpr int kDecodeWaves = 8;
// Chunks travel global -> LDS without passing through registers (global_load_lds), four per wave in
// flight, each wave into its own slots: codes of K (1 KB), codes of V (1 KB), the 32 parameter words.
constexpr int kDecodeStages = 4;
constexpr int kDecodeSlotBytes = 1024 + 1024 + 128;
// These write M0, which the compiler reserves and does not accept on a clobber list: the decode kernel
// holds nothing for which the compiler sets or reads M0 itself, and each helper sets it before its load.
__device__ __forceinline__ void kv_lds_dma16(const void *g, uint32_t lds_wave_base) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off" : : "s"(lds_wave_base), "v"(g) : "memory");
}
__device__ __forceinline__ void kv_lds_dma4(const void *g, uint32_t lds_wave_base) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %1, off" : : "s"(lds_wave_base), "v"(g) : "memory");
}
// With few sequences the (sequence, KV head) grid leaves CUs idle: gridDim.z > 1 cuts every sequence's
// chunks into that many ranges, one workgroup each, which write (maximum, denominator, numerator[128])
// per head to `partial` instead of the output; kv_decode_merge_kernel combines them.
constexpr int kPartialStride = kHeadDim + 2;
template <bool BF16, int G>
__global__ __launch_bounds__(64 * kDecodeWaves) void kv_decode_i4_mfma_kernel(uint16_t *o, const uint16_t *q, KvLayout c,
                                                                              int num_qo_heads, float sm_scale_log2,
                                                                              float *partial) {
  // the waves' partial results meet, after the loop, in the memory of the slots
  __shared__ uint4 slots[kDecodeWaves * kDecodeStages * kDecodeSlotBytes / 16];
  static_assert(sizeof(float) * kDecodeWaves * G * (kHeadDim + 4) <= sizeof(slots), "the merge area lies inside the slots");
  float(*part_o)[G][kHeadDim] = reinterpret_cast<float(*)[G][kHeadDim]>(slots);
  float(*part_s)[G][4] = reinterpret_cast<float(*)[G][4]>(reinterpret_cast<float *>(slots) + kDecodeWaves * G * kHeadDim);  // m, l, D (1024 * sum of P), Z (sum of p * zero)
  const int b = blockIdx.x, h = blockIdx.y;
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int r16 = lane & 15, g = lane >> 4;
  const int p0 = c.indptr[b], np = c.indptr[b + 1] - p0;
  const int len = np > 0 ? (np - 1) * c.page_size + c.last_page_offset[b] : 0;
  constexpr float kNegBig = -1e30f;

  // Q^T operand: lane (head r16, group g) holds dims 32g + 8m + kDimOfElem[e] for MFMA m, the
  // elements of odd dims (high nibbles) divided by 16
  v8h qop[4];
  float qsum = 0.0f, qoff = 0.0f;
  {
    const bool real = r16 < G;
    const uint16_t *qrow = q + ((size_t)b * num_qo_heads + h * G + (real ? r16 : 0)) * kHeadDim + 32 * g;
#pragma unroll
    for (int m = 0; m < 4; ++m) {
      const uint4 raw = reinterpret_cast<const uint4 *>(qrow)[m];
      const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const int dim = kDimOfElem[e];
        float f = from_bits<BF16>(w[dim >> 1] >> (16 * (dim & 1)));
        if (!real) f = 0.0f;
        const _Float16 hq = (_Float16)f;                 // exact for bf16 inputs inside the fp16 range
        const _Float16 hs = (dim & 1) ? hq * (_Float16)0.0625f : hq;
        qsum += (float)hq;
        qoff += 1024.0f * (float)hs;                     // what the 1024 of this element's codes adds to a score
        qop[m][e] = hs;
      }
    }
    qsum += __shfl_xor(qsum, 16);
    qsum += __shfl_xor(qsum, 32);
    qoff += __shfl_xor(qoff, 16);
    qoff += __shfl_xor(qoff, 32);
  }

  NibbleConsts nib = {0x64006400u, 0x000f000fu, 0x00f000f0u};
  asm volatile("" : "+s"(nib.one_k), "+v"(nib.lo), "+v"(nib.hi));
  float m_run = kNegBig, l_run = 0.0f, d_run = 0.0f, z_run = 0.0f;
  v4f oacc[8];
#pragma unroll
  for (int j = 0; j < 8; ++j) oacc[j] = v4f{0.f, 0.f, 0.f, 0.f};

  const int nchunks = (len + 15) >> 4;
  const int ch_beg = (int)((long)nchunks * blockIdx.z / gridDim.z), ch_end = (int)((long)nchunks * (blockIdx.z + 1) / gridDim.z);
  // this wave's chunks: ch_beg + wave + kDecodeWaves * k, k = 0 .. n_mine-1
  const int n_mine = ch_end > ch_beg + wave ? (ch_end - ch_beg - wave + kDecodeWaves - 1) / kDecodeWaves : 0;
  const uint32_t slot_base = (uint32_t)reinterpret_cast<uintptr_t>(slots) + wave * (kDecodeStages * kDecodeSlotBytes);
  // The pages of this wave's chunks, 64 at a time, one per lane: inside the loop a page is a readlane,
  // not a load (a load there would be waited for with vmcnt(0), draining the chunks in flight; that
  // happens once per 64 chunks).
  int pages = 0;
  auto load_pages = [&](int k0) {
    const int kk = k0 + lane;
    pages = kk < n_mine ? c.indices[p0 + ((ch_beg + wave + kDecodeWaves * kk) << 4) / c.page_size] : 0;
  };
  auto page_of = [&](int k) { return __builtin_amdgcn_readlane(pages, k & 63); };  // k in the block last loaded
  // V travels so that the dword a lane needs of token 4g+i sits at 256 i + 4 lane of the slot: the lane
  // that fetches 16 bytes into position L of the slot takes token 4 ((L >> 2) & 3) + (L >> 4), piece L & 3
  const int v_tok = 4 * ((lane >> 2) & 3) + (lane >> 4), v_piece = lane & 3;
  auto issue = [&](int k, int page) {  // three instructions per chunk and wave: vmcnt counts on it
    if (k >= n_mine) return;  // wave-uniform
    const int t0 = (ch_beg + wave + kDecodeWaves * k) << 4, slot0 = t0 % c.page_size;
    const size_t krow0 = kv_row(c, page, 0, h, slot0), vrow0 = kv_row(c, page, 1, h, slot0);
    const uint32_t dst = slot_base + (k % kDecodeStages) * kDecodeSlotBytes;
    kv_lds_dma16(c.data + (krow0 + r16) * kRowBytes + 16 * g, dst);                   // K: token r16, bytes 16g .. 16g+15
    kv_lds_dma16(c.data + (vrow0 + v_tok) * kRowBytes + 16 * v_piece, dst + 1024);
    if (lane < 32) kv_lds_dma4(c.param + (lane < 16 ? krow0 + lane : vrow0 + lane - 16), dst + 2048);
  };
  load_pages(0);
  issue(0, page_of(0));
  issue(1, page_of(1));
  issue(2, page_of(2));
  for (int k = 0; k < n_mine; ++k) {
    const int ch = ch_beg + wave + kDecodeWaves * k;
    const int t0 = ch << 4;
    if (((k + 3) & 63) == 0) load_pages(k + 3);
    issue(k + 3, page_of(k + 3));
    const int younger = n_mine - 1 - k;  // chunks asked for after this one
    if (younger >= 3)
      asm volatile("s_waitcnt vmcnt(9)" ::: "memory");
    else if (younger == 2)
      asm volatile("s_waitcnt vmcnt(6)" ::: "memory");
    else if (younger == 1)
      asm volatile("s_waitcnt vmcnt(3)" ::: "memory");
    else
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    const uint8_t *slot = reinterpret_cast<const uint8_t *>(slots) + wave * (kDecodeStages * kDecodeSlotBytes) +
                          (k % kDecodeStages) * kDecodeSlotBytes;
    const uint4 kq = reinterpret_cast<const uint4 *>(slot)[lane];
    uint32_t vd[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) vd[i] = reinterpret_cast<const uint32_t *>(slot + 1024 + 256 * i)[lane];
    const uint4 kpar = reinterpret_cast<const uint4 *>(slot + 2048)[g];
    const uint4 vpar = reinterpret_cast<const uint4 *>(slot + 2048 + 64)[g];
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // the slot is read before a later request may overwrite it

    v4f sacc = {0.f, 0.f, 0.f, 0.f};
    sacc = __builtin_amdgcn_mfma_f32_16x16x32_f16(k_operand(kq.x, nib), qop[0], sacc, 0, 0, 0);
    sacc = __builtin_amdgcn_mfma_f32_16x16x32_f16(k_operand(kq.y, nib), qop[1], sacc, 0, 0, 0);
    sacc = __builtin_amdgcn_mfma_f32_16x16x32_f16(k_operand(kq.z, nib), qop[2], sacc, 0, 0, 0);
    sacc = __builtin_amdgcn_mfma_f32_16x16x32_f16(k_operand(kq.w, nib), qop[3], sacc, 0, 0, 0);

    const uint32_t kp[4] = {kpar.x, kpar.y, kpar.z, kpar.w}, vp[4] = {vpar.x, vpar.y, vpar.z, vpar.w};
    // scores -> running maximum -> P (times the V scales, as fp16) and this chunk's sums.  Only a
    // sequence's last chunk has rows past the end (they may hold anything): every other chunk takes
    // the variant without the row masks (the choice is wave-uniform).
    v2h p01, p23;
    float corr, psum = 0.0f, pasum, pz = 0.0f;
    auto scores_to_p = [&](auto whole_c) {
      constexpr bool WHOLE = decltype(whole_c)::value;
      float sc[4], mx = m_run;
#pragma unroll
      for (int v = 0; v < 4; ++v) {
        const float ks = from_bits<BF16>(kp[v]), kz = from_bits<BF16>(kp[v] >> 16);
        sc[v] = (ks * (sacc[v] - qoff) - kz * qsum) * sm_scale_log2;
        if (!WHOLE && !(t0 + 4 * g + v < len)) sc[v] = kNegBig;
        mx = fmaxf(mx, sc[v]);
      }
      mx = max_over_lane_groups(mx);
      corr = __builtin_amdgcn_exp2f(m_run - mx);
      m_run = mx;
      float pr[4];
#pragma unroll
      for (int v = 0; v < 4; ++v) {
        const bool valid = WHOLE || t0 + 4 * g + v < len;
        const float pv = __builtin_amdgcn_exp2f(sc[v] - mx);
        const float vs = valid ? from_bits<BF16>(vp[v]) : 0.0f, vz = valid ? from_bits<BF16>(vp[v] >> 16) : 0.0f;
        psum += pv;
        pz = __builtin_fmaf(pv, vz, pz);
        pr[v] = pv * vs;
      }
      p01 = v2h{(_Float16)pr[0], (_Float16)pr[1]};
      p23 = v2h{(_Float16)pr[2], (_Float16)pr[3]};
    };
    if (t0 + 16 <= len)
      scores_to_p(std::true_type{});
    else
      scores_to_p(std::false_type{});
    // the sum of the four fp16 values as the second product sees them
    const v2h ones = {(_Float16)1.0f, (_Float16)1.0f};
    pasum = __builtin_amdgcn_fdot2(p01, ones, __builtin_amdgcn_fdot2(p23, ones, 0.0f, false), false);
    const v4h pa = {p01[0], p01[1], p23[0], p23[1]};
    l_run = l_run * corr + psum;
    d_run = d_run * corr + 1024.0f * pasum;
    z_run = z_run * corr + pz;
    if (__any(corr != 1.0f)) {  // the running maximum of some head moved: rescale the accumulators
      float cr[4];
#pragma unroll
      for (int v = 0; v < 4; ++v)
        cr[v] = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, corr), v));
#pragma unroll
      for (int j = 0; j < 8; ++j)
#pragma unroll
        for (int v = 0; v < 4; ++v) oacc[j][v] *= cr[v];
    }
    // V operands: byte bb of the four token dwords -> codes 2bb (low nibbles) and 2bb+1 (high nibbles)
#define ARCQ_PV(BB)                                                                                             \
  {                                                                                                             \
    const uint32_t t01 = __builtin_amdgcn_perm(vd[1], vd[0], 0x0c040c00u + 0x00010001u * (BB));                 \
    const uint32_t t23 = __builtin_amdgcn_perm(vd[3], vd[2], 0x0c040c00u + 0x00010001u * (BB));                 \
    v2u lo, hi;                                                                                                 \
    lo[0] = (t01 & nib.lo) | nib.one_k;                                                                         \
    lo[1] = (t23 & nib.lo) | nib.one_k;                                                                         \
    hi[0] = (t01 & nib.hi) | nib.one_k;                                                                         \
    hi[1] = (t23 & nib.hi) | nib.one_k;                                                                         \
    oacc[2 * (BB)] = __builtin_amdgcn_mfma_f32_16x16x16f16(pa, __builtin_bit_cast(v4h, lo), oacc[2 * (BB)], 0, 0, 0);      \
    oacc[2 * (BB) + 1] =                                                                                        \
        __builtin_amdgcn_mfma_f32_16x16x16f16(pa, __builtin_bit_cast(v4h, hi), oacc[2 * (BB) + 1], 0, 0, 0);    \
  }
    ARCQ_PV(0) ARCQ_PV(1) ARCQ_PV(2) ARCQ_PV(3)
#undef ARCQ_PV
  }

  // per-wave totals of the softmax sums over the four lane groups, then merge the waves
  l_run += __shfl_xor(l_run, 16);
  l_run += __shfl_xor(l_run, 32);
  d_run += __shfl_xor(d_run, 16);
  d_run += __shfl_xor(d_run, 32);
  z_run += __shfl_xor(z_run, 16);
  z_run += __shfl_xor(z_run, 32);
  __syncthreads();  // every wave is done with its slots
  if (g == 0) {
    if (r16 < G) {
      part_s[wave][r16][0] = m_run;
      part_s[wave][r16][1] = l_run;
      part_s[wave][r16][2] = d_run;
      part_s[wave][r16][3] = z_run;
    }
#pragma unroll
    for (int j = 0; j < 8; ++j)
#pragma unroll
      for (int v = 0; v < G; ++v) part_o[wave][v][8 * r16 + j] = oacc[j][v];   // rows 4g+v = heads, g == 0
  }
  __syncthreads();
  for (int idx = threadIdx.x; idx < G * kHeadDim; idx += 64 * kDecodeWaves) {
    const int hh = idx / kHeadDim, dim = idx - hh * kHeadDim;
    float M = kNegBig;
#pragma unroll
    for (int w = 0; w < kDecodeWaves; ++w) M = fmaxf(M, part_s[w][hh][0]);
    const float unscale = (dim & 1) ? 0.0625f : 1.0f;  // odd dims were accumulated as 16 n
    float num = 0.0f, den = 0.0f;
#pragma unroll
    for (int w = 0; w < kDecodeWaves; ++w) {
      const float wgt = __builtin_amdgcn_exp2f(part_s[w][hh][0] - M);
      num = __builtin_fmaf(wgt, (part_o[w][hh][dim] - part_s[w][hh][2]) * unscale - part_s[w][hh][3], num);
      den = __builtin_fmaf(wgt, part_s[w][hh][1], den);
    }
    if (gridDim.z > 1) {
      float *dst = partial + (((size_t)b * num_qo_heads + h * G + hh) * gridDim.z + blockIdx.z) * kPartialStride;
      dst[2 + dim] = num;
      if (dim == 0) {
        dst[0] = M;
        dst[1] = den;
      }
      continue;
    }
    const float out = den > 0.0f ? num / den : 0.0f;
    o[((size_t)b * num_qo_heads + h * G + hh) * kHeadDim + dim] = (uint16_t)to_bits<BF16>(out);
  }
}

// one workgroup of 128 threads per (sequence, query head): softmax-weighted sum of the ranges' partials
template <bool BF16>
__global__ __launch_bounds__(128) void kv_decode_merge_kernel(uint16_t *o, const float *partial, int splits) {
  const float *src = partial + (size_t)blockIdx.x * splits * kPartialStride;
  float M = -1e30f;
  for (int z = 0; z < splits; ++z) M = fmaxf(M, src[z * kPartialStride]);
  float num = 0.0f, den = 0.0f;
  for (int z = 0; z < splits; ++z) {
    const float wgt = __builtin_amdgcn_exp2f(src[z * kPartialStride] - M);
    num = __builtin_fmaf(wgt, src[z * kPartialStride + 2 + threadIdx.x], num);
    den = __builtin_fmaf(wgt, src[z * kPartialStride + 1], den);
  }
  const float out = den > 0.0f ? num / den : 0.0f;
  o[(size_t)blockIdx.x * kHeadDim + threadIdx.x] = (uint16_t)to_bits<BF16>(out);
}

int check_layout(const void *kv_data, const void *kv_param, const int32_t *kv_indptr, const int32_t *kv_indices,
                 const int32_t *last_page_offset, int n_layers, int layer_idx, int heads, int page_size, int head_dim,
                 int dtype) {
  if (dtype != ARCQ_DTYPE_F16 && dtype != ARCQ_DTYPE_BF16) return ARCQ_ERR_FORMAT;
  if (head_dim != kHeadDim || n_layers < 1 || layer_idx < 0 || layer_idx >= n_layers || heads < 1 || page_size < 1)
    return ARCQ_ERR_SHAPE;
  if (!kv_data || !kv_param || !kv_indptr || !kv_indices || !last_page_offset) return ARCQ_ERR_NULL;
  if (!aligned16(kv_data) || ((uintptr_t)kv_param & 3)) return ARCQ_ERR_ALIGN;
  return ARCQ_OK;
}

}  // namespace
}  // namespace arcq

extern "C" {

int arcq_kv_append_i4(const void *k, const void *v, int dtype, int batch, const int32_t *seqlen_indptr, int max_new_tokens,
                      void *kv_data, void *kv_param, const int32_t *kv_indptr, const int32_t *kv_indices,
                      const int32_t *last_page_offset, int n_layers, int layer_idx, int num_kv_heads, int page_size,
                      int head_dim, void *stream) {
  using namespace arcq;
  const int rc = check_layout(kv_data, kv_param, kv_indptr, kv_indices, last_page_offset, n_layers, layer_idx,
                              num_kv_heads, page_size, head_dim, dtype);
  if (rc != ARCQ_OK) return rc;
  if (batch < 0 || max_new_tokens < 0) return ARCQ_ERR_SHAPE;
  if (batch == 0 || max_new_tokens == 0) return ARCQ_OK;
  if (!k || !v) return ARCQ_ERR_NULL;
  if (!aligned16(k) || !aligned16(v)) return ARCQ_ERR_ALIGN;
  KvLayout c{static_cast<uint8_t *>(kv_data), static_cast<uint32_t *>(kv_param), kv_indptr, kv_indices,
             last_page_offset,               n_layers,                           layer_idx, num_kv_heads, page_size};
  const long rows = (long)max_new_tokens * num_kv_heads;
  int gy = (int)((rows + 15) / 16);
  if (gy > 256) gy = 256;
  dim3 grid(batch, gy);
  if (dtype == ARCQ_DTYPE_BF16)
    hipLaunchKernelGGL(kv_append_i4_kernel<true>, grid, dim3(256), 0, static_cast<hipStream_t>(stream),
                       static_cast<const uint16_t *>(k), static_cast<const uint16_t *>(v), seqlen_indptr, c);
  else
    hipLaunchKernelGGL(kv_append_i4_kernel<false>, grid, dim3(256), 0, static_cast<hipStream_t>(stream),
                       static_cast<const uint16_t *>(k), static_cast<const uint16_t *>(v), seqlen_indptr, c);
  ARCQ_HIP_TRY(hipGetLastError());
  return ARCQ_OK;
}

int arcq_rope_kv_append_i4(const void *qkv, int ld, int dtype, int batch, int num_qo_heads, const void *cos_table,
                           const void *sin_table, int max_positions, const int32_t *positions, void *q_out,
                           void *kv_data, void *kv_param, const int32_t *kv_indptr, const int32_t *kv_indices,
                           const int32_t *last_page_offset, int n_layers, int layer_idx, int num_kv_heads, int page_size,
                           int head_dim, void *stream) {
  using namespace arcq;
  const int rc = check_layout(kv_data, kv_param, kv_indptr, kv_indices, last_page_offset, n_layers, layer_idx,
                              num_kv_heads, page_size, head_dim, dtype);
  if (rc != ARCQ_OK) return rc;
  const long rows = (long)num_qo_heads + 2L * num_kv_heads;
  if (batch < 0 || num_qo_heads < 1 || max_positions < 1 || ld < rows * kHeadDim || ld % 8 != 0) return ARCQ_ERR_SHAPE;
  if (batch == 0) return ARCQ_OK;
  if (!qkv || !cos_table || !sin_table || !positions || !q_out) return ARCQ_ERR_NULL;
  if (!aligned16(qkv) || !aligned16(cos_table) || !aligned16(sin_table) || !aligned16(q_out)) return ARCQ_ERR_ALIGN;
  KvLayout c{static_cast<uint8_t *>(kv_data), static_cast<uint32_t *>(kv_param), kv_indptr, kv_indices,
             last_page_offset,               n_layers,                           layer_idx, num_kv_heads, page_size};
  dim3 grid(batch, (unsigned)((rows + 15) / 16));
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (dtype == ARCQ_DTYPE_BF16)
    hipLaunchKernelGGL(rope_kv_append_i4_kernel<true>, grid, dim3(256), 0, st, static_cast<const uint16_t *>(qkv), ld,
                       static_cast<const uint16_t *>(cos_table), static_cast<const uint16_t *>(sin_table), max_positions,
                       positions, static_cast<uint16_t *>(q_out), num_qo_heads, c);
  else
    hipLaunchKernelGGL(rope_kv_append_i4_kernel<false>, grid, dim3(256), 0, st, static_cast<const uint16_t *>(qkv), ld,
                       static_cast<const uint16_t *>(cos_table), static_cast<const uint16_t *>(sin_table), max_positions,
                       positions, static_cast<uint16_t *>(q_out), num_qo_heads, c);
  ARCQ_HIP_TRY(hipGetLastError());
  return ARCQ_OK;
}

int arcq_rope(const void *qkv, int ld, int dtype, long tokens, int q_len, int pos0, int num_qo_heads, int num_kv_heads,
              int head_dim, const void *cos_table, const void *sin_table, int max_positions, void *q_out, void *k_out,
              void *stream) {
  using namespace arcq;
  if (dtype != ARCQ_DTYPE_F16 && dtype != ARCQ_DTYPE_BF16) return ARCQ_ERR_FORMAT;
  const long heads = (long)num_qo_heads + num_kv_heads;
  if (head_dim != kHeadDim || tokens < 0 || q_len < 1 || num_qo_heads < 1 || num_kv_heads < 0 || max_positions < 1 ||
      ld < heads * kHeadDim || ld % 8 != 0)
    return ARCQ_ERR_SHAPE;
  if (tokens == 0) return ARCQ_OK;
  if (!qkv || !cos_table || !sin_table || !q_out || (num_kv_heads > 0 && !k_out)) return ARCQ_ERR_NULL;
  if (!aligned16(qkv) || !aligned16(cos_table) || !aligned16(sin_table) || !aligned16(q_out) || !aligned16(k_out))
    return ARCQ_ERR_ALIGN;
  const long rows = tokens * heads;
  const unsigned grid = (unsigned)std::min<long>((rows + 15) / 16, 16384);
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (dtype == ARCQ_DTYPE_BF16)
    hipLaunchKernelGGL(rope_rows_kernel<true>, dim3(grid), dim3(256), 0, st, static_cast<const uint16_t *>(qkv), ld,
                       static_cast<const uint16_t *>(cos_table), static_cast<const uint16_t *>(sin_table), max_positions,
                       q_len, pos0, rows, num_qo_heads, num_kv_heads, static_cast<uint16_t *>(q_out),
                       static_cast<uint16_t *>(k_out));
  else
    hipLaunchKernelGGL(rope_rows_kernel<false>, dim3(grid), dim3(256), 0, st, static_cast<const uint16_t *>(qkv), ld,
                       static_cast<const uint16_t *>(cos_table), static_cast<const uint16_t *>(sin_table), max_positions,
                       q_len, pos0, rows, num_qo_heads, num_kv_heads, static_cast<uint16_t *>(q_out),
                       static_cast<uint16_t *>(k_out));
  ARCQ_HIP_TRY(hipGetLastError());
  return ARCQ_OK;
}

int arcq_kv_store_i4(const void *k_codes, const void *v_codes, const void *k_param, const void *v_param, int batch,
                     const int32_t *seqlen_indptr, int max_new_tokens, void *kv_data, void *kv_param,
                     const int32_t *kv_indptr, const int32_t *kv_indices, const int32_t *last_page_offset, int n_layers,
                     int layer_idx, int num_kv_heads, int page_size, int head_dim, void *stream) {
  using namespace arcq;
  const int rc = check_layout(kv_data, kv_param, kv_indptr, kv_indices, last_page_offset, n_layers, layer_idx,
                              num_kv_heads, page_size, head_dim, ARCQ_DTYPE_F16);
  if (rc != ARCQ_OK) return rc;
  if (batch < 0 || max_new_tokens < 0) return ARCQ_ERR_SHAPE;
  if (batch == 0 || max_new_tokens == 0) return ARCQ_OK;
  if (!k_codes || !v_codes || !k_param || !v_param) return ARCQ_ERR_NULL;
  if (((uintptr_t)k_codes | (uintptr_t)v_codes | (uintptr_t)k_param | (uintptr_t)v_param) & 3) return ARCQ_ERR_ALIGN;
  KvLayout c{static_cast<uint8_t *>(kv_data), static_cast<uint32_t *>(kv_param), kv_indptr, kv_indices,
             last_page_offset,               n_layers,                           layer_idx, num_kv_heads, page_size};
  const long rows = (long)max_new_tokens * num_kv_heads;
  int gy = (int)((rows + 15) / 16);
  if (gy > 256) gy = 256;
  hipLaunchKernelGGL(kv_store_i4_kernel, dim3(batch, gy), dim3(256), 0, static_cast<hipStream_t>(stream),
                     static_cast<const uint32_t *>(k_codes), static_cast<const uint32_t *>(v_codes),
                     static_cast<const uint32_t *>(k_param), static_cast<const uint32_t *>(v_param), seqlen_indptr, c);
  ARCQ_HIP_TRY(hipGetLastError());
  return ARCQ_OK;
}

int arcq_kv_decode_i4(void *o, const void *q, int dtype, int batch, int num_qo_heads, const void *kv_data,
                      const void *kv_param, const int32_t *kv_indptr, const int32_t *kv_indices,
                      const int32_t *last_page_offset, int n_layers, int layer_idx, int num_kv_heads, int page_size,
                      int head_dim, float sm_scale, void *stream) {
  using namespace arcq;
  const int rc = check_layout(kv_data, kv_param, kv_indptr, kv_indices, last_page_offset, n_layers, layer_idx,
                              num_kv_heads, page_size, head_dim, dtype);
  if (rc != ARCQ_OK) return rc;
  if (batch < 0 || num_qo_heads < num_kv_heads || num_qo_heads % num_kv_heads != 0) return ARCQ_ERR_SHAPE;
  const int G = num_qo_heads / num_kv_heads;
  if (G != 1 && G != 2 && G != 4) return ARCQ_ERR_SHAPE;  // query heads per KV head
  if (batch == 0) return ARCQ_OK;
  if (!o || !q) return ARCQ_ERR_NULL;
  if (!aligned16(o) || !aligned16(q)) return ARCQ_ERR_ALIGN;
  KvLayout c{const_cast<uint8_t *>(static_cast<const uint8_t *>(kv_data)),
             const_cast<uint32_t *>(static_cast<const uint32_t *>(kv_param)),
             kv_indptr,
             kv_indices,
             last_page_offset,
             n_layers,
             layer_idx,
             num_kv_heads,
             page_size};
  const float sl2 = sm_scale * 1.4426950408889634f;
  const bool mfma = page_size % 16 == 0;
  // few (sequence, KV head) pairs: cut the sequences so that about two workgroups per CU exist (the
  // lengths live on the device, so the cut is by count only; a range without tokens costs nothing).
  // The ranges' partial sums go through the stream's scratch buffer.
  hipStream_t st = static_cast<hipStream_t>(stream);
  int splits = 1;
  float *partial = nullptr;
  if (mfma) {
    const long pairs = (long)batch * num_kv_heads;
    const int split_env = tuning().kv_decode_splits;
    splits = split_env > 0 ? split_env : (pairs >= 256 ? 1 : (int)((512 + pairs - 1) / pairs));
    if (splits > 16) splits = 16;
    if (splits > 1 &&
        (size_t)batch * num_qo_heads * splits * kPartialStride * sizeof(float) > kWorkspaceBytes[kWsDecode])
      splits = 1;
    if (splits > 1) {
      int status = ARCQ_OK;
      partial = static_cast<float *>(stream_workspace(kWsDecode, st, &status));
      if (!partial) return status;
    }
  }
  dim3 grid(batch, num_kv_heads, splits);
  uint16_t *op = static_cast<uint16_t *>(o);
  const uint16_t *qp = static_cast<const uint16_t *>(q);
#define ARCQ_LAUNCH_DECODE(BF, GG)                                                                                \
  do {                                                                                                            \
    if (mfma)                                                                                                     \
      hipLaunchKernelGGL((kv_decode_i4_mfma_kernel<BF, GG>), grid, dim3(64 * kDecodeWaves), 0, st, op, qp, c,    \
                         num_qo_heads, sl2, partial);                                                             \
    else                                                                                                          \
      hipLaunchKernelGGL((kv_decode_i4_kernel<BF, GG>), dim3(batch, num_kv_heads), dim3(256), 0, st, op, qp, c,  \
                         num_qo_heads, sl2);                                                                      \
  } while (0)
  if (dtype == ARCQ_DTYPE_BF16) {
    if (G == 1) ARCQ_LAUNCH_DECODE(true, 1);
    else if (G == 2) ARCQ_LAUNCH_DECODE(true, 2);
    else ARCQ_LAUNCH_DECODE(true, 4);
  } else {
    if (G == 1) ARCQ_LAUNCH_DECODE(false, 1);
    else if (G == 2) ARCQ_LAUNCH_DECODE(false, 2);
    else ARCQ_LAUNCH_DECODE(false, 4);
  }
#undef ARCQ_LAUNCH_DECODE
  ARCQ_HIP_TRY(hipGetLastError());
  if (splits > 1) {
    if (dtype == ARCQ_DTYPE_BF16)
      hipLaunchKernelGGL(kv_decode_merge_kernel<true>, dim3(batch * num_qo_heads), dim3(128), 0, st, op, partial, splits);
    else
      hipLaunchKernelGGL(kv_decode_merge_kernel<false>, dim3(batch * num_qo_heads), dim3(128), 0, st, op, partial, splits);
    ARCQ_HIP_TRY(hipGetLastError());
  }
  return ARCQ_OK;
}

}  // extern "C"
