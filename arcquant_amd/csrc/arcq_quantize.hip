// arcq_quantize.hip -- reorder + block-FP4 quantize (+ ARC residual channels, + fused RMSNorm)
// for gfx950.  HBM-bound: one pass over the bf16 rows, coalesced 128-bit loads into LDS, the
// channel gather done out of LDS, 64-bit packed-code stores.
//
// One workgroup walks rows r = blockIdx.x, blockIdx.x + gridDim.x, ...; reorder_index (and
// gamma for the fused op) are staged in LDS once per workgroup.  A thread owns 16 consecutive
// reordered channels ("unit"): a whole NVFP4 block, or half an MXFP4 block whose other half
// sits in the neighbouring lane (one cross-lane max).
#include <hip/hip_runtime.h>

#include "arcq_internal.h"
#include "arcq_math.h"

namespace arcq {
namespace {

enum { MODE_X = 0, MODE_W = 1, MODE_NORM = 2 };
constexpr int kThreads = 256;

struct QuantParams {
  const uint16_t *x;      // bf16 [rows, K]
  const uint16_t *gamma;  // bf16 [K] (MODE_NORM)
  const int16_t *idx;     // [K]
  uint8_t *codes;         // [rows, (K+S)/2]
  uint8_t *scales;        // [rows, (K+S)/G]
  const float *d_gscale;  // optional device scalar
  float gscale;
  float eps;
  int rows, K, S;
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

template <int FMT>
__device__ __forceinline__ void store_unit(uint8_t *crow, uint8_t *srow, int unit, uint2 packed, uint32_t sbyte) {
  *reinterpret_cast<uint2 *>(crow + unit * 8) = packed;
  if (FMT == ARCQ_FMT_NVFP4) {
    srow[unit] = (uint8_t)sbyte;
  } else if ((unit & 1) == 0) {
    srow[unit >> 1] = (uint8_t)sbyte;
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
    __syncthreads();  // the previous row has been consumed (first pass: nothing pending)
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
      __syncthreads();
      double tot = 0.0;
#pragma unroll
      for (int w = 0; w < kThreads / 64; ++w) tot += red[w];
      const float var = (float)(tot / (double)K);
      rstd = 1.0f / sqrtf(var + p.eps);
    } else {
      __syncthreads();
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

__global__ void check_index_kernel(const int16_t *idx, int K, int *bad) {
  extern __shared__ uint4 smem[];
  uint32_t *seen = reinterpret_cast<uint32_t *>(smem);
  for (int i = threadIdx.x; i < (K + 31) / 32; i += blockDim.x) seen[i] = 0u;
  __syncthreads();
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
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (fmt == ARCQ_FMT_NVFP4) {
    if (mode == MODE_X) return launch_quantize<ARCQ_FMT_NVFP4, MODE_X>(p, st);
    if (mode == MODE_W) return launch_quantize<ARCQ_FMT_NVFP4, MODE_W>(p, st);
    return launch_quantize<ARCQ_FMT_NVFP4, MODE_NORM>(p, st);
  }
  if (mode == MODE_X) return launch_quantize<ARCQ_FMT_MXFP4, MODE_X>(p, st);
  if (mode == MODE_W) return launch_quantize<ARCQ_FMT_MXFP4, MODE_W>(p, st);
  return launch_quantize<ARCQ_FMT_MXFP4, MODE_NORM>(p, st);
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
