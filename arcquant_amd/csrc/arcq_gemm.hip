// arcq_gemm.hip -- augmented-K block-scaled FP4 GEMM for gfx950:
//   C[M,N] (bf16) = alpha * dq(A)[M,K'] @ dq(B)[N,K']^T, fp32 accumulation.
//
// MXFP4 runs on the scaled FP4 matrix instruction (v_mfma_scale_f32_32x32x64_f8f6f4): a lane
// feeds 32 consecutive K elements (16 bytes of codes) of one row plus that block's E8M0 byte.
// NVFP4's block-16 scales with a 3-bit mantissa have no hardware path: codes are decoded
// exactly (code value x scale has at most 6 significant bits) to bf16 in registers and fed to
// v_mfma_f32_32x32x16_bf16.
//
// The weight matrix takes the "A" operand slot and the activations the "B" slot, so that a
// lane ends up holding four consecutive output columns n of one row m and stores 8 bytes.
#include <hip/hip_runtime.h>

#include "arcq_internal.h"
#include "arcq_math.h"

namespace arcq {
namespace {

typedef int v8i __attribute__((ext_vector_type(8)));
typedef int v4i __attribute__((ext_vector_type(4)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef __bf16 v8bf __attribute__((ext_vector_type(8)));

struct GemmParams {
  const uint8_t *a_codes, *a_scales;  // activations, M rows
  const uint8_t *b_codes, *b_scales;  // weights, N rows
  uint16_t *c;                        // bf16 [M,N]
  const float *d_alpha_a, *d_alpha_b;
  float alpha;
  int M, N, Kp;
};

__device__ __forceinline__ float effective_alpha(const GemmParams &p) {
  float a = p.alpha;
  if (p.d_alpha_a && p.d_alpha_b) {
    a *= (*p.d_alpha_a) * (*p.d_alpha_b);
  } else if (p.d_alpha_a) {
    a *= *p.d_alpha_a;
  } else if (p.d_alpha_b) {
    a *= *p.d_alpha_b;
  }
  return a;
}

// One 32x32 accumulator tile -> C.  acc[v] is (n = n0 + 8*(v/4) + 4*(lane/32) + v%4, m = m0 + lane%32).
__device__ __forceinline__ void store_tile(const GemmParams &p, const v16f &acc, int m0, int n0, int lane, float alpha) {
  const int m = m0 + (lane & 31);
  if (m >= p.M) return;
  uint16_t *crow = p.c + (size_t)m * p.N;
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    const int n = n0 + 8 * q + 4 * (lane >> 5);
    uint32_t h[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) h[j] = f32_to_bf16_bits(acc[4 * q + j] * alpha);
    if (n + 3 < p.N && (p.N & 3) == 0) {
      *reinterpret_cast<uint2 *>(crow + n) = make_uint2(h[0] | (h[1] << 16), h[2] | (h[3] << 16));
    } else {
#pragma unroll
      for (int j = 0; j < 4; ++j)
        if (n + j < p.N) crow[n + j] = (uint16_t)h[j];
    }
  }
}

// ---------------------------------------------------------------------------------------------
// Baseline kernels: operands straight from global memory into registers.  Correct for every
// shape the entry point accepts; the tuned kernels below are checked against the same oracle.
// Workgroup = 4 waves in 2x2, wave tile 64(n) x 64(m).
// ---------------------------------------------------------------------------------------------
constexpr int kWgN = 128, kWgM = 128;

__global__ __launch_bounds__(256) void gemm_mxfp4_direct(GemmParams p) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int n_base = blockIdx.x * kWgN + (wave & 1) * 64;
  const int m_base = blockIdx.y * kWgM + (wave >> 1) * 64;
  const int kbytes = p.Kp >> 1, ksc = p.Kp >> 5;
  const int r = lane & 31, half = lane >> 5;
  // rows past the edge read the last valid row; their results are never stored
  const uint8_t *wrow[2], *xrow[2], *wsc[2], *xsc[2];
#pragma unroll
  for (int t = 0; t < 2; ++t) {
    const int n = min(n_base + 32 * t + r, p.N - 1), m = min(m_base + 32 * t + r, p.M - 1);
    wrow[t] = p.b_codes + (size_t)n * kbytes + 16 * half;
    xrow[t] = p.a_codes + (size_t)m * kbytes + 16 * half;
    wsc[t] = p.b_scales + (size_t)n * ksc + half;
    xsc[t] = p.a_scales + (size_t)m * ksc + half;
  }
  v16f acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.0f;

  for (int k = 0; k < p.Kp; k += 64) {
    v8i wf[2], xf[2];
    int ws[2], xs[2];
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      const uint4 wq = *reinterpret_cast<const uint4 *>(wrow[t] + (k >> 1));
      const uint4 xq = *reinterpret_cast<const uint4 *>(xrow[t] + (k >> 1));
      wf[t] = v8i{(int)wq.x, (int)wq.y, (int)wq.z, (int)wq.w, 0, 0, 0, 0};
      xf[t] = v8i{(int)xq.x, (int)xq.y, (int)xq.z, (int)xq.w, 0, 0, 0, 0};
      ws[t] = wsc[t][k >> 5];
      xs[t] = xsc[t][k >> 5];
    }
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int j = 0; j < 2; ++j)
        acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(wf[i], xf[j], acc[i][j], 4, 4, 0, ws[i], 0, xs[j]);
  }
  const float alpha = effective_alpha(p);
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j) store_tile(p, acc[i][j], m_base + 32 * j, n_base + 32 * i, lane, alpha);
}

// 8 e2m1 codes (one dword, element 0 in the low nibble) times an NVFP4 block scale -> 8 bf16.
// Exact: |code value| has 2 significant bits, the scale 4.
__device__ __forceinline__ v8bf decode8_nvfp4(uint32_t codes, float s) {
  v8bf out;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const float f = e2m1_value((codes >> (4 * i)) & 15u) * s;
    out[i] = __builtin_bit_cast(__bf16, (uint16_t)(f2u(f) >> 16));
  }
  return out;
}

__global__ __launch_bounds__(256) void gemm_nvfp4_direct(GemmParams p) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int n_base = blockIdx.x * kWgN + (wave & 1) * 64;
  const int m_base = blockIdx.y * kWgM + (wave >> 1) * 64;
  const int kbytes = p.Kp >> 1, ksc = p.Kp >> 4;
  const int r = lane & 31, half = lane >> 5;
  const uint8_t *wrow[2], *xrow[2], *wsc[2], *xsc[2];
#pragma unroll
  for (int t = 0; t < 2; ++t) {
    const int n = min(n_base + 32 * t + r, p.N - 1), m = min(m_base + 32 * t + r, p.M - 1);
    wrow[t] = p.b_codes + (size_t)n * kbytes + 4 * half;
    xrow[t] = p.a_codes + (size_t)m * kbytes + 4 * half;
    wsc[t] = p.b_scales + (size_t)n * ksc;
    xsc[t] = p.a_scales + (size_t)m * ksc;
  }
  v16f acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.0f;

  // one MFMA step covers K=16 = one NVFP4 block: lanes 0-31 take its first 8 elements, 32-63 the rest
  for (int k = 0; k < p.Kp; k += 16) {
    v8bf wf[2], xf[2];
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      const uint32_t wc = *reinterpret_cast<const uint32_t *>(wrow[t] + (k >> 1));
      const uint32_t xc = *reinterpret_cast<const uint32_t *>(xrow[t] + (k >> 1));
      wf[t] = decode8_nvfp4(wc, nvfp4_scale_value(wsc[t][k >> 4]));
      xf[t] = decode8_nvfp4(xc, nvfp4_scale_value(xsc[t][k >> 4]));
    }
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int j = 0; j < 2; ++j)
        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(wf[i], xf[j], acc[i][j], 0, 0, 0);
  }
  const float alpha = effective_alpha(p);
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j) store_tile(p, acc[i][j], m_base + 32 * j, n_base + 32 * i, lane, alpha);
}

}  // namespace
}  // namespace arcq

extern "C" int arcq_matmul(const void *a_codes, const void *a_scales, const void *b_codes, const void *b_scales,
                           int M, int N, int Kp, int fmt, float alpha, const float *d_alpha_a,
                           const float *d_alpha_b, void *c, void *stream) {
  using namespace arcq;
  if (fmt != ARCQ_FMT_NVFP4 && fmt != ARCQ_FMT_MXFP4) return ARCQ_ERR_FORMAT;
  if (M < 0 || N < 0 || Kp < 64 || Kp % 64 != 0) return ARCQ_ERR_SHAPE;
  if (M == 0 || N == 0) return ARCQ_OK;
  if (!a_codes || !a_scales || !b_codes || !b_scales || !c) return ARCQ_ERR_NULL;
  if (!aligned16(a_codes) || !aligned16(b_codes) || !aligned16(c)) return ARCQ_ERR_ALIGN;
  GemmParams p;
  p.a_codes = static_cast<const uint8_t *>(a_codes);
  p.a_scales = static_cast<const uint8_t *>(a_scales);
  p.b_codes = static_cast<const uint8_t *>(b_codes);
  p.b_scales = static_cast<const uint8_t *>(b_scales);
  p.c = static_cast<uint16_t *>(c);
  p.d_alpha_a = d_alpha_a;
  p.d_alpha_b = d_alpha_b;
  p.alpha = alpha;
  p.M = M;
  p.N = N;
  p.Kp = Kp;
  hipStream_t st = static_cast<hipStream_t>(stream);
  dim3 grid((N + kWgN - 1) / kWgN, (M + kWgM - 1) / kWgM);
  if (fmt == ARCQ_FMT_MXFP4)
    hipLaunchKernelGGL(gemm_mxfp4_direct, grid, dim3(256), 0, st, p);
  else
    hipLaunchKernelGGL(gemm_nvfp4_direct, grid, dim3(256), 0, st, p);
  ARCQ_HIP_TRY(hipGetLastError());
  return ARCQ_OK;
}
