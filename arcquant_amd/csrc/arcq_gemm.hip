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
#include <stdlib.h>

#include <algorithm>
#include <mutex>
#include <type_traits>

#include "arcq_internal.h"
#include "arcq_math.h"
#include "arcq_swiglu.h"

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
  // split-K (tiled kernels): blockIdx.y selects one of k_slices ranges of K steps and the workgroup
  // writes its fp32 partial tile to partial[slice][M][N] instead of C; splitk_reduce_kernel adds them
  float *partial = nullptr;
  int k_slices = 1;
  // optional residual, bf16 [M,N]: C = bf16(bf16(alpha * acc) + residual), what a bf16 add of the
  // rounded GEMM output and the residual gives
  const uint16_t *residual = nullptr;
  // grouped GEMM (tiled kernels): rows seg[e] .. seg[e+1]-1 of A and C belong to segment e, whose weights
  // start seg_b_codes / seg_b_scales bytes after those of segment e-1; d_alpha_a / d_alpha_b are arrays
  // indexed by segment.  A workgroup rewrites its copy of these parameters to its segment's sub-problem.
  const int *seg = nullptr;
  int n_seg = 0;
  size_t seg_b_codes = 0, seg_b_scales = 0;
  // fused SwiGLU epilogue (tiled kernels): the weight rows alternate gate, up, gate, up ..., so that output
  // columns 2j and 2j+1 are gate_j and up_j of one token and sit in one lane; c then is bf16 [M, N/2] and
  // receives act_fn(gate) * up formed from the bf16-rounded GEMM outputs, exactly what the unfused sequence
  // (GEMM, then silu and multiply in bf16) gives.  absmax_bits: NULL, or one word per segment (one word when
  // not grouped) that collects max |output| as the bits of a non-negative float (zeroed by the caller).
  int swiglu = 0;
  uint32_t *absmax_bits = nullptr;
  int seg_index = 0;
};

// Grouped launches: maps the workgroup to (segment, tile) and turns p into that segment's problem (M = its
// rows, operand pointers moved to its first row and its weights).  lin: tile number inside the segment, in
// the order the ungrouped kernels use.  The launch holds an upper bound of the tile count; workgroups
// beyond the real count return false.  G: elements per scale byte.
template <int BM, int BN, int G>
__device__ __forceinline__ bool enter_segment(GemmParams &p, int &lin) {
  const int tiles_n = (p.N + BN - 1) / BN;
  const int per_xcd = gridDim.x >> 3;  // the grid is a multiple of 8: contiguous runs of tiles per XCD
  lin = (blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);
  const int rows = p.M;
  int beg = min(max(p.seg[0], 0), rows);
  for (int e = 0; e < p.n_seg; ++e) {
    const int end = min(max(p.seg[e + 1], beg), rows);  // offsets that do not grow or leave the tensor: empty segments
    const int cnt = end - beg;
    const int t = ((cnt + BM - 1) / BM) * tiles_n;
    if (lin < t) {
      const size_t kbytes = p.Kp >> 1, ksc = p.Kp / G;
      p.a_codes += (size_t)beg * kbytes;
      p.a_scales += (size_t)beg * ksc;
      p.c += (size_t)beg * (p.swiglu ? p.N >> 1 : p.N);
      if (p.residual) p.residual += (size_t)beg * p.N;
      p.b_codes += (size_t)e * p.seg_b_codes;
      p.b_scales += (size_t)e * p.seg_b_scales;
      if (p.d_alpha_a) p.d_alpha_a += e;
      if (p.d_alpha_b) p.d_alpha_b += e;
      p.M = cnt;
      p.seg_index = e;
      return true;
    }
    lin -= t;
    beg = end;
  }
  return false;
}

// two bf16 pairs + two bf16 pairs, each sum rounded to bf16
__device__ __forceinline__ uint32_t add_bf16_pair(uint32_t a, uint32_t b) {
  return pack_bf16_rne(u2f(a << 16) + u2f(b << 16), u2f(a & 0xffff0000u) + u2f(b & 0xffff0000u));
}
__device__ __forceinline__ uint2 add_bf16_x4(uint2 a, uint2 b) {
  return make_uint2(add_bf16_pair(a.x, b.x), add_bf16_pair(a.y, b.y));
}

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
  if (m0 + 32 <= p.M && n0 + 32 <= p.N && (p.N & 3) == 0) {  // tile fully inside: no per-element checks
    uint16_t *crow = p.c + (size_t)m * p.N + n0 + 4 * (lane >> 5);
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      uint2 v = make_uint2(pack_bf16_rne(acc[4 * q] * alpha, acc[4 * q + 1] * alpha),
                           pack_bf16_rne(acc[4 * q + 2] * alpha, acc[4 * q + 3] * alpha));
      if (p.residual) v = add_bf16_x4(v, *reinterpret_cast<const uint2 *>(p.residual + (crow - p.c) + 8 * q));
      *reinterpret_cast<uint2 *>(crow + 8 * q) = v;
    }
    return;
  }
  if (m >= p.M) return;
  uint16_t *crow = p.c + (size_t)m * p.N;
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    const int n = n0 + 8 * q + 4 * (lane >> 5);
    uint32_t h[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) h[j] = f32_to_bf16_bits(acc[4 * q + j] * alpha);
    if (p.residual) {
      const uint16_t *rrow = p.residual + (size_t)m * p.N;
#pragma unroll
      for (int j = 0; j < 4; ++j)
        if (n + j < p.N) h[j] = f32_to_bf16_bits(bf16_bits_to_f32(h[j]) + bf16_bits_to_f32(rrow[n + j]));
    }
    if (n + 3 < p.N && (p.N & 3) == 0) {
      *reinterpret_cast<uint2 *>(crow + n) = make_uint2(h[0] | (h[1] << 16), h[2] | (h[3] << 16));
    } else {
#pragma unroll
      for (int j = 0; j < 4; ++j)
        if (n + j < p.N) crow[n + j] = (uint16_t)h[j];
    }
  }
}

// One 32x32 accumulator tile that lies inside C, with 16-byte stores: lanes r and r + 32 hold the two halves of
// eight consecutive columns of row r for every q; one half-wave swap (v_permlane32_swap) per register pair gives
// the lower lane all eight columns of an even q and the upper lane those of the odd q behind it.
// c: this lane's address for q = 0 (row m0 + lane % 32, column n0 + 8 * (lane / 32)); res: the same into the residual, or NULL.
__device__ __forceinline__ void store_tile_rows16(const v16f &acc, uint16_t *c, const uint16_t *res, float alpha) {
#pragma unroll
  for (int h = 0; h < 2; ++h) {  // q = 2h (lower lanes) and 2h + 1 (upper lanes)
    const uint32_t e0 = pack_bf16_rne(acc[8 * h] * alpha, acc[8 * h + 1] * alpha);
    const uint32_t e1 = pack_bf16_rne(acc[8 * h + 2] * alpha, acc[8 * h + 3] * alpha);
    const uint32_t o0 = pack_bf16_rne(acc[8 * h + 4] * alpha, acc[8 * h + 5] * alpha);
    const uint32_t o1 = pack_bf16_rne(acc[8 * h + 6] * alpha, acc[8 * h + 7] * alpha);
    // swap(upper lanes of the first operand, lower lanes of the second): lower lanes end up with (own even q,
    // partner's even q), upper lanes with (partner's odd q, own odd q)
    const auto s0 = __builtin_amdgcn_permlane32_swap(e0, o0, false, false);
    const auto s1 = __builtin_amdgcn_permlane32_swap(e1, o1, false, false);
    uint4 v = make_uint4(s0[0], s1[0], s0[1], s1[1]);
    if (res) {
      const uint4 rv = *reinterpret_cast<const uint4 *>(res + 16 * h);
      v = make_uint4(add_bf16_pair(v.x, rv.x), add_bf16_pair(v.y, rv.y), add_bf16_pair(v.z, rv.z), add_bf16_pair(v.w, rv.w));
    }
    *reinterpret_cast<uint4 *>(c + 16 * h) = v;
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


// ---------------------------------------------------------------------------------------------
// Tiled MXFP4 kernel: 256 threads = 2x2 waves, workgroup tile (64*WN) x (64*WM), K step 256.
// Requires K' % 128 == 0 (scale rows are then dword-aligned and a K step ends on a dword).
//
// Global -> LDS goes through LDS-direct loads (global_load_lds_dwordx4 / _dword): no staging
// registers, a wave's 64 lanes fill consecutive LDS in lane order.  A code-tile row is 128 bytes =
// 8 chunks of 16 bytes (one MX block each); lane l of a load fetches row l/8 and, instead of
// chunk l%8, chunk (l%8) ^ ((row>>1)&7): global reads still cover whole 128-byte lines, while the
// 16 lanes of an MFMA operand read (16 consecutive rows, same chunk) hit 16 different 16-byte
// bank groups.  The E8M0 bytes of the step (8 per row) travel the same way, 4 bytes per lane.
// Two LDS stages: the loads of step k+1 are in flight while step k is multiplied.
// Every vector-memory instruction of the main loop is one of these loads, written as inline asm
// and waited for explicitly before the barrier -- the compiler's wait-count pass would otherwise
// put a vmcnt(0) in front of LDS reads and drain the prefetch in the middle of the MFMAs.
//
// Inside a K step a lane with half index kh = lane/32 consumes blocks 4*kh .. 4*kh+3 in its four
// MFMAs, so its four E8M0 bytes are one dword of the row-major scale array and the byte is
// picked by the instruction's op_sel.
// ---------------------------------------------------------------------------------------------
// These write M0.  The compiler reserves M0 and refuses it on a clobber list ("may lead to undefined
// behaviour"), so the contract is kept by hand: the kernels that use these helpers contain nothing for
// which the compiler would set or read M0 itself (no LDS-direct builtins, no indirect register
// indexing, no s_sendmsg), and every helper sets M0 before its load.
__device__ __forceinline__ void lds_dma16(const void *g, uint32_t lds_wave_base) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off"
               :
               : "s"(lds_wave_base), "v"(g)
               : "memory");
}

// The same with a wave-uniform base address and a 32-bit byte offset per lane.
__device__ __forceinline__ void lds_dma16_at(const void *base, uint32_t lane_offset, uint32_t lds_wave_base) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
               :
               : "s"(lds_wave_base), "v"(lane_offset), "s"(base)
               : "memory");
}

__device__ __forceinline__ void lds_dma4(const void *g, uint32_t lds_wave_base) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %1, off" : : "s"(lds_wave_base), "v"(g) : "memory");
}

__device__ __forceinline__ void wait_dma_and_sync() {
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
  __builtin_amdgcn_s_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}

template <int WN, int WM, int NWM>
__device__ __forceinline__ void store_workgroup_tile_swiglu_fwd(const GemmParams &p, v16f (&acc)[WN][WM], uint8_t *ldsA,
                                                                uint8_t *ldsB, int m_base, int n_base, int wave, int lane);

// Epilogue shared by the tiled kernels: acc[i][j] is the 32x32 tile (n-tile i, m-tile j) of the
// wave tile.  The workgroup's waves form a 2 (along N) x NWM (along M) grid, wave = n + 2 * m.
// ldsA / ldsB: two LDS areas of at least NWM*32*WM*64*WN bytes each, free for reuse.
template <int WN, int WM, int NWM = 2>
__device__ __forceinline__ void store_workgroup_tile(const GemmParams &p, v16f (&acc)[WN][WM], uint8_t *ldsA,
                                                     uint8_t *ldsB, int m_base, int n_base, int wave, int lane) {
  constexpr int BN = 64 * WN, BM = 32 * WM * NWM;
  const int r = lane & 31, kh = lane >> 5;
  const int wn0 = (wave & 1) * 32 * WN, wm0 = (wave >> 1) * 32 * WM;
  if (p.swiglu) return store_workgroup_tile_swiglu_fwd<WN, WM, NWM>(p, acc, ldsA, ldsB, m_base, n_base, wave, lane);
  if (p.partial) {  // split-K: the unscaled fp32 tile of this K range
    float *part = p.partial + (size_t)blockIdx.y * p.M * p.N;
#pragma unroll
    for (int i = 0; i < WN; ++i)
#pragma unroll
      for (int j = 0; j < WM; ++j) {
        const int m = m_base + wm0 + 32 * j + r;
        if (m >= p.M) continue;
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const int n = n_base + wn0 + 32 * i + 8 * q + 4 * kh;
          float *dst = part + (size_t)m * p.N + n;
          if (n + 3 < p.N && (p.N & 3) == 0) {
            *reinterpret_cast<float4 *>(dst) =
                make_float4(acc[i][j][4 * q], acc[i][j][4 * q + 1], acc[i][j][4 * q + 2], acc[i][j][4 * q + 3]);
          } else {
#pragma unroll
            for (int e = 0; e < 4; ++e)
              if (n + e < p.N) dst[e] = acc[i][j][4 * q + e];
          }
        }
      }
    return;
  }
  const float alpha = effective_alpha(p);
  constexpr bool kPow2 = (WN & (WN - 1)) == 0;  // the swizzled transpose below needs 4*WN lanes per row to be a power of two
  if (kPow2 && m_base + BM <= p.M && n_base + BN <= p.N && (p.N & 7) == 0) {
    // Whole tile inside C: transpose each wave's tile through LDS (free now) so that every store
    // instruction writes whole rows of the wave tile, 16 bytes per lane.
    wait_dma_and_sync();  // every wave is done reading operands
    constexpr int RB = 64 * WN;                       // bytes per row of the wave tile
    constexpr int LPR = 4 * WN;                       // lanes per row when reading 16 bytes each
    uint8_t *region = (wave < NWM ? ldsA : ldsB) + (wave % NWM) * (32 * WM * RB);
#pragma unroll
    for (int i = 0; i < WN; ++i)
#pragma unroll
      for (int j = 0; j < WM; ++j) {
        const int m = 32 * j + r;
        const int sw = (m & (LPR - 1)) << 1;          // even: keeps 8-byte chunk pairs adjacent
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const v16f &a = acc[i][j];                  // the hardware's round-to-nearest-even convert
          const int c = 8 * i + 2 * q + kh;           // 8-byte chunk of the row
          *reinterpret_cast<uint2 *>(region + m * RB + ((c ^ sw) << 3)) =
              make_uint2(pack_bf16_rne(a[4 * q] * alpha, a[4 * q + 1] * alpha),
                         pack_bf16_rne(a[4 * q + 2] * alpha, a[4 * q + 3] * alpha));
        }
      }
    const int rr = lane / LPR, t = lane % LPR;
    uint16_t *cbase = p.c + (size_t)(m_base + wm0) * p.N + n_base + wn0 + 8 * t;
#pragma unroll
    for (int it = 0; it < (32 * WM * LPR) / 64; ++it) {
      const int m = it * (64 / LPR) + rr;
      const int sw = (m & (LPR - 1)) << 1;
      uint4 v = *reinterpret_cast<const uint4 *>(region + m * RB + (((2 * t) ^ sw) << 3));
      if (p.residual) {
        const uint4 rv = *reinterpret_cast<const uint4 *>(p.residual + (cbase - p.c) + (size_t)m * p.N);
        v = make_uint4(add_bf16_pair(v.x, rv.x), add_bf16_pair(v.y, rv.y), add_bf16_pair(v.z, rv.z),
                       add_bf16_pair(v.w, rv.w));
      }
      *reinterpret_cast<uint4 *>(cbase + (size_t)m * p.N) = v;
    }
    return;
  }
#pragma unroll
  for (int i = 0; i < WN; ++i)
#pragma unroll
    for (int j = 0; j < WM; ++j)
      store_tile(p, acc[i][j], m_base + wm0 + 32 * j, n_base + wn0 + 32 * i, lane, alpha);
}

// Fused SwiGLU epilogue of the tiled kernels (p.swiglu): a lane's four consecutive columns of one row are
// (gate_j, up_j, gate_j+1, up_j+1); each is rounded to bf16 as the plain epilogue would store it, and the two
// products act_fn(gate) * up leave as one dword.  Whole tiles go through LDS so that every store
// instruction writes 16 bytes per lane along output rows; ragged tiles store dwords with bounds checks.
template <int WN, int WM, int NWM>
__device__ __forceinline__ void store_workgroup_tile_swiglu(const GemmParams &p, v16f (&acc)[WN][WM], uint8_t *ldsA,
                                                            uint8_t *ldsB, int m_base, int n_base, int wave, int lane) {
  constexpr int BN = 64 * WN, BM = 32 * WM * NWM;
  const int r = lane & 31, kh = lane >> 5;
  const int wn0 = (wave & 1) * 32 * WN, wm0 = (wave >> 1) * 32 * WM;
  const float alpha = effective_alpha(p);
  const int No = p.N >> 1;  // output columns
  uint32_t amax = 0u;       // max |t| of this lane as bf16 bits without the sign
  auto product = [&](const v16f &a, int q) {  // the hardware's RNE convert: the bits f32_to_bf16_bits gives
    return swiglu_pair(pack_bf16_rne(a[4 * q] * alpha, a[4 * q + 2] * alpha),
                       pack_bf16_rne(a[4 * q + 1] * alpha, a[4 * q + 3] * alpha));
  };
  auto track = [&](uint32_t t) {
    const uint32_t lo = t & 0x7fffu, hi = (t >> 16) & 0x7fffu;
    amax = lo > amax ? lo : amax;
    amax = hi > amax ? hi : amax;
  };
  constexpr bool kPow2 = (WN & (WN - 1)) == 0;
  if (kPow2 && m_base + BM <= p.M && n_base + BN <= p.N && (No & 7) == 0) {
    wait_dma_and_sync();  // every wave is done reading operands
    constexpr int RB = 32 * WN;   // bytes per row of the wave tile: 16 * WN products
    constexpr int LPR = 2 * WN;   // lanes per row when reading 16 bytes each
    uint8_t *region = (wave < NWM ? ldsA : ldsB) + (wave % NWM) * (32 * WM * RB);
#pragma unroll
    for (int i = 0; i < WN; ++i)
#pragma unroll
      for (int j = 0; j < WM; ++j) {
        const int m = 32 * j + r;
        const int sw = m & (LPR - 1);                 // swizzle of the row's 16-byte groups
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const uint32_t t = product(acc[i][j], q);
          track(t);
          const int c = 8 * i + 2 * q + kh;           // dword of the row
          *reinterpret_cast<uint32_t *>(region + m * RB + ((((c >> 2) ^ sw) << 2) | (c & 3)) * 4) = t;
        }
      }
    const int rr = lane / LPR, tq = lane % LPR;
    uint16_t *cbase = p.c + (size_t)(m_base + wm0) * No + ((n_base + wn0) >> 1) + 8 * tq;
#pragma unroll
    for (int it = 0; it < (32 * WM * LPR) / 64; ++it) {
      const int m = it * (64 / LPR) + rr;
      const int sw = m & (LPR - 1);
      const uint4 v = *reinterpret_cast<const uint4 *>(region + m * RB + ((tq ^ sw) << 4));
      *reinterpret_cast<uint4 *>(cbase + (size_t)m * No) = v;
    }
  } else {
#pragma unroll
    for (int i = 0; i < WN; ++i)
#pragma unroll
      for (int j = 0; j < WM; ++j) {
        const int m = m_base + wm0 + 32 * j + r;
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const int n = n_base + wn0 + 32 * i + 8 * q + 4 * kh;
          const uint32_t t = product(acc[i][j], q);   // every lane computes (the special-value test of the
          if (m < p.M && n + 3 < p.N) {               // activation function is a vote of the whole wave)
            track(t);
            *reinterpret_cast<uint32_t *>(p.c + (size_t)m * No + (n >> 1)) = t;
          }
        }
      }
  }
  if (p.absmax_bits) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
      const uint32_t v = (uint32_t)__shfl_xor((int)amax, o);
      amax = v > amax ? v : amax;
    }
    if (lane == 0 && amax) atomicMax(p.absmax_bits + p.seg_index, amax << 16);  // bf16 bits -> fp32 bits
  }
}

template <int WN, int WM, int NWM>
__device__ __forceinline__ void store_workgroup_tile_swiglu_fwd(const GemmParams &p, v16f (&acc)[WN][WM], uint8_t *ldsA,
                                                                uint8_t *ldsB, int m_base, int n_base, int wave, int lane) {
  store_workgroup_tile_swiglu<WN, WM, NWM>(p, acc, ldsA, ldsB, m_base, n_base, wave, lane);
}

// An FP4 operand of the scaled MFMA is 4 registers; the builtin's type has 8, the upper 4 unused.
__device__ __forceinline__ v8i fp4_operand(uint4 q) {
  const v4i v = {(int)q.x, (int)q.y, (int)q.z, (int)q.w};
  return __builtin_shufflevector(v, v, 0, 1, 2, 3, -1, -1, -1, -1);
}

// Scheduling pattern of one MXFP4 sub-step: NM MFMAs with NR LDS reads (the next sub-step's operands)
// spread behind them, the first MFMAs taking the larger shares.
template <int NM, int NR, int M = 0>
struct MfmaReadPattern {
  static __device__ __forceinline__ void apply() {
    if constexpr (M < NM) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      constexpr int R = (NR + NM - 1 - M) / NM;
      if constexpr (R > 0) __builtin_amdgcn_sched_group_barrier(0x100, R, 0);
      MfmaReadPattern<NM, NR, M + 1>::apply();
    }
  }
};

template <int WN, int WM, int NS = 2, int NWM = 2, bool PERSIST = false>
__global__ __launch_bounds__(128 * NWM) void gemm_mxfp4_tiled(GemmParams p) {
  // waves: 2 along N x NWM along M (wave = n + 2 * m), each with WN x WM accumulator tiles of 32 x 32
  constexpr int BN = 64 * WN, BM = 32 * WM * NWM, NW = 2 * NWM;
  // PERSIST (eight-wave tiles, plain launches): at most one workgroup per CU walks the tiles of its XCD's run.
  // The stages and the scale pairs keep alternating across tiles, so the first stage of the next tile is
  // requested during the last K step of the current one, and the finished tile leaves straight from the
  // accumulator registers (no LDS, no barrier) while those requests are on their way.
  static_assert(!PERSIST || (NWM == 4 && NS == 2 && WN == 4 && WM == 2), "persistent workgroups are built on the 256x256 requesting-wave layout");
  // Eight waves (two per SIMD): the first wave of every SIMD requests the whole next stage, the second one
  // goes straight to its MFMAs, so the matrix pipe works while the requests queue up in the load unit.
  constexpr bool kLoaderWaves = NWM == 4 && NS == 2;
  constexpr int NLW = kLoaderWaves ? NW / 2 : NW;  // waves that request the stages

  constexpr int RPI = 8 * NLW;   // rows of 128 code bytes that one load instruction of the requesting waves covers
  static_assert(NS == 2 || (NS == 4 && WN == 2 && WM <= 2 && NWM == 2), "the four-stage ring's wait counts are those of the 128x64 and 128x128 tiles");
  static_assert(!kLoaderWaves || (BN / 64 <= NLW && BM / 64 <= NLW), "one scale load per operand and requesting wave");
  __shared__ uint4 sW[NS * BN * 8], sX[NS * BM * 8];  // code tiles, NS stages each
  __shared__ uint4 sWs[NS * BN], sXs[NS * BM];        // 16 scale bytes per row (two K steps), NS stages each
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int kbytes = p.Kp >> 1, ksc = p.Kp >> 5;

  // tile of this workgroup: consecutive workgroup ids go to different XCDs (8 of them, each with
  // its own L2), so hand each XCD a contiguous run of tiles that walk down M for a fixed weight tile
  int lin;
  int run_left = 0, run_step = 0;  // PERSIST: tiles of this XCD's run still ahead of `lin`, distance between this workgroup's tiles
  if (p.seg) {
    if (!enter_segment<BM, BN, 32>(p, lin)) return;
  } else {
    const int total = ((p.M + BM - 1) / BM) * ((p.N + BN - 1) / BN);
    const int per_xcd = (total + 7) >> 3;
    if constexpr (PERSIST) {
      const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
      run_step = gridDim.x >> 3;
      const int run_end = min(total, (xcd + 1) * per_xcd);
      lin = xcd * per_xcd + slot;
      if (lin >= run_end) return;
      run_left = run_end - lin;
    } else {
      lin = (blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);
      if (lin >= total) return;
    }
  }
  const int tiles_m = (p.M + BM - 1) / BM;
  int n_base = (lin / tiles_m) * BN, m_base = (lin % tiles_m) * BM;

  const int nk = (p.Kp + 255) >> 8;
  const bool short_last = (p.Kp & 255) != 0;  // then the last step has 4 valid blocks (K' % 256 == 128)

  // ---- global -> LDS plan: codes
  const int ld_row = (tid >> 3) & (RPI - 1);                     // + RPI*i
  const int ld_q = (tid & 7) ^ ((ld_row >> 1) & 7);              // chunk fetched by this lane
  // With requesting waves the addresses are a wave-uniform base (operand + K offset) plus a 32-bit byte
  // offset per lane (the host sends operands of 4 GiB and more to the four-wave kernels).
  constexpr int NPW = kLoaderWaves ? 1 : BN / RPI, NPX = kLoaderWaves ? 1 : BM / RPI;
  // (persistent workgroups see whole tiles only: no row is clamped, the rows of one lane are RPI * kbytes apart,
  // and one offset per operand is enough: the multiples go into the scalar base)
  constexpr int NOW = kLoaderWaves && !PERSIST ? BN / RPI : 1, NOX = kLoaderWaves && !PERSIST ? BM / RPI : 1;
  const uint8_t *wsrc[NPW], *xsrc[NPX];
  uint32_t wvo[NOW], xvo[NOX];
  uint32_t wsvo = 0, xsvo = 0;
  const int npairs = (nk + 1) >> 1;
  const int sc_shift = max(0, npairs * 16 - ksc);
  auto lane_offsets = [&](int nb, int mb) {  // requesting waves: this lane's byte offsets into the operands for a tile
#pragma unroll
    for (int i = 0; i < NOW; ++i) wvo[i] = (uint32_t)min(nb + RPI * i + ld_row, p.N - 1) * (uint32_t)kbytes + ld_q * 16;
#pragma unroll
    for (int i = 0; i < NOX; ++i) xvo[i] = (uint32_t)min(mb + RPI * i + ld_row, p.M - 1) * (uint32_t)kbytes + ld_q * 16;
    wsvo = (uint32_t)min(nb + 64 * min(wave, BN / 64 - 1) + lane, p.N - 1) * (uint32_t)ksc;
    xsvo = (uint32_t)min(mb + 64 * min(wave, BM / 64 - 1) + lane, p.M - 1) * (uint32_t)ksc;
  };
  if constexpr (kLoaderWaves) {
    lane_offsets(n_base, m_base);
  } else {
#pragma unroll
    for (int i = 0; i < BN / RPI; ++i)
      wsrc[i] = p.b_codes + (size_t)min(n_base + RPI * i + ld_row, p.N - 1) * kbytes + ld_q * 16;
#pragma unroll
    for (int i = 0; i < BM / RPI; ++i)
      xsrc[i] = p.a_codes + (size_t)min(m_base + RPI * i + ld_row, p.M - 1) * kbytes + ld_q * 16;
  }
  // ---- scales: a lane fetches 16 bytes = the E8M0 bytes of one row for a PAIR of K steps; one
  // load instruction covers 64 rows.  Instruction j of the weights goes to wave j%NW, of the
  // activations to wave (j+BN/64)%NW; with requesting waves, instruction j of either operand to wave j.
  // If the row ends inside the last pair, the 16-byte window is
  // shifted back to end at the row end (sc_shift bytes; K' % 128 == 0 makes it a multiple of 4).
  constexpr int NPS = kLoaderWaves ? 1 : BN / 64, NPT = kLoaderWaves ? 1 : BM / 64;
  const uint8_t *wssrc[NPS], *xssrc[NPT];
  if constexpr (!kLoaderWaves) {
#pragma unroll
    for (int j = 0; j < BN / 64; ++j) wssrc[j] = p.b_scales + (size_t)min(n_base + 64 * j + lane, p.N - 1) * ksc;
#pragma unroll
    for (int j = 0; j < BM / 64; ++j) xssrc[j] = p.a_scales + (size_t)min(m_base + 64 * j + lane, p.M - 1) * ksc;
  }
  const uint32_t lw0 = (uint32_t)reinterpret_cast<uintptr_t>(sW) + (wave % NLW) * 1024;
  const uint32_t lx0 = (uint32_t)reinterpret_cast<uintptr_t>(sX) + (wave % NLW) * 1024;
  const uint32_t lws0 = (uint32_t)reinterpret_cast<uintptr_t>(sWs);
  const uint32_t lxs0 = (uint32_t)reinterpret_cast<uintptr_t>(sXs);

  // sb / pb: K steps and scale pairs of the tiles this workgroup has finished (0 unless PERSIST): the stage of a
  // step and of a pair alternate across tiles
  int step_base = 0, pair_base = 0;
  auto issue = [&](int kt, int sb, int pb) {
    const int st = (kt + sb) & (NS - 1);
    // a short last step has only chunks 0..3: fetch those twice; the products of the absent blocks
    // are zeroed in compute()
    const bool clip = short_last && kt == nk - 1;
    if constexpr (kLoaderWaves) {
      const uint8_t *wb = p.b_codes + kt * 128, *xb = p.a_codes + kt * 128;
      const uint32_t back = (clip && ld_q >= 4) ? 64u : 0u;
      const size_t rows_step = PERSIST ? (size_t)RPI * kbytes : 0;
#pragma unroll
      for (int i = 0; i < BN / RPI; ++i)
        lds_dma16_at(wb + i * rows_step, wvo[PERSIST ? 0 : i] - back, lw0 + st * (BN * 128) + i * (RPI * 128));
#pragma unroll
      for (int i = 0; i < BM / RPI; ++i)
        lds_dma16_at(xb + i * rows_step, xvo[PERSIST ? 0 : i] - back, lx0 + st * (BM * 128) + i * (RPI * 128));
      if ((kt & 1) == 0) {  // scales of steps kt and kt+1
        const int pair = kt >> 1, sst = (pair + pb) & (NS - 1);
        const int soff = pair * 16 - (pair == npairs - 1 ? sc_shift : 0);
        if (wave < BN / 64) lds_dma16_at(p.b_scales + soff, wsvo, lws0 + sst * (BN * 16) + wave * 1024);
        if (wave < BM / 64) lds_dma16_at(p.a_scales + soff, xsvo, lxs0 + sst * (BM * 16) + wave * 1024);
      }
    } else {
    const int koff = kt * 128 - ((clip && ld_q >= 4) ? 64 : 0);
#pragma unroll
    for (int i = 0; i < NPW; ++i) lds_dma16(wsrc[i] + koff, lw0 + st * (BN * 128) + i * (RPI * 128));
#pragma unroll
    for (int i = 0; i < NPX; ++i) lds_dma16(xsrc[i] + koff, lx0 + st * (BM * 128) + i * (RPI * 128));
    if ((kt & 1) == 0) {  // scales of steps kt and kt+1
      const int pair = kt >> 1, sst = (pair + pb) & (NS - 1);
      const int soff = pair * 16 - (pair == npairs - 1 ? sc_shift : 0);
#pragma unroll
      for (int j = 0; j < NPS; ++j)
        if ((j % NW) == wave) lds_dma16(wssrc[j] + soff, lws0 + sst * (BN * 16) + j * 1024);
#pragma unroll
      for (int j = 0; j < NPT; ++j)
        if (((j + BN / 64) % NW) == wave) lds_dma16(xssrc[j] + soff, lxs0 + sst * (BM * 16) + j * 1024);
    }
    }
  };

  // ---- LDS -> MFMA operands
  const int r = lane & 31, kh = lane >> 5;
  const int swz = (r >> 1) & 7;
  const int wn0 = (wave & 1) * 32 * WN, wm0 = (wave >> 1) * 32 * WM;   // wave tile inside the workgroup tile
  int w_rd[4], x_rd[4];                                                   // chunk index for tile 0, per sub-step
#pragma unroll
  for (int ks = 0; ks < 4; ++ks) {
    w_rd[ks] = (wn0 + r) * 8 + ((4 * kh + ks) ^ swz);
    x_rd[ks] = (wm0 + r) * 8 + ((4 * kh + ks) ^ swz);
  }
  const int ws_rd = (wn0 + r) * 4, xs_rd = (wm0 + r) * 4;                // first dword of the row's 16 scale bytes

  v16f acc[WN][WM];
#pragma unroll
  for (int i = 0; i < WN; ++i)
#pragma unroll
    for (int j = 0; j < WM; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.0f;

  // One K step.  TAIL: the short last step (blocks 4..7 absent): lanes with kh = 1 multiply zeros.
  // The operand reads of sub-step ks+1 go out between the MFMAs of sub-step ks (two register sets,
  // one read behind each of the first MFMAs), so neither their issue nor their latency idles the matrix pipe.
  auto compute = [&](int kt, auto tail) {
    constexpr bool TAIL = decltype(tail)::value;
    const int st = (kt + step_base) & (NS - 1), sst = ((kt >> 1) + pair_base) & (NS - 1);
    const uint4 *cw = sW + st * (BN * 8), *cx = sX + st * (BM * 8);
    // this lane's four scale bytes of the step inside the row's 16-byte pair window; a lane whose
    // blocks are absent (short last step) may point past it and is clamped: its operands are zero
    const int sdw = min(3, (kt & 1) * 2 + ((kt >> 1) == npairs - 1 ? (sc_shift >> 2) : 0) + kh);
    const int *cws = reinterpret_cast<const int *>(sWs) + sst * (BN * 4) + sdw;
    const int *cxs = reinterpret_cast<const int *>(sXs) + sst * (BM * 4) + sdw;
    int ws[WN], xs[WM];
    uint4 wq[2][WN], xq[2][WM];
    auto fetch = [&](int ks, int b) {  // in the order in which the MFMAs need them
#pragma unroll
      for (int t = 0; t < (WN > WM ? WN : WM); ++t) {
        if (t < WM) xq[b][t] = cx[x_rd[ks] + t * 256];
        if (t < WN) wq[b][t] = cw[w_rd[ks] + t * 256];
      }
    };
#pragma unroll
    for (int i = 0; i < WN; ++i) ws[i] = cws[ws_rd + i * 128];
#pragma unroll
    for (int j = 0; j < WM; ++j) xs[j] = cxs[xs_rd + j * 128];
    fetch(0, 0);
#define ARCQ_MX_SUBSTEP(KS)                                                                                   \
  {                                                                                                           \
    if (KS < 3) fetch(KS + 1, (KS + 1) & 1);                                                                  \
    v8i wf[WN], xf[WM];                                                                                       \
    _Pragma("unroll") for (int i = 0; i < WN; ++i) {                                                          \
      uint4 q = wq[KS & 1][i];                                                                                \
      if (TAIL && kh) q = make_uint4(0, 0, 0, 0);                                                             \
      wf[i] = fp4_operand(q);                                                                                 \
    }                                                                                                         \
    _Pragma("unroll") for (int j = 0; j < WM; ++j) {                                                          \
      uint4 q = xq[KS & 1][j];                                                                                \
      if (TAIL && kh) q = make_uint4(0, 0, 0, 0);                                                             \
      xf[j] = fp4_operand(q);                                                                                 \
    }                                                                                                         \
    _Pragma("unroll") for (int i = 0; i < WN; ++i) _Pragma("unroll") for (int j = 0; j < WM; ++j)             \
        acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(wf[i], xf[j], acc[i][j], 4, 4, KS, ws[i], \
                                                                     KS, xs[j]);                              \
    if (KS < 3) MfmaReadPattern<WN * WM, WN + WM>::apply();                                                   \
    __builtin_amdgcn_sched_barrier(0);                                                                        \
  }
    ARCQ_MX_SUBSTEP(0)
    ARCQ_MX_SUBSTEP(1)
    ARCQ_MX_SUBSTEP(2)
    ARCQ_MX_SUBSTEP(3)
#undef ARCQ_MX_SUBSTEP
  };

  // this workgroup's K steps: all of them, or with split-K a range that starts on a pair of steps
  // (the scale bytes travel in pairs)
  const int kt_beg = 2 * (int)((long)npairs * blockIdx.y / p.k_slices);
  const int kt_end = min(nk, 2 * (int)((long)npairs * (blockIdx.y + 1) / p.k_slices));
  const bool tail = short_last && kt_end == nk;
  const int nfull = tail ? kt_end - 1 : kt_end;
  // NS - 1 steps are on their way while one is computed.  With two stages the wait for a step is a
  // wait for everything; with four, the two younger steps stay outstanding: this wave issued
  // 2*WN + 2*WM code loads for each of them and, for the even one of the two, its share of the scale
  // loads (128x64 tile: one instruction for waves 0..2, none for wave 3; 128x128: one for every wave),
  // and vmcnt counts in issue order.
  const bool scale_wave = WM == 2 || wave < 3;
  auto wait_step = [&](int younger) {  // younger: steps issued after the one waited for
    if (NS == 4 && younger >= 2) {
      if (WM == 2)
        asm volatile("s_waitcnt vmcnt(17)" ::: "memory");
      else if (scale_wave)
        asm volatile("s_waitcnt vmcnt(13)" ::: "memory");
      else
        asm volatile("s_waitcnt vmcnt(12)" ::: "memory");
    } else if (!PERSIST || wave < NLW) {
      // (persistent workgroups: the waves that request nothing have only a finished tile's stores outstanding,
      // and those may drain behind the next tile's first steps)
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
  };
  const bool requests = wave < NLW;
#pragma unroll
  for (int a = 0; a < NS - 1; ++a)
    if (kt_beg + a < kt_end && requests) issue(kt_beg + a, 0, 0);
  if constexpr (!PERSIST) {
    for (int kt = kt_beg; kt < nfull; ++kt) {
      wait_step(kt_end - 1 - kt);  // the stage of step kt is complete; everyone is done with the stage of step kt-1
      if (kt + NS - 1 < kt_end && requests) issue(kt + NS - 1, 0, 0);
      compute(kt, std::false_type{});
    }
    if (tail && kt_beg < kt_end) {
      wait_step(0);
      compute(nk - 1, std::true_type{});
    }
    store_workgroup_tile<WN, WM, NWM>(p, acc, reinterpret_cast<uint8_t *>(sW), reinterpret_cast<uint8_t *>(sX), m_base,
                                      n_base, wave, lane);
  } else {
    // (the host sends only problems made of whole tiles here: M % BM == 0, N % BN == 0)
    const float alpha = effective_alpha(p);
    for (;;) {
      const bool more = run_left > run_step;  // this workgroup has another tile
      const int cur_n = n_base, cur_m = m_base;
      auto request_next_tile = [&]() {  // during the last step: the next tile's first stage goes out before it is multiplied
        if (!more) return;
        lin += run_step;
        n_base = (lin / tiles_m) * BN;
        m_base = (lin % tiles_m) * BM;
        if (requests) {
          lane_offsets(n_base, m_base);
          issue(0, step_base + nk, pair_base + npairs);
        }
      };
      for (int kt = 0; kt < nfull; ++kt) {
        wait_step(0);
        if (kt + 1 < nk) {
          if (requests) issue(kt + 1, step_base, pair_base);
        } else {
          request_next_tile();
        }
        compute(kt, std::false_type{});
      }
      if (tail) {
        wait_step(0);
        request_next_tile();
        compute(nk - 1, std::true_type{});
      }
      // The finished tile leaves through the stage that the last step has just been multiplied from: it stays
      // free until the next tile's second step is requested, which happens behind the barrier of its first
      // step, i.e. after every wave's epilogue.  Each wave transposes its own 32-row slabs in an 8 KB piece of
      // that stage (wave-local: the one barrier here only says that everyone is done reading operands), so that
      // every store instruction writes whole rows of the wave tile, 16 bytes per lane.
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
      __builtin_amdgcn_s_barrier();
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
      {
        const int st_last = (nk - 1 + step_base) & 1;
        uint8_t *region = reinterpret_cast<uint8_t *>(wave < 4 ? sW + st_last * (BN * 8) : sX + st_last * (BM * 8)) + (wave & 3) * 8192;
        static_assert(BN * 128 >= 4 * 8192 && BM * 128 >= 4 * 8192 && 32 * 64 * WN == 8192, "8 KB per wave inside one stage of either operand");
        constexpr int RB = 64 * WN, LPR = 4 * WN;   // bytes per row of the wave tile, lanes per row at 16 bytes each
        // (the lane number is made opaque here: the LDS addresses below do not depend on the tile, and hoisted out
        // of the tile loop they would be spilled and reloaded one by one)
        int lane_e = lane;
        asm volatile("" : "+v"(lane_e));
        const int r_e = lane_e & 31, kh_e = lane_e >> 5;
        const int rr = lane_e / LPR, t = lane_e % LPR;
#pragma unroll
        for (int j = 0; j < WM; ++j) {
          const int sw = (r_e & (LPR - 1)) << 1;
#pragma unroll
          for (int i = 0; i < WN; ++i) {
#pragma unroll
            for (int q = 0; q < 4; ++q) {
              const v16f &a = acc[i][j];
              const int c = 8 * i + 2 * q + kh_e;  // 8-byte chunk of the row
              *reinterpret_cast<uint2 *>(region + r_e * RB + ((c ^ sw) << 3)) =
                  make_uint2(pack_bf16_rne(a[4 * q] * alpha, a[4 * q + 1] * alpha), pack_bf16_rne(a[4 * q + 2] * alpha, a[4 * q + 3] * alpha));
            }
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.0f;
          }
          uint16_t *cbase = p.c + (size_t)(cur_m + wm0 + 32 * j) * p.N + cur_n + wn0 + 8 * t;
#pragma unroll
          for (int it = 0; it < (32 * LPR) / 64; ++it) {
            const int m = it * (64 / LPR) + rr;
            const int swr = (m & (LPR - 1)) << 1;
            uint4 v = *reinterpret_cast<const uint4 *>(region + m * RB + (((2 * t) ^ swr) << 3));
            if (p.residual) {
              const uint4 rv = *reinterpret_cast<const uint4 *>(p.residual + (cbase - p.c) + (size_t)m * p.N);
              v = make_uint4(add_bf16_pair(v.x, rv.x), add_bf16_pair(v.y, rv.y), add_bf16_pair(v.z, rv.z), add_bf16_pair(v.w, rv.w));
            }
            *reinterpret_cast<uint4 *>(cbase + (size_t)m * p.N) = v;
          }
        }
      }
      if (!more) break;
      run_left -= run_step;
      step_base += nk;
      pair_base += npairs;
    }
  }
}

// ---------------------------------------------------------------------------------------------
// Tiled NVFP4 kernel: same workgroup tiling, LDS-direct loads and LDS layout as the MXFP4 kernel
// (a 16-byte chunk is two NVFP4 blocks), but the block scales (1+m/8)*2^e have no hardware path:
// every wave decodes its operands to fp16 in registers -- code value x scale has at most 6
// significant bits and lies in [2^-10, 2688], exact in fp16 -- and multiplies them with
// v_mfma_f32_32x32x16_f16.  Since the scale is applied per element, an MFMA K step need not be a
// block: a lane reads one 16-byte chunk and feeds its four dwords (8 codes each) to four MFMAs,
// lanes 0-31 from chunk 4*0+cp, lanes 32-63 from chunk 4*1+cp.
// Decode of 8 codes (one dword): four v_cvt_scalef32_pk_f16_fp4 (two codes each, exact) and four
// packed fp16 multiplies by the block scale: 8 VALU instructions per 8 values.
// Requires K' % 128 == 0.
// ---------------------------------------------------------------------------------------------
typedef _Float16 v8h __attribute__((ext_vector_type(8)));
typedef uint32_t v4u __attribute__((ext_vector_type(4)));

// fp16 bits of two NVFP4 scale bytes sitting in bits 7:0 and 23:16: (1+m/8)*2^(e-9) = (b<<7) + 0x1800
__device__ __forceinline__ uint32_t nv_scale_pair_f16(uint32_t two_bytes) { return (two_bytes << 7) + 0x18001800u; }

// packed fp16 multiply of both halves of a by the LOW (HI=false) or HIGH half of s.  Plain vector
// code, not inline asm: the compiler folds the broadcast into op_sel and, unlike with asm, keeps
// the wait states the matrix pipe needs between a VALU write and an MFMA reading that register.
typedef _Float16 v2h __attribute__((ext_vector_type(2)));
template <bool HI>
__device__ __forceinline__ uint32_t pk_mul_f16_bcast(uint32_t a, uint32_t s) {
  const v2h av = __builtin_bit_cast(v2h, a), sv = __builtin_bit_cast(v2h, s);
  const _Float16 k = HI ? sv[1] : sv[0];
  const v2h kv = {k, k};
  return __builtin_bit_cast(uint32_t, av * kv);
}

template <bool HI>
__device__ __forceinline__ v8h decode8_nvfp4_f16(uint32_t codes, uint32_t scale_pair) {
  // hardware FP4 -> fp16 conversion, two codes per instruction (low nibble first), then one packed
  // multiply by the block scale: 8 VALU instructions per 8 values
  v4u d;
  d[0] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(codes, 1.0f, 0));
  d[1] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(codes, 1.0f, 1));
  d[2] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(codes, 1.0f, 2));
  d[3] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(codes, 1.0f, 3));
#pragma unroll
  for (int k = 0; k < 4; ++k) d[k] = pk_mul_f16_bcast<HI>(d[k], scale_pair);
  return __builtin_bit_cast(v8h, d);
}

template <int WN, int WM, int NWM = 2>
__global__ __launch_bounds__(128 * NWM) void gemm_nvfp4_tiled(GemmParams p) {
  // waves: 2 along N x NWM along M (wave = n + 2 * m), each with WN x WM accumulator tiles of 32 x 32
  constexpr int BN = 64 * WN, BM = 32 * WM * NWM, NW = 2 * NWM;
  constexpr int RPI = 16 * NWM;  // rows of 128 code bytes that one load instruction of the workgroup covers
  __shared__ uint4 sW[2 * BN * 8], sX[2 * BM * 8];  // code tiles, two stages each
  constexpr int BMS = BM < 64 ? 64 : BM;            // a scale load instruction covers 64 rows (clamped to the last one)
  __shared__ uint4 sWs[2 * BN], sXs[2 * BMS];       // 16 scale bytes per row per K step, two stages each
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int kbytes = p.Kp >> 1, ksc = p.Kp >> 4;

  int lin;
  if (p.seg) {
    if (!enter_segment<BM, BN, 16>(p, lin)) return;
  } else {
    const int total = ((p.M + BM - 1) / BM) * ((p.N + BN - 1) / BN);
    const int per_xcd = (total + 7) >> 3;
    lin = (blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);
    if (lin >= total) return;
  }
  const int tiles_m = (p.M + BM - 1) / BM;
  const int n_base = (lin / tiles_m) * BN, m_base = (lin % tiles_m) * BM;

  const int nk = (p.Kp + 255) >> 8;
  const bool short_last = (p.Kp & 255) != 0;  // then the last step has chunks 0..3 and 8 scale bytes

  const int ld_row = tid >> 3;
  const int ld_q = (tid & 7) ^ ((ld_row >> 1) & 7);
  const uint8_t *wsrc[BN / RPI], *xsrc[BM / RPI];
#pragma unroll
  for (int i = 0; i < BN / RPI; ++i)
    wsrc[i] = p.b_codes + (size_t)min(n_base + RPI * i + ld_row, p.N - 1) * kbytes + ld_q * 16;
#pragma unroll
  for (int i = 0; i < BM / RPI; ++i)
    xsrc[i] = p.a_codes + (size_t)min(m_base + RPI * i + ld_row, p.M - 1) * kbytes + ld_q * 16;
  // scales: one lane = the 16 scale bytes of one row for this K step; instruction j (64 rows) of
  // the weights goes to wave j%4, of the activations to wave (j+WN)%4.  In a short last step the
  // window is shifted back by 8 bytes so that it ends with the row.
  const uint8_t *wssrc[BN / 64], *xssrc[BMS / 64];
#pragma unroll
  for (int j = 0; j < BN / 64; ++j) wssrc[j] = p.b_scales + (size_t)min(n_base + 64 * j + lane, p.N - 1) * ksc;
#pragma unroll
  for (int j = 0; j < BMS / 64; ++j) xssrc[j] = p.a_scales + (size_t)min(m_base + 64 * j + lane, p.M - 1) * ksc;
  const uint32_t lw0 = (uint32_t)reinterpret_cast<uintptr_t>(sW) + wave * 1024;
  const uint32_t lx0 = (uint32_t)reinterpret_cast<uintptr_t>(sX) + wave * 1024;
  const uint32_t lws0 = (uint32_t)reinterpret_cast<uintptr_t>(sWs);
  const uint32_t lxs0 = (uint32_t)reinterpret_cast<uintptr_t>(sXs);

  auto issue = [&](int kt) {
    const int st = kt & 1;
    const bool clip = short_last && kt == nk - 1;
    const int koff = kt * 128 - ((clip && ld_q >= 4) ? 64 : 0);
    const int soff = kt * 16 - (clip ? 8 : 0);
#pragma unroll
    for (int i = 0; i < BN / RPI; ++i) lds_dma16(wsrc[i] + koff, lw0 + st * (BN * 128) + i * (RPI * 128));
#pragma unroll
    for (int i = 0; i < BM / RPI; ++i) lds_dma16(xsrc[i] + koff, lx0 + st * (BM * 128) + i * (RPI * 128));
#pragma unroll
    for (int j = 0; j < BN / 64; ++j)
      if ((j % NW) == wave) lds_dma16(wssrc[j] + soff, lws0 + st * (BN * 16) + j * 1024);
#pragma unroll
    for (int j = 0; j < BMS / 64; ++j)
      if (((j + BN / 64) % NW) == wave) lds_dma16(xssrc[j] + soff, lxs0 + st * (BMS * 16) + j * 1024);
  };

  const int r = lane & 31, kh = lane >> 5;
  const int swz = (r >> 1) & 7;
  const int wn0 = (wave & 1) * 32 * WN, wm0 = (wave >> 1) * 32 * WM;
  int w_rd[4], x_rd[4];
#pragma unroll
  for (int cp = 0; cp < 4; ++cp) {
    w_rd[cp] = (wn0 + r) * 8 + ((4 * kh + cp) ^ swz);
    x_rd[cp] = (wm0 + r) * 8 + ((4 * kh + cp) ^ swz);
  }

  v16f acc[WN][WM];
#pragma unroll
  for (int i = 0; i < WN; ++i)
#pragma unroll
    for (int j = 0; j < WM; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.0f;

  // One K step = 16 MFMA sub-steps (4 chunks x 4 dwords).  TAIL: chunks 4..7 absent -> lanes with
  // kh = 1 contribute zeros.  Software pipeline inside the wave: while the MFMAs of sub-step s
  // run in the matrix pipe, the VALU decodes the operands of sub-step s+1 into a second register
  // set, and the codes of the next chunk are read from LDS one chunk ahead.  The compiler is told
  // to issue one MFMA, then a slice of the decode, and so on (sched_group_barrier), because a wave
  // issues in order and back-to-back MFMAs would leave the VALU idle.
  auto compute = [&](int kt, auto tail) {
    constexpr bool TAIL = decltype(tail)::value;
    const int st = kt & 1;
    const uint4 *cw = sW + st * (BN * 8), *cx = sX + st * (BM * 8);
    // this lane's 8 scale bytes (blocks 8*kh .. 8*kh+7 of the step) as fp16 pairs:
    // sp[.][0] = blocks (0,2), [1] = (1,3), [2] = (4,6), [3] = (5,7) relative to 8*kh
    const int sq = TAIL ? 1 : kh;  // short last step: the 8 valid bytes sit in the upper half of the window
    uint32_t wsp[WN][4], xsp[WM][4];
#pragma unroll
    for (int i = 0; i < WN; ++i) {
      const uint2 b = reinterpret_cast<const uint2 *>(sWs + st * BN + wn0 + r + 32 * i)[sq];
      wsp[i][0] = nv_scale_pair_f16(b.x & 0x00ff00ffu);
      wsp[i][1] = nv_scale_pair_f16((b.x >> 8) & 0x00ff00ffu);
      wsp[i][2] = nv_scale_pair_f16(b.y & 0x00ff00ffu);
      wsp[i][3] = nv_scale_pair_f16((b.y >> 8) & 0x00ff00ffu);
    }
#pragma unroll
    for (int j = 0; j < WM; ++j) {
      const uint2 b = reinterpret_cast<const uint2 *>(sXs + st * BMS + wm0 + r + 32 * j)[sq];
      xsp[j][0] = nv_scale_pair_f16(b.x & 0x00ff00ffu);
      xsp[j][1] = nv_scale_pair_f16((b.x >> 8) & 0x00ff00ffu);
      xsp[j][2] = nv_scale_pair_f16(b.y & 0x00ff00ffu);
      xsp[j][3] = nv_scale_pair_f16((b.y >> 8) & 0x00ff00ffu);
    }
    uint4 wq[2][WN], xq[2][WM];   // codes of chunk cp (buffer cp&1)
    v8h wf[2][WN], xf[2][WM];     // decoded operands of sub-step s (buffer s&1)
    auto fetch = [&](int cp) {
#pragma unroll
      for (int i = 0; i < WN; ++i) {
        wq[cp & 1][i] = cw[w_rd[cp] + i * 256];
        if (TAIL && kh) wq[cp & 1][i] = make_uint4(0, 0, 0, 0);
      }
#pragma unroll
      for (int j = 0; j < WM; ++j) {
        xq[cp & 1][j] = cx[x_rd[cp] + j * 256];
        if (TAIL && kh) xq[cp & 1][j] = make_uint4(0, 0, 0, 0);
      }
    };
    // dword d of chunk cp holds 8 codes of block 2cp + d/2: scale pair index (cp>>1)*2 + (d>>1),
    // low half for even cp, high half for odd cp
    auto decode = [&](int s) {
      const int cp = s >> 2, d = s & 3, b = s & 1;
#pragma unroll
      for (int i = 0; i < WN; ++i) {
        const uint4 q = wq[cp & 1][i];
        const uint32_t c = d == 0 ? q.x : d == 1 ? q.y : d == 2 ? q.z : q.w;
        const uint32_t sp = wsp[i][(cp >> 1) * 2 + (d >> 1)];
        wf[b][i] = (cp & 1) ? decode8_nvfp4_f16<true>(c, sp) : decode8_nvfp4_f16<false>(c, sp);
      }
#pragma unroll
      for (int j = 0; j < WM; ++j) {
        const uint4 q = xq[cp & 1][j];
        const uint32_t c = d == 0 ? q.x : d == 1 ? q.y : d == 2 ? q.z : q.w;
        const uint32_t sp = xsp[j][(cp >> 1) * 2 + (d >> 1)];
        xf[b][j] = (cp & 1) ? decode8_nvfp4_f16<true>(c, sp) : decode8_nvfp4_f16<false>(c, sp);
      }
    };
    fetch(0);
    decode(0);
#pragma unroll
    for (int s = 0; s < 16; ++s) {
      __builtin_amdgcn_sched_barrier(0);
      if ((s & 3) == 0 && s < 12) fetch((s >> 2) + 1);  // next chunk's codes, one chunk ahead
      if (s < 15) decode(s + 1);
#pragma unroll
      for (int i = 0; i < WN; ++i)
#pragma unroll
        for (int j = 0; j < WM; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(wf[s & 1][i], xf[s & 1][j], acc[i][j], 0, 0, 0);
      // issue order for this sub-step: LDS reads first, then MFMA / VALU interleaved
      if ((s & 3) == 0 && s < 12) __builtin_amdgcn_sched_group_barrier(0x100, WN + WM, 0);
#pragma unroll
      for (int g = 0; g < WN * WM; ++g) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x002, (8 * (WN + WM) + WN * WM - 1) / (WN * WM), 0);
      }
    }
    __builtin_amdgcn_sched_barrier(0);
  };

  const int kt_beg = (int)((long)nk * blockIdx.y / p.k_slices), kt_end = (int)((long)nk * (blockIdx.y + 1) / p.k_slices);
  const bool tail = short_last && kt_end == nk;
  const int nfull = tail ? kt_end - 1 : kt_end;
  if (kt_beg < kt_end) issue(kt_beg);
  for (int kt = kt_beg; kt < nfull; ++kt) {
    wait_dma_and_sync();
    if (kt + 1 < kt_end) issue(kt + 1);
    compute(kt, std::false_type{});
  }
  if (tail && kt_beg < kt_end) {
    wait_dma_and_sync();
    compute(nk - 1, std::true_type{});
  }
  store_workgroup_tile<WN, WM, NWM>(p, acc, reinterpret_cast<uint8_t *>(sW), reinterpret_cast<uint8_t *>(sX), m_base,
                                    n_base, wave, lane);
}

#ifdef ARCQ_EXPERIMENTS
// ---------------------------------------------------------------------------------------------
// EXPERIMENT (built only with -DARCQ_EXPERIMENTS, reached only through ARCQ_GEMM_KERNEL=86 / 46; measured slower than
// the kernel above: 963 against 826 us on gate_up at M = 4096).
// NVFP4 at large M: every operand value is decoded ONCE per workgroup.  In the kernel above each wave decodes
// the operand rows it multiplies, so a weight row is decoded by every wave along M and an activation row by
// every wave along N, and the decode instructions (six per MFMA) share the issue slots of the one wave per SIMD
// with the MFMAs.  Here the workgroup's eight waves (2 along N x 4 along M, wave tile 128 x 64, two waves per
// SIMD) first act as decoders: per K step of 64 elements a thread takes 32 codes of one weight row and 32 of
// one activation row straight from global memory (16 bytes and two scale bytes each), decodes them exactly to
// fp16 (code value x block scale has six significant bits) and writes them into an fp16 tile in LDS -- two
// stages of 2 x 256 rows x 128 bytes -- and then as multipliers: v_mfma_f32_32x32x16_f16 on 16-byte operand
// reads from that tile, two decode instructions per MFMA instead of six.  The decode of step t+1 is interleaved
// with the MFMAs of step t, its codes were requested during step t-1; one barrier per step.
// Requires K' % 128 == 0.
// ---------------------------------------------------------------------------------------------
template <int NWM>  // waves along M: 4 = eight waves of 128 x 64 (two per SIMD), 2 = four waves of 128 x 128
__global__ __launch_bounds__(128 * NWM) void gemm_nvfp4_lds16(GemmParams p) {
  constexpr int WN = 4, WM = 8 / NWM, BN = 256, BM = 256, NT = 128 * NWM, IPT = 512 / NT;  // IPT: decoder items per thread and operand
  __shared__ uint4 sT[2 * (BN + BM) * 8];  // stage s: fp16 weights [BN rows x 8 chunks] at s*(BN+BM)*8, activations behind them
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int kbytes = p.Kp >> 1, ksc = p.Kp >> 4;

  int lin;
  if (p.seg) {
    if (!enter_segment<BM, BN, 16>(p, lin)) return;
  } else {
    const int total = ((p.M + BM - 1) / BM) * ((p.N + BN - 1) / BN);
    const int per_xcd = (total + 7) >> 3;
    lin = (blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);
    if (lin >= total) return;
  }
  const int tiles_m = (p.M + BM - 1) / BM;
  const int n_base = (lin / tiles_m) * BN, m_base = (lin % tiles_m) * BM;
  const int nk = p.Kp >> 6;  // K steps of 64 elements: 32 code bytes and 4 scale bytes per row

  // ---- decoder role: item (row, half h of the step's 64 elements) of either tile; a thread takes items tid + it * NT
  const int d_h = tid & 1;
  int d_row[IPT], d_swz[IPT];
  const uint8_t *wc[IPT], *xc[IPT], *wsc[IPT], *xsc[IPT];
  // chunk c (16 bytes = 8 fp16) of row `row` sits at row * 8 + (c ^ ((row >> 1) & 7)): rows two apart use different
  // chunk slots and neighbouring rows different halves of the banks, so neither the decoders' 16-byte writes nor the
  // multipliers' 16-byte reads (32 consecutive rows, one chunk) collide
#pragma unroll
  for (int it = 0; it < IPT; ++it) {
    d_row[it] = (tid + it * NT) >> 1;
    d_swz[it] = (d_row[it] >> 1) & 7;
    wc[it] = p.b_codes + (size_t)min(n_base + d_row[it], p.N - 1) * kbytes + 16 * d_h;
    xc[it] = p.a_codes + (size_t)min(m_base + d_row[it], p.M - 1) * kbytes + 16 * d_h;
    wsc[it] = p.b_scales + (size_t)min(n_base + d_row[it], p.N - 1) * ksc + 2 * d_h;
    xsc[it] = p.a_scales + (size_t)min(m_base + d_row[it], p.M - 1) * ksc + 2 * d_h;
  }
  struct Codes { uint4 w[IPT], x[IPT]; uint32_t ws[IPT], xs[IPT]; };
  auto request = [&](int kt, Codes &c) {
#pragma unroll
    for (int it = 0; it < IPT; ++it) {
      c.w[it] = *reinterpret_cast<const uint4 *>(wc[it] + 32 * kt);
      c.x[it] = *reinterpret_cast<const uint4 *>(xc[it] + 32 * kt);
      c.ws[it] = *reinterpret_cast<const uint16_t *>(wsc[it] + 4 * kt);
      c.xs[it] = *reinterpret_cast<const uint16_t *>(xsc[it] + 4 * kt);
    }
  };
  // dword D (8 codes) of a thread's 32 codes + its block's scale byte -> chunk 4 * d_h + D of the row's fp16 tile
  // (dwords 0, 1 belong to the first of the two blocks, 2, 3 to the second)
  auto decode_dword = [&](const uint4 &q, uint32_t two_scales, uint4 *tile_row, int d_swz, auto dsel) {
    constexpr int D = decltype(dsel)::value;
    const uint32_t sp = nv_scale_pair_f16((two_scales & 0xffu) | ((two_scales & 0xff00u) << 8));  // (block 0, block 1) as fp16
    const uint32_t c = D == 0 ? q.x : D == 1 ? q.y : D == 2 ? q.z : q.w;
    const v8h v = D < 2 ? decode8_nvfp4_f16<false>(c, sp) : decode8_nvfp4_f16<true>(c, sp);
    tile_row[(4 * d_h + D) ^ d_swz] = __builtin_bit_cast(uint4, v);
  };
  auto decode_part = [&](const Codes &c, int stage, auto dsel) {  // a quarter of a step: 16 * IPT VALU instructions, 2 * IPT LDS writes
    uint4 *base = sT + stage * ((BN + BM) * 8);
#pragma unroll
    for (int it = 0; it < IPT; ++it) {
      decode_dword(c.w[it], c.ws[it], base + d_row[it] * 8, d_swz[it], dsel);
      decode_dword(c.x[it], c.xs[it], base + BN * 8 + d_row[it] * 8, d_swz[it], dsel);
    }
  };
  auto decode_step = [&](const Codes &c, int stage) {
    decode_part(c, stage, std::integral_constant<int, 0>{});
    decode_part(c, stage, std::integral_constant<int, 1>{});
    decode_part(c, stage, std::integral_constant<int, 2>{});
    decode_part(c, stage, std::integral_constant<int, 3>{});
  };

  // ---- multiplier role
  const int r = lane & 31, kh = lane >> 5;
  const int swz = (r >> 1) & 7;
  const int wn0 = (wave & 1) * 32 * WN, wm0 = (wave >> 1) * 32 * WM;
  int w_rd[4], x_rd[4];  // chunk 2 * ks + kh of this lane's row in operand tile 0, per sub-step of 16 elements
#pragma unroll
  for (int ks = 0; ks < 4; ++ks) {
    w_rd[ks] = (wn0 + r) * 8 + ((2 * ks + kh) ^ swz);
    x_rd[ks] = BN * 8 + (wm0 + r) * 8 + ((2 * ks + kh) ^ swz);
  }
  v16f acc[WN][WM];
#pragma unroll
  for (int i = 0; i < WN; ++i)
#pragma unroll
    for (int j = 0; j < WM; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.0f;

  auto lds_sync = [&]() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
  };

  Codes ca, cb;  // the codes of the next step and of the one after it
  request(0, ca);
  if (nk > 1) request(1, cb);
  decode_step(ca, 0);
  lds_sync();
  // One K step: the MFMAs of step kt and, if MORE, the decode of step kt + 1 (codes in cb, requested a step ago)
  // into the other stage.  MORE is a compile-time flag so that a sub-step stays one basic block and the MFMAs,
  // the decode instructions and the LDS traffic can be interleaved in it.
  auto step = [&](int kt, auto more_t) {
    constexpr bool MORE = decltype(more_t)::value;
    const uint4 *t = sT + (kt & 1) * ((BN + BM) * 8);
    uint4 wq[2][WN], xq[2][WM];
    auto fetch = [&](int ks, int b) {
#pragma unroll
      for (int i = 0; i < (WN > WM ? WN : WM); ++i) {
        if (i < WM) xq[b][i] = t[x_rd[ks] + i * 256];
        if (i < WN) wq[b][i] = t[w_rd[ks] + i * 256];
      }
    };
    fetch(0, 0);
    // a quarter of the next step's decode (2 x (4 converts + 4 multiplies), two 16-byte LDS writes) rides behind the
    // eight MFMAs of every sub-step: one MFMA, two decode instructions, and the operand reads of the next sub-step
#define ARCQ_L16_SUBSTEP(KS)                                                                                     \
  {                                                                                                              \
    if (KS < 3) fetch(KS + 1, (KS + 1) & 1);                                                                     \
    if (MORE) decode_part(cb, (kt + 1) & 1, std::integral_constant<int, KS>{});                                  \
    _Pragma("unroll") for (int i = 0; i < WN; ++i) _Pragma("unroll") for (int j = 0; j < WM; ++j)                \
        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(v8h, wq[KS & 1][i]),               \
                                                          __builtin_bit_cast(v8h, xq[KS & 1][j]), acc[i][j], 0, 0, 0); \
    _Pragma("unroll") for (int g = 0; g < WN * WM; ++g) {                                                        \
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);                                                         \
      if (MORE) __builtin_amdgcn_sched_group_barrier(0x002, 2, 0);                                               \
      if (KS < 3 && g < WN + WM) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);                              \
      if (MORE && g >= WN * WM - 2 * IPT) __builtin_amdgcn_sched_group_barrier(0x200, 1, 0);                     \
    }                                                                                                            \
    __builtin_amdgcn_sched_barrier(0);                                                                           \
  }
    ARCQ_L16_SUBSTEP(0)
    ARCQ_L16_SUBSTEP(1)
    ARCQ_L16_SUBSTEP(2)
    ARCQ_L16_SUBSTEP(3)
#undef ARCQ_L16_SUBSTEP
  };
  for (int kt = 0; kt + 1 < nk; ++kt) {
    if (kt + 2 < nk) request(kt + 2, ca);  // two steps ahead, into the register set decoded during the previous step
    step(kt, std::true_type{});
    {
      const Codes tmp = ca;
      ca = cb;
      cb = tmp;
    }
    lds_sync();
  }
  step(nk - 1, std::false_type{});
  lds_sync();
  store_workgroup_tile<WN, WM, NWM>(p, acc, reinterpret_cast<uint8_t *>(sT), reinterpret_cast<uint8_t *>(sT + (BN + BM) * 8), m_base,
                                    n_base, wave, lane);
}

template <int NWM>
int launch_nvfp4_lds16(const GemmParams &p, hipStream_t st) {
  const int total = ((p.M + 255) / 256 + (p.seg ? p.n_seg : 0)) * ((p.N + 255) / 256);
  const int grid = ((total + 7) / 8) * 8;
  hipLaunchKernelGGL(gemm_nvfp4_lds16<NWM>, dim3(grid), dim3(128 * NWM), 0, st, p);
  ARCQ_HIP_TRY(hipGetLastError());
  return ARCQ_OK;
}
#endif  // ARCQ_EXPERIMENTS

// ---------------------------------------------------------------------------------------------
// Skinny kernels for M <= 64 (decode batches): the GEMM is a stream of the weight matrix, read
// exactly once, so nothing is staged through LDS.  A workgroup owns 16 weight rows; its NW waves
// take the K steps of 128 round-robin in pairs (split-K: with four waves wave w does steps 2w, 2w+1, 2w+8, 2w+9, ...:
// a pair of steps is one whole 128-byte line of every row, and the four waves walk neighbouring lines) and their partial sums meet in LDS.  A lane loads
// the 16 bytes (32 codes) the 16x16 MFMA wants from it straight from global memory: row lane%16,
// K group lane/16, i.e. 64 contiguous bytes per row and step.  The activations (<= 64 rows) come
// from L2 the same way, one 16-column tile at a time, each reusing the weight registers.
// Requires K' % 128 == 0 and 16-byte aligned scale arrays.
// ---------------------------------------------------------------------------------------------
typedef float v4f __attribute__((ext_vector_type(4)));

template <int MT, int AT, int NW>
__device__ __forceinline__ void skinny_reduce_store(const GemmParams &p, v4f (&acc)[AT * MT], float (*red)[MT * AT][64][4],
                                                    int wave, int lane) {
  if (wave > 0) {
#pragma unroll
    for (int j = 0; j < AT * MT; ++j) *reinterpret_cast<v4f *>(red[wave - 1][j][lane]) = acc[j];
  }
  __syncthreads();
  if (wave > 0) return;
  const float alpha = effective_alpha(p);
#pragma unroll
  for (int i = 0; i < AT; ++i) {
    const int n0 = ((int)blockIdx.x * AT + i) * 16 + 4 * (lane >> 4);
#pragma unroll
    for (int j = 0; j < MT; ++j) {
      v4f t = acc[i * MT + j];
#pragma unroll
      for (int w = 0; w < NW - 1; ++w) t += *reinterpret_cast<const v4f *>(red[w][i * MT + j][lane]);
      const int m = 16 * j + (lane & 15);
      if (m >= p.M) continue;
      uint16_t *dst = p.c + (size_t)m * p.N + n0;
      if (n0 + 3 < p.N && (p.N & 3) == 0) {
        const uint32_t lo = pack_bf16_rne(t[0] * alpha, t[1] * alpha), hi = pack_bf16_rne(t[2] * alpha, t[3] * alpha);
        uint2 v = make_uint2(lo, hi);
        if (p.residual) v = add_bf16_x4(v, *reinterpret_cast<const uint2 *>(p.residual + (dst - p.c)));
        *reinterpret_cast<uint2 *>(dst) = v;
      } else {
#pragma unroll
        for (int v = 0; v < 4; ++v)
          if (n0 + v < p.N) {
            uint32_t hb = f32_to_bf16_bits(t[v] * alpha);
            if (p.residual) hb = f32_to_bf16_bits(bf16_bits_to_f32(hb) + bf16_bits_to_f32(p.residual[(dst - p.c) + v]));
            dst[v] = (uint16_t)hb;
          }
      }
    }
  }
}

template <int MT, int AT, int NW>
__global__ __launch_bounds__(64 * NW) void gemm_mxfp4_skinny(GemmParams p) {
  __shared__ float red[NW - 1][MT * AT][64][4];
  constexpr int D = (MT * AT >= 4) ? 4 : 8;  // K steps whose loads are in flight together
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int r = lane & 15, g = lane >> 4;
  const int T = p.Kp >> 7;
  const size_t rowb = (size_t)(p.Kp >> 1), rows = (size_t)(p.Kp >> 5);
  const uint8_t *wc[AT], *ws[AT], *xc[MT], *xs[MT];
#pragma unroll
  for (int i = 0; i < AT; ++i) {
    const int n = min(((int)blockIdx.x * AT + i) * 16 + r, p.N - 1);
    wc[i] = p.b_codes + n * rowb + 16 * g;
    ws[i] = p.b_scales + n * rows;
  }
#pragma unroll
  for (int j = 0; j < MT; ++j) {
    const int m = min(16 * j + r, p.M - 1);
    xc[j] = p.a_codes + m * rowb + 16 * g;
    xs[j] = p.a_scales + m * rows;
  }
  v4f acc[AT * MT];
#pragma unroll
  for (int j = 0; j < AT * MT; ++j) acc[j] = v4f{0.f, 0.f, 0.f, 0.f};
  const uint32_t sh = 8u * (uint32_t)g;
  for (int t0 = 2 * wave; t0 < T; t0 += NW * D) {
    uint4 a[AT][D], b[MT][D];
    uint32_t sa[AT][D], sb[MT][D];
#pragma unroll
    for (int d = 0; d < D; ++d) {
      const int t = t0 + 2 * NW * (d >> 1) + (d & 1);
      if (t < T) {  // uniform over the wave
#pragma unroll
        for (int i = 0; i < AT; ++i) {
          a[i][d] = *reinterpret_cast<const uint4 *>(wc[i] + 64 * t);
          sa[i][d] = *reinterpret_cast<const uint32_t *>(ws[i] + 4 * t);
        }
#pragma unroll
        for (int j = 0; j < MT; ++j) {
          b[j][d] = *reinterpret_cast<const uint4 *>(xc[j] + 64 * t);
          sb[j][d] = *reinterpret_cast<const uint32_t *>(xs[j] + 4 * t);
        }
      }
    }
#pragma unroll
    for (int d = 0; d < D; ++d) {
      if (t0 + 2 * NW * (d >> 1) + (d & 1) < T) {
#pragma unroll
        for (int i = 0; i < AT; ++i)
#pragma unroll
          for (int j = 0; j < MT; ++j)
            acc[i * MT + j] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(
                fp4_operand(a[i][d]), fp4_operand(b[j][d]), acc[i * MT + j], 4, 4, 0, (int)(sa[i][d] >> sh), 0,
                (int)(sb[j][d] >> sh));
      }
    }
  }
  skinny_reduce_store<MT, AT, NW>(p, acc, red, wave, lane);
}

// NVFP4: the same walk; a lane's 16 bytes are two blocks of 16, decoded to fp16 eight codes at a
// time and fed to four v_mfma_f32_16x16x32_f16.  Which K index a lane supplies to which of the four
// is free as long as both operands agree: here MFMA d of a step takes K = 128t + 32*(lane/16) + 8d..+7.
template <int MT, int NW>
__global__ __launch_bounds__(64 * NW) void gemm_nvfp4_skinny(GemmParams p) {
  __shared__ float red[NW - 1][MT][64][4];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int r = lane & 15, g = lane >> 4;
  const int T = p.Kp >> 7;
  const size_t rowb = (size_t)(p.Kp >> 1), rows = (size_t)(p.Kp >> 4);
  const int n = min((int)blockIdx.x * 16 + r, p.N - 1);
  const uint8_t *wc = p.b_codes + n * rowb + 16 * g;
  const uint8_t *ws = p.b_scales + n * rows + 2 * g;
  const uint8_t *xc[MT], *xs[MT];
#pragma unroll
  for (int j = 0; j < MT; ++j) {
    const int m = min(16 * j + r, p.M - 1);
    xc[j] = p.a_codes + m * rowb + 16 * g;
    xs[j] = p.a_scales + m * rows + 2 * g;
  }
  v4f acc[MT];
#pragma unroll
  for (int j = 0; j < MT; ++j) acc[j] = v4f{0.f, 0.f, 0.f, 0.f};
  constexpr int D = MT >= 4 ? 2 : 4;  // K steps whose loads are in flight together
  for (int t0 = 2 * wave; t0 < T; t0 += NW * D) {
    uint4 aq[D], bq[MT][D];
    uint32_t as2[D], bs2[MT][D];
#pragma unroll
    for (int d = 0; d < D; ++d) {
      const int t = t0 + 2 * NW * (d >> 1) + (d & 1);
      if (t < T) {  // uniform over the wave
        aq[d] = *reinterpret_cast<const uint4 *>(wc + 64 * t);
        as2[d] = *reinterpret_cast<const uint16_t *>(ws + 8 * t);
#pragma unroll
        for (int j = 0; j < MT; ++j) {
          bq[j][d] = *reinterpret_cast<const uint4 *>(xc[j] + 64 * t);
          bs2[j][d] = *reinterpret_cast<const uint16_t *>(xs[j] + 8 * t);
        }
      }
    }
#pragma unroll
    for (int d = 0; d < D; ++d) {
      if (t0 + 2 * NW * (d >> 1) + (d & 1) < T) {
        const uint32_t ap = nv_scale_pair_f16((as2[d] & 0xffu) | ((as2[d] & 0xff00u) << 8));
        const v8h a0 = decode8_nvfp4_f16<false>(aq[d].x, ap), a1 = decode8_nvfp4_f16<false>(aq[d].y, ap);
        const v8h a2 = decode8_nvfp4_f16<true>(aq[d].z, ap), a3 = decode8_nvfp4_f16<true>(aq[d].w, ap);
#pragma unroll
        for (int j = 0; j < MT; ++j) {
          const uint32_t bp = nv_scale_pair_f16((bs2[j][d] & 0xffu) | ((bs2[j][d] & 0xff00u) << 8));
          const uint4 q = bq[j][d];
          acc[j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a0, decode8_nvfp4_f16<false>(q.x, bp), acc[j], 0, 0, 0);
          acc[j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a1, decode8_nvfp4_f16<false>(q.y, bp), acc[j], 0, 0, 0);
          acc[j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a2, decode8_nvfp4_f16<true>(q.z, bp), acc[j], 0, 0, 0);
          acc[j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a3, decode8_nvfp4_f16<true>(q.w, bp), acc[j], 0, 0, 0);
        }
      }
    }
  }
  skinny_reduce_store<MT, 1, NW>(p, acc, red, wave, lane);
}

// NW waves per workgroup split K among them: eight where the layer is narrow (few workgroups, one wave
// per SIMD otherwise), four where the grid alone fills the machine
template <int FMT, int MT, int AT>
int launch_skinny(const GemmParams &p, hipStream_t st) {
  const int grid = (p.N + 16 * AT - 1) / (16 * AT);
  const bool eight = grid <= 512 && AT == 1;
  if (FMT == ARCQ_FMT_MXFP4) {
    if (eight)
      hipLaunchKernelGGL((gemm_mxfp4_skinny<MT, 1, 8>), dim3(grid), dim3(512), 0, st, p);
    else
      hipLaunchKernelGGL((gemm_mxfp4_skinny<MT, AT, 4>), dim3(grid), dim3(256), 0, st, p);
  } else {
    if (eight)
      hipLaunchKernelGGL((gemm_nvfp4_skinny<MT, 8>), dim3(grid), dim3(512), 0, st, p);
    else
      hipLaunchKernelGGL((gemm_nvfp4_skinny<MT, 4>), dim3(grid), dim3(256), 0, st, p);
  }
  ARCQ_HIP_TRY(hipGetLastError());
  return ARCQ_OK;
}

template <int FMT>
int launch_skinny_for(const GemmParams &p, hipStream_t st) {
  if (p.M <= 16) return launch_skinny<FMT, 1, 1>(p, st);
  if (p.M <= 32) return launch_skinny<FMT, 2, 1>(p, st);
  return launch_skinny<FMT, 4, 1>(p, st);
}

template <int WN, int WM, int NWM = 2>
int launch_nvfp4_tiled(const GemmParams &p, hipStream_t st) {
  constexpr int BN = 64 * WN, BM = 32 * WM * NWM;
  // grouped: every segment may end in one partial tile of rows
  const int total = ((p.M + BM - 1) / BM + (p.seg ? p.n_seg : 0)) * ((p.N + BN - 1) / BN);
  const int grid = ((total + 7) / 8) * 8;
  hipLaunchKernelGGL((gemm_nvfp4_tiled<WN, WM, NWM>), dim3(grid, p.k_slices), dim3(128 * NWM), 0, st, p);
  ARCQ_HIP_TRY(hipGetLastError());
  return ARCQ_OK;
}

template <int WN, int WM, int NS = 2, int NWM = 2>
int launch_mxfp4_tiled(const GemmParams &p, hipStream_t st) {
  constexpr int BN = 64 * WN, BM = 32 * WM * NWM;
  // grouped: every segment may end in one partial tile of rows
  const int total = ((p.M + BM - 1) / BM + (p.seg ? p.n_seg : 0)) * ((p.N + BN - 1) / BN);
  const int grid = ((total + 7) / 8) * 8;  // whole groups of 8 so that the XCD split covers every tile
  hipLaunchKernelGGL((gemm_mxfp4_tiled<WN, WM, NS, NWM>), dim3(grid, p.k_slices), dim3(128 * NWM), 0, st, p);
  ARCQ_HIP_TRY(hipGetLastError());
  return ARCQ_OK;
}

// The eight-wave tiles as persistent workgroups, one per CU at most (plain launches: no expert segments, no fused
// SwiGLU, K not cut)
template <int WN, int WM>
int launch_mxfp4_persistent(const GemmParams &p, hipStream_t st) {
  constexpr int BN = 64 * WN, BM = 32 * WM * 4;
  const int total = ((p.M + BM - 1) / BM) * ((p.N + BN - 1) / BN);
  const int grid = std::min(256, ((total + 7) / 8) * 8);  // whole groups of 8: one slot per XCD and group
  hipLaunchKernelGGL((gemm_mxfp4_tiled<WN, WM, 2, 4, true>), dim3(grid), dim3(512), 0, st, p);
  ARCQ_HIP_TRY(hipGetLastError());
  return ARCQ_OK;
}

// Split-K for few rows of activations and narrow layers: a 128x64 tile grid alone leaves most CUs idle
// (N = 4096, M = 64: 32 workgroups), so K is cut into slices, one workgroup per (tile, slice), each
// writing its fp32 partial tile; this kernel adds the slices in order and writes bf16.  The kernel
// boundary makes the partials visible; nothing is accumulated atomically, so results are
// reproducible.
__global__ __launch_bounds__(256) void splitk_reduce_kernel(GemmParams p) {
  const size_t total4 = ((size_t)p.M * p.N) >> 2, plane = (size_t)p.M * p.N;
  const float alpha = effective_alpha(p);
  for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < total4; i += (size_t)gridDim.x * 256) {
    float4 t = reinterpret_cast<const float4 *>(p.partial)[i];
    for (int k = 1; k < p.k_slices; ++k) {
      const float4 u = reinterpret_cast<const float4 *>(p.partial + (size_t)k * plane)[i];
      t.x += u.x, t.y += u.y, t.z += u.z, t.w += u.w;
    }
    const uint32_t lo = pack_bf16_rne(t.x * alpha, t.y * alpha), hi = pack_bf16_rne(t.z * alpha, t.w * alpha);
    uint2 v = make_uint2(lo, hi);
    if (p.residual) v = add_bf16_x4(v, reinterpret_cast<const uint2 *>(p.residual)[i]);
    reinterpret_cast<uint2 *>(p.c)[i] = v;
  }
}

// Which kernel runs a problem, decided on the host from the shape alone (so that every entry point
// that shares this plan computes the same bits).  kernel: 0 = direct, 1 = skinny, <WN><WM> = tiled
// (214 / 224: MXFP4 with the four-stage ring); slices > 1: split-K over 128x64 tiles, which needs
// slices * M * N fp32 words of scratch.
struct GemmPlan {
  int kernel = 0;
  int slices = 1;
  size_t scratch_bytes() const { return slices > 1 ? scratch : 0; }
  size_t scratch = 0;
};

// the largest scratch the plan ever asks for (the stream workspaces are this big)
constexpr size_t kSplitMaxBytes = kWorkspaceBytes[kWsSplitK];

GemmPlan plan_gemm(int M, int N, int Kp, int fmt, bool scales_aligned) {
  GemmPlan plan;
  const Tuning &tune = tuning();
  const int force = tune.gemm_kernel, split_env = tune.gemm_splitk;
  const bool fast_ok = Kp % 128 == 0 && scales_aligned;
  // Measured crossover against the tiled kernels (weights streaming from HBM): the skinny kernels
  // re-read the activations from L2 once per 16 weight rows, which costs more the larger M and N are.
  const bool skinny_wins = fmt == ARCQ_FMT_MXFP4
                               ? (N <= 4096 || (N <= 8192 && (M <= 32 || Kp >= 8192)) || M <= 4)
                               : (N <= 8192 || M <= 16);
  // Narrow layers with a decode batch of tens of rows: 128x64 tiles with K cut into slices (measured
  // against the skinny and the plain tiled kernels with the weights streaming from HBM; two launches,
  // so it pays only where the single launch is far from the weight stream's time).
  int split = 0;
  bool one_round_21 = false;  // 128x64 tiles, no more of them than CUs, K not cut
  // NVFP4 on a wide layer with up to 32 rows: decoding bounds the 128x64 tile (every weight row decoded by both
  // of its M-waves, 64 activation rows multiplied of which at most 32 are real), so workgroups of two waves along
  // N with a 64x32 tile -- each weight row decoded once -- and K in two slices to fill the CUs
  // (gate_up 28672 x 4096: 30.7 -> 24.7 us at M = 16, 28.7 -> 26.7 at M = 32; slower on the narrow layers)
  // (only while the two slices fit the 8 MiB array of the entry point that allocates nothing, which serves
  // every decode batch: N up to 32768 at 32 rows)
  const bool small_nv = fmt == ARCQ_FMT_NVFP4 && split_env == 0 && force < 0 && M >= 8 && M <= 32 && N >= 16384 && Kp < 8192 &&
                        (size_t)2 * M * N * sizeof(float) <= kNoAllocScratchBytes;
  if (split_env > 1) split = M <= 512 ? split_env : 0;
  else if (small_nv) split = 2;
  else if (split_env == 0 && force < 0 && M <= 64 && N <= 8192) {
    if (Kp >= 8192 && M >= 24) split = 8;
    else if (Kp < 8192 && N > 4096 && M > (fmt == ARCQ_FMT_MXFP4 ? 16 : 32)) split = 4;
  } else if (split_env == 0 && force < 0 && M > 64 && M <= 512) {
    // Up to a few hundred rows on a narrow layer: the larger tiles leave most CUs without a workgroup,
    // and a workgroup's time is its number of K steps times the memory latency, whatever M is.  As
    // many 128x64 tiles x K slices as there are CUs when K is long (NVFP4, whose workgroups fit two to a CU:
    // two slices anyway; the MXFP4 ring kernel has one workgroup per CU, and a second round costs more than
    // the slices save: down projection at M = 512, 38 us uncut against 49 us in two slices).
    const long tiles21 = (long)((M + 63) / 64) * ((N + 127) / 128);
    if (tiles21 <= 256) {
      int sl = Kp >= 8192 ? (fmt == ARCQ_FMT_MXFP4 ? (int)(256 / tiles21) : std::max(2, (int)(256 / tiles21))) : 1;
      if (fmt == ARCQ_FMT_NVFP4 && Kp < 8192) sl = (int)(256 / tiles21);  // no ring there: slices hide the latency
      if (sl >= 2) split = std::min(sl, 8);
      else one_round_21 = true;
    }
  }
  if (split > 1 && fast_ok && Kp >= 512 && (N & 3) == 0) {
    const int slices = std::min(split, (Kp + 255) / 256 / 2);
    const size_t bytes = (size_t)slices * M * N * sizeof(float);
    if (slices > 1 && bytes <= kSplitMaxBytes) {
      plan.kernel = fmt == ARCQ_FMT_MXFP4 ? 214 : ((small_nv || force == 11) ? 11 : 21);
      plan.slices = slices;
      plan.scratch = bytes;
      return plan;
    }
  }
  if (fast_ok && (force == 1 || (force < 0 && skinny_wins)) && M <= 64) {
    plan.kernel = 1;
    return plan;
  }
  // the tiled kernels fetch scale bytes in 16-byte windows that are shifted back at the end of a row:
  // the row must be at least one window long (K' >= 512 for MXFP4, 256 for NVFP4)
  const bool tiled_ok = fast_ok && Kp >= 512;
  if (fmt == ARCQ_FMT_MXFP4 && force != 0 && tiled_ok) {
    // Tile choice from a small cost model: rounds of resident workgroups x cost of one round.
    // 256x256 tiles run ~1.4x faster per flop than 256x128 ones (LDS reads per MFMA) and 128x128
    // ones ~0.75x; 128x128 workgroups fit two to a CU.  Units: a 256x128 tile = 2.  The 256x256 tile runs as
    // eight waves of 128x64 (kernel 84; two waves per SIMD: one wave's waits for LDS data and for the next
    // stage overlap with the other's MFMAs), 7-16 % faster than as four waves of 128x128 (kernel 44); likewise
    // the 256x128 tile as eight waves of 128x32 (kernel 82), ~5 % faster than as four waves of 128x64 (42).
    const long t44 = (long)((M + 255) / 256) * ((N + 255) / 256), t42 = (long)((M + 127) / 128) * ((N + 255) / 256);
    const long t22 = (long)((M + 127) / 128) * ((N + 127) / 128);
    const double c44 = (double)((t44 + 255) / 256) * 2.8, c42 = (double)((t42 + 255) / 256) * 1.9;
    const double c22 = t22 <= 256 ? 1.33 : (double)((t22 + 511) / 512) * 2.67;
    // Problems of one round of workgroups are bounded by the memory latency of their K steps, not by
    // the matrix cores: the smallest tile that still fits one round (most CUs busy), with three K steps
    // in flight instead of one (four-stage LDS ring, one workgroup per CU).  The same ring measured
    // no gain for NVFP4, whose steps are long: decoding bounds them.
    const long t21 = (long)((M + 63) / 64) * ((N + 127) / 128);
    const int pick = t21 <= 256 ? 214
                                : (t22 <= 256 ? 224
                                              : (M <= 128 ? 21
                                                          : (M < 512 ? 22
                                                                     : (c44 < c42 && c44 < c22 ? 84 : (c42 <= c22 ? 82 : 22)))));
    const bool known = force == 44 || force == 84 || force == 82 || force == 42 || force == 224 || force == 22 ||
                       force == 214 || force == 21;
    plan.kernel = known ? force : pick;
    return plan;
  }
  if (fmt == ARCQ_FMT_NVFP4 && force != 0 && tiled_ok) {
    // 256x256 tiles where they fill at least three quarters of the CUs (they decode each operand row for the
    // fewest MFMAs); with fewer of them half the machine idles (4096 x 4096 at M = 2048: 128 tiles, 105 us
    // against 74 us with 256x128 tiles), so the next smaller tile that still fills it
    const long t44 = (long)((M + 255) / 256) * ((N + 255) / 256), t42 = (long)((M + 127) / 128) * ((N + 255) / 256);
    const int pick = t44 >= 192 ? 44 : (M > 128 && !one_round_21 ? (t42 >= 192 ? 42 : 22) : 21);
#ifdef ARCQ_EXPERIMENTS
    const bool known = force == 44 || force == 84 || force == 86 || force == 46 || force == 42 || force == 22 || force == 21 || force == 11;
#else
    const bool known = force == 44 || force == 42 || force == 22 || force == 21 || force == 11;
#endif
    plan.kernel = known ? force : pick;  // a forced kernel that NVFP4 does not have is ignored
    return plan;
  }
  plan.kernel = 0;
  return plan;
}

int run_gemm(GemmParams p, const GemmPlan &plan, int fmt, float *scratch, hipStream_t st) {
  if (plan.slices > 1) {
    p.k_slices = plan.slices;
    p.partial = scratch;
    const int rc = fmt == ARCQ_FMT_MXFP4 ? launch_mxfp4_tiled<2, 1, 4>(p, st)
                   : (plan.kernel == 11 ? launch_nvfp4_tiled<1, 1, 1>(p, st) : launch_nvfp4_tiled<2, 1>(p, st));
    if (rc != ARCQ_OK) return rc;
    const size_t total4 = ((size_t)p.M * p.N) >> 2;
    hipLaunchKernelGGL(splitk_reduce_kernel, dim3((unsigned)std::min<size_t>((total4 + 255) / 256, 1024)), dim3(256), 0,
                       st, p);
    ARCQ_HIP_TRY(hipGetLastError());
    return ARCQ_OK;
  }
  if (plan.kernel == 1)
    return fmt == ARCQ_FMT_MXFP4 ? launch_skinny_for<ARCQ_FMT_MXFP4>(p, st) : launch_skinny_for<ARCQ_FMT_NVFP4>(p, st);
  if (fmt == ARCQ_FMT_MXFP4) {
    // the eight-wave kernels address an operand's rows with 32-bit byte offsets from its base
    const bool wide = (size_t)std::max(p.M, p.N) * (size_t)(p.Kp >> 1) >= ((size_t)1 << 32);
    // persistent workgroups: plain launches over whole tiles
    // and more of them than one round of workgroups: with a single tile per CU there is nothing to overlap
    // (gate_up at M = 4096, seven tiles per CU: 333 -> 325 us; qkv, one and a half: 77.5 -> 74.9; one round: 1-3 % slower)
    const bool persist = !p.seg && !p.swiglu && tuning().gemm_persist != 0 && p.M % 256 == 0 && p.N % 256 == 0 &&
                         (long)(p.M / 256) * (p.N / 256) > 256;
    switch (wide && plan.kernel == 84 ? 44 : (wide && plan.kernel == 82 ? 42 : plan.kernel)) {
      case 44: return launch_mxfp4_tiled<4, 4>(p, st);
      // 256x256 tile, eight waves of 128x64, and 256x128 tile, eight waves of 128x32
      case 84: return persist ? launch_mxfp4_persistent<4, 2>(p, st) : launch_mxfp4_tiled<4, 2, 2, 4>(p, st);
      case 82: return launch_mxfp4_tiled<4, 1, 2, 4>(p, st);
      case 42: return launch_mxfp4_tiled<4, 2>(p, st);
      case 224: return launch_mxfp4_tiled<2, 2, 4>(p, st);
      case 22: return launch_mxfp4_tiled<2, 2>(p, st);
      case 214: return launch_mxfp4_tiled<2, 1, 4>(p, st);
      case 21: return launch_mxfp4_tiled<2, 1>(p, st);
      default: break;
    }
  } else {
    switch (plan.kernel) {
      case 44: return launch_nvfp4_tiled<4, 4>(p, st);
#ifdef ARCQ_EXPERIMENTS
      case 84: return launch_nvfp4_tiled<4, 2, 4>(p, st);  // 256x256 tile, eight waves of 128x64
      case 86: return launch_nvfp4_lds16<4>(p, st);       // 256x256 tile, operands decoded once per workgroup: eight waves,
      case 46: return launch_nvfp4_lds16<2>(p, st);       // four waves
#endif
      case 42: return launch_nvfp4_tiled<4, 2>(p, st);
      case 22: return launch_nvfp4_tiled<2, 2>(p, st);
      case 21: return launch_nvfp4_tiled<2, 1>(p, st);
      case 11: return launch_nvfp4_tiled<1, 1, 1>(p, st);  // 64x32 tile, two waves along N
      default: break;
    }
  }
  // the direct kernels know neither the fused SwiGLU epilogue (half as many output columns) nor expert segments
  if (p.swiglu || p.seg) return ARCQ_ERR_SHAPE;
  const dim3 grid((p.N + kWgN - 1) / kWgN, (p.M + kWgM - 1) / kWgM);
  if (fmt == ARCQ_FMT_MXFP4)
    hipLaunchKernelGGL(gemm_mxfp4_direct, grid, dim3(256), 0, st, p);
  else
    hipLaunchKernelGGL(gemm_nvfp4_direct, grid, dim3(256), 0, st, p);
  ARCQ_HIP_TRY(hipGetLastError());
  return ARCQ_OK;
}

// argument checks shared by the entry points; fills p
int check_gemm_args(const void *a_codes, const void *a_scales, const void *b_codes, const void *b_scales, int M, int N,
                    int Kp, int fmt, float alpha, const float *d_alpha_a, const float *d_alpha_b, const void *residual,
                    void *c, GemmParams *p) {
  if (fmt != ARCQ_FMT_NVFP4 && fmt != ARCQ_FMT_MXFP4) return ARCQ_ERR_FORMAT;
  if (M < 0 || N < 0 || Kp < 64 || Kp % 64 != 0) return ARCQ_ERR_SHAPE;
  if (M == 0 || N == 0) return ARCQ_OK;
  if (!a_codes || !a_scales || !b_codes || !b_scales || !c) return ARCQ_ERR_NULL;
  if (!aligned16(a_codes) || !aligned16(b_codes) || !aligned16(c)) return ARCQ_ERR_ALIGN;
  p->a_codes = static_cast<const uint8_t *>(a_codes);
  p->a_scales = static_cast<const uint8_t *>(a_scales);
  p->b_codes = static_cast<const uint8_t *>(b_codes);
  p->b_scales = static_cast<const uint8_t *>(b_scales);
  p->c = static_cast<uint16_t *>(c);
  p->d_alpha_a = d_alpha_a;
  p->d_alpha_b = d_alpha_b;
  p->alpha = alpha;
  p->M = M;
  p->N = N;
  p->Kp = Kp;
  p->residual = static_cast<const uint16_t *>(residual);
  return ARCQ_OK;
}

int matmul_impl(const void *a_codes, const void *a_scales, const void *b_codes, const void *b_scales, int M, int N,
                int Kp, int fmt, float alpha, const float *d_alpha_a, const float *d_alpha_b, const void *residual,
                void *c, void *stream) {
  GemmParams p;
  const int rc = check_gemm_args(a_codes, a_scales, b_codes, b_scales, M, N, Kp, fmt, alpha, d_alpha_a, d_alpha_b,
                                 residual, c, &p);
  if (rc != ARCQ_OK || M == 0 || N == 0) return rc;
  hipStream_t st = static_cast<hipStream_t>(stream);
  const GemmPlan plan = plan_gemm(M, N, Kp, fmt, aligned16(a_scales) && aligned16(b_scales));
  float *scratch = nullptr;
  if (plan.slices > 1) {
    int status = ARCQ_OK;
    scratch = static_cast<float *>(stream_workspace(kWsSplitK, st, &status));
    if (!scratch) return status;
  }
  return run_gemm(p, plan, fmt, scratch, st);
}

// ---------------------------------------------------------------------------------------------
// arcq_matmul_noalloc: the split-K partial tiles in a fixed array of the code object instead of
// allocated memory, for callers that cannot allocate.  `scratch` below is the host-side stand-in of
// that array, not a device address: its address on each device comes from hipGetSymbolAddress, once
// per device, and only that pointer is handed to kernels.
// ---------------------------------------------------------------------------------------------
constexpr int kNoAllocMaxDevices = 64;

}  // namespace
}  // namespace arcq

static __device__ __align__(256) unsigned char scratch[arcq::kNoAllocScratchBytes];

namespace arcq {
namespace {

// device address of `scratch` on the current device (each device holds its own copy); nullptr + status on failure
float *noalloc_scratch(int *status) {
  static std::mutex mu;
  static float *addr[kNoAllocMaxDevices];
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) {
    *status = note_hip_error(e);
    return nullptr;
  }
  if (dev < 0 || dev >= kNoAllocMaxDevices) {
    *status = ARCQ_ERR_WORKSPACE;
    return nullptr;
  }
  std::lock_guard<std::mutex> lock(mu);
  if (!addr[dev]) {
    void *ptr = nullptr;
    e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !ptr) {
      *status = note_hip_error(e != hipSuccess ? e : hipErrorInvalidSymbol);
      return nullptr;
    }
    addr[dev] = static_cast<float *>(ptr);
  }
  return addr[dev];
}

}  // namespace

int noalloc_prepare() {
  int status = ARCQ_OK;
  return noalloc_scratch(&status) ? ARCQ_OK : status;
}
}  // namespace arcq

extern "C" int arcq_matmul_noalloc(const void *a_codes, const void *a_scales, const void *b_codes, const void *b_scales,
                                   int M, int N, int Kp, int fmt, float alpha, const float *d_alpha_a,
                                   const float *d_alpha_b, void *c, void *stream) {
  using namespace arcq;
  GemmParams p;
  const int rc = check_gemm_args(a_codes, a_scales, b_codes, b_scales, M, N, Kp, fmt, alpha, d_alpha_a, d_alpha_b,
                                 nullptr, c, &p);
  if (rc != ARCQ_OK || M == 0 || N == 0) return rc;
  const GemmPlan plan = plan_gemm(M, N, Kp, fmt, aligned16(a_scales) && aligned16(b_scales));
  if (plan.scratch_bytes() > kNoAllocScratchBytes) return ARCQ_ERR_WORKSPACE;  // beyond the fixed array: nothing is launched
  float *ws = nullptr;
  if (plan.slices > 1) {
    int status = ARCQ_OK;
    ws = noalloc_scratch(&status);
    if (!ws) return status;
    // every word of the partial tiles that the reduction reads is written by this call's first
    // launch, so nothing of the previous call's contents has to be cleared
  }
  return run_gemm(p, plan, fmt, ws, static_cast<hipStream_t>(stream));
}

extern "C" size_t arcq_matmul_noalloc_limit(void) { return arcq::kNoAllocScratchBytes; }

extern "C" size_t arcq_matmul_scratch_bytes(int M, int N, int Kp, int fmt) {
  if ((fmt != ARCQ_FMT_NVFP4 && fmt != ARCQ_FMT_MXFP4) || M <= 0 || N <= 0 || Kp < 64 || Kp % 64 != 0) return 0;
  return arcq::plan_gemm(M, N, Kp, fmt, true).scratch_bytes();
}

extern "C" int arcq_matmul(const void *a_codes, const void *a_scales, const void *b_codes, const void *b_scales,
                           int M, int N, int Kp, int fmt, float alpha, const float *d_alpha_a,
                           const float *d_alpha_b, void *c, void *stream) {
  return arcq::matmul_impl(a_codes, a_scales, b_codes, b_scales, M, N, Kp, fmt, alpha, d_alpha_a, d_alpha_b, nullptr, c,
                           stream);
}

extern "C" int arcq_matmul_add(const void *a_codes, const void *a_scales, const void *b_codes, const void *b_scales,
                               int M, int N, int Kp, int fmt, float alpha, const float *d_alpha_a,
                               const float *d_alpha_b, const void *residual, void *c, void *stream) {
  if (!residual) return ARCQ_ERR_NULL;
  if (!arcq::aligned16(residual)) return ARCQ_ERR_ALIGN;
  return arcq::matmul_impl(a_codes, a_scales, b_codes, b_scales, M, N, Kp, fmt, alpha, d_alpha_a, d_alpha_b, residual, c,
                           stream);
}

namespace arcq {
namespace {

int grouped_matmul_impl(const void *a_codes, const void *a_scales, const void *b_codes, const void *b_scales,
                        const int *seg_offsets, int n_seg, int M, int N, int Kp, int fmt, float alpha,
                        const float *d_alpha_a, const float *d_alpha_b, const void *residual, void *c, bool swiglu,
                        float *d_absmax, void *stream) {
  GemmParams p;
  const int rc = check_gemm_args(a_codes, a_scales, b_codes, b_scales, M, N, Kp, fmt, alpha, d_alpha_a, d_alpha_b,
                                 residual, c, &p);
  if (rc != ARCQ_OK || M == 0 || N == 0) return rc;
  if (n_seg < 1 || Kp % 128 != 0 || Kp < 512) return ARCQ_ERR_SHAPE;  // the tiled kernels' shapes only
  if (swiglu && (N % 16 != 0 || residual)) return ARCQ_ERR_SHAPE;
  if (!seg_offsets) return ARCQ_ERR_NULL;
  if (!aligned16(a_scales) || !aligned16(b_scales) || (residual && !aligned16(residual))) return ARCQ_ERR_ALIGN;
  const int G = fmt == ARCQ_FMT_NVFP4 ? 16 : 32;
  p.seg = seg_offsets;
  p.n_seg = n_seg;
  p.seg_b_codes = (size_t)N * (Kp >> 1);
  p.seg_b_scales = (size_t)N * (Kp / G);
  p.swiglu = swiglu ? 1 : 0;
  p.absmax_bits = reinterpret_cast<uint32_t *>(d_absmax);
  // Tile from the rows an average segment holds (the real counts live on the device).  The larger tiles are
  // faster per flop, but every segment ends in a partly empty tile of rows and skewed routing leaves some
  // segments far below the average.  Measured on 8 segments of skewed sizes (a Mixtral block's two GEMMs and
  // what runs between them): NVFP4, 8192 rows of 195..3120 per segment: 128x128 tiles 3.51 ms, 256x128 3.70,
  // 256x256 3.86-3.96; MXFP4 with the eight-wave 256x256 kernel against 128x128 tiles: 0.66 / 0.74 ms at 2048
  // rows, 1.00 / 1.03 at 4096, 1.18 / 1.32 at 6144, 1.52 / 1.65 at 8192.
  const int avg = M / n_seg;
  GemmPlan plan;
  const int force = tuning().gemm_kernel;
  if (fmt == ARCQ_FMT_MXFP4)
    plan.kernel = avg >= 256 ? 84 : (avg >= 96 ? 22 : 21);
  else
    plan.kernel = avg >= 2048 ? 44 : (avg >= 96 ? 22 : 21);
  if (force == 84 || force == 44 || force == 42 || force == 22 || force == 21) plan.kernel = force;
  return run_gemm(p, plan, fmt, nullptr, static_cast<hipStream_t>(stream));
}

__global__ void scales_from_absmax_kernel(float *v, int n, float divisor) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  const float scale = v[i] / divisor;
  v[i] = scale == 0.0f ? 1.0f : scale;
}

}  // namespace
}  // namespace arcq

extern "C" int arcq_grouped_matmul(const void *a_codes, const void *a_scales, const void *b_codes, const void *b_scales,
                                   const int *seg_offsets, int n_seg, int M, int N, int Kp, int fmt, float alpha,
                                   const float *d_alpha_a, const float *d_alpha_b, const void *residual, void *c,
                                   void *stream) {
  return arcq::grouped_matmul_impl(a_codes, a_scales, b_codes, b_scales, seg_offsets, n_seg, M, N, Kp, fmt, alpha,
                                   d_alpha_a, d_alpha_b, residual, c, false, nullptr, stream);
}

extern "C" int arcq_grouped_matmul_swiglu(const void *a_codes, const void *a_scales, const void *b_codes,
                                          const void *b_scales, const int *seg_offsets, int n_seg, int M, int N, int Kp,
                                          int fmt, float alpha, const float *d_alpha_a, const float *d_alpha_b, void *t,
                                          float *d_absmax, void *stream) {
  return arcq::grouped_matmul_impl(a_codes, a_scales, b_codes, b_scales, seg_offsets, n_seg, M, N, Kp, fmt, alpha,
                                   d_alpha_a, d_alpha_b, nullptr, t, true, d_absmax, stream);
}

extern "C" int arcq_matmul_swiglu(const void *a_codes, const void *a_scales, const void *b_codes, const void *b_scales,
                                  int M, int N, int Kp, int fmt, float alpha, const float *d_alpha_a,
                                  const float *d_alpha_b, void *t, float *d_absmax, void *stream) {
  using namespace arcq;
  GemmParams p;
  const int rc = check_gemm_args(a_codes, a_scales, b_codes, b_scales, M, N, Kp, fmt, alpha, d_alpha_a, d_alpha_b,
                                 nullptr, t, &p);
  if (rc != ARCQ_OK || M == 0 || N == 0) return rc;
  if (Kp % 128 != 0 || Kp < 512 || N % 16 != 0) return ARCQ_ERR_SHAPE;  // the tiled kernels' shapes only
  if (!aligned16(a_scales) || !aligned16(b_scales)) return ARCQ_ERR_ALIGN;
  p.swiglu = 1;
  p.absmax_bits = reinterpret_cast<uint32_t *>(d_absmax);
  GemmPlan plan = plan_gemm(M, N, Kp, fmt, true);
  const int id = plan.kernel;  // (a kernel forced through the environment may not exist for this format)
  const bool tiled = plan.slices == 1 && (id == 84 || id == 44 || id == 42 || id == 22 || id == 21 ||
                                          (fmt == ARCQ_FMT_MXFP4 && (id == 82 || id == 224 || id == 214)));
  if (!tiled) {  // the decode-batch kernels and split-K have no fused epilogue: a small tile instead
    plan = GemmPlan();
    plan.kernel = M > 64 ? 22 : 21;
  }
  return run_gemm(p, plan, fmt, nullptr, static_cast<hipStream_t>(stream));
}

extern "C" int arcq_scales_from_absmax(float *d_values, int n, float divisor, void *stream) {
  if (n < 0 || !(divisor > 0.0f)) return ARCQ_ERR_SHAPE;
  if (n == 0) return ARCQ_OK;
  if (!d_values) return ARCQ_ERR_NULL;
  hipLaunchKernelGGL(arcq::scales_from_absmax_kernel, dim3((n + 255) / 256), dim3(256), 0, static_cast<hipStream_t>(stream),
                     d_values, n, divisor);
  ARCQ_HIP_TRY(hipGetLastError());
  return ARCQ_OK;
}
