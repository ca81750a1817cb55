// arcq_probe.hip -- MEASUREMENT ONLY, not part of the product library: plain copy kernels in several launch
// shapes for gfx950.  bench.py times them on the headline launch's bytes as the streaming ceiling of the box, and
// the rocprofv3 FETCH_SIZE / WRITE_SIZE readings are calibrated on them.  Built into libarcq_probe.so.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/arcq_probe.h"

namespace arcq {
namespace {

inline bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// Plain streaming kernels: read n16_in 16-byte words, write the first n16_out of them back (n16_out <= n16_in).
// U independent loads are in flight per thread before the first use; NT: non-temporal stores.  A thread's
// U words of one round are `stride` apart, so every load instruction of a wave covers 1 KB of consecutive bytes.
typedef uint32_t v4u32 __attribute__((ext_vector_type(4)));
template <int U, bool NT>
__global__ __launch_bounds__(256) void stream_probe_kernel(const v4u32 *src, v4u32 *dst, size_t n16_in, size_t n16_out) {
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  v4u32 acc = {0u, 0u, 0u, 0u};
  for (size_t i0 = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i0 < n16_in; i0 += U * stride) {
    v4u32 v[U];
#pragma unroll
    for (int j = 0; j < U; ++j) {
      const size_t i = i0 + j * stride;
      v[j] = i < n16_in ? (NT ? __builtin_nontemporal_load(src + i) : src[i]) : acc;
    }
#pragma unroll
    for (int j = 0; j < U; ++j) {
      const size_t i = i0 + j * stride;
      if (i < n16_out) {
        if (NT) __builtin_nontemporal_store(v[j], dst + i);
        else dst[i] = v[j];
      } else if (i < n16_in) {
        acc ^= v[j];
      }
    }
  }
  if ((acc.x ^ acc.y ^ acc.z ^ acc.w) == 0x9e3779b9u && n16_out) dst[0] = acc;  // keeps the reads alive
}

// The same through LDS-direct loads (the path the wave-per-row quantizer takes): a wave brings 4 KB into a
// slot of its own with four load instructions, reads it back and stores what is to be written.
__global__ __launch_bounds__(1024) void stream_probe_lds_kernel(const v4u32 *src, v4u32 *dst, size_t n16_in, size_t n16_out) {
  extern __shared__ uint4 smem[];
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const uint32_t slot_addr = (uint32_t)reinterpret_cast<uintptr_t>(smem) + wave * 4096;
  const v4u32 *slot = reinterpret_cast<const v4u32 *>(smem) + wave * 256;
  const size_t nblk = (n16_in + 255) >> 8;  // 4 KB blocks; the last one may be partial: it is read by plain loads
  v4u32 acc = {0u, 0u, 0u, 0u};
  for (size_t b = (size_t)blockIdx.x * 16 + wave; b < nblk; b += (size_t)gridDim.x * 16) {
    const size_t i0 = b << 8;
    if (i0 + 256 <= n16_in) {
      const uint8_t *g = reinterpret_cast<const uint8_t *>(src + i0) + 16 * lane;
      asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\t"
                   "global_load_lds_dwordx4 %1, off\n\tglobal_load_lds_dwordx4 %1, off offset:1024\n\t"
                   "global_load_lds_dwordx4 %1, off offset:2048\n\tglobal_load_lds_dwordx4 %1, off offset:3072\n\t"
                   "s_waitcnt vmcnt(0)"
                   :
                   : "s"(slot_addr), "v"(g)
                   : "memory");
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const v4u32 v = slot[j * 64 + lane];
        const size_t i = i0 + j * 64 + lane;
        if (i < n16_out) __builtin_nontemporal_store(v, dst + i);
        else acc ^= v;
      }
    } else {
      for (size_t i = i0 + lane; i < n16_in; i += 64) {
        const v4u32 v = src[i];
        if (i < n16_out) dst[i] = v;
        else acc ^= v;
      }
    }
  }
  if ((acc.x ^ acc.y ^ acc.z ^ acc.w) == 0x9e3779b9u && n16_out) dst[0] = acc;
}


// Register-only matrix-pipe loops: what the MFMA units sustain with the operands the GEMMs feed them, with no
// loads, LDS traffic or barriers.  Every wave keeps NACC independent 32x32 accumulators and four operand registers
// per side, filled from `src` (4096 words: zeros, random bits, decoded-FP4-like fp16 values ...: the rate depends
// on the data, the chip lowers its clock under the multipliers' switching power).  KIND 0: v_mfma_scale_f32_32x32x64_f8f6f4
// with FP4 operands and E8M0 block scales (the MXFP4 GEMM's instruction), 1: v_mfma_f32_32x32x16_f16 (NVFP4's),
// 2: v_mfma_f32_32x32x16_bf16 (the bf16 baseline's).
typedef float v16f __attribute__((ext_vector_type(16)));
typedef int v8i __attribute__((ext_vector_type(8)));
typedef _Float16 v8h __attribute__((ext_vector_type(8)));
typedef __bf16 v8bf __attribute__((ext_vector_type(8)));
typedef int v4i_t __attribute__((ext_vector_type(4)));

template <int KIND, int NACC>
__global__ __launch_bounds__(512) void mfma_rate_kernel(const int *src, float *out, int iters) {
  v8i a[4], b[4];
  for (int i = 0; i < 4; ++i)
    for (int j = 0; j < 8; ++j) {
      a[i][j] = src[(threadIdx.x * 8 + j + i * 17) & 4095];
      b[i][j] = src[(threadIdx.x * 8 + j + i * 29 + 5) & 4095];
    }
  int sa[4], sb[4];
  for (int i = 0; i < 4; ++i) {
    sa[i] = (src[(threadIdx.x + i) & 4095] & 0x03030303) + 0x7e7e7e7e;  // E8M0 bytes near 2^0
    sb[i] = (src[(threadIdx.x + 9 + i) & 4095] & 0x03030303) + 0x7e7e7e7e;
  }
  v16f acc[NACC];
  for (int i = 0; i < NACC; ++i)
    for (int v = 0; v < 16; ++v) acc[i][v] = 0.f;
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int ks = 0; ks < 4; ++ks)
#pragma unroll
      for (int i = 0; i < NACC; ++i) {
        if (KIND == 0) {
          acc[i] = ks == 0   ? __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a[i & 3], b[(i >> 2) & 3], acc[i], 4, 4, 0, sa[i & 3], 0, sb[(i >> 2) & 3])
                   : ks == 1 ? __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a[i & 3], b[(i >> 2) & 3], acc[i], 4, 4, 1, sa[i & 3], 1, sb[(i >> 2) & 3])
                   : ks == 2 ? __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a[i & 3], b[(i >> 2) & 3], acc[i], 4, 4, 2, sa[i & 3], 2, sb[(i >> 2) & 3])
                             : __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a[i & 3], b[(i >> 2) & 3], acc[i], 4, 4, 3, sa[i & 3], 3, sb[(i >> 2) & 3]);
        } else {
          const v4i_t al = {a[i & 3][0], a[i & 3][1], a[i & 3][2], a[i & 3][3]}, bl = {b[(i >> 2) & 3][0], b[(i >> 2) & 3][1], b[(i >> 2) & 3][2], b[(i >> 2) & 3][3]};
          if (KIND == 1)
            acc[i] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(v8h, al), __builtin_bit_cast(v8h, bl), acc[i], 0, 0, 0);
          else
            acc[i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(v8bf, al), __builtin_bit_cast(v8bf, bl), acc[i], 0, 0, 0);
        }
      }
  }
  float s = 0;
  for (int i = 0; i < NACC; ++i)
    for (int v = 0; v < 16; ++v) s += acc[i][v];
  out[blockIdx.x * blockDim.x + threadIdx.x] = s;
}

}  // namespace
}  // namespace arcq

extern "C" {

int arcq_stream_probe_variant(const void *src, void *dst, size_t bytes_in, size_t bytes_out, int variant, void *stream) {
  if (!src || !dst) return ARCQ_PROBE_ERR_NULL;
  if (bytes_out > bytes_in || (bytes_in & 15) || (bytes_out & 15)) return ARCQ_PROBE_ERR_SHAPE;
  if (!arcq::aligned16(src) || !arcq::aligned16(dst)) return ARCQ_PROBE_ERR_ALIGN;
  if (variant < 0 || variant >= arcq_stream_probe_variants()) return ARCQ_PROBE_ERR_SHAPE;
  if (bytes_in == 0) return ARCQ_PROBE_OK;
  hipStream_t st = static_cast<hipStream_t>(stream);
  const arcq::v4u32 *s = static_cast<const arcq::v4u32 *>(src);
  arcq::v4u32 *d = static_cast<arcq::v4u32 *>(dst);
  const size_t n_in = bytes_in / 16, n_out = bytes_out / 16;
  // grids: "resident" = what the chip holds at once (8 workgroups of 256 threads on each of 256 CUs);
  // "one round" = every thread reads its U words and is done
  const auto one_round = [&](int u) { return (unsigned)((n_in + (size_t)256 * u - 1) / ((size_t)256 * u)); };
#define ARCQ_PROBE(U, NT, GRID) \
  hipLaunchKernelGGL((arcq::stream_probe_kernel<U, NT>), dim3(GRID), dim3(256), 0, st, s, d, n_in, n_out)
  switch (variant) {
    case 0: ARCQ_PROBE(1, false, 2048); break;
    case 1: ARCQ_PROBE(4, false, 2048); break;
    case 2: ARCQ_PROBE(4, true, 2048); break;
    case 3: ARCQ_PROBE(8, true, 2048); break;
    case 4: ARCQ_PROBE(4, true, 1024); break;
    case 5: ARCQ_PROBE(8, true, 1024); break;
    case 6: ARCQ_PROBE(4, true, one_round(4)); break;
    case 7: ARCQ_PROBE(8, true, one_round(8)); break;
    case 8: ARCQ_PROBE(2, true, one_round(2)); break;
    default:
      hipLaunchKernelGGL(arcq::stream_probe_lds_kernel, dim3(variant == 9 ? 256 : 512), dim3(1024), 65536, st, s, d, n_in, n_out);
  }
#undef ARCQ_PROBE
  return hipGetLastError() == hipSuccess ? ARCQ_PROBE_OK : ARCQ_PROBE_ERR_LAUNCH;
}

int arcq_stream_probe_variants(void) { return 11; }

int arcq_stream_probe(const void *src, void *dst, size_t bytes_in, size_t bytes_out, void *stream) {
  return arcq_stream_probe_variant(src, dst, bytes_in, bytes_out, 0, stream);
}


int arcq_mfma_rate_probe(int kind, int waves_per_simd, int iters, const void *src, void *out, void *stream) {
  if (!src || !out) return ARCQ_PROBE_ERR_NULL;
  if (kind < 0 || kind > 2 || (waves_per_simd != 1 && waves_per_simd != 2) || iters < 1) return ARCQ_PROBE_ERR_SHAPE;
  hipStream_t st = static_cast<hipStream_t>(stream);
  const int *s = static_cast<const int *>(src);
  float *o = static_cast<float *>(out);
  const dim3 grid(256), block(256 * waves_per_simd);  // one workgroup per CU
#define ARCQ_RATE(K, NACC) hipLaunchKernelGGL((arcq::mfma_rate_kernel<K, NACC>), grid, block, 0, st, s, o, iters)
  if (kind == 0) ARCQ_RATE(0, 8);  // eight independent accumulators per wave: half a wave's register file
  else if (kind == 1) ARCQ_RATE(1, 8);
  else ARCQ_RATE(2, 8);
#undef ARCQ_RATE
  return hipGetLastError() == hipSuccess ? ARCQ_PROBE_OK : ARCQ_PROBE_ERR_LAUNCH;
}

double arcq_mfma_rate_probe_flops(int kind, int waves_per_simd, int iters) {
  // 256 CUs x 4 SIMDs x waves x iters x 4 sub-steps x accumulators x flops of one instruction
  const double per_instr = kind == 0 ? 2.0 * 32 * 32 * 64 : 2.0 * 32 * 32 * 16;
  const int nacc = 8;
  return 256.0 * 4 * waves_per_simd * (double)iters * 4 * nacc * per_instr;
}

}  // extern "C"
