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

}  // extern "C"
