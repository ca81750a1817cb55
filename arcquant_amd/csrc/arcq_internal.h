// arcq_internal.h -- shared between the translation units of libarcq_hip.so (not installed).
#ifndef ARCQ_INTERNAL_H_
#define ARCQ_INTERNAL_H_

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/arcq.h"

namespace arcq {

// Records a failed HIP call for arcq_last_hip_error() and maps it to ARCQ_ERR_LAUNCH.
int note_hip_error(hipError_t e);

inline bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

#define ARCQ_HIP_TRY(expr)                                   \
  do {                                                       \
    hipError_t _e = (expr);                                  \
    if (_e != hipSuccess) return ::arcq::note_hip_error(_e); \
  } while (0)

// Scratch memory of the kernels that need some beyond their inputs and outputs.  One buffer per
// (device, stream, kind), allocated on the first call that needs it (or by arcq_prepare_stream) and
// kept until the process ends, so that a captured graph may hold its address.  Work on one stream is
// serialised, so two calls never share a buffer unless they share a stream.
enum WorkspaceKind {
  kWsTensorScale = 0,  // (maximum, arrival counter) pairs of arcq_tensor_scale, one per 128-byte line, and from byte 2048
                       // the workgroups' slots of the one-launch scale + quantizer (zeroed once)
  kWsSplitK = 1,       // fp32 partial tiles of the split-K GEMM
  kWsDecode = 2,       // partial softmax sums of the split decode attention
  kWsKinds = 3
};
constexpr size_t kWorkspaceBytes[kWsKinds] = {4096, 32u << 20, 8u << 20};

// The buffer of `kind` for (current device, stream).  Returns nullptr and sets *status when there is
// none and none can be made: ARCQ_ERR_WORKSPACE while `stream` is capturing (an allocation there
// would break the capture), ARCQ_ERR_LAUNCH when the allocation fails.
void *stream_workspace(int kind, hipStream_t stream, int *status);

// Frees the buffers of (current device, stream) and forgets the pair; ARCQ_OK also when there were none.
int release_stream_workspace(hipStream_t stream);

// Size of the fixed device array behind arcq_matmul_noalloc.  The GEMM planner also reads it: the plans it
// makes for decode batches must fit the array, so that arcq_matmul and arcq_matmul_noalloc serve the same shapes.
constexpr size_t kNoAllocScratchBytes = 8u << 20;

// Resolves the device address of that array on the current device (once per device; no allocation).
int noalloc_prepare();

// Overrides for tuning runs, read from the environment once, when the library is first used:
//   ARCQ_GEMM_KERNEL=<WN><WM>   force a GEMM tile (84 / 82 = 256x256 / 256x128 as eight waves, 44, 42, 22, 21, 11; 214 / 224 = four-stage
//                               ring; 1 = skinny, 0 = direct); a number the format has no kernel for is ignored
//   ARCQ_GEMM_SPLITK=<slices>   force split-K for M <= 512 (1 = never split)
//   ARCQ_GEMM_PERSIST=<0|1>     0 = the eight-wave MXFP4 tiles as one workgroup per tile instead of persistent workgroups
//   ARCQ_QUANT_GRID=<n>         workgroups of the row quantizers
//   ARCQ_QUANT_KERNEL=<1|2|3>   1 = never, 2 = always take the wave-per-row quantizer where it has an instance;
//                               3 = the four-units-per-thread kernel of the rows beyond 16384 channels from 1024 channels on
//   ARCQ_KV_DECODE_SPLITS=<n>   ranges per sequence of the decode attention
//   ARCQ_RESIDENT_SPIN_US=<n>   how long a workgroup of the one-launch scale + quantizer waits for the others before it takes
//                               the tensor's maximum by itself (0: at once; -1: always two launches instead)
// Unset (the normal case) every field keeps the value below and the dispatch is the measured one.
struct Tuning {
  int gemm_kernel = -1;
  int gemm_splitk = 0;
  int gemm_persist = 1;
  int quant_grid = 0;
  int quant_kernel = 0;
  int kv_decode_splits = 0;
  int resident_spin_us = 200;
};
const Tuning &tuning();

}  // namespace arcq
#endif  // ARCQ_INTERNAL_H_
