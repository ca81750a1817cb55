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

}  // namespace arcq
#endif  // ARCQ_INTERNAL_H_
