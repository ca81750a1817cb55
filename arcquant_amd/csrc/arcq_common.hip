// arcq_common.hip -- status strings, version, last-error bookkeeping of libarcq_hip.so.
#include <hip/hip_runtime.h>

#include "arcq_internal.h"

namespace arcq {
namespace {
thread_local int g_last_hip_error = 0;
}

int note_hip_error(hipError_t e) {
  g_last_hip_error = static_cast<int>(e);
  return ARCQ_ERR_LAUNCH;
}
}  // namespace arcq

extern "C" {

int arcq_version(void) { return 100; }  // 0.1.0

const char *arcq_status_string(int status) {
  switch (status) {
    case ARCQ_OK: return "ok";
    case ARCQ_ERR_NULL: return "a required pointer is NULL";
    case ARCQ_ERR_SHAPE: return "unsupported shape (need K % 32 == 0, 32 <= K <= 32736, select_num % G == 0, "
                                "select_num <= K, K' % 64 == 0 for matmul)";
    case ARCQ_ERR_FORMAT: return "unknown format (expected ARCQ_FMT_NVFP4 or ARCQ_FMT_MXFP4)";
    case ARCQ_ERR_ALIGN: return "a pointer is not 16-byte aligned";
    case ARCQ_ERR_LAUNCH: return "HIP launch failed";
    case ARCQ_ERR_INDEX: return "reorder_index is not a permutation of 0..K-1";
    default: return "unknown status";
  }
}

int arcq_last_hip_error(void) { return arcq::g_last_hip_error; }

}  // extern "C"
