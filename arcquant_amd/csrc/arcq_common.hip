// arcq_common.hip -- status strings, version, last-error bookkeeping, per-stream scratch memory and
// the tuning overrides of libarcq_hip.so.
#include <hip/hip_runtime.h>
#include <stdlib.h>

#include <mutex>
#include <vector>

#include "arcq_internal.h"

namespace arcq {
namespace {
thread_local int g_last_hip_error = 0;

struct WorkspaceEntry {
  int device;
  hipStream_t stream;
  void *ptr[kWsKinds];
};
std::mutex g_ws_mutex;
std::vector<WorkspaceEntry> g_ws;  // a few entries: one per (device, stream) that ever needed scratch
}  // namespace

int note_hip_error(hipError_t e) {
  g_last_hip_error = static_cast<int>(e);
  return ARCQ_ERR_LAUNCH;
}

void *stream_workspace(int kind, hipStream_t stream, int *status) {
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) {
    *status = note_hip_error(e);
    return nullptr;
  }
  std::lock_guard<std::mutex> lock(g_ws_mutex);
  WorkspaceEntry *ent = nullptr;
  for (auto &w : g_ws)
    if (w.device == dev && w.stream == stream) ent = &w;
  if (ent && ent->ptr[kind]) return ent->ptr[kind];
  // nothing yet: allocate, unless the stream is being captured (hipMalloc there would end the capture)
  hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
  if (hipStreamIsCapturing(stream, &cap) != hipSuccess) (void)hipGetLastError();
  if (cap != hipStreamCaptureStatusNone) {
    *status = ARCQ_ERR_WORKSPACE;
    return nullptr;
  }
  void *p = nullptr;
  e = hipMalloc(&p, kWorkspaceBytes[kind]);
  if (e == hipSuccess && kind == kWsTensorScale) {
    e = hipMemsetAsync(p, 0, kWorkspaceBytes[kind], stream);  // ordered in front of the first kernel that uses it
    if (e != hipSuccess) (void)hipFree(p);
  }
  if (e != hipSuccess) {
    (void)hipGetLastError();
    *status = note_hip_error(e);
    return nullptr;
  }
  if (!ent) {
    g_ws.push_back(WorkspaceEntry{dev, stream, {nullptr, nullptr, nullptr}});
    ent = &g_ws.back();
  }
  ent->ptr[kind] = p;
  return p;
}

int release_stream_workspace(hipStream_t stream) {
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return note_hip_error(e);
  void *ptr[kWsKinds] = {nullptr, nullptr, nullptr};
  {
    std::lock_guard<std::mutex> lock(g_ws_mutex);
    for (size_t i = 0; i < g_ws.size(); ++i)
      if (g_ws[i].device == dev && g_ws[i].stream == stream) {
        for (int k = 0; k < kWsKinds; ++k) ptr[k] = g_ws[i].ptr[k];
        g_ws.erase(g_ws.begin() + (long)i);
        break;
      }
  }
  int rc = ARCQ_OK;
  for (int k = 0; k < kWsKinds; ++k)
    if (ptr[k]) {
      e = hipFree(ptr[k]);  // waits for the device: no kernel still reads the buffer afterwards
      if (e != hipSuccess) rc = note_hip_error(e);
    }
  return rc;
}

const Tuning &tuning() {
  static const Tuning t = [] {
    Tuning v;
    if (const char *e = getenv("ARCQ_GEMM_KERNEL")) v.gemm_kernel = atoi(e);
    if (const char *e = getenv("ARCQ_GEMM_SPLITK")) v.gemm_splitk = atoi(e);
    if (const char *e = getenv("ARCQ_GEMM_PERSIST")) v.gemm_persist = atoi(e);
    if (const char *e = getenv("ARCQ_QUANT_GRID")) v.quant_grid = atoi(e);
    if (const char *e = getenv("ARCQ_QUANT_KERNEL")) v.quant_kernel = atoi(e);
    if (const char *e = getenv("ARCQ_KV_DECODE_SPLITS")) v.kv_decode_splits = atoi(e);
    if (const char *e = getenv("ARCQ_RESIDENT_SPIN_US")) v.resident_spin_us = atoi(e);
    return v;
  }();
  return t;
}
}  // namespace arcq

extern "C" {

int arcq_version(void) { return 200; }  // 0.2.0

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
    case ARCQ_ERR_WORKSPACE: return "scratch memory unavailable: the stream is being captured and has none yet (call "
                                    "arcq_prepare_stream before the capture), or the problem exceeds the fixed scratch "
                                    "of a non-allocating entry point";
    default: return "unknown status";
  }
}

int arcq_last_hip_error(void) { return arcq::g_last_hip_error; }

int arcq_prepare_stream(void *stream) {
  hipStream_t st = static_cast<hipStream_t>(stream);
  for (int kind = 0; kind < arcq::kWsKinds; ++kind) {
    int status = ARCQ_OK;
    if (!arcq::stream_workspace(kind, st, &status)) return status;
  }
  return arcq::noalloc_prepare();  // the fixed array of arcq_matmul_noalloc: its address on this device
}

int arcq_release_stream(void *stream) { return arcq::release_stream_workspace(static_cast<hipStream_t>(stream)); }

}  // extern "C"
