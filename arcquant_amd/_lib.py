"""ctypes binding of libarcq_hip.so (the C ABI declared in include/arcq.h).

There is no fallback: if the HIP library has not been built, loading raises and every
operator with it.
"""
from __future__ import annotations

import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "csrc", "libarcq_hip.so")
HEADER_PATH = os.path.join(_HERE, "..", "include", "arcq.h")

NVFP4 = 0
MXFP4 = 1
FORMATS = {"NVFP4": NVFP4, "MXFP4": MXFP4}

_lib = None


class ArcqError(RuntimeError):
    def __init__(self, status: int, where: str):
        self.status = status
        msg = lib().arcq_status_string(status).decode()
        hip = lib().arcq_last_hip_error() if status == 5 else 0
        super().__init__(f"{where}: {msg} (arcq status {status}" + (f", hipError {hip})" if hip else ")"))


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            f"{LIB_PATH} is missing: build it with `python -m arcquant_amd.build` "
            "(hipcc, --offload-arch=gfx950). arcquant_amd has no non-HIP path.")
    L = ctypes.CDLL(LIB_PATH)
    vp, i, f, sz = ctypes.c_void_p, ctypes.c_int, ctypes.c_float, ctypes.c_size_t
    L.arcq_version.restype = i
    L.arcq_status_string.argtypes = [i]
    L.arcq_status_string.restype = ctypes.c_char_p
    L.arcq_last_hip_error.restype = i
    L.arcq_prepare_stream.argtypes = [vp]
    L.arcq_prepare_stream.restype = i
    L.arcq_release_stream.argtypes = [vp]
    L.arcq_release_stream.restype = i
    L.arcq_group_size.argtypes = [i]
    L.arcq_group_size.restype = i
    L.arcq_codes_bytes.argtypes = [i, i, i]
    L.arcq_codes_bytes.restype = sz
    L.arcq_scales_bytes.argtypes = [i, i, i, i]
    L.arcq_scales_bytes.restype = sz
    quant = [vp, i, i, vp, i, i, f, vp, vp, vp, vp]
    L.arcq_reorder_quantize_x.argtypes = quant
    L.arcq_reorder_quantize_w.argtypes = quant
    L.arcq_rmsnorm_quantize_x.argtypes = [vp, vp, f, i, i, vp, i, i, f, vp, vp, vp, vp]
    L.arcq_swiglu_quantize_x.argtypes = [vp, vp, i, i, i, vp, i, i, f, vp, vp, vp, vp]
    L.arcq_swiglu_absmax.argtypes = [vp, vp, i, i, i, vp, vp]
    L.arcq_tensor_scale.argtypes = [vp, vp, i, i, i, f, vp, vp]
    L.arcq_reorder_quantize_x_absmax.argtypes = [vp, i, i, vp, i, i, f, vp, vp, vp, vp]
    L.arcq_kv_append_i4.argtypes = [vp, vp, i, i, vp, i, vp, vp, vp, vp, vp, i, i, i, i, i, vp]
    L.arcq_rope_kv_append_i4.argtypes = [vp, i, i, i, i, vp, vp, i, vp, vp, vp, vp, vp, vp, vp, i, i, i, i, i, vp]
    L.arcq_rope.argtypes = [vp, i, i, ctypes.c_long, i, i, i, i, i, vp, vp, i, vp, vp, vp]
    L.arcq_kv_store_i4.argtypes = [vp, vp, vp, vp, i, vp, i, vp, vp, vp, vp, vp, i, i, i, i, i, vp]
    L.arcq_kv_decode_i4.argtypes = [vp, vp, i, i, i, vp, vp, vp, vp, vp, i, i, i, i, i, f, vp]
    L.arcq_matmul.argtypes = [vp, vp, vp, vp, i, i, i, i, f, vp, vp, vp, vp]
    L.arcq_matmul_add.argtypes = [vp, vp, vp, vp, i, i, i, i, f, vp, vp, vp, vp, vp]
    if hasattr(L, "arcq_matmul_noalloc"):
        L.arcq_matmul_noalloc.argtypes = L.arcq_matmul.argtypes
        L.arcq_matmul_noalloc.restype = i
        L.arcq_matmul_noalloc_limit.restype = sz
        L.arcq_matmul_scratch_bytes.argtypes = [i, i, i, i]
        L.arcq_matmul_scratch_bytes.restype = sz
    L.arcq_grouped_reorder_quantize_x.argtypes = [vp, i, i, vp, i, vp, i, i, vp, vp, vp, vp]
    L.arcq_grouped_swiglu_quantize_x.argtypes = [vp, vp, i, i, i, vp, i, vp, i, i, vp, vp, vp, vp]
    L.arcq_grouped_tensor_scale.argtypes = [vp, vp, i, i, i, vp, i, f, vp, vp]
    L.arcq_grouped_matmul.argtypes = [vp, vp, vp, vp, vp, i, i, i, i, i, f, vp, vp, vp, vp, vp]
    L.arcq_grouped_matmul_swiglu.argtypes = [vp, vp, vp, vp, vp, i, i, i, i, i, f, vp, vp, vp, vp, vp]
    L.arcq_matmul_swiglu.argtypes = [vp, vp, vp, vp, i, i, i, i, f, vp, vp, vp, vp, vp]
    L.arcq_scales_from_absmax.argtypes = [vp, i, f, vp]
    for name in ("arcq_grouped_matmul_swiglu", "arcq_matmul_swiglu", "arcq_scales_from_absmax"):
        getattr(L, name).restype = i
    L.arcq_moe_combine.argtypes = [vp, vp, vp, i, i, i, i, vp, vp]
    L.arcq_moe_combine.restype = i
    L.arcq_moe_route.argtypes = [vp, i, i, i, i, vp, vp, vp, vp, vp, vp, vp, sz, vp]
    L.arcq_moe_route.restype = i
    L.arcq_moe_route_workspace_bytes.argtypes = [i, i]
    L.arcq_moe_route_workspace_bytes.restype = sz
    for name in ("arcq_grouped_reorder_quantize_x", "arcq_grouped_swiglu_quantize_x", "arcq_grouped_tensor_scale",
                 "arcq_grouped_matmul"):
        getattr(L, name).restype = i
    L.arcq_check_index.argtypes = [vp, i, vp]
    L.arcq_dequantize.argtypes = [vp, vp, i, i, i, vp, vp]
    for name in ("arcq_reorder_quantize_x", "arcq_reorder_quantize_w", "arcq_rmsnorm_quantize_x", "arcq_matmul",
                 "arcq_check_index", "arcq_dequantize", "arcq_swiglu_quantize_x", "arcq_swiglu_absmax",
                 "arcq_kv_append_i4", "arcq_kv_store_i4", "arcq_kv_decode_i4"):
        getattr(L, name).restype = i
    _lib = L
    return L


PROBE_LIB_PATH = os.path.join(_HERE, "csrc", "libarcq_probe.so")
_probe = None


def probe_lib() -> ctypes.CDLL:
    """libarcq_probe.so (include/arcq_probe.h): plain copy kernels, for measurement only -- bench.py's streaming
    ceiling and the calibration of the rocprofv3 traffic counters.  No operator loads it."""
    global _probe
    if _probe is None:
        if not os.path.exists(PROBE_LIB_PATH):
            raise RuntimeError(f"{PROBE_LIB_PATH} is missing: build it with `python -m arcquant_amd.build`")
        P = ctypes.CDLL(PROBE_LIB_PATH)
        vp, i, sz = ctypes.c_void_p, ctypes.c_int, ctypes.c_size_t
        P.arcq_stream_probe.argtypes = [vp, vp, sz, sz, vp]
        P.arcq_stream_probe.restype = i
        P.arcq_stream_probe_variant.argtypes = [vp, vp, sz, sz, i, vp]
        P.arcq_stream_probe_variant.restype = i
        P.arcq_stream_probe_variants.restype = i
        P.arcq_mfma_rate_probe.argtypes = [i, i, i, vp, vp, vp]
        P.arcq_mfma_rate_probe.restype = i
        P.arcq_mfma_rate_probe_flops.argtypes = [i, i, i]
        P.arcq_mfma_rate_probe_flops.restype = ctypes.c_double
        _probe = P
    return _probe


def check(status: int, where: str) -> None:
    if status != 0:
        raise ArcqError(status, where)


# ------------------------------------------------------------------------------------------
# launch plumbing shared by the operator modules: torch is asked for the current stream and the
# current device through its cheapest entry points, since a decode step is a chain of launches
# of a few microseconds each and the host must keep ahead of them
# ------------------------------------------------------------------------------------------
GROUP_SIZE = {NVFP4: 16, MXFP4: 32}


def stream_of(t) -> ctypes.c_void_p:
    """torch's current stream on t's device, as the `void *stream` of the C ABI"""
    import torch
    try:
        return ctypes.c_void_p(torch._C._cuda_getCurrentRawStream(t.device.index))
    except AttributeError:                       # a torch without the raw-stream hook
        return ctypes.c_void_p(torch.cuda.current_stream(t.device).cuda_stream)


class on_device_of:
    """`with on_device_of(t):` makes t's device current for the launch; free when it already is"""
    __slots__ = ("idx", "prev")

    def __init__(self, t):
        self.idx = t.device.index

    def __enter__(self):
        import torch
        self.prev = torch.cuda.current_device()
        if self.prev != self.idx:
            torch.cuda.set_device(self.idx)

    def __exit__(self, *exc):
        if self.prev != self.idx:
            import torch
            torch.cuda.set_device(self.prev)
        return False

