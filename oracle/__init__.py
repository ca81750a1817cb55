"""CPU oracle for the ARC quantized-linear path -- TEST INFRASTRUCTURE ONLY.

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may import
this package; the shipped op surface (arcquant_amd) never does.

Two restatements of the reference's fake-quant arithmetic live here:

* ``arcq_oracle.c`` (loaded through ctypes below): scalar C, one IEEE rounding
  per operation, returns packed codes + scale bytes + dequantised values.
* ``fakequant_torch.py``: the same sequence of torch tensor operations the
  reference runs (model/quantize.py:14-59,145-201,287-343), used to cross-check
  the C code and as the timed host-CPU baseline.
"""
from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

NVFP4 = 0
MXFP4 = 1
_FMT = {"NVFP4": NVFP4, "MXFP4": MXFP4, NVFP4: NVFP4, MXFP4: MXFP4}
_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libarcq_oracle.so")
_lib = None


def fmt_id(fmt) -> int:
    return _FMT[fmt]


def group_size(fmt) -> int:
    return 16 if fmt_id(fmt) == NVFP4 else 32


def build(force: bool = False) -> str:
    """Compile the C oracle with gcc (a few hundred ms)."""
    src = os.path.join(_HERE, "arcq_oracle.c")
    if force or not os.path.exists(_LIB_PATH) or os.path.getmtime(_LIB_PATH) < os.path.getmtime(src):
        subprocess.check_call(["make", "-s", "-C", _HERE, "-B", "libarcq_oracle.so"])
    return _LIB_PATH


def build_hostmath(force: bool = False) -> str:
    """Compile host_math.cpp: the kernels' scalar arithmetic (arcquant_amd/csrc/arcq_math.h) built for the host
    with the exhaustive checks of its shortcuts.  Test scaffolding, like the rest of this package."""
    path = os.path.join(_HERE, "libarcq_hostmath.so")
    deps = [os.path.join(_HERE, "host_math.cpp"), os.path.join(_HERE, "..", "arcquant_amd", "csrc", "arcq_math.h")]
    if force or not os.path.exists(path) or any(os.path.getmtime(path) < os.path.getmtime(d) for d in deps):
        subprocess.check_call(["make", "-s", "-C", _HERE, "-B", "libarcq_hostmath.so"])
    return path


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        L = ctypes.CDLL(_LIB_PATH)
        vp, i, f = ctypes.c_void_p, ctypes.c_int, ctypes.c_float
        L.arcq_oracle_quantize_x.argtypes = [vp, i, i, vp, i, i, f, vp, vp, vp]
        L.arcq_oracle_quantize_w.argtypes = [vp, i, i, vp, i, i, f, vp, vp, vp]
        L.arcq_oracle_rmsnorm_quantize_x.argtypes = [vp, vp, f, i, i, vp, i, i, f, vp, vp, vp, vp]
        L.arcq_oracle_dequantize.argtypes = [vp, vp, i, i, i, vp]
        L.arcq_oracle_matmul.argtypes = [vp, vp, vp, vp, i, i, i, i, f, vp]
        for name in ("e2m1", "ue4m3", "ue8m0"):
            getattr(L, f"arcq_oracle_{name}_many").argtypes = [vp, i, vp, vp]
        L.oq_scale_value.argtypes = [i, ctypes.c_uint8]
        L.oq_scale_value.restype = f
        _lib = L
    return _lib


def _bf16_bits(t) -> np.ndarray:
    """torch bf16 tensor (CPU) or uint16 ndarray -> contiguous uint16 ndarray."""
    if isinstance(t, np.ndarray):
        assert t.dtype == np.uint16
        return np.ascontiguousarray(t)
    import torch

    assert t.dtype == torch.bfloat16, t.dtype
    return np.ascontiguousarray(t.detach().cpu().contiguous().view(torch.int16).numpy().view(np.uint16))


def _idx(idx, K):
    if idx is None:
        return None
    if not isinstance(idx, np.ndarray):
        idx = idx.detach().cpu().numpy()
    idx = np.ascontiguousarray(idx.astype(np.int16))
    assert idx.shape == (K,)
    return idx


def _ptr(a):
    return None if a is None else a.ctypes.data_as(ctypes.c_void_p)


def _quant(fn_name, x, idx, S, fmt, gscale, want_dq, extra=None):
    xb = _bf16_bits(x)
    M, K = xb.shape
    f = fmt_id(fmt)
    G = group_size(f)
    Kp = K + S
    codes = np.empty((M, Kp // 2), np.uint8)
    scales = np.empty((M, Kp // G), np.uint8)
    dq = np.empty((M, Kp), np.float32) if want_dq else None
    ix = _idx(idx, K)
    fn = getattr(lib(), fn_name)
    if extra is None:
        rc = fn(_ptr(xb), M, K, _ptr(ix), S, f, float(gscale), _ptr(codes), _ptr(scales), _ptr(dq))
        normed = None
    else:
        gamma, eps, want_normed = extra
        gb = _bf16_bits(gamma)
        assert gb.shape == (K,)
        normed = np.empty((M, K), np.uint16) if want_normed else None
        rc = fn(_ptr(xb), _ptr(gb), float(eps), M, K, _ptr(ix), S, f, float(gscale), _ptr(codes), _ptr(scales),
                _ptr(dq), _ptr(normed))
    if rc != 0:
        raise ValueError(f"{fn_name}: rc={rc} (M={M} K={K} S={S} fmt={fmt})")
    out = {"codes": codes, "scales": scales, "dq": dq}
    if normed is not None:
        out["normed"] = normed
    return out


def quantize_x(x, idx, S, fmt, gscale=1.0, want_dq=False):
    """fake_reorder_quantize_x (quantize.py:314-343) with the gather folded in."""
    return _quant("arcq_oracle_quantize_x", x, idx, S, fmt, gscale, want_dq)


def quantize_w(w, idx, S, fmt, gscale=1.0, want_dq=False):
    """fake_reorder_quantize_w (quantize.py:287-312) with the gather folded in."""
    return _quant("arcq_oracle_quantize_w", w, idx, S, fmt, gscale, want_dq)


def rmsnorm_quantize_x(x, gamma, eps, idx, S, fmt, gscale=1.0, want_dq=False, want_normed=False):
    return _quant("arcq_oracle_rmsnorm_quantize_x", x, idx, S, fmt, gscale, want_dq, (gamma, eps, want_normed))


def dequantize(codes, scales, fmt):
    codes = np.ascontiguousarray(codes, np.uint8)
    scales = np.ascontiguousarray(scales, np.uint8)
    rows, half = codes.shape
    out = np.empty((rows, half * 2), np.float32)
    rc = lib().arcq_oracle_dequantize(_ptr(codes), _ptr(scales), rows, half * 2, fmt_id(fmt), _ptr(out))
    assert rc == 0
    return out


def matmul(ca, sa, cb, sb, fmt, alpha=1.0):
    """alpha * dq(A) @ dq(B)^T accumulated in fp64 (small shapes only: O(MNK) scalar)."""
    ca, sa, cb, sb = (np.ascontiguousarray(a, np.uint8) for a in (ca, sa, cb, sb))
    M, half = ca.shape
    N = cb.shape[0]
    Y = np.empty((M, N), np.float32)
    rc = lib().arcq_oracle_matmul(_ptr(ca), _ptr(sa), _ptr(cb), _ptr(sb), M, N, half * 2, fmt_id(fmt), float(alpha),
                                  _ptr(Y))
    assert rc == 0
    return Y


def _many(name, a):
    a = np.ascontiguousarray(a, np.float32).ravel()
    val = np.empty_like(a)
    byte = np.empty(a.shape, np.uint8)
    getattr(lib(), f"arcq_oracle_{name}_many")(_ptr(a), a.size, _ptr(val), _ptr(byte))
    return val, byte


def e2m1(n):
    return _many("e2m1", n)


def ue4m3(t):
    return _many("ue4m3", t)


def ue8m0(t):
    return _many("ue8m0", t)


def scale_values(scales, fmt):
    """scale bytes -> fp32 values."""
    s = np.asarray(scales, np.uint8).astype(np.int32)
    if fmt_id(fmt) == NVFP4:
        return np.ldexp(1.0 + (s & 7) / 8.0, (s >> 3) - 9).astype(np.float32)
    return np.ldexp(1.0, s - 127).astype(np.float32)
