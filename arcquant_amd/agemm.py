"""Drop-in for the reference's ``agemm`` extension module on PyTorch-ROCm.

Same four operators, same positional arguments and return values as the pybind11 module the
reference builds from kernels/src/bindings.cpp:547-575:

    matmul(A, B, SFA, SFB, scale)                          -> bf16 [M, N]
    reorder_quantize_x(X, reorder_index, KE)               -> (QX, SFX)
    reorder_quantize_w(W, reorder_index, KE)               -> (QW, SFW)
    rmsnorm_quantize_x(X, W, eps, reorder_index, KE)       -> (QX, SFX)

plus keyword-only extensions the reference does not have:

    fmt="NVFP4" | "MXFP4"   block format (the reference's kernels are NVFP4 only)
    global_scale            fp32 tensor scale the values are divided by inside the kernel, as
                            fake_reorder_quantize_x does (model/quantize.py:330); a python
                            float or a 0-dim CUDA tensor (read on the device, no host sync).
                            The reference's callers pass X / scale instead, which rounds to
                            bf16 first (model/qLlamaLayer.py:76).

PyTorch is used for device memory and the current stream only; all arithmetic happens in
libarcq_hip.so through its C ABI (include/arcq.h).  Errors surface as RuntimeError, like the
reference's ``std::runtime_error`` (bindings.cpp:157-159).
"""
from __future__ import annotations

import ctypes

import torch

from . import _lib
from ._lib import FORMATS, ArcqError  # noqa: F401

__all__ = ["matmul", "reorder_quantize_x", "reorder_quantize_w", "rmsnorm_quantize_x", "init_kv_i4", "append_kv_i4",
           "batch_decode_i4", "swiglu_quantize_x", "tensor_scale", "prepare_stream", "release_stream", "dequantize", "check_index",
           "unpack_codes", "scale_values", "grouped_tensor_scale", "grouped_reorder_quantize_x",
           "grouped_swiglu_quantize_x", "grouped_matmul", "moe_route", "moe_combine", "matmul_swiglu",
           "grouped_matmul_swiglu", "interleave_gate_up"]


def _fmt_id(fmt) -> int:
    try:
        return FORMATS[fmt] if isinstance(fmt, str) else FORMATS[{0: "NVFP4", 1: "MXFP4"}[int(fmt)]]
    except KeyError:
        raise RuntimeError(f"unknown quantization format {fmt!r} (expected 'NVFP4' or 'MXFP4')") from None


_stream = _lib.stream_of
_on_device = _lib.on_device_of


def _require(t: torch.Tensor, name: str, dtype, ndim=None):
    if not isinstance(t, torch.Tensor):
        raise RuntimeError(f"{name} must be a torch.Tensor")
    if t.dtype != dtype:
        raise RuntimeError(f"expected {name} to have dtype {dtype}, but got {t.dtype}")
    if not t.is_cuda:
        raise RuntimeError(f"{name} must be on the GPU (got {t.device})")
    if ndim is not None and t.dim() != ndim:
        raise RuntimeError(f"{name} must be {ndim}-D (got shape {tuple(t.shape)})")
    if not t.is_contiguous():
        raise RuntimeError(f"{name} must be contiguous")
    return t


def _scalar(value, device):
    """python float / 0-dim tensor -> (host float, device pointer or None, keep-alive)."""
    if value is None:
        return 1.0, None, None
    if isinstance(value, torch.Tensor):
        if value.numel() != 1:
            raise RuntimeError("scale must be a scalar")
        if value.is_cuda:
            if value.dtype == torch.float32 and value.device == device:
                return 1.0, ctypes.c_void_p(value.data_ptr()), value
            v = value.detach().to(device=device, dtype=torch.float32).reshape(1)
            return 1.0, ctypes.c_void_p(v.data_ptr()), v
        return float(value), None, None
    return float(value), None, None


def _quantize(entry, X, gamma, eps, reorder_index, KE, fmt, global_scale):
    f = _fmt_id(fmt)
    L = _lib.lib()
    _require(X, "X", torch.bfloat16, 2)
    _require(reorder_index, "reorder_index", torch.int16, 1)
    M, K = X.shape
    if reorder_index.numel() != K:
        raise RuntimeError(f"reorder_index has {reorder_index.numel()} entries, expected K={K}")
    if reorder_index.device != X.device:
        raise RuntimeError("reorder_index must be on the same device as X")
    KE = int(KE)
    G = _lib.GROUP_SIZE[f]
    if K % 32 or K < 32 or K > 32736 or KE < 0 or KE > K or KE % G:
        raise RuntimeError(f"Value error in {entry}: K={K}, KE={KE} not supported for {fmt} "
                           f"(need K % 32 == 0, 32 <= K <= 32736, KE % {G} == 0, KE <= K)")
    QX = torch.empty((M, (K + KE) // 2), dtype=torch.uint8, device=X.device)
    SFX = torch.empty((M * ((K + KE) // G),), dtype=torch.uint8, device=X.device)
    if isinstance(global_scale, str):
        if global_scale != "absmax" or entry != "arcq_reorder_quantize_x":
            raise RuntimeError("global_scale must be a number or a tensor (reorder_quantize_x also takes 'absmax')")
        scale = torch.empty((), dtype=torch.float32, device=X.device)
        with _on_device(X):
            rc = L.arcq_reorder_quantize_x_absmax(X.data_ptr(), M, K, reorder_index.data_ptr(), KE, f, 2688.0, scale.data_ptr(),
                                                  QX.data_ptr(), SFX.data_ptr(), _stream(X))
        _lib.check(rc, "arcq_reorder_quantize_x_absmax")
        return QX, SFX, scale
    gs, d_gs, keep = _scalar(global_scale, X.device)
    with _on_device(X):
        if gamma is None:
            rc = getattr(L, entry)(X.data_ptr(), M, K, reorder_index.data_ptr(), KE, f, gs, d_gs, QX.data_ptr(),
                                   SFX.data_ptr(), _stream(X))
        else:
            _require(gamma, "W", torch.bfloat16, 1)
            if gamma.numel() != K or gamma.device != X.device:
                raise RuntimeError(f"RMSNorm weight must have K={K} entries on X's device")
            rc = L.arcq_rmsnorm_quantize_x(X.data_ptr(), gamma.data_ptr(), float(eps), M, K,
                                           reorder_index.data_ptr(), KE, f, gs, d_gs, QX.data_ptr(),
                                           SFX.data_ptr(), _stream(X))
    _lib.check(rc, entry)
    del keep
    return QX, SFX


def reorder_quantize_x(X, reorder_index, KE, *, fmt="NVFP4", global_scale=None):
    """agemm.reorder_quantize_x (kernels/src/bindings.cpp:122-163).
    X bf16 [M,K]; reorder_index int16 [K]; returns QX u8 [M,(K+KE)/2], SFX u8 [M*(K+KE)/G].
    global_scale="absmax" forms the NVFP4 tensor scale max|X| / 2688 on the device as part of the call (what the
    reference's callers compute with torch first, model/qLlamaLayer.py:73-77) and returns it as a third value:
    one launch and one pass over X while X fits the chip's LDS (up to 4096 rows of up to 4096 channels)."""
    return _quantize("arcq_reorder_quantize_x", X, None, 0.0, reorder_index, KE, fmt, global_scale)


def reorder_quantize_w(W, reorder_index, KE, *, fmt="NVFP4", global_scale=None):
    """agemm.reorder_quantize_w (kernels/src/bindings.cpp:170-210)."""
    return _quantize("arcq_reorder_quantize_w", W, None, 0.0, reorder_index, KE, fmt, global_scale)


def rmsnorm_quantize_x(X, W, eps, reorder_index, KE, *, fmt="NVFP4", global_scale=None):
    """agemm.rmsnorm_quantize_x (kernels/src/bindings.cpp:216-254); W is the RMSNorm weight bf16 [K]."""
    return _quantize("arcq_rmsnorm_quantize_x", X, W, eps, reorder_index, KE, fmt, global_scale)


def tensor_scale(x, divisor=2688.0):
    """NVFP4 tensor scale max|x| / divisor of bf16 activations [M, K] (rows may be strided) as a 0-dim
    fp32 tensor on x's device, 1 for an all-zero tensor: what the reference's callers compute with torch
    ahead of the quantizer (model/qLlamaLayer.py:73-77), in one launch."""
    if not isinstance(x, torch.Tensor) or x.dtype != torch.bfloat16 or not x.is_cuda or x.dim() != 2 or x.stride(1) != 1:
        raise RuntimeError("tensor_scale takes a 2-D bf16 CUDA tensor with unit stride along its last dimension")
    M, K = x.shape
    ld = x.stride(0) if M > 1 else K
    if K % 8 or ld % 8 or x.data_ptr() % 16:
        raise RuntimeError(f"Value error in tensor_scale: K={K}, row stride {ld} not supported")
    out = torch.empty((), dtype=torch.float32, device=x.device)
    with _on_device(x):
        rc = _lib.lib().arcq_tensor_scale(x.data_ptr(), None, ld, M, K, float(divisor), out.data_ptr(), _stream(x))
    _lib.check(rc, "arcq_tensor_scale")
    return out


def swiglu_quantize_x(gate, up, reorder_index, KE, *, fmt="NVFP4", global_scale=None):
    """act_fn(gate) * up -> quantized activations in one pass (no counterpart in the reference's
    module; its layers do silu, multiply and quantize as separate ops, model/qLlamaLayer.py:432-439).
    gate, up: bf16 [M, K] views with the same row stride and unit column stride, e.g. the two
    halves of a fused gate_up output.  global_scale: None / float / 0-dim CUDA tensor;
    "absmax" computes the NVFP4 tensor scale max|t| / 2688 on the device first and returns it
    as a third value."""
    f = _fmt_id(fmt)
    L = _lib.lib()
    for t, name in ((gate, "gate"), (up, "up")):
        if not isinstance(t, torch.Tensor) or t.dtype != torch.bfloat16 or not t.is_cuda or t.dim() != 2:
            raise RuntimeError(f"{name} must be a 2-D bf16 CUDA tensor")
        if t.stride(1) != 1:
            raise RuntimeError(f"{name} must have unit stride along its last dimension")
    if gate.shape != up.shape or gate.stride(0) != up.stride(0) or gate.device != up.device:
        raise RuntimeError("gate and up must have the same shape, row stride and device")
    _require(reorder_index, "reorder_index", torch.int16, 1)
    M, K = gate.shape
    ld = gate.stride(0) if M > 1 else K
    KE = int(KE)
    G = _lib.GROUP_SIZE[f]
    if K % 32 or K < 32 or K > 32736 or KE < 0 or KE > K or KE % G or reorder_index.numel() != K or ld % 8:
        raise RuntimeError(f"Value error in swiglu_quantize_x: K={K}, KE={KE}, row stride {ld} not supported for {fmt}")
    want_scale = isinstance(global_scale, str)
    with _on_device(gate):
        if want_scale:
            if global_scale != "absmax":
                raise RuntimeError("global_scale must be a number, a tensor or 'absmax'")
            global_scale = torch.empty((), dtype=torch.float32, device=gate.device)
            _lib.check(L.arcq_tensor_scale(gate.data_ptr(), up.data_ptr(), ld, M, K, 2688.0, global_scale.data_ptr(),
                                           _stream(gate)), "arcq_tensor_scale")
        gs, d_gs, keep = _scalar(global_scale, gate.device)
        QX = torch.empty((M, (K + KE) // 2), dtype=torch.uint8, device=gate.device)
        SFX = torch.empty((M * ((K + KE) // G),), dtype=torch.uint8, device=gate.device)
        rc = L.arcq_swiglu_quantize_x(gate.data_ptr(), up.data_ptr(), ld, M, K, reorder_index.data_ptr(), KE, f, gs,
                                      d_gs, QX.data_ptr(), SFX.data_ptr(), _stream(gate))
    _lib.check(rc, "arcq_swiglu_quantize_x")
    del keep
    return (QX, SFX, global_scale) if want_scale else (QX, SFX)


def _infer_fmt(A, SFA, fmt):
    if fmt is not None:
        return _fmt_id(fmt)
    M, half = A.shape
    n = SFA.numel()
    if n == M * (2 * half // 16):
        return FORMATS["NVFP4"]
    if n == M * (2 * half // 32):
        return FORMATS["MXFP4"]
    raise RuntimeError(f"cannot tell the block format from SFA ({n} scale bytes for {M}x{2 * half} values)")


def matmul(A, B, SFA, SFB, scale, *, fmt=None, residual=None):
    """agemm.matmul (kernels/src/bindings.cpp:99-120): bf16 [M,N] = scale * dq(A) @ dq(B)^T.

    A u8 [M,K'/2], B u8 [N,K'/2], SFA/SFB as returned by the quantizers.  ``scale`` may be a
    python float (as in the reference), a 0-dim tensor, or a pair of 0-dim CUDA tensors
    (scale_x, scale_w) whose product is formed on the device -- the last two avoid the host sync
    the reference's float argument forces (model/qLinearLayer.py:69).  ``residual`` bf16 [M,N]: added
    in the epilogue, with the result of ``matmul(...) + residual`` bit for bit.
    """
    _require(A, "A", torch.uint8, 2)
    _require(B, "B", torch.uint8, 2)
    _require(SFA, "SFA", torch.uint8)
    _require(SFB, "SFB", torch.uint8)
    if A.shape[1] != B.shape[1]:
        raise RuntimeError(f"A and B disagree on K': {2 * A.shape[1]} vs {2 * B.shape[1]}")
    f = _infer_fmt(A, SFA, fmt)
    L = _lib.lib()
    M, N, Kp = A.shape[0], B.shape[0], 2 * A.shape[1]
    G = _lib.GROUP_SIZE[f]
    if SFA.numel() != M * (Kp // G) or SFB.numel() != N * (Kp // G):
        raise RuntimeError("scale buffers do not match the code buffers")
    if Kp % 64:
        raise RuntimeError(f"Value error in matmul: K'={Kp} must be a multiple of 64")
    if isinstance(scale, (tuple, list)):
        sa, sb = scale
        ha, da, ka = _scalar(sa, A.device)
        hb, db, kb = _scalar(sb, A.device)
        alpha = ha * hb
    else:
        alpha, da, ka = _scalar(scale, A.device)
        db, kb = None, None
    C = torch.empty((M, N), dtype=torch.bfloat16, device=A.device)
    with _on_device(A):
        if residual is None:
            rc = L.arcq_matmul(A.data_ptr(), SFA.data_ptr(), B.data_ptr(), SFB.data_ptr(), M, N, Kp, f, alpha, da, db,
                               C.data_ptr(), _stream(A))
        else:
            _require(residual, "residual", torch.bfloat16, 2)
            if tuple(residual.shape) != (M, N) or residual.device != A.device:
                raise RuntimeError(f"residual must be bf16 [{M}, {N}] on A's device")
            rc = L.arcq_matmul_add(A.data_ptr(), SFA.data_ptr(), B.data_ptr(), SFB.data_ptr(), M, N, Kp, f, alpha, da,
                                   db, residual.data_ptr(), C.data_ptr(), _stream(A))
    _lib.check(rc, "arcq_matmul")
    del ka, kb
    return C


# ------------------------------------------------------------------------------------------
# grouped operators for mixture-of-experts blocks: rows sorted by expert, `seg` int32 [E+1] row
# offsets on the device, one launch per step for all experts and no host read-back
# (model/qMixtralLayer.py:458-471 walks the experts in Python instead)
# ------------------------------------------------------------------------------------------

def _seg(seg, device):
    _require(seg, "seg", torch.int32, 1)
    if seg.device != device or seg.numel() < 2:
        raise RuntimeError("seg must be an int32 tensor [experts + 1] on the operands' device")
    return seg.numel() - 1


def _rows_2d(t, name):
    if not isinstance(t, torch.Tensor) or t.dtype != torch.bfloat16 or not t.is_cuda or t.dim() != 2 or t.stride(1) != 1:
        raise RuntimeError(f"{name} must be a 2-D bf16 CUDA tensor with unit stride along its last dimension")
    M, K = t.shape
    ld = t.stride(0) if M > 1 else K
    if ld % 8 or t.data_ptr() % 16:
        raise RuntimeError(f"{name}: row stride {ld} / alignment not supported")
    return M, K, ld


def grouped_tensor_scale(x, seg, divisor=2688.0, *, up=None):
    """NVFP4 tensor scales max|x_e| / divisor of each expert's rows of x (bf16 [M, K]) as fp32 [E] on the
    device (1 for an expert without rows); with `up`, of act_fn(x) * up (x = gate)."""
    M, K, ld = _rows_2d(x, "x")
    E = _seg(seg, x.device)
    if up is not None:
        if _rows_2d(up, "up") != (M, K, ld):
            raise RuntimeError("gate and up must have the same shape and row stride")
    out = torch.empty(E, dtype=torch.float32, device=x.device)
    with _on_device(x):
        rc = _lib.lib().arcq_grouped_tensor_scale(x.data_ptr(), None if up is None else up.data_ptr(), ld, M, K,
                                                  seg.data_ptr(), E, float(divisor), out.data_ptr(), _stream(x))
    _lib.check(rc, "arcq_grouped_tensor_scale")
    return out


def _grouped_quantize(gate, up, seg, reorder_index, KE, fmt, global_scales):
    f = _fmt_id(fmt)
    M, K, ld = _rows_2d(gate, "x" if up is None else "gate")
    E = _seg(seg, gate.device)
    _require(reorder_index, "reorder_index", torch.int16, 2)
    KE = int(KE)
    G = _lib.GROUP_SIZE[f]
    if tuple(reorder_index.shape) != (E, K) or reorder_index.device != gate.device:
        raise RuntimeError(f"reorder_index must be int16 [{E}, {K}] on the operands' device")
    if K % 32 or K < 32 or K > 32736 or KE < 0 or KE > K or KE % G:
        raise RuntimeError(f"Value error in grouped quantizer: K={K}, KE={KE} not supported for {fmt}")
    if global_scales is not None:
        _require(global_scales, "global_scales", torch.float32, 1)
        if global_scales.numel() != E or global_scales.device != gate.device:
            raise RuntimeError(f"global_scales must be fp32 [{E}] on the operands' device")
    QX = torch.empty((M, (K + KE) // 2), dtype=torch.uint8, device=gate.device)
    SFX = torch.empty((M * ((K + KE) // G),), dtype=torch.uint8, device=gate.device)
    L = _lib.lib()
    d_gs = None if global_scales is None else global_scales.data_ptr()
    with _on_device(gate):
        if up is None:
            if ld != K:
                raise RuntimeError("x must be contiguous")
            rc = L.arcq_grouped_reorder_quantize_x(gate.data_ptr(), M, K, seg.data_ptr(), E, reorder_index.data_ptr(), KE,
                                                   f, d_gs, QX.data_ptr(), SFX.data_ptr(), _stream(gate))
        else:
            rc = L.arcq_grouped_swiglu_quantize_x(gate.data_ptr(), up.data_ptr(), ld, M, K, seg.data_ptr(), E,
                                                  reorder_index.data_ptr(), KE, f, d_gs, QX.data_ptr(), SFX.data_ptr(),
                                                  _stream(gate))
    _lib.check(rc, "grouped quantizer")
    return QX, SFX


def grouped_reorder_quantize_x(X, seg, reorder_index, KE, *, fmt="NVFP4", global_scales=None):
    """reorder_quantize_x over tokens sorted by expert: row r in seg[e] .. seg[e+1]-1 is quantized with
    reorder_index[e] and tensor scale global_scales[e] (None: 1).  X bf16 [M, K] contiguous."""
    return _grouped_quantize(X, None, seg, reorder_index, KE, fmt, global_scales)


def grouped_swiglu_quantize_x(gate, up, seg, reorder_index, KE, *, fmt="NVFP4", global_scales=None):
    """swiglu_quantize_x over tokens sorted by expert; global_scales: fp32 [E], None, or "absmax" (the
    per-expert NVFP4 scales are computed on the device first and returned as a third value)."""
    if isinstance(global_scales, str):
        if global_scales != "absmax":
            raise RuntimeError("global_scales must be a tensor, None or 'absmax'")
        gs = grouped_tensor_scale(gate, seg, 2688.0, up=up)
        return _grouped_quantize(gate, up, seg, reorder_index, KE, fmt, gs) + (gs,)
    if _rows_2d(up, "up") != _rows_2d(gate, "gate"):
        raise RuntimeError("gate and up must have the same shape and row stride")
    return _grouped_quantize(gate, up, seg, reorder_index, KE, fmt, global_scales)


def grouped_matmul(A, B, SFA, SFB, seg, scale_a=None, scale_b=None, *, fmt=None, residual=None):
    """Rows seg[e] .. seg[e+1]-1 of bf16 [M, N] = scale_a[e] * scale_b[e] * dq(A rows) @ dq(B[e])^T.
    A u8 [M, K'/2]; B u8 [E, N, K'/2], SFB u8 [E * N * K'/G]: the experts' quantized weights stacked;
    scale_a / scale_b fp32 [E] on the device or None."""
    _require(A, "A", torch.uint8, 2)
    _require(B, "B", torch.uint8, 3)
    _require(SFA, "SFA", torch.uint8)
    _require(SFB, "SFB", torch.uint8)
    E = _seg(seg, A.device)
    if B.shape[0] != E or A.shape[1] != B.shape[2]:
        raise RuntimeError(f"B must be [{E}, N, {A.shape[1]}]")
    f = _infer_fmt(A, SFA, fmt)
    M, N, Kp = A.shape[0], B.shape[1], 2 * A.shape[1]
    G = _lib.GROUP_SIZE[f]
    if SFA.numel() != M * (Kp // G) or SFB.numel() != E * N * (Kp // G):
        raise RuntimeError("scale buffers do not match the code buffers")
    if Kp % 128 or Kp < 512:
        raise RuntimeError(f"Value error in grouped_matmul: K'={Kp} must be a multiple of 128, at least 512")
    ptrs = []
    for t, name in ((scale_a, "scale_a"), (scale_b, "scale_b")):
        if t is None:
            ptrs.append(None)
            continue
        _require(t, name, torch.float32, 1)
        if t.numel() != E or t.device != A.device:
            raise RuntimeError(f"{name} must be fp32 [{E}] on A's device")
        ptrs.append(t.data_ptr())
    if residual is not None:
        _require(residual, "residual", torch.bfloat16, 2)
        if tuple(residual.shape) != (M, N) or residual.device != A.device:
            raise RuntimeError(f"residual must be bf16 [{M}, {N}] on A's device")
    C = torch.empty((M, N), dtype=torch.bfloat16, device=A.device)
    with _on_device(A):
        rc = _lib.lib().arcq_grouped_matmul(A.data_ptr(), SFA.data_ptr(), B.data_ptr(), SFB.data_ptr(), seg.data_ptr(), E,
                                            M, N, Kp, f, 1.0, ptrs[0], ptrs[1],
                                            None if residual is None else residual.data_ptr(), C.data_ptr(), _stream(A))
    _lib.check(rc, "arcq_grouped_matmul")
    return C


def interleave_gate_up(w_gate, w_up):
    """[F, K] gate and up weights -> [2F, K] with rows gate_0, up_0, gate_1, up_1, ...: the row order the
    SwiGLU-fused GEMMs expect (quantize the result with reorder_quantize_w as usual)."""
    if w_gate.shape != w_up.shape:
        raise RuntimeError("gate and up weights must have the same shape")
    return torch.stack((w_gate, w_up), dim=1).reshape(2 * w_gate.shape[0], w_gate.shape[1]).contiguous()


def _absmax_to_scales(buf, divisor):
    with _on_device(buf):
        _lib.check(_lib.lib().arcq_scales_from_absmax(buf.data_ptr(), buf.numel(), float(divisor), _stream(buf)),
                   "arcq_scales_from_absmax")
    return buf


def matmul_swiglu(A, B, SFA, SFB, scale, *, fmt=None, tensor_scale=False):
    """matmul for a fused gate/up projection whose weight rows alternate gate, up (interleave_gate_up), with
    act_fn(gate) * up formed in the epilogue: returns t bf16 [M, N/2], bit-identical to
    ``h = matmul(...); F.silu(h_gate) * h_up`` in bf16, without h going through memory.  tensor_scale=True
    also returns the NVFP4 tensor scale max|t| / 2688 of t (0-dim fp32 device tensor, 1 for all zeros)."""
    _require(A, "A", torch.uint8, 2)
    _require(B, "B", torch.uint8, 2)
    _require(SFA, "SFA", torch.uint8)
    _require(SFB, "SFB", torch.uint8)
    if A.shape[1] != B.shape[1]:
        raise RuntimeError(f"A and B disagree on K': {2 * A.shape[1]} vs {2 * B.shape[1]}")
    f = _infer_fmt(A, SFA, fmt)
    M, N, Kp = A.shape[0], B.shape[0], 2 * A.shape[1]
    G = _lib.GROUP_SIZE[f]
    if SFA.numel() != M * (Kp // G) or SFB.numel() != N * (Kp // G):
        raise RuntimeError("scale buffers do not match the code buffers")
    if Kp % 128 or Kp < 512 or N % 16:
        raise RuntimeError(f"Value error in matmul_swiglu: K'={Kp} (multiple of 128, >= 512), N={N} (multiple of 16)")
    if isinstance(scale, (tuple, list)):
        ha, da, ka = _scalar(scale[0], A.device)
        hb, db, kb = _scalar(scale[1], A.device)
        alpha = ha * hb
    else:
        alpha, da, ka = _scalar(scale, A.device)
        db, kb = None, None
    T = torch.empty((M, N // 2), dtype=torch.bfloat16, device=A.device)
    amax = torch.zeros(1, dtype=torch.float32, device=A.device) if tensor_scale else None
    with _on_device(A):
        rc = _lib.lib().arcq_matmul_swiglu(A.data_ptr(), SFA.data_ptr(), B.data_ptr(), SFB.data_ptr(), M, N, Kp, f, alpha,
                                           da, db, T.data_ptr(), None if amax is None else amax.data_ptr(), _stream(A))
    _lib.check(rc, "arcq_matmul_swiglu")
    del ka, kb
    if tensor_scale:
        return T, _absmax_to_scales(amax, 2688.0).reshape(())
    return T


def grouped_matmul_swiglu(A, B, SFA, SFB, seg, scale_a=None, scale_b=None, *, fmt=None, tensor_scale=False):
    """grouped_matmul with the SwiGLU epilogue of matmul_swiglu (B[e] rows alternate gate, up): t bf16 [M, N/2];
    tensor_scale=True also returns the per-expert NVFP4 tensor scales max|t_e| / 2688 as fp32 [E]."""
    _require(A, "A", torch.uint8, 2)
    _require(B, "B", torch.uint8, 3)
    _require(SFA, "SFA", torch.uint8)
    _require(SFB, "SFB", torch.uint8)
    E = _seg(seg, A.device)
    if B.shape[0] != E or A.shape[1] != B.shape[2]:
        raise RuntimeError(f"B must be [{E}, N, {A.shape[1]}]")
    f = _infer_fmt(A, SFA, fmt)
    M, N, Kp = A.shape[0], B.shape[1], 2 * A.shape[1]
    G = _lib.GROUP_SIZE[f]
    if SFA.numel() != M * (Kp // G) or SFB.numel() != E * N * (Kp // G):
        raise RuntimeError("scale buffers do not match the code buffers")
    if Kp % 128 or Kp < 512 or N % 16:
        raise RuntimeError(f"Value error in grouped_matmul_swiglu: K'={Kp}, N={N}")
    ptrs = []
    for t, name in ((scale_a, "scale_a"), (scale_b, "scale_b")):
        if t is None:
            ptrs.append(None)
            continue
        _require(t, name, torch.float32, 1)
        if t.numel() != E or t.device != A.device:
            raise RuntimeError(f"{name} must be fp32 [{E}] on A's device")
        ptrs.append(t.data_ptr())
    T = torch.empty((M, N // 2), dtype=torch.bfloat16, device=A.device)
    amax = torch.zeros(E, dtype=torch.float32, device=A.device) if tensor_scale else None
    with _on_device(A):
        rc = _lib.lib().arcq_grouped_matmul_swiglu(A.data_ptr(), SFA.data_ptr(), B.data_ptr(), SFB.data_ptr(),
                                                   seg.data_ptr(), E, M, N, Kp, f, 1.0, ptrs[0], ptrs[1], T.data_ptr(),
                                                   None if amax is None else amax.data_ptr(), _stream(A))
    _lib.check(rc, "arcq_grouped_matmul_swiglu")
    if tensor_scale:
        return T, _absmax_to_scales(amax, 2688.0)
    return T


def moe_route(router_logits, top_k):
    """Routing of a mixture-of-experts block in two launches (model/qMixtralLayer.py:441-452 and the bookkeeping
    of its loop over experts): softmax in fp32, top-k, weights divided by their sum, bf16.  Returns
    (sel int32 [T, k], weight bf16 [T, k], seg_offsets int32 [E+1], position int64 [T*k], token_of_row int32
    [T*k], weight_of_row bf16 [T*k]); rows of one expert keep ascending (token, slot) order.  Among equal
    probabilities the lower expert number is taken."""
    if router_logits.dim() != 2 or router_logits.dtype not in (torch.bfloat16, torch.float32) or not router_logits.is_cuda:
        raise RuntimeError("moe_route: router_logits must be a bf16 or fp32 [tokens, experts] tensor on the GPU")
    router_logits = router_logits.contiguous()
    T, E = router_logits.shape
    if not 1 <= top_k <= min(8, E) or E > 64:
        raise RuntimeError(f"Value error in moe_route: experts={E}, top_k={top_k}")
    dev = router_logits.device
    sel = torch.empty((T, top_k), dtype=torch.int32, device=dev)
    weight = torch.empty((T, top_k), dtype=torch.bfloat16, device=dev)
    seg = torch.empty(E + 1, dtype=torch.int32, device=dev)
    position = torch.empty(T * top_k, dtype=torch.int64, device=dev)
    tok = torch.empty(T * top_k, dtype=torch.int32, device=dev)
    ws = torch.empty(T * top_k, dtype=torch.bfloat16, device=dev)
    L = _lib.lib()
    nbytes = L.arcq_moe_route_workspace_bytes(T, E)
    work = torch.empty(max(nbytes, 4), dtype=torch.uint8, device=dev)
    with _on_device(router_logits):
        rc = L.arcq_moe_route(router_logits.data_ptr(), int(router_logits.dtype == torch.float32), T, E, top_k,
                              sel.data_ptr(), weight.data_ptr(), seg.data_ptr(), position.data_ptr(), tok.data_ptr(),
                              ws.data_ptr(), work.data_ptr(), work.numel(), _stream(router_logits))
    _lib.check(rc, "arcq_moe_route")
    return sel, weight, seg, position, tok, ws


def moe_combine(y, position, weight, tokens, top_k):
    """out[t] = sum over token t's experts (ascending expert number) of bf16(y[row] * weight[row]), partial sums
    rounded to bf16: the weighting and index_add_ of model/qMixtralLayer.py:466-471 in one launch.
    y bf16 [pairs, H] in expert-sorted order, position int64 [tokens * top_k] (row of y per (token, slot)),
    weight bf16 [pairs] in sorted order."""
    _require(y, "y", torch.bfloat16, 2)
    _require(position, "position", torch.int64, 1)
    _require(weight, "weight", torch.bfloat16, 1)
    pairs, H = y.shape
    if position.numel() != tokens * top_k or weight.numel() != pairs or H % 8 or not 1 <= top_k <= 8:
        raise RuntimeError(f"Value error in moe_combine: pairs={pairs}, H={H}, tokens={tokens}, top_k={top_k}")
    out = torch.empty((tokens, H), dtype=torch.bfloat16, device=y.device)
    with _on_device(y):
        rc = _lib.lib().arcq_moe_combine(y.data_ptr(), position.data_ptr(), weight.data_ptr(), tokens, H, top_k, pairs,
                                         out.data_ptr(), _stream(y))
    _lib.check(rc, "arcq_moe_combine")
    return out


def prepare_stream(device=None) -> None:
    """Allocate the library's scratch buffers for torch's current stream on `device` (arcq_prepare_stream).
    Needed once per stream before a capture on it: a captured call cannot allocate."""
    dev = torch.device("cuda", torch.cuda.current_device()) if device is None else torch.device(device)
    probe = torch.empty(0, device=dev)
    with _on_device(probe):
        _lib.check(_lib.lib().arcq_prepare_stream(_stream(probe)), "arcq_prepare_stream")


def release_stream(stream=None) -> None:
    """Free the library's scratch buffers of a torch stream (default: the current one) on its device
    (arcq_release_stream): for streams about to be destroyed.  Never while a graph captured on the stream may
    still be replayed -- the graph holds the buffers' addresses."""
    st = torch.cuda.current_stream() if stream is None else stream
    with torch.cuda.device(st.device):
        _lib.check(_lib.lib().arcq_release_stream(ctypes.c_void_p(st.cuda_stream)), "arcq_release_stream")


# The three INT4 KV-cache operators of the reference's module (kernels/src/bindings.cpp:576-578), so that a
# caller written against `agemm` (model/kv_cache.py:49-80) finds them here; same keyword arguments.
from .kv_cache import append_kv_i4, batch_decode_i4, init_kv_i4  # noqa: E402,F401


# ------------------------------------------------------------------------------------------
# helpers for tests and debugging (no counterpart in the reference)
# ------------------------------------------------------------------------------------------

def dequantize(Q, SF, *, fmt):
    """codes + scale bytes -> fp32 values q*s [rows, K'] on the device."""
    f = _fmt_id(fmt)
    _require(Q, "Q", torch.uint8, 2)
    _require(SF, "SF", torch.uint8)
    rows, Kp = Q.shape[0], 2 * Q.shape[1]
    out = torch.empty((rows, Kp), dtype=torch.float32, device=Q.device)
    with _on_device(Q):
        rc = _lib.lib().arcq_dequantize(Q.data_ptr(), SF.data_ptr(), rows, Kp, f, out.data_ptr(), _stream(Q))
    _lib.check(rc, "arcq_dequantize")
    return out


def check_index(reorder_index) -> None:
    """Raises RuntimeError unless reorder_index (int16, CUDA) is a permutation of 0..K-1."""
    _require(reorder_index, "reorder_index", torch.int16, 1)
    with _on_device(reorder_index):
        rc = _lib.lib().arcq_check_index(reorder_index.data_ptr(), reorder_index.numel(), _stream(reorder_index))
    _lib.check(rc, "arcq_check_index")


def unpack_codes(Q: torch.Tensor) -> torch.Tensor:
    """u8 [rows, K'/2] -> u8 [rows, K'] of 4-bit codes (element 2j was the low nibble of byte j)."""
    return torch.stack([Q & 15, Q >> 4], dim=-1).reshape(Q.shape[0], -1)


def scale_values(SF: torch.Tensor, *, fmt) -> torch.Tensor:
    """scale bytes -> fp32 values (NVFP4: (1+(b&7)/8)*2^((b>>3)-9); MXFP4: 2^(b-127))."""
    b = SF.to(torch.int32)
    if _fmt_id(fmt) == FORMATS["NVFP4"]:
        return torch.ldexp(1.0 + (b & 7).float() / 8.0, (b >> 3) - 9)
    return torch.ldexp(torch.ones_like(b, dtype=torch.float32), b - 127)
