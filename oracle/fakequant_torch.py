"""Torch restatement of the reference's fake-quant path -- TEST INFRASTRUCTURE ONLY.

It issues the same torch tensor operations, in the same order and dtypes, as
model/quantize.py of the reference (cited per function), so that library-level
behaviour (torch.log2, torch.round, argmin's first-minimum rule, fp32 division)
is the reference's own.  On top of the values the reference returns, the block
routines also hand back what they were computed from -- grid index and block
scale -- so codes and scale bytes can be compared with the C oracle and the GPU.

This is also the "reference CPU fake-quant path" that bench.py times on the host.
"""
from __future__ import annotations

import numpy as np
import torch

E2M1_GRID = (-6.0, -4.0, -3.0, -2.0, -1.5, -1.0, -0.5, 0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0)
# grid position -> 4-bit code (sign<<3 | magnitude index), zero always 0x0
GRID_TO_CODE = torch.tensor([0xF, 0xE, 0xD, 0xC, 0xB, 0xA, 0x9, 0x0, 0x1, 0x2, 0x3, 0x4, 0x5, 0x6, 0x7],
                            dtype=torch.uint8)


def nearest_e2m1(t: torch.Tensor, chunk: int = 1 << 20):
    """quantize.py:14-22 -- argmin over |t[...,None] - grid|.  Returns (values, grid index).

    The reference materialises the whole [..., 15] difference tensor at once; here
    it is done in slices of ``chunk`` elements so a 4096x4096 input does not need
    1 GB -- the per-element arithmetic is identical.
    """
    grid = torch.tensor(E2M1_GRID, device=t.device, dtype=t.dtype)
    flat = t.reshape(-1)
    pos = torch.empty(flat.shape, dtype=torch.int64, device=t.device)
    for lo in range(0, flat.numel(), chunk):
        seg = flat[lo:lo + chunk]
        pos[lo:lo + chunk] = torch.argmin(torch.abs(seg.unsqueeze(-1) - grid), dim=-1)
    pos = pos.view(t.shape)
    return grid[pos], pos


def round_ue4m3(s: torch.Tensor) -> torch.Tensor:
    """quantize.py:40-49."""
    s = torch.clamp(s, min=2e-3, max=448.0)
    e = torch.floor(torch.log2(s + 1e-9))
    frac = s / (2 ** e) - 1.0
    frac_q = torch.round(frac * 8) / 8
    return (1 + frac_q) * (2 ** e)


def round_ue8m0(s: torch.Tensor) -> torch.Tensor:
    """quantize.py:54-59."""
    e = torch.ceil(torch.log2(s + 1e-9))
    e = torch.clamp(e, min=-127, max=127)
    return 2 ** e


def blockwise(t: torch.Tensor, fmt: str, detail: bool = False):
    """quantize.py:145-172 (NVFP4, groups of 16) / 174-201 (MXFP4, groups of 32)."""
    g = 16 if fmt == "NVFP4" else 32
    shape = t.shape
    pad = (g - shape[-1] % g) % g
    if pad:
        t = torch.nn.functional.pad(t, (0, pad))
    blk = t.reshape(-1, g)
    amax = torch.max(torch.abs(blk), dim=1, keepdim=True)[0]
    s = amax / 6.0
    s[s == 0] = 1e-9
    s = round_ue4m3(s) if fmt == "NVFP4" else round_ue8m0(s)
    q, pos = nearest_e2m1(blk / s)
    out = (q * s).view(t.shape)
    if pad:
        out = out[..., :-pad]
    out = out.view(shape)
    if detail:
        assert not pad
        return out, pos.view(shape), s.view(*shape[:-1], shape[-1] // g)
    return out


def tensor_scale(t: torch.Tensor, fmt: str) -> torch.Tensor:
    """quantize.py:290-295 / 317-322: signed max / 2688 for NVFP4, 1.0 otherwise."""
    if fmt == "NVFP4":
        return torch.max(t).to(torch.float32) / (448.0 * 6.0)
    return torch.tensor(1.0, device=t.device, dtype=torch.float32)


def fake_quantize_x(x: torch.Tensor, select_num: int, fmt: str):
    """quantize.py:314-343 with reorder_index = arange (the callers gather first,
    model/qLlamaLayer.py:84-86).  Returns what the reference returns:
    (values [M,K+S] in x.dtype, per-row amax, tensor scale)."""
    scale = tensor_scale(x, fmt)
    x32 = x.to(torch.float32) / scale
    row_amax = x32.abs().max(dim=1, keepdim=True)[0]
    if select_num == 0:
        return blockwise(x32, fmt).to(x.dtype), row_amax.to(x.dtype), scale.to(x.dtype)
    q = blockwise(x32, fmt)
    err = x32 - q
    q_err = blockwise(err[:, -select_num:], fmt)
    out = torch.cat([q, q_err], dim=1) * scale
    return out.to(x.dtype), row_amax.to(x.dtype), scale.to(x.dtype)


def fake_quantize_w(w: torch.Tensor, select_num: int, fmt: str):
    """quantize.py:287-312 with reorder_index = arange.  Values are NOT multiplied
    back by the tensor scale (quantize.py:311-312)."""
    scale = tensor_scale(w, fmt)
    w32 = w.to(torch.float32) / scale
    row_amax = w32.abs().max(dim=1, keepdim=True)[0]
    if select_num == 0:
        return blockwise(w32, fmt).to(w.dtype), row_amax.to(w.dtype), scale.to(w.dtype)
    q = torch.cat([blockwise(w32, fmt), blockwise(w32[:, -select_num:], fmt)], dim=1)
    return q.to(w.dtype), row_amax.to(w.dtype), scale.to(w.dtype)


def fake_linear(x, w, idx, select_num, fmt):
    """One ARC linear on the fake path: model/qLlamaLayer.py:79-86 (activation side),
    model/qLinearLayer.py:58,71 (weight side, F.linear).  For NVFP4 the weight's
    tensor scale is applied to the output, which the reference's real-kernel path
    does through alpha (qLinearLayer.py:69)."""
    ix = idx.to(torch.int64)
    qx, _, _ = fake_quantize_x(torch.index_select(x, 1, ix), select_num, fmt)
    qw, _, sw = fake_quantize_w(torch.index_select(w, 1, ix), select_num, fmt)
    y = torch.nn.functional.linear(qx, qw)
    return y * sw if fmt == "NVFP4" else y


# ---------------------------------------------------------------------------------------------
# codes / scale bytes from the same intermediates (for comparison with the C oracle and the GPU)
# ---------------------------------------------------------------------------------------------

def scale_bytes(s: torch.Tensor, fmt: str) -> np.ndarray:
    """Exact re-encoding of block scale values: NVFP4 ((e+9)<<3 | m8), MXFP4 (e+127)."""
    m, e = np.frexp(s.detach().cpu().numpy().astype(np.float64))  # s = m*2^e, m in [0.5,1)
    if fmt == "NVFP4":
        m8 = (m * 2 - 1) * 8
        assert np.all(m8 == np.round(m8)), "scale is not (1+k/8)*2^e"
        return (((e - 1 + 9) << 3) | m8.astype(np.int64)).astype(np.uint8)
    assert np.all(m == 0.5), "scale is not a power of two"
    return (e - 1 + 127).astype(np.uint8)


def pack_positions(pos: torch.Tensor) -> np.ndarray:
    c = GRID_TO_CODE[pos.cpu()].numpy()
    return (c[..., 0::2] | (c[..., 1::2] << 4)).astype(np.uint8)


def quantize_x_detailed(x: torch.Tensor, idx, select_num: int, fmt: str, gscale: float):
    """Same arithmetic as fake_quantize_x for a given tensor scale, returning
    packed codes [M,(K+S)/2], scale bytes [M,(K+S)/G] and values q*s [M,K+S]."""
    if idx is not None:
        x = torch.index_select(x, 1, idx.to(torch.int64))
    x32 = x.to(torch.float32) / torch.tensor(gscale, dtype=torch.float32)
    q, pos, s = blockwise(x32, fmt, detail=True)
    if select_num:
        err = x32 - q
        qe, pe, se = blockwise(err[:, -select_num:].contiguous(), fmt, detail=True)
        q, pos, s = torch.cat([q, qe], 1), torch.cat([pos, pe], 1), torch.cat([s, se], 1)
    return pack_positions(pos), scale_bytes(s, fmt), q


def quantize_w_detailed(w: torch.Tensor, idx, select_num: int, fmt: str, gscale: float):
    if idx is not None:
        w = torch.index_select(w, 1, idx.to(torch.int64))
    w32 = w.to(torch.float32) / torch.tensor(gscale, dtype=torch.float32)
    q, pos, s = blockwise(w32, fmt, detail=True)
    if select_num:
        qe, pe, se = blockwise(w32[:, -select_num:].contiguous(), fmt, detail=True)
        q, pos, s = torch.cat([q, qe], 1), torch.cat([pos, pe], 1), torch.cat([s, se], 1)
    return pack_positions(pos), scale_bytes(s, fmt), q


def hf_rmsnorm(x: torch.Tensor, gamma: torch.Tensor, eps: float) -> torch.Tensor:
    """benchmarks/modeling_arc.py:237-242 (the HF LlamaRMSNorm formula)."""
    h = x.to(torch.float32)
    var = h.pow(2).mean(-1, keepdim=True)
    h = h * torch.rsqrt(var + eps)
    return gamma * h.to(x.dtype)
