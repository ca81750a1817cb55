"""Torch restatement of the reference's INT4 KV-cache arithmetic -- TEST INFRASTRUCTURE ONLY.

asym_quantize_and_pack_i4 follows model/kv_cache.py:23-37 op for op in eager mode, i.e. every
elementwise op rounds to the tensor dtype (fp16 or bf16); the reference wraps the function in
torch.jit.script, whose fuser may keep intermediates in fp32 on some devices -- that variant is not
restated, and no vectors of the reference pin either one: parity unpinned beyond the formula.
decode_attention is the textbook softmax(q K^T / sqrt(d)) V in fp64 over the dequantized cache
(n * scale - zero, model/kv_cache.py:39-43); the reference's kernel lives in a patched FlashInfer
that is not in its tree, so its internal precision is unknown: parity unpinned, tolerance in the tests.
"""
import torch


def asym_quantize_and_pack_i4(x: torch.Tensor):
    maxq = 15
    xmax = torch.amax(x, dim=-1, keepdim=True)
    xmin = torch.amin(x, dim=-1, keepdim=True)
    scale = (xmax - xmin).clamp(min=1e-5) / maxq
    zero = -xmin
    q = torch.clamp(torch.round((x + zero) / scale), 0, maxq)
    q = q.to(dtype=torch.uint8)
    q = q[..., 0::2] | (q[..., 1::2] << 4)
    return q, scale, zero


def unpack(q: torch.Tensor) -> torch.Tensor:
    return torch.stack((q & 0x0F, (q >> 4) & 0x0F), dim=-1).view(*q.shape[:-1], q.shape[-1] * 2)


def gather_sequence(pages, params, indptr, indices, last_page_offset, layer, b):
    """codes [len, heads, 128] (uint8 values 0..15) and (scale, zero) [len, heads, 2] fp64 of
    sequence b, for k and v"""
    page_size = pages.shape[4]
    ids = indices[indptr[b]:indptr[b + 1]].tolist()
    n = (len(ids) - 1) * page_size + int(last_page_offset[b]) if ids else 0
    out = []
    if not ids:                                    # a sequence without pages
        heads = pages.shape[3]
        empty = (torch.zeros(0, heads, 128, dtype=torch.uint8), torch.zeros(0, heads, 2, dtype=torch.float64))
        return [empty, empty]
    for kv in (0, 1):
        codes = torch.cat([unpack(pages[p, layer, kv]) for p in ids], dim=1)[:, :n]       # [heads, len, 128]
        par = torch.cat([params[p, layer, kv] for p in ids], dim=1)[:, :n].double()        # [heads, len, 2]
        out.append((codes.permute(1, 0, 2), par.permute(1, 0, 2)))
    return out


def decode_attention(q, pages, params, indptr, indices, last_page_offset, layer, sm_scale=None):
    """q [batch, q_heads, 128] -> fp64 [batch, q_heads, 128]"""
    batch, qh, d = q.shape
    heads = pages.shape[3]
    g = qh // heads
    sm_scale = d ** -0.5 if sm_scale is None else sm_scale
    out = torch.zeros(batch, qh, d, dtype=torch.float64)
    for b in range(batch):
        (kc, kp), (vc, vp) = gather_sequence(pages, params, indptr, indices, last_page_offset, layer, b)
        if kc.shape[0] == 0:
            continue
        k = kc.double() * kp[..., :1] - kp[..., 1:]                                          # [len, heads, 128]
        v = vc.double() * vp[..., :1] - vp[..., 1:]
        for h in range(qh):
            s = (k[:, h // g] @ q[b, h].double()) * sm_scale
            p = torch.softmax(s, dim=0)
            out[b, h] = p @ v[:, h // g]
    return out
