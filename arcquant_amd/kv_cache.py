"""INT4 paged KV cache and decode attention: counterpart of the reference's model/kv_cache.py on
libarcq_hip.so.

    init_kv_i4 / append_kv_i4 / batch_decode_i4   the reference's three ops (model/kv_cache.py:49-80,
                                                  kernels/src/bindings.cpp:287-413), same keyword arguments
    quantize_append                               asym_quantize_and_pack_i4 (model/kv_cache.py:23-37)
                                                  fused with the append: one launch instead of ~15
    MultiLayerPagedKVCache4Bit                    the cache container (model/kv_cache.py:139-307)

Differences from the reference container: it is not a transformers.Cache subclass (that base class
changed across transformers versions); sequences may have different lengths (the reference raises
when page counts differ, model/kv_cache.py:286-287); the (scale, zero) pairs are stored in the
model dtype, fp16 or bf16 (the reference stores fp16 only); query heads may outnumber KV heads
(grouped-query attention), which the reference's kernel does not take.
"""
from __future__ import annotations

import ctypes
import functools
import math
from typing import Optional

import numpy as np
import torch

from . import _lib

_DTYPES = {torch.float16: 0, torch.bfloat16: 1}


_stream = _lib.stream_of


def _ptr(t):
    return ctypes.c_void_p(t.data_ptr()) if t is not None else None


def _container_dims(kv_data, kv_param):
    if kv_data.dim() != 6 or kv_param.dim() != 6 or kv_data.dtype != torch.uint8:
        raise RuntimeError("kv_data must be u8 [pages, layers, 2, heads, page_size, head_dim/2] and kv_param "
                           "[pages, layers, 2, heads, page_size, 2]")
    if not (kv_data.is_contiguous() and kv_param.is_contiguous() and kv_data.is_cuda and kv_param.is_cuda):
        raise RuntimeError("kv_data and kv_param must be contiguous CUDA tensors")
    if kv_param.dtype not in _DTYPES:
        raise RuntimeError("kv_param must be float16 or bfloat16")
    n_layers, heads, page_size = kv_data.shape[1], kv_data.shape[3], kv_data.shape[4]
    return n_layers, heads, page_size, kv_data.shape[5] * 2


def _check_table(kv_indptr, kv_indices, last_page_offset):
    for t in (kv_indptr, kv_indices, last_page_offset):
        if t.dtype != torch.int32 or not t.is_cuda or not t.is_contiguous():
            raise RuntimeError("kv_indptr, kv_indices and last_page_offset must be contiguous int32 CUDA tensors")


def quantize_append(kv_data, kv_param, kv_indptr, kv_indices, last_page_offset, k, v, layer_idx, seqlen_indptr=None,
                    max_new_tokens=None):
    """Quantize k, v [tokens, kv_heads, 128] (fp16 / bf16, the dtype of kv_param) per (token, head) as
    model/kv_cache.py:23-37 does and write them into their pages.  The page table describes the cache
    after the append.  seqlen_indptr int32 [batch+1]: offsets of each sequence's new tokens (prefill);
    None: one new token per sequence."""
    n_layers, heads, page_size, head_dim = _container_dims(kv_data, kv_param)
    _check_table(kv_indptr, kv_indices, last_page_offset)
    if k.dtype != kv_param.dtype or v.dtype != k.dtype or k.shape != v.shape or k.dim() != 3:
        raise RuntimeError("k and v must be [tokens, kv_heads, head_dim] tensors of kv_param's dtype")
    if k.shape[1] != heads or k.shape[2] != head_dim or not (k.is_contiguous() and v.is_contiguous()):
        raise RuntimeError("k / v do not match the cache's heads / head_dim or are not contiguous")
    batch = last_page_offset.numel()
    if seqlen_indptr is None:
        if k.shape[0] != batch:
            raise RuntimeError("without seqlen_indptr there must be exactly one new token per sequence")
        max_new_tokens = 1
    elif max_new_tokens is None:
        max_new_tokens = int(k.shape[0])
    with _lib.on_device_of(k):
        rc = _lib.lib().arcq_kv_append_i4(_ptr(k), _ptr(v), _DTYPES[k.dtype], batch, _ptr(seqlen_indptr),
                                          int(max_new_tokens), _ptr(kv_data), _ptr(kv_param), _ptr(kv_indptr),
                                          _ptr(kv_indices), _ptr(last_page_offset), n_layers, int(layer_idx), heads,
                                          page_size, head_dim, _stream(k))
    _lib.check(rc, "arcq_kv_append_i4")


def rope_tables(max_positions, head_dim, dtype, device, base=10000.0):
    """cos / sin [max_positions, head_dim/2] in `dtype`, computed as the rotary embedding of the layers
    computes them per step (fp32 position x inverse frequency, cos / sin in fp32, cast)."""
    inv_freq = 1.0 / (base ** (torch.arange(0, head_dim, 2, device=device).float() / head_dim))
    freqs = torch.outer(torch.arange(max_positions, device=device, dtype=torch.float32), inv_freq)
    return freqs.cos().to(dtype).contiguous(), freqs.sin().to(dtype).contiguous()


def rope(qkv, q_len, pos0, num_qo_heads, num_kv_heads, cos_table, sin_table):
    """Rotary embedding of the query and key heads of a fused qkv projection output [tokens, (q + 2 kv
    heads) * 128] (rows may be strided); token t sits at position pos0 + t % q_len.  Returns the rotated
    q [tokens, num_qo_heads, 128] and k [tokens, num_kv_heads, 128]; same values as torch's
    q * cos + rotate_half(q) * sin in qkv's dtype (model/qLlamaLayer.py:30-64)."""
    if qkv.dim() != 2 or qkv.dtype not in _DTYPES or qkv.stride(1) != 1 or not qkv.is_cuda:
        raise RuntimeError("qkv must be a 2-D fp16 / bf16 CUDA tensor with unit stride along its last dimension")
    tokens = qkv.shape[0]
    if qkv.shape[1] < (num_qo_heads + 2 * num_kv_heads) * 128 or tokens % q_len:
        raise RuntimeError("qkv does not match the head counts or q_len")
    for t in (cos_table, sin_table):
        if t.dtype != qkv.dtype or t.dim() != 2 or t.shape[1] != 64 or not t.is_contiguous():
            raise RuntimeError("cos / sin tables must be contiguous [positions, 64] of qkv's dtype")
    q = torch.empty(tokens, num_qo_heads, 128, dtype=qkv.dtype, device=qkv.device)
    k = torch.empty(tokens, num_kv_heads, 128, dtype=qkv.dtype, device=qkv.device)
    ld = qkv.stride(0) if tokens > 1 else qkv.shape[1]
    with _lib.on_device_of(qkv):
        rc = _lib.lib().arcq_rope(_ptr(qkv), int(ld), _DTYPES[qkv.dtype], tokens, int(q_len), int(pos0),
                                  int(num_qo_heads), int(num_kv_heads), 128, _ptr(cos_table), _ptr(sin_table),
                                  int(cos_table.shape[0]), _ptr(q), _ptr(k), _stream(qkv))
    _lib.check(rc, "arcq_rope")
    return q, k


def rope_quantize_append(qkv, num_qo_heads, cos_table, sin_table, positions, kv_data, kv_param, kv_indptr, kv_indices,
                         last_page_offset, layer_idx, q_out=None):
    """One decode step between the qkv projection and the attention (model/qLlamaLayer.py:316-327):
    rotary embedding of the new token's query and key heads, quantized append of its key and value heads.
    qkv [batch, (num_qo_heads + 2 * kv_heads) * 128] (rows may be strided); returns the rotated queries
    [batch, num_qo_heads, 128].  The page table describes the cache after the append."""
    n_layers, heads, page_size, head_dim = _container_dims(kv_data, kv_param)
    _check_table(kv_indptr, kv_indices, last_page_offset)
    batch = last_page_offset.numel()
    if qkv.dim() != 2 or qkv.shape[0] != batch or qkv.dtype != kv_param.dtype or qkv.stride(1) != 1:
        raise RuntimeError("qkv must be [batch, (query heads + 2 * kv heads) * head_dim] in kv_param's dtype")
    if qkv.shape[1] < (num_qo_heads + 2 * heads) * head_dim:
        raise RuntimeError("qkv rows are too short for the head counts")
    for t in (cos_table, sin_table):
        if t.dtype != qkv.dtype or t.dim() != 2 or t.shape[1] != head_dim // 2 or not t.is_contiguous():
            raise RuntimeError("cos / sin tables must be contiguous [positions, head_dim/2] of qkv's dtype")
    if positions.dtype != torch.int32 or positions.numel() != batch or not positions.is_cuda:
        raise RuntimeError("positions must be an int32 CUDA tensor [batch]")
    if q_out is None:
        q_out = torch.empty(batch, num_qo_heads, head_dim, dtype=qkv.dtype, device=qkv.device)
    with _lib.on_device_of(qkv):
        rc = _lib.lib().arcq_rope_kv_append_i4(_ptr(qkv), int(qkv.stride(0)), _DTYPES[qkv.dtype], batch,
                                               int(num_qo_heads), _ptr(cos_table), _ptr(sin_table),
                                               int(cos_table.shape[0]), _ptr(positions), _ptr(q_out), _ptr(kv_data),
                                               _ptr(kv_param), _ptr(kv_indptr), _ptr(kv_indices),
                                               _ptr(last_page_offset), n_layers, int(layer_idx), heads, page_size,
                                               head_dim, _stream(qkv))
    _lib.check(rc, "arcq_rope_kv_append_i4")
    return q_out


def _store(kv_data, kv_param, kv_indptr, kv_indices, last_page_offset, k, v, k_param, v_param, seqlen_indptr, layer_idx):
    n_layers, heads, page_size, head_dim = _container_dims(kv_data, kv_param)
    _check_table(kv_indptr, kv_indices, last_page_offset)
    if k.dtype != torch.uint8 or v.dtype != torch.uint8 or k.shape != v.shape or k.dim() != 3:
        raise RuntimeError("k and v must be u8 [tokens, kv_heads, head_dim/2] (already quantized)")
    if k.shape[1] != heads or k.shape[2] * 2 != head_dim:
        raise RuntimeError("k / v do not match the cache's heads / head_dim")
    for p in (k_param, v_param):
        if p.dtype != kv_param.dtype or tuple(p.shape) != (k.shape[0], heads, 2):
            raise RuntimeError("k_param / v_param must be [tokens, kv_heads, 2] of kv_param's dtype")
    k, v, k_param, v_param = (t.contiguous() for t in (k, v, k_param, v_param))
    batch = last_page_offset.numel()
    max_new = 1 if seqlen_indptr is None else int(k.shape[0])
    with _lib.on_device_of(k):
        rc = _lib.lib().arcq_kv_store_i4(_ptr(k), _ptr(v), _ptr(k_param), _ptr(v_param), batch, _ptr(seqlen_indptr),
                                         max_new, _ptr(kv_data), _ptr(kv_param), _ptr(kv_indptr), _ptr(kv_indices),
                                         _ptr(last_page_offset), n_layers, int(layer_idx), heads, page_size, head_dim,
                                         _stream(k))
    _lib.check(rc, "arcq_kv_store_i4")


def init_kv_i4(kv_data, kv_param, kv_indptr, kv_indices, last_page_offset, k, v, k_param, v_param, seqlen_indptr,
               layer_idx):
    """model/kv_cache.py:49-60: prefill rows, already quantized, into their pages."""
    _store(kv_data, kv_param, kv_indptr, kv_indices, last_page_offset, k, v, k_param, v_param, seqlen_indptr, layer_idx)


def append_kv_i4(kv_data, kv_param, kv_indptr, kv_indices, last_page_offset, k, v, k_param, v_param, layer_idx):
    """model/kv_cache.py:63-73: one already quantized token per sequence."""
    _store(kv_data, kv_param, kv_indptr, kv_indices, last_page_offset, k, v, k_param, v_param, None, layer_idx)


def batch_decode_i4(o, q, kv_data, kv_param, kv_indptr, kv_indices, last_page_offset, layer_idx, sm_scale=None):
    """model/kv_cache.py:75-80: o[b, h] = softmax(q[b, h] K_b^T / sqrt(head_dim)) V_b over the INT4 pages.
    q, o: [batch, query heads, 128] in kv_param's dtype; query heads = 1, 2 or 4 x KV heads."""
    n_layers, heads, page_size, head_dim = _container_dims(kv_data, kv_param)
    _check_table(kv_indptr, kv_indices, last_page_offset)
    if q.dim() != 3 or o.shape != q.shape or q.dtype != kv_param.dtype or o.dtype != q.dtype:
        raise RuntimeError("q and o must be [batch, heads, head_dim] tensors of kv_param's dtype")
    if not (q.is_contiguous() and o.is_contiguous()) or q.shape[2] != head_dim:
        raise RuntimeError("q / o must be contiguous with the cache's head_dim")
    if sm_scale is None:
        sm_scale = 1.0 / math.sqrt(head_dim)
    with _lib.on_device_of(q):
        rc = _lib.lib().arcq_kv_decode_i4(_ptr(o), _ptr(q), _DTYPES[q.dtype], q.shape[0], q.shape[1], _ptr(kv_data),
                                          _ptr(kv_param), _ptr(kv_indptr), _ptr(kv_indices), _ptr(last_page_offset),
                                          n_layers, int(layer_idx), heads, page_size, head_dim, float(sm_scale),
                                          _stream(q))
    _lib.check(rc, "arcq_kv_decode_i4")
    return o


class MultiLayerPagedKVCache4Bit:
    """model/kv_cache.py:139-307.  update() during prefill stores the new keys / values and returns
    them unchanged (prefill attention runs on them directly); during decode it appends the one new
    token per sequence and returns a callable that maps the query [batch, 1, heads, 128] to the
    attention output, as the reference's does."""

    def __init__(self, batch_size, page_size, max_seq_len, device, n_layers, num_heads, head_dim,
                 dtype=torch.float16):
        if head_dim != 128:
            raise ValueError("head_dim must be 128")
        self.batch_size, self.page_size, self.max_seq_len = batch_size, page_size, max_seq_len
        self.device, self.n_layers, self.num_heads, self.head_dim = device, n_layers, num_heads, head_dim
        max_page_cnt = self.page_cnt_from_length(max_seq_len)
        self.pages = torch.zeros((max_page_cnt * batch_size, n_layers, 2, num_heads, page_size, head_dim // 2),
                                 dtype=torch.uint8, device=device)
        self.scales = torch.zeros((max_page_cnt * batch_size, n_layers, 2, num_heads, page_size, 2), dtype=dtype,
                                  device=device)
        self._needs_init = [True] * n_layers
        self.lengths = [0] * batch_size          # host mirror of the sequence lengths
        # The page table lives in tensors allocated once and updated in place, so that a captured HIP
        # graph of a decode step keeps reading the right addresses.  `positions` holds the position of
        # each sequence's newest token (for rotary embeddings inside a graph).
        mk = lambda n: torch.zeros(n, dtype=torch.int32, device=device)
        self._indptr, self._indices = mk(batch_size + 1), mk(max(1, max_page_cnt * batch_size))
        self._counters = mk(2 * batch_size)       # last_page_offset | positions: one add advances both
        self._last, self.positions = self._counters[:batch_size], self._counters[batch_size:]
        self._specs = None
        self._rope = None                         # cos / sin tables of decode_step, built on first use
        self.external_step = False                # True: the caller advances the cache with begin_step()

    def page_cnt_from_length(self, length):
        return (length + self.page_size - 1) // self.page_size

    @property
    def length(self):
        return max(self.lengths)

    @property
    def seen_tokens(self):
        return self.length

    def get_seq_length(self, layer_idx: Optional[int] = 0) -> int:
        return self.length

    def _build_specs(self):
        """page table for the current lengths: sequence b owns pages b, b + batch, b + 2*batch, ...
        (model/kv_cache.py:293-296); built on the host with numpy, one small upload per array"""
        ps, nb = self.page_size, self.batch_size
        lens = np.asarray(self.lengths, dtype=np.int64)
        cnt = (lens + ps - 1) // ps
        maxc = int(cnt.max()) if nb else 0
        if maxc * nb > self.pages.shape[0]:
            raise ValueError(f"KV cache capacity exceeded: {int(lens.max())} tokens, built for {self.max_seq_len}")
        indptr = np.zeros(nb + 1, dtype=np.int32)
        indptr[1:] = np.cumsum(cnt)
        grid = np.arange(maxc, dtype=np.int64)[None, :] * nb + np.arange(nb, dtype=np.int64)[:, None]
        indices = grid[np.arange(maxc)[None, :] < cnt[:, None]].astype(np.int32)
        off = lens % ps
        last = np.where((lens != 0) & (off == 0), ps, off).astype(np.int32)
        self._indptr.copy_(torch.from_numpy(indptr))
        if indices.size:
            self._indices[:indices.size].copy_(torch.from_numpy(indices))
        self._last.copy_(torch.from_numpy(last))
        self.positions.copy_(torch.from_numpy(np.maximum(lens - 1, 0).astype(np.int32)))
        self._specs = {"kv_data": self.pages, "kv_param": self.scales, "kv_indptr": self._indptr,
                       "kv_indices": self._indices, "last_page_offset": self._last}
        return self._specs

    def _advance_one_token(self):
        """every sequence grows by one token: unless one of them starts a new page, only
        last_page_offset changes, and that is one in-place add on the device"""
        ps = self.page_size
        new_page = any(n % ps == 0 for n in self.lengths)        # length n -> n + 1 opens page n // ps
        self.lengths = [n + 1 for n in self.lengths]
        if new_page or self._specs is None:
            self._build_specs()
        else:
            self._counters.add_(1)

    def begin_step(self):
        """Advance every sequence by one token ahead of a decode step whose launches are replayed from
        a captured graph: the host-side bookkeeping happens here, the graph only launches kernels.
        Use with external_step = True."""
        self._advance_one_token()

    def get_cache_specs_for_flash_infer(self, attention_mask=None):
        return self._specs if self._specs is not None else self._build_specs()

    def update(self, key_states, value_states, layer_idx, cache_kwargs=None):
        """key_states / value_states: [batch, new tokens, kv heads, 128]"""
        b_sz, added, heads, head_dim = key_states.shape
        assert b_sz == self.batch_size and heads == self.num_heads and head_dim == self.head_dim
        mask = (cache_kwargs or {}).get("attention_mask")
        if self._needs_init[layer_idx]:
            if mask is not None:
                new = [int(n) for n in mask.sum(dim=-1).tolist()]     # valid tokens per sequence
            else:
                new = [added] * b_sz
            if layer_idx == 0:
                self.lengths = [a + n for a, n in zip(self.lengths, new)]
                self._build_specs()
            self._needs_init[layer_idx] = False
            k = key_states.reshape(b_sz * added, heads, head_dim)
            v = value_states.reshape(b_sz * added, heads, head_dim)
            if mask is not None:
                keep = mask.reshape(-1).bool()
                k, v = k[keep], v[keep]
            offs = [0]
            for n in new:
                offs.append(offs[-1] + n)
            seq_indptr = torch.tensor(offs, dtype=torch.int32, device=self.device)
            quantize_append(k=k.contiguous(), v=v.contiguous(), layer_idx=layer_idx, seqlen_indptr=seq_indptr,
                            max_new_tokens=max(new), **self._specs)
            return key_states, value_states
        assert added == 1
        if layer_idx == 0 and not self.external_step:
            self._advance_one_token()
        quantize_append(k=key_states.reshape(b_sz, heads, head_dim).contiguous(),
                        v=value_states.reshape(b_sz, heads, head_dim).contiguous(), layer_idx=layer_idx, **self._specs)
        return functools.partial(self._attend, layer_idx=layer_idx)

    def decode_step(self, qkv, num_qo_heads, layer_idx):
        """The decode step of one layer from its fused qkv projection [batch, (q + 2 kv heads) * 128]:
        rotary embedding at the positions of the new tokens, quantized append, attention over the pages.
        Returns [batch, num_qo_heads * 128]."""
        assert not self._needs_init[layer_idx], "decode_step comes after the prefill of this layer"
        if layer_idx == 0 and not self.external_step:
            self._advance_one_token()
        if self._rope is None:
            self._rope = rope_tables(self.pages.shape[0] // self.batch_size * self.page_size, self.head_dim,
                                     self.scales.dtype, self.device)
        q = rope_quantize_append(qkv, num_qo_heads, self._rope[0], self._rope[1], self.positions,
                                 layer_idx=layer_idx, **self._specs)
        out = torch.empty_like(q)
        batch_decode_i4(out, q, layer_idx=layer_idx, **self._specs)
        return out.view(q.shape[0], -1)

    def _attend(self, q, layer_idx):
        batch, q_len, q_heads, head_dim = q.shape
        assert q_len == 1
        q3 = q.reshape(batch, q_heads, head_dim).contiguous()
        out = torch.empty_like(q3)
        batch_decode_i4(out, q3, layer_idx=layer_idx, **self._specs)
        return out.unsqueeze(1)
