"""Layer-level callers of the ARC hot path: counterparts of the reference's Python layer code,
built on arcquant_amd.agemm (libarcq_hip.so) and nothing else.

    reorder_quantize_x      model/qLlamaLayer.py:73-86     (activation quantizer + NVFP4 tensor scale)
    QLinearLayer            model/qLinearLayer.py:30-81    (quantized weights, forward on the tuple)
    RMSNormQuant            benchmarks/modeling_arc.py:211-227 (fused RMSNorm -> quantize)
    LlamaMLP / LlamaAttention / LlamaDecoderLayer
                            model/qLlamaLayer.py:281-443, benchmarks/modeling_arc.py:80-330
    MixtralSparseMoeBlock   model/qMixtralLayer.py:388-543

The protocol between a quantizer and the linears that consume it is the reference's tuple
``(qx, scale_x, scale, bsz, q_len)`` (model/qLinearLayer.py:66): packed codes, block-scale bytes,
tensor scale, and the shape to restore.

What differs from the reference, on purpose:
  * nothing synchronises with the host.  The reference calls torch.cuda.synchronize() after every
    quantizer and every GEMM (model/qLlamaLayer.py:298, model/qLinearLayer.py:73) and turns the
    tensor scales into python floats (an implicit .item()); here the NVFP4 tensor scales stay
    0-dim device tensors that the kernels read themselves.
  * x / scale is done inside the quantizer in fp32 (model/quantize.py:330), not in bf16 before it
    (model/qLlamaLayer.py:76).
  * quant_type 'MXFP4' runs the real kernels too; the reference falls back to fake-quantized bf16
    tensors and F.linear for it (model/qLinearLayer.py:71).
  * the MoE block sorts tokens by expert on the device and runs every step of the expert MLPs as one
    grouped launch over all experts, with no read-back, instead of one torch.where (a host sync) and
    five launches per expert.
"""
from __future__ import annotations

import math
from typing import Optional

import torch
import torch.nn as nn
import torch.nn.functional as F

from . import agemm
from . import kv_cache as _kvc

NVFP4_RANGE = 448.0 * 6.0   # model/qLlamaLayer.py:74


def _tensor_scale(t: torch.Tensor, signed: bool) -> torch.Tensor:
    """NVFP4 tensor scale as a 0-dim fp32 device tensor.  Activations: max|x| / 2688
    (model/qLlamaLayer.py:74); weights: the signed max (model/qLinearLayer.py:26).  A zero tensor
    gets scale 1 (the reference would divide by zero)."""
    if not signed and t.is_cuda and t.dtype == torch.bfloat16 and t.dim() == 2 and t.stride(1) == 1 and \
            t.shape[1] % 8 == 0 and t.stride(0) % 8 == 0 and t.data_ptr() % 16 == 0:
        return agemm.tensor_scale(t, NVFP4_RANGE)               # one launch, same value
    m = (t.max() if signed else t.abs().max()).float()
    # tensor / tensor: an IEEE division.  Dividing by a python number would make torch multiply by
    # the rounded reciprocal on the GPU, one ulp away from the CPU result for many inputs.
    m = m / torch.full_like(m, NVFP4_RANGE)
    return torch.where(m == 0, torch.ones_like(m), m)


def reorder_quantize_x(x, reorder_index, select_num, quant_type="NVFP4"):
    """model/qLlamaLayer.py:79-86: x bf16 [tokens, K] -> (qx, scale_x, scale)."""
    if quant_type == "NVFP4":
        if x.is_cuda and x.dtype == torch.bfloat16 and x.dim() == 2 and x.is_contiguous():
            # scale and quantizer as one call: one launch and one pass over x while it fits the chip's LDS
            return agemm.reorder_quantize_x(x, reorder_index, select_num, fmt="NVFP4", global_scale="absmax")
        scale = _tensor_scale(x, signed=False)
        qx, scale_x = agemm.reorder_quantize_x(x, reorder_index, select_num, fmt="NVFP4", global_scale=scale)
        return qx, scale_x, scale
    qx, scale_x = agemm.reorder_quantize_x(x, reorder_index, select_num, fmt=quant_type)
    return qx, scale_x, 1.0


def swiglu_quantize_tokens(gate_up, inter, reorder_index, select_num, quant_type="NVFP4"):
    """act_fn(gate) * up -> quantized tuple in one fused pass over the output of a fused gate_up
    projection ([..., 2*inter]: gate first).  Same values as quantize_tokens(F.silu(gate) * up, ...),
    without the [tokens, inter] intermediate going through memory three times."""
    if gate_up.dim() == 3:
        bsz, q_len, _ = gate_up.shape
        flat = gate_up.reshape(bsz * q_len, -1)
    else:
        bsz, q_len = None, gate_up.shape[0]
        flat = gate_up
    gate, up = flat[:, :inter], flat[:, inter:]
    if quant_type == "NVFP4":
        qx, sfx, scale = agemm.swiglu_quantize_x(gate, up, reorder_index, select_num, fmt="NVFP4",
                                                 global_scale="absmax")
    else:
        qx, sfx = agemm.swiglu_quantize_x(gate, up, reorder_index, select_num, fmt=quant_type)
        scale = 1.0
    return qx, sfx, scale, bsz, q_len


def quantize_tokens(hidden_states, reorder_index, select_num, quant_type="NVFP4"):
    """[bsz, q_len, K] or [tokens, K] -> the 5-tuple a QLinearLayer takes."""
    if hidden_states.dim() == 3:
        bsz, q_len, _ = hidden_states.shape
        flat = hidden_states.reshape(bsz * q_len, -1)
    else:
        bsz, q_len = None, hidden_states.shape[0]
        flat = hidden_states
    qx, sfx, scale = reorder_quantize_x(flat.contiguous(), reorder_index, select_num, quant_type)
    return qx, sfx, scale, bsz, q_len


class QLinearLayer(nn.Module):
    """model/qLinearLayer.py:30-81.  Weights are quantized once at construction with the input
    channels reordered by `reorder_index` and the last `select_num` of them repeated."""

    def __init__(self, originalLayer: nn.Linear, select_num, reorder_index, out_reorder_index=None,
                 quant_type="NVFP4"):
        super().__init__()
        self.in_features = originalLayer.in_features
        self.out_features = originalLayer.out_features
        self.select_num = int(select_num)
        self.quant_type = quant_type
        w = originalLayer.weight.data
        if not w.is_cuda:
            raise RuntimeError("QLinearLayer quantizes on the GPU: move the layer to a cuda device first")
        w = w.to(torch.bfloat16).contiguous()
        idx = reorder_index.to(device=w.device, dtype=torch.int16).contiguous()
        if quant_type == "NVFP4":
            scale = _tensor_scale(w, signed=True)
            W, scale_w = agemm.reorder_quantize_w(w, idx, self.select_num, fmt="NVFP4", global_scale=scale)
        else:
            scale = torch.ones((), dtype=torch.float32, device=w.device)
            W, scale_w = agemm.reorder_quantize_w(w, idx, self.select_num, fmt=quant_type)
        self.register_buffer("W", W)
        self.register_buffer("scale_w", scale_w)
        self.register_buffer("scale", scale)
        if originalLayer.bias is not None:
            self.register_buffer("bias", originalLayer.bias.data.to(torch.bfloat16))
        else:
            self.bias = None

    @torch.no_grad()
    def forward(self, x, residual=None):
        """residual [..., out_features]: added to the output (in the GEMM's epilogue when the layer has
        no bias), same bits as `self(x) + residual`"""
        qx, scale_x, scale, bsz, q_len = x
        alpha = (scale, self.scale) if isinstance(scale, torch.Tensor) else (float(scale), self.scale)
        fused = residual is not None and self.bias is None
        y = agemm.matmul(qx, self.W, scale_x, self.scale_w, alpha, fmt=self.quant_type,
                         residual=residual.reshape(-1, self.out_features).contiguous() if fused else None)
        if self.bias is not None:
            y = y + self.bias
        if residual is not None and not fused:
            y = y + residual.reshape(-1, self.out_features)
        if bsz is not None:
            return y.reshape(bsz, q_len, -1)
        return y.reshape(q_len, -1)

    @torch.no_grad()
    def forward_swiglu(self, x, tensor_scale):
        """for a gate/up projection whose weight rows alternate gate, up: act_fn(gate) * up [tokens, out/2]
        straight from the GEMM's epilogue (and its NVFP4 tensor scale when asked), same bits as
        ``h = self(x); F.silu(h_gate) * h_up``"""
        qx, scale_x, scale, bsz, q_len = x
        alpha = (scale, self.scale) if isinstance(scale, torch.Tensor) else (float(scale), self.scale)
        return agemm.matmul_swiglu(qx, self.W, scale_x, self.scale_w, alpha, fmt=self.quant_type,
                                   tensor_scale=tensor_scale)


class RMSNormQuant(nn.Module):
    """benchmarks/modeling_arc.py:211-227: RMSNorm fused with the activation quantizer; returns the
    tuple directly (tensor scale 1, as the reference's op has none)."""

    def __init__(self, weight, eps, select_num, reorder_index, quant_type="NVFP4"):
        super().__init__()
        self.register_buffer("weight", weight.to(torch.bfloat16).contiguous())
        self.register_buffer("reorder_index", reorder_index.to(torch.int16).contiguous())
        self.variance_epsilon = float(eps)
        self.select_num = int(select_num)
        self.quant_type = quant_type

    @torch.no_grad()
    def forward(self, hidden_states):
        bsz, q_len, _ = hidden_states.shape
        flat = hidden_states.reshape(bsz * q_len, -1).contiguous()
        A, SFA = agemm.rmsnorm_quantize_x(flat, self.weight, self.variance_epsilon, self.reorder_index,
                                          self.select_num, fmt=self.quant_type)
        return A, SFA, 1.0, bsz, q_len


def _rotate_half(x):
    h = x.shape[-1] // 2
    return torch.cat((-x[..., h:], x[..., :h]), dim=-1)


def rotary_pos_emb(q, k, beg, base=10000.0):
    """benchmarks/modeling_arc.py:63-78: rotary embedding for positions beg .. beg+seqlen.
    beg may also be an int32 tensor [batch] of per-sequence positions (one new token each), read on the
    device -- what a decode step replayed from a captured graph needs."""
    dim, seqlen = q.shape[-1], q.shape[-2]
    inv_freq = 1.0 / (base ** (torch.arange(0, dim, 2, device=q.device).float() / dim))
    if isinstance(beg, torch.Tensor):
        t = beg.to(torch.float32)[:, None] + torch.arange(seqlen, device=q.device, dtype=torch.float32)[None, :]
        freqs = t[:, :, None] * inv_freq[None, None, :]                     # [batch, seqlen, dim/2]
        emb = torch.cat((freqs, freqs), dim=-1)[:, None]                    # [batch, 1, seqlen, dim]
    else:
        t = torch.arange(beg, beg + seqlen, device=q.device, dtype=torch.float32)
        freqs = torch.outer(t, inv_freq)
        emb = torch.cat((freqs, freqs), dim=-1)[None, None]
    cos, sin = emb.cos().to(q.dtype), emb.sin().to(q.dtype)
    return q * cos + _rotate_half(q) * sin, k * cos + _rotate_half(k) * sin


def _linear(out_features, in_features, std, device, gen):
    lin = nn.Linear(in_features, out_features, bias=False, device=device, dtype=torch.bfloat16)
    w = torch.randn(out_features, in_features, generator=gen) * std
    lin.weight.data.copy_(w.to(torch.bfloat16))
    return lin


class LlamaMLP(nn.Module):
    """SwiGLU MLP with gate and up projections fused into one [2*inter, hidden] linear
    (model/qLlamaLayer.py:380-443 with the fusion of benchmark configuration 4), followed by the fused
    SwiGLU -> quantize pass.  interleave=True instead interleaves the fused weight's rows (gate_0, up_0,
    gate_1, ...) and forms act_fn(gate) * up in the GEMM's epilogue, so that the [tokens, 2*inter] projection
    output never goes through memory: the same bits, but not the default here, because on one large GEMM with
    256x256 tiles (one workgroup per CU) the epilogue's activation arithmetic is exposed and costs more than
    the pass it saves (16384 tokens, MXFP4: 2.01 against 1.73 ms for GEMM + quantizer; NVFP4 3.95 against
    3.81).  The MoE block's grouped GEMMs run 128x128 tiles, two workgroups per CU, where one workgroup's
    epilogue hides behind the other's main loop: there it is the default and a gain."""

    def __init__(self, gate_up: nn.Linear, down: nn.Linear, select_num_in, select_num_down, in_index, down_index,
                 quant_type="NVFP4", interleave=False):
        super().__init__()
        self.inter = down.in_features
        kp = gate_up.in_features + int(select_num_in)
        self.interleaved = bool(interleave) and kp % 128 == 0 and kp >= 512 and self.inter % 8 == 0 and \
            gate_up.bias is None
        if self.interleaved:
            w = gate_up.weight.data
            il = nn.Linear(gate_up.in_features, 2 * self.inter, bias=False, device=w.device, dtype=w.dtype)
            il.weight.data.copy_(agemm.interleave_gate_up(w[:self.inter], w[self.inter:]))
            gate_up = il
        self.gate_up_proj = QLinearLayer(gate_up, select_num_in, in_index, quant_type=quant_type)
        self.down_proj = QLinearLayer(down, select_num_down, down_index, quant_type=quant_type)
        self.register_buffer("down_reorder_index", down_index.to(torch.int16))
        self.quant_type = quant_type

    @torch.no_grad()
    def forward(self, x, residual=None):
        """x: the tuple of the already quantized (normalised) hidden states; residual: added to the output"""
        sel = self.down_proj.select_num
        if getattr(self, "interleaved", False):
            nv = self.quant_type == "NVFP4"
            r = self.gate_up_proj.forward_swiglu(x, nv)
            t, scale = r if nv else (r, 1.0)
            qx, sfx = agemm.reorder_quantize_x(t, self.down_reorder_index, sel, fmt=self.quant_type,
                                               global_scale=scale if nv else None)
            return self.down_proj((qx, sfx, scale, x[3], x[4]), residual)
        gu = self.gate_up_proj(x)
        if self.inter <= 32736 and self.inter % 32 == 0:
            return self.down_proj(swiglu_quantize_tokens(gu, self.inter, self.down_reorder_index, sel, self.quant_type),
                                  residual)
        t = F.silu(gu[..., :self.inter]) * gu[..., self.inter:]
        return self.down_proj(quantize_tokens(t, self.down_reorder_index, sel, self.quant_type), residual)


class LlamaAttention(nn.Module):
    """Grouped-query attention with a fused qkv projection, bf16 SDPA and a preallocated bf16 KV
    cache (model/qLlamaLayer.py:207-378; the INT4 paged cache of model/kv_cache.py is a separate path)."""

    def __init__(self, qkv: nn.Linear, o: nn.Linear, num_heads, num_kv_heads, select_num_in, select_num_o, in_index,
                 o_index, quant_type="NVFP4"):
        super().__init__()
        self.num_heads, self.num_kv_heads = num_heads, num_kv_heads
        self.head_dim = o.in_features // num_heads
        self.qkv_proj = QLinearLayer(qkv, select_num_in, in_index, quant_type=quant_type)
        self.o_proj = QLinearLayer(o, select_num_o, o_index, quant_type=quant_type)
        self.register_buffer("o_reorder_index", o_index.to(torch.int16))
        self.quant_type = quant_type
        self._rope = None                    # cos / sin tables of the fused rotary embedding, built on first use

    @torch.no_grad()
    def forward(self, x, kv_cache=None, past_len=0, layer_idx=0, residual=None):
        """x: quantized hidden states (tuple); residual: added to the output.  kv_cache: None, or (k, v) bf16 [bsz, kv_heads, L, d]
        holding past_len valid positions (the new keys/values are written behind them), or an
        arcquant_amd.kv_cache.MultiLayerPagedKVCache4Bit (INT4 pages; decode attention then runs on
        the quantized cache, model/qLlamaLayer.py:334-338 with model/kv_cache.py:214-279)."""
        bsz, q_len = x[3], x[4]
        d, nh, nkv = self.head_dim, self.num_heads, self.num_kv_heads
        qkv = self.qkv_proj(x)
        if kv_cache is not None and not isinstance(kv_cache, tuple) and q_len == 1 and \
                not kv_cache._needs_init[layer_idx]:
            # decode over the INT4 pages: rotary embedding + quantized append in one launch, then attention
            out = kv_cache.decode_step(qkv.view(bsz, -1), nh, layer_idx).view(bsz, 1, nh * d)
            return self.o_proj(quantize_tokens(out, self.o_reorder_index, self.o_proj.select_num, self.quant_type),
                               residual)
        v = qkv[..., (nh + nkv) * d:].view(bsz, q_len, nkv, d).transpose(1, 2)
        if isinstance(past_len, int) and d == 128:
            # rotary embedding of q and k in one pass over the projection output (same values as
            # rotary_pos_emb below: every product and the sum rounded to bf16)
            need = past_len + q_len
            if self._rope is None or self._rope[0].shape[0] < need:
                self._rope = _kvc.rope_tables(max(need, 4096), d, qkv.dtype, qkv.device)
            q, k = _kvc.rope(qkv.view(bsz * q_len, -1), q_len, past_len, nh, nkv, *self._rope)
            q = q.view(bsz, q_len, nh, d).transpose(1, 2)
            k = k.view(bsz, q_len, nkv, d).transpose(1, 2)
        else:
            q = qkv[..., :nh * d].view(bsz, q_len, nh, d).transpose(1, 2)
            k = qkv[..., nh * d:(nh + nkv) * d].view(bsz, q_len, nkv, d).transpose(1, 2)
            q, k = rotary_pos_emb(q, k, past_len)
        if kv_cache is not None and not isinstance(kv_cache, tuple):
            r = kv_cache.update(k.transpose(1, 2), v.transpose(1, 2), layer_idx)
            if callable(r):                                   # decode: attention over the INT4 pages
                out = r(q.transpose(1, 2)).reshape(bsz, q_len, nh * d)
                return self.o_proj(quantize_tokens(out, self.o_reorder_index, self.o_proj.select_num,
                                                   self.quant_type), residual)
            kv_cache = None                                   # prefill: attend to the fresh keys / values
        if kv_cache is not None:
            kc, vc = kv_cache
            kc[:, :, past_len:past_len + q_len] = k
            vc[:, :, past_len:past_len + q_len] = v
            k, v = kc[:, :, :past_len + q_len], vc[:, :, :past_len + q_len]
        if q_len == 1:
            mask, causal = None, False
        elif isinstance(past_len, int) and past_len == 0:
            mask, causal = None, True
        elif isinstance(past_len, int):
            # a chunk of new tokens behind past_len cached ones: new token i sees the cache and the new
            # tokens up to itself (the lower-right aligned mask of model/qLlamaLayer.py's attention_mask)
            total = past_len + q_len
            mask = torch.ones(q_len, total, dtype=torch.bool, device=q.device).tril(diagonal=past_len)
            causal = False
        else:
            raise RuntimeError("a device-side past_len (graph replay) is for decode steps: one new token per sequence")
        out = F.scaled_dot_product_attention(q, k, v, attn_mask=mask, is_causal=causal, enable_gqa=(nkv != nh))
        out = out.transpose(1, 2).reshape(bsz, q_len, nh * d)
        return self.o_proj(quantize_tokens(out, self.o_reorder_index, self.o_proj.select_num, self.quant_type), residual)


class LlamaDecoderLayer(nn.Module):
    """One decoder layer: x + attn(norm_quant(x)), then + mlp(norm_quant(.)), with both RMSNorms
    fused into the quantizer (benchmarks/modeling_arc.py:262-330)."""

    def __init__(self, hidden, inter, num_heads, num_kv_heads, eps=1e-5, select_num=256, select_num_down=256,
                 quant_type="NVFP4", indices=None, seed=4, device="cuda"):
        super().__init__()
        gen = torch.Generator().manual_seed(seed)
        d = hidden // num_heads
        ident = lambda n: torch.arange(n, dtype=torch.int16, device=device)
        idx = indices or {}
        in_attn = idx.get("attn_in", ident(hidden))
        in_mlp = idx.get("mlp_in", ident(hidden))
        o_idx = idx.get("o_in", ident(hidden))
        down_idx = idx.get("down_in", ident(inter))
        self.linears = {   # the bf16 originals, kept for comparisons; not registered, not used in forward
            "qkv": _linear((num_heads + 2 * num_kv_heads) * d, hidden, 0.02, device, gen),
            "o": _linear(hidden, hidden, 0.02, device, gen),
            "gate_up": _linear(2 * inter, hidden, 0.02, device, gen),
            "down": _linear(hidden, inter, 0.02, device, gen),
        }
        g1 = (torch.rand(hidden, generator=gen) + 0.5).to(torch.bfloat16).to(device)
        g2 = (torch.rand(hidden, generator=gen) + 0.5).to(torch.bfloat16).to(device)
        self.input_layernorm = RMSNormQuant(g1, eps, select_num, in_attn, quant_type)
        self.post_attention_layernorm = RMSNormQuant(g2, eps, select_num, in_mlp, quant_type)
        self.self_attn = LlamaAttention(self.linears["qkv"], self.linears["o"], num_heads, num_kv_heads, select_num,
                                        select_num, in_attn, o_idx, quant_type)
        self.mlp = LlamaMLP(self.linears["gate_up"], self.linears["down"], select_num, select_num_down, in_mlp,
                            down_idx, quant_type)

    @torch.no_grad()
    def forward(self, hidden_states, kv_cache=None, past_len=0, layer_idx=0):
        # both residual adds happen in the epilogues of the o and down projections
        h = self.self_attn(self.input_layernorm(hidden_states), kv_cache, past_len, layer_idx, residual=hidden_states)
        return self.mlp(self.post_attention_layernorm(h), residual=h)


class SplitQLinear(nn.Module):
    """Several QLinearLayers over one quantized input, outputs concatenated along the features: q / k / v
    (or gate / up) kept as the reference keeps them, each with the tensor scale of its own weight
    (model/qLinearLayer.py:25-28), where the fused layers above have one scale for the stacked weight."""

    def __init__(self, parts):
        super().__init__()
        self.parts = nn.ModuleList(parts)
        self.select_num = parts[0].select_num
        self.out_features = sum(p.out_features for p in parts)

    @torch.no_grad()
    def forward(self, x, residual=None):
        y = torch.cat([p(x) for p in self.parts], dim=-1)
        return y if residual is None else y + residual


class LlamaRMSNorm(nn.Module):
    """HF's LlamaRMSNorm (benchmarks/modeling_arc.py:237-242): fp32 statistics, the normalised value and
    its product with the weight each rounded to the input dtype.  model/qLlamaLayer.py:180-197 keeps the
    model's own norm in front of the quantizer; RMSNormQuant is the fused form."""

    def __init__(self, weight, eps):
        super().__init__()
        self.register_buffer("weight", weight.to(torch.bfloat16).contiguous())
        self.variance_epsilon = float(eps)

    @torch.no_grad()
    def forward(self, hidden_states):
        dt = hidden_states.dtype
        h = hidden_states.to(torch.float32)
        h = h * torch.rsqrt(h.pow(2).mean(-1, keepdim=True) + self.variance_epsilon)
        return self.weight * h.to(dt)


CALIBRATION_KEY = "layers.{}.{}.{}.{}"     # model/qLlamaLayer.py:236: layer, block, projection, 'input'


def _calibrated(select_nums, reorder_index, i, block, proj, device):
    key = CALIBRATION_KEY.format(i, block, proj, "input")
    if key not in select_nums or key not in reorder_index:
        raise KeyError(f"calibration files hold no entry {key}")
    return int(select_nums[key]), reorder_index[key].to(device=device, dtype=torch.int16).contiguous()


class QLlamaAttention(LlamaAttention):
    """model/qLlamaLayer.py:207-378 with the reference's constructor arguments: the projections of the
    original attention block and the two calibration dicts (reorder_indices.py:88-97) keyed
    'layers.{i}.self_attn.{q,k,v,o}_proj.input'.  q, k and v stay separate QLinearLayers with their own
    NVFP4 tensor scales, so the weight codes are the reference's; they share one quantized input, taken
    with q_proj's entry as the reference does (model/qLlamaLayer.py:297)."""

    def __init__(self, q_proj, k_proj, v_proj, o_proj, num_heads, num_kv_heads, select_nums, reorder_index, i,
                 quant_type="NVFP4"):
        nn.Module.__init__(self)
        dev = q_proj.weight.device
        self.num_heads, self.num_kv_heads = num_heads, num_kv_heads
        self.head_dim = o_proj.in_features // num_heads
        self.layer_idx = i
        parts = []
        for name, lin in (("q_proj", q_proj), ("k_proj", k_proj), ("v_proj", v_proj)):
            sel, idx = _calibrated(select_nums, reorder_index, i, "self_attn", name, dev)
            parts.append(QLinearLayer(lin, sel, idx, quant_type=quant_type))
        self.qkv_proj = SplitQLinear(parts)
        self.q_proj, self.k_proj, self.v_proj = parts
        sel_q, idx_q = _calibrated(select_nums, reorder_index, i, "self_attn", "q_proj", dev)
        sel_o, idx_o = _calibrated(select_nums, reorder_index, i, "self_attn", "o_proj", dev)
        for p in parts[1:]:
            if p.select_num != sel_q:
                raise ValueError("k_proj / v_proj read q_proj's quantized input: their select_num must equal q_proj's")
        self.o_proj = QLinearLayer(o_proj, sel_o, idx_o, quant_type=quant_type)
        self.register_buffer("q_reorder_index", idx_q)
        self.register_buffer("o_reorder_index", idx_o)
        self.quant_type = quant_type
        self._rope = None


class QLlamaMLP(LlamaMLP):
    """model/qLlamaLayer.py:380-443: gate_proj and up_proj separate (own tensor scales), one quantized
    input taken with up_proj's entry (model/qLlamaLayer.py:429), keys 'layers.{i}.mlp.{gate,up,down}_proj.input'."""

    def __init__(self, gate_proj, up_proj, down_proj, select_nums, reorder_index, i, quant_type="NVFP4"):
        nn.Module.__init__(self)
        dev = gate_proj.weight.device
        self.inter = down_proj.in_features
        sel_g, idx_g = _calibrated(select_nums, reorder_index, i, "mlp", "gate_proj", dev)
        sel_u, idx_u = _calibrated(select_nums, reorder_index, i, "mlp", "up_proj", dev)
        sel_d, idx_d = _calibrated(select_nums, reorder_index, i, "mlp", "down_proj", dev)
        if sel_g != sel_u:
            raise ValueError("gate_proj reads up_proj's quantized input: their select_num must be equal")
        self.gate_proj = QLinearLayer(gate_proj, sel_g, idx_g, quant_type=quant_type)
        self.up_proj = QLinearLayer(up_proj, sel_u, idx_u, quant_type=quant_type)
        self.gate_up_proj = SplitQLinear([self.gate_proj, self.up_proj])
        self.down_proj = QLinearLayer(down_proj, sel_d, idx_d, quant_type=quant_type)
        self.register_buffer("up_reorder_index", idx_u)
        self.register_buffer("down_reorder_index", idx_d)
        self.layer_idx = i
        self.quant_type = quant_type


class QLlamaDecoderLayer(nn.Module):
    """model/qLlamaLayer.py:88-176 built the reference's way: from a decoder layer's own linears and norm
    weights plus the calibration dicts.  The norms stay the model's (torch) and every quantizer takes the
    NVFP4 tensor scale max|x|/2688 of its input, as model/qLlamaLayer.py:73-86 does; fuse_norm=True swaps
    in the fused RMSNorm -> quantize operator (tensor scale 1: benchmarks/modeling_arc.py:211-227)."""

    attention_class = QLlamaAttention
    mlp_class = QLlamaMLP

    def __init__(self, linears, norm_weights, eps, num_heads, num_kv_heads, select_nums, reorder_index, layer_idx,
                 quant_type="NVFP4", fuse_norm=False):
        super().__init__()
        self.self_attn = self.attention_class(linears["q_proj"], linears["k_proj"], linears["v_proj"], linears["o_proj"],
                                              num_heads, num_kv_heads, select_nums, reorder_index, layer_idx, quant_type)
        self.mlp = self.mlp_class(linears["gate_proj"], linears["up_proj"], linears["down_proj"], select_nums,
                                  reorder_index, layer_idx, quant_type)
        self.quant_type = quant_type
        self.layer_idx = layer_idx
        if fuse_norm:
            self.input_layernorm = RMSNormQuant(norm_weights[0], eps, self.self_attn.q_proj.select_num,
                                                self.self_attn.q_reorder_index, quant_type)
            self.post_attention_layernorm = RMSNormQuant(norm_weights[1], eps, self.mlp.up_proj.select_num,
                                                         self.mlp.up_reorder_index, quant_type)
        else:
            self.input_layernorm = LlamaRMSNorm(norm_weights[0], eps)
            self.post_attention_layernorm = LlamaRMSNorm(norm_weights[1], eps)
        self.fuse_norm = bool(fuse_norm)

    @torch.no_grad()
    def forward(self, hidden_states, kv_cache=None, past_len=0, layer_idx=None):
        li = self.layer_idx if layer_idx is None else layer_idx
        a, m = self.self_attn, self.mlp
        t = self.input_layernorm(hidden_states)
        if not self.fuse_norm:
            t = quantize_tokens(t, a.q_reorder_index, a.q_proj.select_num, self.quant_type)
        h = a(t, kv_cache, past_len, li, residual=hidden_states)
        t = self.post_attention_layernorm(h)
        if not self.fuse_norm:
            t = quantize_tokens(t, m.up_reorder_index, m.up_proj.select_num, self.quant_type)
        return m(t, residual=h)


class MixtralExpertMLP(nn.Module):
    """model/qMixtralLayer.py:466-543: w2(act(w1 x) * w3 x) on a ragged set of tokens.  w1 and w3 share their
    input and are one quantized linear whose rows alternate w1_0, w3_0, w1_1, ... (act(w1 x) * w3 x then comes
    out of that GEMM's epilogue); interleave=False stacks them [w1 | w3] with a separate SwiGLU -> quantize pass."""

    def __init__(self, w1: nn.Linear, w3: nn.Linear, w2: nn.Linear, select_num, in_index, w2_index, quant_type="NVFP4",
                 interleave=True):
        super().__init__()
        self.ffn = w1.out_features
        kp = w1.in_features + int(select_num)
        self.interleaved = bool(interleave) and kp % 128 == 0 and kp >= 512 and self.ffn % 8 == 0
        w13 = nn.Linear(w1.in_features, 2 * self.ffn, bias=False, device=w1.weight.device, dtype=torch.bfloat16)
        if self.interleaved:
            w13.weight.data.copy_(agemm.interleave_gate_up(w1.weight.data, w3.weight.data))
        else:
            w13.weight.data.copy_(torch.cat([w1.weight.data, w3.weight.data], dim=0))
        self.w13 = QLinearLayer(w13, select_num, in_index, quant_type=quant_type)   # w1 and w3 share their input
        self.w2 = QLinearLayer(w2, select_num, w2_index, quant_type=quant_type)
        self.register_buffer("w1_reorder_index", in_index.to(torch.int16))
        self.register_buffer("w2_reorder_index", w2_index.to(torch.int16))
        self.quant_type = quant_type

    @torch.no_grad()
    def forward(self, x):
        xq = quantize_tokens(x, self.w1_reorder_index, self.w13.select_num, self.quant_type)
        if self.interleaved:
            nv = self.quant_type == "NVFP4"
            r = self.w13.forward_swiglu(xq, nv)
            t, scale = r if nv else (r, 1.0)
            qx, sfx = agemm.reorder_quantize_x(t, self.w2_reorder_index, self.w2.select_num, fmt=self.quant_type,
                                               global_scale=scale if nv else None)
            return self.w2((qx, sfx, scale, None, t.shape[0]))
        h = self.w13(xq)
        if self.ffn <= 32736 and self.ffn % 32 == 0:
            return self.w2(swiglu_quantize_tokens(h, self.ffn, self.w2_reorder_index, self.w2.select_num,
                                                  self.quant_type))
        t = F.silu(h[:, :self.ffn]) * h[:, self.ffn:]
        return self.w2(quantize_tokens(t, self.w2_reorder_index, self.w2.select_num, self.quant_type))


class MixtralSparseMoeBlock(nn.Module):
    """model/qMixtralLayer.py:388-464: softmax router in fp32, top-k, renormalised weights, every
    token processed by its experts without capacity limits.

    The reference walks the experts in Python (one torch.where, i.e. one host synchronisation, and five
    launches per expert).  Here the (token, slot) pairs are sorted by expert on the device and each step of
    the expert MLP is one grouped launch over all experts -- tensor scales, quantizer, w1|w3 GEMM, fused
    SwiGLU quantizer, w2 GEMM -- reading the experts' row ranges from a device tensor: nothing is read back
    to the host.  The experts' quantized weights are stacked for that; each expert module keeps views of
    its part.  grouped=False keeps the per-expert loop (one read-back of the counts)."""

    def __init__(self, gate: nn.Linear, experts, top_k=2, grouped=True):
        super().__init__()
        self.gate = gate
        self.experts = nn.ModuleList(experts)
        self.num_experts = len(experts)
        self.top_k = top_k
        e0 = experts[0]
        same = all(ex.w13.W.shape == e0.w13.W.shape and ex.w2.W.shape == e0.w2.W.shape and
                   ex.interleaved == e0.interleaved and
                   ex.quant_type == e0.quant_type and ex.w13.select_num == e0.w13.select_num and
                   ex.w2.select_num == e0.w2.select_num and ex.w13.bias is None and ex.w2.bias is None
                   for ex in experts)
        kp13, kp2 = 2 * e0.w13.W.shape[1], 2 * e0.w2.W.shape[1]
        self.grouped = bool(grouped) and same and kp13 % 128 == 0 and kp2 % 128 == 0 and min(kp13, kp2) >= 512 and \
            e0.ffn <= 32736 and e0.ffn % 32 == 0 and e0.w13.in_features <= 32736
        if self.grouped:
            self.quant_type, self.ffn, self.interleaved = e0.quant_type, e0.ffn, e0.interleaved
            for name in ("w13", "w2"):
                W = torch.stack([getattr(ex, name).W for ex in experts])
                SF = torch.cat([getattr(ex, name).scale_w for ex in experts])
                sc = torch.stack([getattr(ex, name).scale.reshape(()) for ex in experts]).to(torch.float32)
                self.register_buffer(f"{name}_W", W)
                self.register_buffer(f"{name}_scale_w", SF)
                self.register_buffer(f"{name}_scale", sc)
                per = SF.numel() // len(experts)
                for i, ex in enumerate(experts):        # the experts keep views, not copies
                    lin = getattr(ex, name)
                    lin.W, lin.scale_w, lin.scale = W[i], SF[i * per:(i + 1) * per], sc[i]
            self.register_buffer("w1_reorder_index", torch.stack([ex.w1_reorder_index for ex in experts]))
            self.register_buffer("w2_reorder_index", torch.stack([ex.w2_reorder_index for ex in experts]))
            self.register_buffer("_expert_ids", torch.arange(self.num_experts, device=W.device))

    def _pair_ids(self, n, device):
        if getattr(self, "_pairs", None) is None or self._pairs.numel() != n or self._pairs.device != device:
            self._pairs = torch.arange(n, device=device)
        return self._pairs

    def _experts_grouped(self, xs, seg):
        """the expert MLPs over tokens sorted by expert: xs bf16 [pairs, hidden], seg int32 [E+1] on the device"""
        e0, qt = self.experts[0], self.quant_type
        nv = qt == "NVFP4"
        gs = agemm.grouped_tensor_scale(xs, seg, NVFP4_RANGE) if nv else None
        q, sf = agemm.grouped_reorder_quantize_x(xs, seg, self.w1_reorder_index, e0.w13.select_num, fmt=qt,
                                                 global_scales=gs)
        if self.interleaved:          # act(w1 x) * w3 x out of the first GEMM's epilogue, with its per-expert maxima
            r = agemm.grouped_matmul_swiglu(q, self.w13_W, sf, self.w13_scale_w, seg, gs, self.w13_scale if nv else None,
                                            fmt=qt, tensor_scale=nv)
            t, gs2 = r if nv else (r, None)
            q2, sf2 = agemm.grouped_reorder_quantize_x(t, seg, self.w2_reorder_index, e0.w2.select_num, fmt=qt,
                                                       global_scales=gs2)
        else:
            h = agemm.grouped_matmul(q, self.w13_W, sf, self.w13_scale_w, seg, gs, self.w13_scale if nv else None, fmt=qt)
            gate, up = h[:, :self.ffn], h[:, self.ffn:]
            if nv:
                q2, sf2, gs2 = agemm.grouped_swiglu_quantize_x(gate, up, seg, self.w2_reorder_index, e0.w2.select_num,
                                                               fmt=qt, global_scales="absmax")
            else:
                q2, sf2 = agemm.grouped_swiglu_quantize_x(gate, up, seg, self.w2_reorder_index, e0.w2.select_num, fmt=qt)
                gs2 = None
        return agemm.grouped_matmul(q2, self.w2_W, sf2, self.w2_scale_w, seg, gs2, self.w2_scale if nv else None, fmt=qt)

    @torch.no_grad()
    def forward(self, hidden_states, router_logits: Optional[torch.Tensor] = None):
        bsz, q_len, hid = hidden_states.shape
        x = hidden_states.reshape(-1, hid)
        if router_logits is None:
            router_logits = self.gate(x)
        fused_route = (x.dtype == torch.bfloat16 and self.num_experts <= 64 and self.top_k <= 8
                       and router_logits.dtype in (torch.bfloat16, torch.float32))
        if fused_route:
            # softmax, top-k, normalised weights and the expert-sorted bookkeeping in two launches
            sel, w, seg, position, tok, ws = agemm.moe_route(router_logits, self.top_k)
            flat_e = sel.reshape(-1)
        else:
            w = F.softmax(router_logits, dim=1, dtype=torch.float)
            w, sel = torch.topk(w, self.top_k, dim=-1)
            w = (w / w.sum(dim=-1, keepdim=True)).to(x.dtype)
            # (token, slot) pairs sorted by expert: one contiguous run of rows per expert
            flat_e = sel.reshape(-1)
            order = torch.argsort(flat_e, stable=True)
            tok = order // self.top_k
            ws = w.reshape(-1).index_select(0, order)
            seg = position = None
        xs = x.index_select(0, tok)
        if self.grouped:
            if seg is None:
                counts = (flat_e[:, None] == self._expert_ids[None, :]).sum(0)      # on the device: no read-back
                seg = torch.zeros(self.num_experts + 1, dtype=torch.int32, device=x.device)
                seg[1:] = torch.cumsum(counts, 0)
            y = self._experts_grouped(xs, seg)
            if hid % 8 == 0 and self.top_k <= 8:
                if position is None:
                    position = torch.empty_like(order)
                    position[order] = self._pair_ids(order.numel(), x.device)        # inverse of the sort
                return agemm.moe_combine(y, position, ws.contiguous(), x.shape[0], self.top_k).reshape(bsz, q_len, hid), \
                    router_logits
            out = torch.zeros_like(x)
            out.index_add_(0, tok, (y * ws[:, None]).to(x.dtype))
            return out.reshape(bsz, q_len, hid), router_logits
        out = torch.zeros_like(x)
        counts = torch.bincount(flat_e, minlength=self.num_experts).tolist()   # the one host read-back
        beg = 0
        for e, n in enumerate(counts):
            if n == 0:
                continue
            y = self.experts[e](xs[beg:beg + n].contiguous()) * ws[beg:beg + n, None]
            out.index_add_(0, tok[beg:beg + n], y.to(x.dtype))
            beg += n
        return out.reshape(bsz, q_len, hid), router_logits


def build_mixtral_block(hidden=4096, ffn=14336, num_experts=8, top_k=2, select_num=128, quant_type="NVFP4",
                        indices=None, seed=5, device="cuda", grouped=True, interleave=True):
    """Random-weight MoE block of benchmark configuration 5; `indices[e]` = (input index, w2 index)."""
    gen = torch.Generator().manual_seed(seed)
    gate = _linear(num_experts, hidden, 1.0 / math.sqrt(hidden), device, gen)
    experts = []
    for e in range(num_experts):
        w1 = _linear(ffn, hidden, 0.02, device, gen)
        w3 = _linear(ffn, hidden, 0.02, device, gen)
        w2 = _linear(hidden, ffn, 0.02, device, gen)
        if indices is not None:
            i_in, i_w2 = indices[e]
        else:
            i_in = torch.arange(hidden, dtype=torch.int16, device=device)
            i_w2 = torch.arange(ffn, dtype=torch.int16, device=device)
        experts.append(MixtralExpertMLP(w1, w3, w2, select_num, i_in, i_w2, quant_type, interleave=interleave))
        del w1, w3, w2
    return MixtralSparseMoeBlock(gate, experts, top_k, grouped=grouped)


class QQwen2Attention(QLlamaAttention):
    """model/qQwenLayer.py:205-357: Qwen2's attention block built the reference's way.  Same calibration keys
    ('layers.{i}.self_attn.{q,k,v,o}_proj.input', :227-249) and the same flow as the Llama block; what differs is
    the model: q_proj / k_proj / v_proj carry a bias, which QLinearLayer adds behind the GEMM
    (model/qLinearLayer.py:75-76), and the geometry (Qwen2.5-7B: hidden 3584, 28 query / 4 KV heads of 128)."""


class QQwen2MLP(QLlamaMLP):
    """model/qQwenLayer.py:360-425: keys 'layers.{i}.mlp.{gate,up,down}_proj.input' (:374-391).  The down
    projection's input is 18944 wide in Qwen2.5-7B: the fused SwiGLU -> quantize pass and the quantizers take
    rows of up to 32736 channels (the reference has dedicated kernels for exactly this width,
    kernels/src/reorder.cu:380-555, dispatch kernels/src/bindings.cpp:141-160)."""


class QQwen2DecoderLayer(QLlamaDecoderLayer):
    """model/qQwenLayer.py:88-176: the decoder layer from its own linears (q / k / v with bias), norm weights and
    the two calibration dicts."""

    attention_class = QQwen2Attention
    mlp_class = QQwen2MLP


MOE_KEY = "layers.{}.{}.{}.{}.{}.{}"     # model/qMixtralLayer.py:488: layer, 'block_sparse_moe', 'experts', expert, projection, 'input'


def _calibrated_expert(select_nums, reorder_index, layer_idx, moe_idx, proj, device):
    key = MOE_KEY.format(layer_idx, "block_sparse_moe", "experts", moe_idx, proj, "input")
    if key not in select_nums or key not in reorder_index:
        raise KeyError(f"calibration files hold no entry {key}")
    return int(select_nums[key]), reorder_index[key].to(device=device, dtype=torch.int16).contiguous()


class QMixtralAttention(QLlamaAttention):
    """model/qMixtralLayer.py:214-386: the four-part keys 'layers.{i}.self_attn.{q,k,v,o}_proj.input' (:246-272)
    and the flow of the Llama block."""


class QMixtralBlockSparseTop2MLP(nn.Module):
    """model/qMixtralLayer.py:474-543 with the reference's constructor arguments: one expert's w1 / w3 / w2 and the
    calibration dicts keyed 'layers.{i}.block_sparse_moe.experts.{e}.w{1,2,3}.input' (:488-508).  w1 and w3 stay
    separate QLinearLayers with their own NVFP4 tensor scales, so the weight codes are the reference's; both read
    the input quantized with w1's entry (:530), so w3's entry has to agree with it."""

    def __init__(self, w1: nn.Linear, w3: nn.Linear, w2: nn.Linear, select_nums, reorder_index, layer_idx, moe_idx,
                 quant_type="NVFP4"):
        super().__init__()
        dev = w1.weight.device
        self.ffn_dim, self.hidden_dim = w1.out_features, w1.in_features
        sel1, idx1 = _calibrated_expert(select_nums, reorder_index, layer_idx, moe_idx, "w1", dev)
        sel3, idx3 = _calibrated_expert(select_nums, reorder_index, layer_idx, moe_idx, "w3", dev)
        sel2, idx2 = _calibrated_expert(select_nums, reorder_index, layer_idx, moe_idx, "w2", dev)
        if sel3 != sel1 or not torch.equal(idx3, idx1):
            raise ValueError("w3 reads w1's quantized input: its select_num and reorder_index must equal w1's")
        self.w1 = QLinearLayer(w1, sel1, idx1, quant_type=quant_type)
        self.w3 = QLinearLayer(w3, sel3, idx3, quant_type=quant_type)
        self.w2 = QLinearLayer(w2, sel2, idx2, quant_type=quant_type)
        self.register_buffer("w1_reorder_index", idx1)
        self.register_buffer("w2_reorder_index", idx2)
        self.quant_type = quant_type

    @torch.no_grad()
    def forward(self, x):
        """x bf16 [tokens of this expert, hidden] (model/qMixtralLayer.py:523-543)"""
        xq = quantize_tokens(x, self.w1_reorder_index, self.w1.select_num, self.quant_type)
        gate, up = self.w1(xq), self.w3(xq)
        if self.ffn_dim <= 32736 and self.ffn_dim % 32 == 0:
            nv = self.quant_type == "NVFP4"
            r = agemm.swiglu_quantize_x(gate, up, self.w2_reorder_index, self.w2.select_num, fmt=self.quant_type,
                                        global_scale="absmax" if nv else None)
            return self.w2((r[0], r[1], r[2] if nv else 1.0, None, x.shape[0]))
        return self.w2(quantize_tokens(F.silu(gate) * up, self.w2_reorder_index, self.w2.select_num, self.quant_type))


class QMixtralSparseMoeBlock(MixtralSparseMoeBlock):
    """model/qMixtralLayer.py:388-471 built the reference's way: the router, every expert's (w1, w3, w2) and the
    calibration dicts; the experts become QMixtralBlockSparseTop2MLP (:419-420).  Routing, the expert-sorted rows
    and the weighted sum are MixtralSparseMoeBlock's; the expert MLPs run as grouped launches over all experts
    (w1 and w3 as two launches: each keeps the tensor scale of its own weight) when the experts agree on shapes
    and select_nums, else as the reference's loop over experts."""

    def __init__(self, gate: nn.Linear, experts, select_nums, reorder_index, i, quant_type="NVFP4", top_k=2,
                 grouped=True):
        nn.Module.__init__(self)
        self.gate = gate
        self.num_experts, self.top_k = len(experts), top_k
        self.experts = nn.ModuleList([QMixtralBlockSparseTop2MLP(w1, w3, w2, select_nums, reorder_index, i, j, quant_type)
                                      for j, (w1, w3, w2) in enumerate(experts)])
        e0 = self.experts[0]
        self.quant_type, self.ffn, self.interleaved = quant_type, e0.ffn_dim, False
        same = all(ex.w1.W.shape == e0.w1.W.shape and ex.w2.W.shape == e0.w2.W.shape and
                   ex.w1.select_num == e0.w1.select_num and ex.w2.select_num == e0.w2.select_num and
                   ex.w1.bias is None and ex.w3.bias is None and ex.w2.bias is None for ex in self.experts)
        kp1, kp2 = 2 * e0.w1.W.shape[1], 2 * e0.w2.W.shape[1]
        self.grouped = bool(grouped) and same and kp1 % 128 == 0 and kp2 % 128 == 0 and min(kp1, kp2) >= 512 and \
            e0.ffn_dim <= 32736 and e0.ffn_dim % 32 == 0 and e0.hidden_dim <= 32736
        if self.grouped:
            for name in ("w1", "w3", "w2"):
                W = torch.stack([getattr(ex, name).W for ex in self.experts])
                SF = torch.cat([getattr(ex, name).scale_w for ex in self.experts])
                sc = torch.stack([getattr(ex, name).scale.reshape(()) for ex in self.experts]).to(torch.float32)
                self.register_buffer(f"{name}_W", W)
                self.register_buffer(f"{name}_scale_w", SF)
                self.register_buffer(f"{name}_scale", sc)
                per = SF.numel() // self.num_experts
                for j, ex in enumerate(self.experts):        # the experts keep views, not copies
                    lin = getattr(ex, name)
                    lin.W, lin.scale_w, lin.scale = W[j], SF[j * per:(j + 1) * per], sc[j]
            self.register_buffer("w1_reorder_index", torch.stack([ex.w1_reorder_index for ex in self.experts]))
            self.register_buffer("w2_reorder_index", torch.stack([ex.w2_reorder_index for ex in self.experts]))
            self.register_buffer("_expert_ids", torch.arange(self.num_experts, device=W.device))

    def _experts_grouped(self, xs, seg):
        e0, qt = self.experts[0], self.quant_type
        nv = qt == "NVFP4"
        gs = agemm.grouped_tensor_scale(xs, seg, NVFP4_RANGE) if nv else None
        q, sf = agemm.grouped_reorder_quantize_x(xs, seg, self.w1_reorder_index, e0.w1.select_num, fmt=qt, global_scales=gs)
        gate = agemm.grouped_matmul(q, self.w1_W, sf, self.w1_scale_w, seg, gs, self.w1_scale if nv else None, fmt=qt)
        up = agemm.grouped_matmul(q, self.w3_W, sf, self.w3_scale_w, seg, gs, self.w3_scale if nv else None, fmt=qt)
        if nv:
            q2, sf2, gs2 = agemm.grouped_swiglu_quantize_x(gate, up, seg, self.w2_reorder_index, e0.w2.select_num, fmt=qt,
                                                           global_scales="absmax")
        else:
            q2, sf2 = agemm.grouped_swiglu_quantize_x(gate, up, seg, self.w2_reorder_index, e0.w2.select_num, fmt=qt)
            gs2 = None
        return agemm.grouped_matmul(q2, self.w2_W, sf2, self.w2_scale_w, seg, gs2, self.w2_scale if nv else None, fmt=qt)


class GraphedDecodeStep:
    """One decoder layer's decode step (one new token per sequence, INT4 paged KV cache) captured
    once as a HIP graph and replayed: the step is a chain of ~20 short launches whose issue cost on
    the host exceeds their run time.  Host-side cache bookkeeping happens in cache.begin_step() before
    the replay; the token positions for the rotary embedding are read from cache.positions on the
    device.  No memset nodes are recorded (buffers are cleared by fill kernels).

    The cache is shared by all layers of a model and must advance once per token, not once per layer:
    only the step with ``advance=True`` (the default for layer_idx 0) calls cache.begin_step(); the steps
    of the other layers run behind it on the advanced cache.  A caller that advances the cache itself
    passes advance=False everywhere.

    All steps of a device are captured on ONE side stream (``stream=`` overrides it): the library's scratch
    buffers belong to a (device, stream) pair and stay with a captured graph, and the steps of a model run one
    after the other, so they can share one set (about 40 MiB) instead of holding one per layer."""

    _capture_streams = {}

    @classmethod
    def capture_stream(cls, device):
        device = torch.device(device)
        key = (device.type, torch.cuda.current_device() if device.index is None else device.index)
        if key not in cls._capture_streams:
            cls._capture_streams[key] = torch.cuda.Stream(device=device)
        return cls._capture_streams[key]

    def __init__(self, layer: LlamaDecoderLayer, cache, batch, hidden, layer_idx=0, warmup=3, advance=None, stream=None):
        self.layer, self.cache, self.layer_idx = layer, cache, layer_idx
        self.advance = (layer_idx == 0) if advance is None else bool(advance)
        cache.external_step = True
        self.x = torch.zeros(batch, 1, hidden, dtype=torch.bfloat16, device=cache.device)
        side = self.capture_stream(cache.device) if stream is None else stream
        side.wait_stream(torch.cuda.current_stream())
        saved = list(cache.lengths)
        # warm-up and capture run on a cache advanced by one token (the slot a real step writes), whichever
        # layer this is; the cache is put back afterwards, and the slot is rewritten by the first real step
        with torch.cuda.stream(side):            # warm-up on a side stream, as graph capture requires
            agemm.prepare_stream(cache.device)   # the library's scratch buffers belong to a stream: the capture
            for _ in range(warmup):              # below runs on this same stream and finds them allocated
                cache.begin_step()
                self._run()
                self._rewind(saved)
        torch.cuda.current_stream().wait_stream(side)
        cache.begin_step()
        self.graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(self.graph, stream=side):
            self.y = self._run()
        self._rewind(saved)

    def _rewind(self, lengths):
        self.cache.lengths = list(lengths)
        self.cache._build_specs()

    def _run(self):
        return self.layer(self.x, self.cache, self.cache.positions, self.layer_idx)

    @torch.no_grad()
    def __call__(self, hidden_states):
        if self.advance:
            self.cache.begin_step()
        if hidden_states.data_ptr() != self.x.data_ptr():    # a caller may write into self.x directly
            self.x.copy_(hidden_states)
        self.graph.replay()
        return self.y
