"""Calibration artefacts of ARCQuant: per-linear channel orders and residual-channel counts.

The reference derives both offline (reorder_indices.py:40-97) and stores them as two torch-saved
dicts keyed by '<module path>.input', e.g. 'layers.3.self_attn.q_proj.input':

    *_reorder_index_*.pt   name -> int64 tensor [K]: channels sorted by calibration statistic,
                           ascending, so that outliers come last (utilize.py:22-64)
    *_select_num_*.pt      name -> int: how many of the last channels get a residual,
                           a multiple of 64 (utilize.py:537-551)

This module reads and writes that format (tensor-only loading: nothing in a file is executed) and
restates the two rules that produce the entries; collecting the activation statistics from a model
is calibration proper and stays outside the hot path.
"""
from __future__ import annotations

import math
from typing import Dict

import torch

NAME_TEMPLATE = "layers.{}.{}.{}.input"   # layer index, block ('self_attn' / 'mlp'), projection
# a Mixtral expert's linears (model/qMixtralLayer.py:488): layer index, expert index, projection ('w1' / 'w2' / 'w3')
MOE_NAME_TEMPLATE = "layers.{}.block_sparse_moe.experts.{}.{}.input"


def reorder_index_from_stat(stat: torch.Tensor) -> torch.Tensor:
    """utilize.py:40-46: channel order = argsort of the per-channel statistic, ascending.  Equal
    statistics keep their original order here (the reference leaves ties to torch.sort)."""
    if stat.dim() != 1:
        raise ValueError("the per-channel statistic must be 1-dimensional")
    return torch.sort(stat, descending=False, stable=True).indices


def is_permutation(idx: torch.Tensor) -> bool:
    """utilize.py:24-38"""
    if not torch.is_tensor(idx) or idx.dim() != 1 or idx.dtype.is_floating_point:
        return False
    n = idx.numel()
    return n == 0 or torch.equal(torch.sort(idx).values, torch.arange(n, device=idx.device, dtype=idx.dtype))


def select_num_from_activations(keys: torch.Tensor, granularity: int = 64) -> int:
    """utilize.py:544-551.  keys: [tokens, K] calibration activations of one linear's input (any
    channel order: the count does not depend on it).  A value counts as an outlier when it exceeds
    one eighth of its token's maximum -- signed values and a signed maximum, as in the reference --
    and select_num = ceil(K * outlier fraction / 64) * 64, at most K."""
    keys = keys.reshape(-1, keys.shape[-1])
    in_features = keys.shape[-1]
    threshold = keys.max(dim=-1, keepdim=True)[0] * 0.125
    ratio = (keys > threshold).sum() / keys.numel()
    n = math.ceil(in_features * float(ratio) / granularity) * granularity
    return min(n, in_features)


def average_bits(in_features: int, select_num: int) -> float:
    """utilize.py:556: 4 code bits + 8/16 scale bits per element, residual channels counted twice"""
    return 4.5 * (in_features + select_num) / in_features


def save_reorder_index(path: str, index: Dict[str, torch.Tensor]) -> None:
    for k, v in index.items():
        if not is_permutation(v):
            raise ValueError(f"{k}: not a permutation")
    torch.save({k: v.to(torch.int64).cpu() for k, v in index.items()}, path)


def save_select_num(path: str, select_num: Dict[str, int]) -> None:
    torch.save({k: int(v) for k, v in select_num.items()}, path)


def load_reorder_index(path: str) -> Dict[str, torch.Tensor]:
    d = torch.load(path, map_location="cpu", weights_only=True)
    for k, v in d.items():
        if not is_permutation(v):
            raise ValueError(f"{path}: entry {k} is not a permutation of its channels")
    return d


def load_select_num(path: str) -> Dict[str, int]:
    d = torch.load(path, map_location="cpu", weights_only=True)
    out = {}
    for k, v in d.items():
        v = int(v)
        if v < 0 or v % 16:
            raise ValueError(f"{path}: select_num {v} for {k} is not a non-negative multiple of 16")
        out[k] = v
    return out


def kernel_index(index: torch.Tensor, device="cuda") -> torch.Tensor:
    """the int16 device tensor the quantizers take (model/qLinearLayer.py:55)"""
    if index.numel() > 32736:
        raise ValueError("the kernels address channels with int16")
    return index.to(device=device, dtype=torch.int16).contiguous()
