"""Seeded synthetic inputs for the parity tests and the bench.

Everything is drawn on the CPU with an explicit torch.Generator so that the development
container and the GPU box see identical bits.  Shapes and distributions follow the benchmark
configurations: Llama-3-8B projection shapes, ~N(0,1) activations with a small fraction of
outlier channels, ~N(0,0.02) weights, reorder_index = ascending argsort of the per-channel
max |x| (the reference's definition, utilize.py:39-45,108).
"""
from __future__ import annotations

import torch


def activations(M, K, seed, outlier_frac=0.01, outlier_gain=40.0):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(M, K, generator=g)
    n_out = max(1, round(outlier_frac * K))
    cols = torch.randperm(K, generator=g)[:n_out]
    x[:, cols] *= outlier_gain
    return x.to(torch.bfloat16)


def weights(N, K, seed, std=0.02):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(N, K, generator=g) * std).to(torch.bfloat16)


def gamma(K, seed):
    g = torch.Generator().manual_seed(seed)
    return (torch.rand(K, generator=g) + 0.5).to(torch.bfloat16)


def reorder_index(x: torch.Tensor) -> torch.Tensor:
    """ascending stable argsort of per-channel max |x| -> int16 [K]"""
    return torch.argsort(x.float().abs().amax(0), stable=True).to(torch.int16)


def nvfp4_tensor_scale(t: torch.Tensor) -> float:
    """the fake path's tensor scale: signed max / (448*6) (model/quantize.py:291,318)"""
    return float(torch.max(t).to(torch.float32) / (448.0 * 6.0))


def tensor_scale(t, fmt) -> float:
    return nvfp4_tensor_scale(t) if fmt == "NVFP4" else 1.0
