"""GPU parity at the benchmark configurations' own shapes.

Config 1: one ARC linear, X 2048x4096 (seed 1, 1 % of channels x40), W 4096x4096 ~N(0, 0.02),
reorder_index from the per-channel max |X|, select_num 128, NVFP4 with the fake path's tensor
scales (model/quantize.py:291, 318): packed codes and scale bytes bit-exact against the C
oracle, Y within 1e-2 relative Frobenius error of dequantize-then-matmul.

Config 3: the augmented-K GEMM at every Llama-3-8B projection shape x every M the bench times,
select_num 256, both formats.  Outputs are large, so two checks per launch, neither of which
touches the library's own dequantizer: a seeded sample of rows x columns (always including the
first and last of each) against the fp64 oracle, and the whole output against torch's fp32
matmul of the operands dequantized by the CPU oracle.  This mirrors the reference's own sweep
(kernels/main.py:7-47: quantize, matmul, compare with F.linear) and model/qLinearLayer.py:65-81.
"""
import numpy as np
import pytest
import torch

import recipes

pytestmark = pytest.mark.gpu
TOL = 1e-2
SHAPES = {"qkv": (6144, 4096), "o": (4096, 4096), "gate_up": (28672, 4096), "down": (4096, 14336)}
MS = [1, 16, 128, 512, 2048, 4096]
S3 = 256


@pytest.fixture(scope="module")
def agemm():
    assert torch.cuda.is_available(), "these tests need the MI355X"
    from arcquant_amd import agemm as m
    return m


def rel_fro(got, want):
    got, want = got.double(), want.double()
    return float((got - want).norm() / want.norm())


def config3_activations(M, K):
    """~N(0,1) rows with the same 1 % of channels x40 for every M (the outlier channels belong to the
    layer, not to the batch), so that one reorder_index serves the weights and every M"""
    cols = torch.randperm(K, generator=torch.Generator().manual_seed(33))[:round(0.01 * K)]
    x = torch.randn(M, K, generator=torch.Generator().manual_seed(3 + M))
    x[:, cols] *= 40.0
    return x.to(torch.bfloat16)


_weights = {}


def quantized_weights(agemm, oracle, name, fmt):
    """weights of one projection, quantized once per (shape, format) on the GPU; the fp32 values of
    the codes come from the CPU oracle's dequantizer"""
    key = (name, fmt)
    if key not in _weights:
        _weights.clear()                       # one projection resident at a time
        N, K = SHAPES[name]
        w = recipes.weights(N, K, seed=3)
        idx = recipes.reorder_index(config3_activations(256, K))
        gw = recipes.tensor_scale(w, fmt)
        b, sfb = agemm.reorder_quantize_w(w.cuda(), idx.cuda(), S3, fmt=fmt, global_scale=gw)
        bc, bs = b.cpu().numpy(), sfb.cpu().numpy().reshape(N, -1)
        dq_b = torch.from_numpy(oracle.dequantize(bc, bs, fmt)).cuda()
        _weights[key] = (idx, gw, b, sfb, bc, bs, dq_b)
    return _weights[key]


def sample(n, count, gen):
    """`count` distinct indices of range(n) that include 0 and n-1, sorted"""
    if n <= count:
        return np.arange(n)
    pick = torch.randperm(n - 2, generator=gen)[:count - 2].numpy() + 1
    return np.sort(np.concatenate([[0, n - 1], pick]))


@pytest.mark.parametrize("M", MS)                       # fastest: the weights of a projection are quantized once
@pytest.mark.parametrize("fmt", ["NVFP4", "MXFP4"])
@pytest.mark.parametrize("name", list(SHAPES))
def test_config3_gemm(agemm, oracle, name, M, fmt):
    N, K = SHAPES[name]
    idx, gw, b, sfb, bc, bs, dq_b = quantized_weights(agemm, oracle, name, fmt)
    x = config3_activations(M, K)
    gx = recipes.tensor_scale(x, fmt)
    print(f"config 3 {name} {fmt} M={M} N={N} K={K} S={S3}", flush=True)
    a, sfa = agemm.reorder_quantize_x(x.cuda(), idx.cuda(), S3, fmt=fmt, global_scale=gx)
    y = agemm.matmul(a, b, sfa, sfb, gx * gw)
    torch.cuda.synchronize()
    assert y.shape == (M, N) and y.dtype == torch.bfloat16
    ac, asc = a.cpu().numpy(), sfa.cpu().numpy().reshape(M, -1)
    # (1) sample of rows x columns against the fp64 oracle
    gen = torch.Generator().manual_seed(M * 31 + N)
    rows, cols = sample(M, 64, gen), sample(N, 256, gen)
    want = oracle.matmul(ac[rows], asc[rows], bc[cols], bs[cols], fmt, alpha=gx * gw)
    got = y[torch.from_numpy(rows).cuda()][:, torch.from_numpy(cols).cuda()].float().cpu()
    assert rel_fro(got, torch.from_numpy(want)) < TOL
    assert torch.allclose(got, torch.from_numpy(want), rtol=2 ** -7, atol=1e-3 * float(np.abs(want).max()))
    # (2) the whole output against fp32 matmul of oracle-dequantized operands
    prev = torch.backends.cuda.matmul.allow_tf32
    torch.backends.cuda.matmul.allow_tf32 = False
    try:
        full = (torch.from_numpy(oracle.dequantize(ac, asc, fmt)).cuda() @ dq_b.T) * (gx * gw)
    finally:
        torch.backends.cuda.matmul.allow_tf32 = prev
    assert rel_fro(y.float(), full) < TOL
    # no element of the output may be off by more than the bf16 rounding of an fp32 sum
    assert torch.allclose(y.float(), full, rtol=2 ** -6, atol=2e-3 * float(full.abs().max()))


def test_config1_arc_linear(agemm, oracle):
    """benchmark configuration 1 at its stated shape"""
    _weights.clear()
    M, K, N, S, fmt = 2048, 4096, 4096, 128, "NVFP4"
    x = recipes.activations(M, K, seed=1, outlier_frac=0.01, outlier_gain=40.0)
    w = recipes.weights(N, K, seed=2)
    idx = recipes.reorder_index(x)
    gx, gw = recipes.tensor_scale(x, fmt), recipes.tensor_scale(w, fmt)
    print(f"config 1 M={M} K={K} N={N} S={S} gx={gx} gw={gw}", flush=True)
    want_a = oracle.quantize_x(x, idx, S, fmt, gx)
    want_b = oracle.quantize_w(w, idx, S, fmt, gw)
    a, sfa = agemm.reorder_quantize_x(x.cuda(), idx.cuda(), S, fmt=fmt, global_scale=gx)
    b, sfb = agemm.reorder_quantize_w(w.cuda(), idx.cuda(), S, fmt=fmt, global_scale=gw)
    assert np.array_equal(a.cpu().numpy(), want_a["codes"])
    assert np.array_equal(sfa.cpu().numpy().reshape(M, -1), want_a["scales"])
    assert np.array_equal(b.cpu().numpy(), want_b["codes"])
    assert np.array_equal(sfb.cpu().numpy().reshape(N, -1), want_b["scales"])
    y = agemm.matmul(a, b, sfa, sfb, gx * gw)
    gen = torch.Generator().manual_seed(1)
    rows, cols = sample(M, 96, gen), sample(N, 384, gen)
    want = oracle.matmul(want_a["codes"][rows], want_a["scales"][rows], want_b["codes"][cols], want_b["scales"][cols],
                         fmt, alpha=gx * gw)
    got = y[torch.from_numpy(rows).cuda()][:, torch.from_numpy(cols).cuda()].float().cpu()
    assert rel_fro(got, torch.from_numpy(want)) < TOL
    prev = torch.backends.cuda.matmul.allow_tf32
    torch.backends.cuda.matmul.allow_tf32 = False
    try:
        full = (torch.from_numpy(oracle.dequantize(want_a["codes"], want_a["scales"], fmt)).cuda()
                @ torch.from_numpy(oracle.dequantize(want_b["codes"], want_b["scales"], fmt)).cuda().T) * (gx * gw)
        y_true = x.cuda().float() @ w.cuda().float().T
    finally:
        torch.backends.cuda.matmul.allow_tf32 = prev
    assert rel_fro(y.float(), full) < TOL
    # the reference's own sanity figure (kernels/main.py:46-47): the quantized linear tracks F.linear
    assert rel_fro(y.float(), y_true) < 0.1
