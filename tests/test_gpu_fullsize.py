"""GPU parity of every operator at the sizes of benchmark configurations 4 and 5, operator by operator against
the CPU oracle (never against the library's own dequantizer, never one HIP path against another).

Configuration 4 is one Llama-3-8B decoder layer (hidden 4096, intermediate 14336, select_num 256) at prefill
8 x 2048 = 16384 tokens and at decode batch 64; its linears are called as model/qLlamaLayer.py:297,364,429,439
call them.  Configuration 5 is a Mixtral block (8 experts, top-2, hidden 4096, intermediate 14336, select_num
128) on 4096 tokens whose (token, expert) pairs follow Zipf(1.1): 8192 rows in segments of
3115 / 1894 / 1141 / 733 / 493 / 347 / 258 / 211 (model/qMixtralLayer.py:458-471, 530-543).

Outputs of this size are compared in full where the oracle takes seconds (the quantizers) and on a seeded
sample of rows x columns that always holds the first and last of each against the fp64 oracle (the GEMMs)."""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

import recipes

pytestmark = pytest.mark.gpu
FMTS = ["NVFP4", "MXFP4"]
TOL = 1e-2
SHAPES = {"qkv": (6144, 4096), "o": (4096, 4096), "gate_up": (28672, 4096), "down": (4096, 14336)}
S4 = 256
ZIPF_ROWS = [3115, 1894, 1141, 733, 493, 347, 258, 211]
S5 = 128


@pytest.fixture(scope="module")
def agemm():
    assert torch.cuda.is_available(), "these tests need the MI355X"
    from arcquant_amd import agemm as m
    return m


def rel_fro(got, want):
    got, want = got.double(), want.double()
    return float((got - want).norm() / want.norm())


def sample(n, count, gen):
    """`count` distinct indices of range(n) that include 0 and n-1, sorted"""
    if n <= count:
        return np.arange(n)
    pick = torch.randperm(n - 2, generator=gen)[:count - 2].numpy() + 1
    return np.sort(np.concatenate([[0, n - 1], pick]))


def compare_rows(tag, got_codes, got_scales, want):
    gc = got_codes.cpu().numpy()
    gs = got_scales.cpu().numpy().reshape(want["scales"].shape)
    bad_s, bad_c = int((gs != want["scales"]).sum()), int((gc != want["codes"]).sum())
    assert bad_s == 0, f"{tag}: {bad_s} of {gs.size} scale bytes differ; first at {np.argwhere(gs != want['scales'])[:3]}"
    assert bad_c == 0, f"{tag}: {bad_c} of {gc.size} code bytes differ; first at {np.argwhere(gc != want['codes'])[:3]}"


def layer_activations(M, K, seed):
    """~N(0,1) rows with 1 % of the channels x40; the outlier channels belong to the layer, not to the batch"""
    cols = torch.randperm(K, generator=torch.Generator().manual_seed(44))[:round(0.01 * K)]
    x = torch.randn(M, K, generator=torch.Generator().manual_seed(seed + M))
    x[:, cols] *= 40.0
    return x.to(torch.bfloat16)


# ---------------------------------------------------------------------------------------------- configuration 4

@pytest.mark.parametrize("fmt", FMTS)
@pytest.mark.parametrize("M", [64, 16384])
def test_config4_rmsnorm_quantize_x(agemm, oracle, fmt, M):
    """the layer's two fused norm -> quantize launches: every row against the oracle"""
    K = 4096
    x = recipes.activations(M, K, seed=400 + M, outlier_frac=0.005, outlier_gain=50.0)
    x[M // 2] = 0                                                    # a padding token
    gam = recipes.gamma(K, seed=41)
    idx = recipes.reorder_index(x)
    print(f"config 4 rmsnorm_quantize_x {fmt} M={M} K={K} S={S4}", flush=True)
    want = oracle.rmsnorm_quantize_x(x, gam, 1e-5, idx, S4, fmt, 1.0)
    q, sf = agemm.rmsnorm_quantize_x(x.cuda(), gam.cuda(), 1e-5, idx.cuda(), S4, fmt=fmt)
    compare_rows(f"rmsnorm {M}x{K}", q, sf, want)


@pytest.mark.parametrize("fmt", FMTS)
@pytest.mark.parametrize("M", [64, 16384])
def test_config4_o_input_quantizer(agemm, oracle, fmt, M):
    """the quantizer in front of the o projection (model/qLlamaLayer.py:364): NVFP4 with the tensor scale
    max|x| / 2688 formed on the device, every row against the oracle run with that very fp32 scale"""
    K = 4096
    x = layer_activations(M, K, seed=410)
    idx = recipes.reorder_index(x)
    xd = x.cuda()
    gs = agemm.tensor_scale(xd) if fmt == "NVFP4" else None
    if gs is not None:
        want_gs = x.float().abs().max() / torch.tensor(2688.0)
        assert float(gs) == float(want_gs)
    print(f"config 4 reorder_quantize_x {fmt} M={M} K={K} S={S4}", flush=True)
    want = oracle.quantize_x(x, idx, S4, fmt, 1.0 if gs is None else float(gs))
    q, sf = agemm.reorder_quantize_x(xd, idx.cuda(), S4, fmt=fmt, global_scale=gs)
    compare_rows(f"reorder_quantize_x {M}x{K}", q, sf, want)


@pytest.mark.parametrize("fmt", FMTS)
@pytest.mark.parametrize("M", [64, 16384])
def test_config4_swiglu_quantize_x(agemm, oracle, fmt, M):
    """the down projection's input (model/qLlamaLayer.py:432-439) formed from the fused gate_up output and
    quantized in one pass, NVFP4 with the tensor scale of the activation's own maximum.  act_fn(gate) * up is
    torch-ROCm's bf16 silu and multiply (the exponential is the platform's; the CPU's differs in the last bit
    of a few values in 10^4); those values, brought to the host, go through the oracle's quantizer: a sample
    of 512 rows (first and last included) bit for bit."""
    K = 14336
    g = torch.Generator().manual_seed(420 + M)
    gu = torch.empty(M, 2 * K, dtype=torch.bfloat16)
    for lo in range(0, M, 2048):                                     # in pieces: the fp32 draw of the whole is 1.9 GB
        hi = min(M, lo + 2048)
        gu[lo:hi] = (torch.randn(hi - lo, 2 * K, generator=g) * 1.5).to(torch.bfloat16)
    gu[:, :7] *= 8.0                                                 # saturated gates and large products
    gu[M // 2] = 0
    gud = gu.cuda()
    gate, up = gud[:, :K], gud[:, K:]
    t = F.silu(gate) * up
    chan_max = t.float().abs().amax(0).cpu()
    idx = torch.argsort(chan_max, stable=True).to(torch.int16)
    print(f"config 4 swiglu_quantize_x {fmt} M={M} K={K} S={S4}", flush=True)
    if fmt == "NVFP4":
        q, sf, gs = agemm.swiglu_quantize_x(gate, up, idx.cuda(), S4, fmt=fmt, global_scale="absmax")
        want_gs = t.abs().max().float() / torch.full((), 2688.0, device="cuda")
        assert float(gs) == float(want_gs)
        gs = float(gs)
    else:
        q, sf = agemm.swiglu_quantize_x(gate, up, idx.cuda(), S4, fmt=fmt)
        gs = 1.0
    rows = sample(M, 512, g)
    rt = torch.from_numpy(rows)
    want = oracle.quantize_x(t[rt.cuda()].cpu(), idx, S4, fmt, gs)
    compare_rows(f"swiglu {M}x{K}", q[rt.cuda()], sf.view(M, -1)[rt.cuda()], want)
    # and with the host's own silu: at most one value in a thousand may land on another code
    t_cpu = F.silu(gu[rt][:, :K]) * gu[rt][:, K:]
    want_cpu = oracle.quantize_x(t_cpu, idx, S4, fmt, gs)
    dc = float((q[rt.cuda()].cpu().numpy() != want_cpu["codes"]).mean())
    assert dc <= 1e-3, dc


_weights = {}


def quantized_weights(agemm, oracle, name, fmt):
    key = (name, fmt)
    if key not in _weights:
        _weights.clear()                       # one projection resident at a time
        N, K = SHAPES[name]
        w = recipes.weights(N, K, seed=4)
        idx = recipes.reorder_index(layer_activations(256, K, seed=430))
        gw = recipes.tensor_scale(w, fmt)
        b, sfb = agemm.reorder_quantize_w(w.cuda(), idx.cuda(), S4, fmt=fmt, global_scale=gw)
        bc, bs = b.cpu().numpy(), sfb.cpu().numpy().reshape(N, -1)
        dq_b = torch.from_numpy(oracle.dequantize(bc, bs, fmt)).cuda()
        _weights[key] = (idx, gw, b, sfb, bc, bs, dq_b)
    return _weights[key]


@pytest.mark.parametrize("M", [64, 16384])
@pytest.mark.parametrize("fmt", FMTS)
@pytest.mark.parametrize("name", list(SHAPES))
def test_config4_gemm(agemm, oracle, name, M, fmt):
    """the layer's four GEMMs at prefill and decode size: 64 rows x 256 columns against the fp64 oracle, and
    the whole output against torch's fp32 matmul of the operands as the CPU oracle dequantizes them"""
    N, K = SHAPES[name]
    idx, gw, b, sfb, bc, bs, dq_b = quantized_weights(agemm, oracle, name, fmt)
    x = layer_activations(M, K, seed=430)
    gx = recipes.tensor_scale(x, fmt)
    print(f"config 4 matmul {name} {fmt} M={M} N={N} K={K} S={S4}", flush=True)
    a, sfa = agemm.reorder_quantize_x(x.cuda(), idx.cuda(), S4, fmt=fmt, global_scale=gx)
    y = agemm.matmul(a, b, sfa, sfb, gx * gw)
    torch.cuda.synchronize()
    assert y.shape == (M, N) and y.dtype == torch.bfloat16
    ac, asc = a.cpu().numpy(), sfa.cpu().numpy().reshape(M, -1)
    gen = torch.Generator().manual_seed(M * 31 + N)
    rows, cols = sample(M, 64, gen), sample(N, 256, gen)
    want = oracle.matmul(ac[rows], asc[rows], bc[cols], bs[cols], fmt, alpha=gx * gw)
    got = y[torch.from_numpy(rows).cuda()][:, torch.from_numpy(cols).cuda()].float().cpu()
    assert rel_fro(got, torch.from_numpy(want)) < TOL
    assert torch.allclose(got, torch.from_numpy(want), rtol=2 ** -7, atol=1e-3 * float(np.abs(want).max()))
    prev = torch.backends.cuda.matmul.allow_tf32
    torch.backends.cuda.matmul.allow_tf32 = False
    try:
        dq_a = torch.from_numpy(oracle.dequantize(ac, asc, fmt)).cuda()
        bound = None
        for lo in range(0, M, 4096):                                 # the fp32 product in slabs of 4096 rows
            full = (dq_a[lo:lo + 4096] @ dq_b.T) * (gx * gw)
            bound = float(full.abs().max()) if bound is None else bound
            part = y[lo:lo + 4096].float()
            assert rel_fro(part, full) < TOL, lo
            assert torch.allclose(part, full, rtol=2 ** -6, atol=2e-3 * bound), lo
            del full, part
    finally:
        torch.backends.cuda.matmul.allow_tf32 = prev


# ---------------------------------------------------------------------------------------------- configuration 5

def zipf_segments():
    return torch.tensor([0] + list(np.cumsum(ZIPF_ROWS)), dtype=torch.int32)


def expert_rows(K, seed):
    """8192 rows sorted by expert, every expert with outlier channels and a magnitude of its own"""
    T = sum(ZIPF_ROWS)
    seg = zipf_segments()
    x = torch.randn(T, K, generator=torch.Generator().manual_seed(seed))
    g = torch.Generator().manual_seed(seed + 1)
    for e in range(len(ZIPF_ROWS)):
        cols = torch.randperm(K, generator=g)[:round(0.01 * K)]
        x[seg[e]:seg[e + 1], cols] *= 40.0
        x[seg[e]:seg[e + 1]] *= (1.0 + 0.25 * e)
    x = x.to(torch.bfloat16)
    idx = torch.stack([recipes.reorder_index(x[seg[e]:seg[e + 1]]) for e in range(len(ZIPF_ROWS))])
    return x, seg, idx


@pytest.mark.parametrize("fmt", FMTS)
@pytest.mark.parametrize("K", [4096, 14336])
def test_config5_grouped_quantizer(agemm, oracle, fmt, K):
    """both grouped quantizer launches of the block (hidden 4096 in front of w1 | w3, intermediate 14336 in
    front of w2): every row of every expert against the oracle with that expert's order and tensor scale"""
    x, seg, idx = expert_rows(K, seed=500 + K)
    T, E = x.shape[0], len(ZIPF_ROWS)
    xd = x.cuda()
    print(f"config 5 grouped_reorder_quantize_x {fmt} K={K} S={S5}", flush=True)
    gs = None
    if fmt == "NVFP4":
        gs = agemm.grouped_tensor_scale(xd, seg.cuda())
        want_gs = [float(x[seg[e]:seg[e + 1]].abs().max().float() / torch.tensor(2688.0)) for e in range(E)]
        assert gs.cpu().tolist() == want_gs
    q, sf = agemm.grouped_reorder_quantize_x(xd, seg.cuda(), idx.cuda(), S5, fmt=fmt, global_scales=gs)
    sf = sf.view(T, -1)
    for e in range(E):
        lo, hi = int(seg[e]), int(seg[e + 1])
        want = oracle.quantize_x(x[lo:hi], idx[e], S5, fmt, 1.0 if gs is None else float(gs[e]))
        compare_rows(f"expert {e}", q[lo:hi], sf[lo:hi], want)


def expert_weights(agemm, N, K, fmt, idx, seed, interleaved=False):
    """E weight matrices quantized one by one (model/qMixtralLayer.py:488-508), stacked for the grouped launch"""
    bq, bsf, gw = [], [], []
    for e in range(len(ZIPF_ROWS)):
        w = recipes.weights(N, K, seed=seed + e, std=0.02 * (1 + 0.1 * e))
        s = recipes.tensor_scale(w, fmt)
        wd = w.cuda()
        if interleaved:
            wd = agemm.interleave_gate_up(wd[:N // 2], wd[N // 2:])
        b, sfb = agemm.reorder_quantize_w(wd, idx[e].cuda(), S5, fmt=fmt, global_scale=s)
        bq.append(b), bsf.append(sfb), gw.append(s)
    return bq, bsf, gw


@pytest.mark.parametrize("fmt", FMTS)
def test_config5_grouped_matmul_w2(agemm, oracle, fmt):
    """the w2 launch: (N, K') = (4096, 14464) over the Zipf segments; per expert 24 rows x 128 columns (first
    and last of both included) against the fp64 oracle with that expert's weights"""
    N, K = 4096, 14336
    x, seg, idx = expert_rows(K, seed=520)
    T, E = x.shape[0], len(ZIPF_ROWS)
    print(f"config 5 grouped_matmul {fmt} N={N} K={K} S={S5}", flush=True)
    gs = agemm.grouped_tensor_scale(x.cuda(), seg.cuda()) if fmt == "NVFP4" else None
    a, sfa = agemm.grouped_reorder_quantize_x(x.cuda(), seg.cuda(), idx.cuda(), S5, fmt=fmt, global_scales=gs)
    bq, bsf, gw = expert_weights(agemm, N, K, fmt, idx, seed=5300)
    gw_d = torch.tensor(gw, dtype=torch.float32).cuda() if fmt == "NVFP4" else None
    y = agemm.grouped_matmul(a, torch.stack(bq), sfa, torch.cat(bsf), seg.cuda(), gs, gw_d)
    torch.cuda.synchronize()
    assert y.shape == (T, N)
    ac, asc = a.cpu().numpy(), sfa.cpu().numpy().reshape(T, -1)
    gen = torch.Generator().manual_seed(52)
    for e in range(E):
        lo, hi = int(seg[e]), int(seg[e + 1])
        rows, cols = lo + sample(hi - lo, 24, gen), sample(N, 128, gen)
        alpha = float(gs[e]) * gw[e] if fmt == "NVFP4" else 1.0
        want = oracle.matmul(ac[rows], asc[rows], bq[e].cpu().numpy()[cols], bsf[e].cpu().numpy().reshape(N, -1)[cols],
                             fmt, alpha=alpha)
        got = y[torch.from_numpy(rows).cuda()][:, torch.from_numpy(cols).cuda()].float().cpu()
        assert rel_fro(got, torch.from_numpy(want)) < TOL, f"expert {e}"
        assert torch.allclose(got, torch.from_numpy(want), rtol=2 ** -7, atol=1e-3 * float(np.abs(want).max())), f"expert {e}"


@pytest.mark.parametrize("fmt", FMTS)
@pytest.mark.parametrize("fused", [False, True])
def test_config5_grouped_matmul_w1w3(agemm, oracle, fmt, fused):
    """the w1 | w3 launch: (N, K') = (28672, 4224) over the Zipf segments, plain (h = x [w1 | w3]^T) and with
    the SwiGLU in its epilogue (weight rows alternating w1_j, w3_j; output act(w1 x) * w3 x, 14336 wide).
    Per expert 24 rows x 128 columns against the fp64 oracle with that expert's weights; for the fused form
    the oracle's two projections are rounded to bf16 and pass through torch's bf16 silu and multiply, as
    model/qMixtralLayer.py:535-540 does, and the comparison allows what one bf16 step of a projection moves."""
    N, K, Fi = 28672, 4096, 14336
    x, seg, idx = expert_rows(K, seed=540)
    T, E = x.shape[0], len(ZIPF_ROWS)
    print(f"config 5 grouped_matmul{'_swiglu' if fused else ''} {fmt} N={N} K={K} S={S5}", flush=True)
    gs = agemm.grouped_tensor_scale(x.cuda(), seg.cuda()) if fmt == "NVFP4" else None
    a, sfa = agemm.grouped_reorder_quantize_x(x.cuda(), seg.cuda(), idx.cuda(), S5, fmt=fmt, global_scales=gs)
    bq, bsf, gw = expert_weights(agemm, N, K, fmt, idx, seed=5500, interleaved=fused)
    gw_d = torch.tensor(gw, dtype=torch.float32).cuda() if fmt == "NVFP4" else None
    B, SFB = torch.stack(bq), torch.cat(bsf)
    if fused:
        y, ts = agemm.grouped_matmul_swiglu(a, B, sfa, SFB, seg.cuda(), gs, gw_d, fmt=fmt, tensor_scale=True)
        assert y.shape == (T, Fi)
    else:
        y = agemm.grouped_matmul(a, B, sfa, SFB, seg.cuda(), gs, gw_d)
        assert y.shape == (T, N)
    torch.cuda.synchronize()
    ac, asc = a.cpu().numpy(), sfa.cpu().numpy().reshape(T, -1)
    gen = torch.Generator().manual_seed(54)
    for e in range(E):
        lo, hi = int(seg[e]), int(seg[e + 1])
        rows = lo + sample(hi - lo, 24, gen)
        alpha = float(gs[e]) * gw[e] if fmt == "NVFP4" else 1.0
        be, se = bq[e].cpu().numpy(), bsf[e].cpu().numpy().reshape(N, -1)
        rt = torch.from_numpy(rows).cuda()
        if not fused:
            cols = sample(N, 128, gen)
            want = torch.from_numpy(oracle.matmul(ac[rows], asc[rows], be[cols], se[cols], fmt, alpha=alpha))
            got = y[rt][:, torch.from_numpy(cols).cuda()].float().cpu()
            assert torch.allclose(got, want, rtol=2 ** -7, atol=1e-3 * float(want.abs().max())), f"expert {e}"
        else:
            cols = sample(Fi, 128, gen)
            hg = torch.from_numpy(oracle.matmul(ac[rows], asc[rows], be[2 * cols], se[2 * cols], fmt, alpha=alpha))
            hu = torch.from_numpy(oracle.matmul(ac[rows], asc[rows], be[2 * cols + 1], se[2 * cols + 1], fmt, alpha=alpha))
            want = (F.silu(hg.to(torch.bfloat16)) * hu.to(torch.bfloat16)).float()
            got = y[rt][:, torch.from_numpy(cols).cuda()].float().cpu()
            assert torch.allclose(got, want, rtol=2 ** -5, atol=4e-3 * float(want.abs().max())), f"expert {e}"
            # the per-expert tensor scale of the epilogue: max |y_e| / 2688 over the expert's whole output
            m = y[lo:hi].abs().max().float() / torch.full((), 2688.0, device="cuda")
            assert float(ts[e]) == float(m), f"expert {e}"
        assert rel_fro(got, want) < TOL, f"expert {e}"
