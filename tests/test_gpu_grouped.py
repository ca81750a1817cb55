"""Grouped operators for mixture-of-experts blocks (tokens sorted by expert, one launch per step for all
experts, segment offsets on the device) against the per-expert path they replace:

* grouped quantizer: codes and scale bytes of every row bit-exact against the C oracle's quantizer run
  on that expert's rows with that expert's reorder_index and tensor scale (model/qMixtralLayer.py:530);
* grouped fused SwiGLU quantizer: bit-identical to the ungrouped operator on each expert's rows;
* grouped GEMM: against the fp64 oracle with each expert's weights (model/qMixtralLayer.py:466-543).
"""
import numpy as np
import pytest
import torch

import recipes

pytestmark = pytest.mark.gpu
FMTS = ["NVFP4", "MXFP4"]


@pytest.fixture(scope="module")
def agemm():
    assert torch.cuda.is_available(), "these tests need the MI355X"
    from arcquant_amd import agemm as m
    return m


def rel_fro(got, want):
    got, want = got.double(), want.double()
    return float((got - want).norm() / want.norm())


def segments(counts):
    return torch.tensor([0] + list(np.cumsum(counts)), dtype=torch.int32)


def expert_scale(t):
    """max|t| / 2688 as the callers compute it in fp32 (model/qLlamaLayer.py:74); 1 for no rows / all zeros"""
    if t.numel() == 0:
        return 1.0
    s = float(t.abs().max().float() / torch.tensor(2688.0))
    return s if s != 0.0 else 1.0


COUNTS = [[5, 0, 17, 1, 300, 0, 64, 9], [40], [0, 0, 3], [130, 131, 2, 700]]


@pytest.mark.parametrize("fmt", FMTS)
@pytest.mark.parametrize("counts", COUNTS)
@pytest.mark.parametrize("K,S", [(4096, 128), (512, 512), (1024, 0), (18944, 256)])
def test_grouped_quantize_matches_per_expert_oracle(agemm, oracle, fmt, counts, K, S):
    T, E = sum(counts), len(counts)
    x = recipes.activations(T, K, seed=7000 + T + K, outlier_frac=0.01, outlier_gain=40.0)
    seg = segments(counts)
    # per-expert channel order from the per-expert channel maxima (experts without rows: a random order)
    g = torch.Generator().manual_seed(E + K)
    idx = torch.stack([recipes.reorder_index(x[seg[e]:seg[e + 1]]) if counts[e] else
                       torch.randperm(K, generator=g).to(torch.int16) for e in range(E)])
    for e in range(E):                      # per-expert magnitudes, so that the tensor scales differ
        x[seg[e]:seg[e + 1]] *= (1.0 + 0.5 * e)
    x = x.to(torch.bfloat16)
    print(f"grouped quantize {fmt} counts={counts} K={K} S={S}", flush=True)
    gs = None
    if fmt == "NVFP4":
        gs = agemm.grouped_tensor_scale(x.cuda(), seg.cuda())
        want_gs = [expert_scale(x[seg[e]:seg[e + 1]]) for e in range(E)]
        assert gs.cpu().tolist() == pytest.approx(want_gs, rel=0, abs=0)
    q, sf = agemm.grouped_reorder_quantize_x(x.cuda(), seg.cuda(), idx.cuda(), S, fmt=fmt, global_scales=gs)
    q, sf = q.cpu().numpy(), sf.cpu().numpy().reshape(T, -1)
    for e in range(E):
        if not counts[e]:
            continue
        lo, hi = int(seg[e]), int(seg[e + 1])
        want = oracle.quantize_x(x[lo:hi], idx[e], S, fmt, 1.0 if gs is None else float(gs[e]))
        assert np.array_equal(sf[lo:hi], want["scales"]), f"expert {e}: scale bytes differ"
        assert np.array_equal(q[lo:hi], want["codes"]), f"expert {e}: codes differ"


@pytest.mark.parametrize("fmt", FMTS)
@pytest.mark.parametrize("counts,F", [([5, 0, 17, 1, 300, 0, 64, 9], 1024), ([700, 3], 1024), ([40, 0, 290], 18944)])
def test_grouped_swiglu_matches_ungrouped(agemm, fmt, counts, F):
    T, E, S = sum(counts), len(counts), 128
    g = torch.Generator().manual_seed(T)
    gu = (torch.randn(T, 2 * F, generator=g) * 2.0).to(torch.bfloat16).cuda()
    seg = segments(counts)
    for e in range(E):
        gu[seg[e]:seg[e + 1]] *= (1.0 + 0.25 * e)
    idx = torch.stack([torch.randperm(F, generator=g).to(torch.int16) for _ in range(E)]).cuda()
    gate, up = gu[:, :F], gu[:, F:]
    print(f"grouped swiglu {fmt} counts={counts}", flush=True)
    if fmt == "NVFP4":
        q, sf, gs = agemm.grouped_swiglu_quantize_x(gate, up, seg.cuda(), idx, S, fmt=fmt, global_scales="absmax")
    else:
        q, sf = agemm.grouped_swiglu_quantize_x(gate, up, seg.cuda(), idx, S, fmt=fmt)
    sf = sf.view(T, -1)
    for e in range(E):
        lo, hi = int(seg[e]), int(seg[e + 1])
        if lo == hi:
            if fmt == "NVFP4":
                assert float(gs[e]) == 1.0
            continue
        if fmt == "NVFP4":
            wq, wsf, wgs = agemm.swiglu_quantize_x(gate[lo:hi], up[lo:hi], idx[e], S, fmt=fmt, global_scale="absmax")
            assert float(wgs) == float(gs[e])
        else:
            wq, wsf = agemm.swiglu_quantize_x(gate[lo:hi], up[lo:hi], idx[e], S, fmt=fmt)
        assert torch.equal(sf[lo:hi], wsf.view(hi - lo, -1)) and torch.equal(q[lo:hi], wq), f"expert {e}"


@pytest.mark.parametrize("fmt", FMTS)
@pytest.mark.parametrize("counts,N,K,S", [([5, 0, 17, 1, 300, 0, 64, 9], 384, 512, 128),
                                           ([40], 256, 1024, 0),
                                           ([0, 0, 3], 130, 448, 64),
                                           ([130, 131, 2, 700], 512, 896, 128),
                                           ([300, 500, 10], 512, 512, 128),
                                           ([1100, 900], 256, 512, 0),
                                           ([2500, 2100], 256, 512, 0)])
def test_grouped_matmul_matches_oracle(agemm, oracle, fmt, counts, N, K, S):
    """The launch picks its tile from the average rows per expert: these cases take the 128x64, 128x128
    and 256x256 tiles; experts without rows, with one row, with ragged last tiles; the residual form as well."""
    T, E = sum(counts), len(counts)
    x = recipes.activations(T, K, seed=8000 + T + N, outlier_frac=0.01, outlier_gain=40.0)
    seg = segments(counts)
    g = torch.Generator().manual_seed(N + K)
    idx = torch.stack([torch.randperm(K, generator=g).to(torch.int16) for _ in range(E)])
    w = [recipes.weights(N, K, seed=8100 + e, std=0.02 * (1 + e)) for e in range(E)]
    print(f"grouped matmul {fmt} counts={counts} N={N} K={K} S={S}", flush=True)
    gs = agemm.grouped_tensor_scale(x.cuda(), seg.cuda()) if fmt == "NVFP4" else None
    a, sfa = agemm.grouped_reorder_quantize_x(x.cuda(), seg.cuda(), idx.cuda(), S, fmt=fmt, global_scales=gs)
    bq, bsf, gw = [], [], []
    for e in range(E):
        s = recipes.tensor_scale(w[e], fmt)
        b, sfb = agemm.reorder_quantize_w(w[e].cuda(), idx[e].cuda(), S, fmt=fmt, global_scale=s)
        bq.append(b), bsf.append(sfb), gw.append(s)
    B, SFB = torch.stack(bq), torch.cat(bsf)
    gw_d = torch.tensor(gw, dtype=torch.float32).cuda() if fmt == "NVFP4" else None
    res = (torch.randn(T, N, generator=g)).to(torch.bfloat16).cuda()
    y = agemm.grouped_matmul(a, B, sfa, SFB, seg.cuda(), gs, gw_d)
    y2 = agemm.grouped_matmul(a, B, sfa, SFB, seg.cuda(), gs, gw_d, residual=res)
    torch.cuda.synchronize()
    assert torch.equal(y2, (y + res))
    ac, asc = a.cpu().numpy(), sfa.cpu().numpy().reshape(T, -1)
    for e in range(E):
        lo, hi = int(seg[e]), int(seg[e + 1])
        if lo == hi:
            continue
        alpha = (float(gs[e]) * gw[e]) if fmt == "NVFP4" else 1.0
        want = oracle.matmul(ac[lo:hi], asc[lo:hi], bq[e].cpu().numpy(), bsf[e].cpu().numpy().reshape(N, -1), fmt, alpha=alpha)
        assert rel_fro(y[lo:hi].float().cpu(), torch.from_numpy(want)) < 1e-2, f"expert {e}"
        assert torch.allclose(y[lo:hi].float().cpu(), torch.from_numpy(want).float(), rtol=2 ** -7,
                              atol=1e-3 * float(np.abs(want).max())), f"expert {e}"


def test_grouped_matmul_ignores_rows_behind_the_last_segment(agemm):
    """seg[E] < M: the rows behind it are not written; offsets that shrink or leave the tensor read as empty segments"""
    T, N, K, S, fmt = 200, 256, 512, 0, "MXFP4"
    x = recipes.activations(T, K, seed=1).cuda()
    idx = torch.arange(K, dtype=torch.int16).cuda()
    a, sfa = agemm.reorder_quantize_x(x, idx, S, fmt=fmt)
    b, sfb = agemm.reorder_quantize_w(recipes.weights(N, K, seed=2).cuda(), idx, S, fmt=fmt)
    whole = agemm.matmul(a, b, sfa, sfb, 1.0, fmt=fmt)
    B, SFB = torch.stack([b, b]), torch.cat([sfb, sfb])
    for seg in ([0, 100, 150], [0, 300, 100], [0, -5, 200]):
        y = agemm.grouped_matmul(a, B, sfa, SFB, torch.tensor(seg, dtype=torch.int32).cuda())
        end = max(0, min(seg[1], T))
        end = max(end, min(seg[2], T))
        assert torch.equal(y[:end], whole[:end]), seg


@pytest.mark.parametrize("top_k", [1, 2, 3])
def test_moe_combine_matches_index_add(agemm, top_k):
    """weights applied and expert outputs summed per token as model/qMixtralLayer.py:466-471 does: expert after
    expert in ascending number into a bf16 tensor of zeros"""
    tokens, H, E = 300, 1032, 6
    g = torch.Generator().manual_seed(top_k)
    sel = torch.stack([torch.randperm(E, generator=g)[:top_k] for _ in range(tokens)])
    w = torch.rand(tokens, top_k, generator=g).to(torch.bfloat16)
    flat = sel.reshape(-1)
    order = torch.argsort(flat, stable=True)
    tok = order // top_k
    y = torch.randn(tokens * top_k, H, generator=g).to(torch.bfloat16)
    ws = w.reshape(-1)[order]
    want = torch.zeros(tokens, H, dtype=torch.bfloat16)
    counts = torch.bincount(flat, minlength=E).tolist()
    beg = 0
    for e, n in enumerate(counts):                 # the reference's loop over experts
        want.index_add_(0, tok[beg:beg + n], y[beg:beg + n] * ws[beg:beg + n, None])
        beg += n
    position = torch.empty_like(order)
    position[order] = torch.arange(order.numel())
    got = agemm.moe_combine(y.cuda(), position.cuda(), ws.cuda(), tokens, top_k)
    assert torch.equal(got.cpu(), want)


@pytest.mark.parametrize("fmt", FMTS)
@pytest.mark.parametrize("M,F,K,S", [(300, 256, 512, 128), (64, 384, 448, 64), (1, 128, 512, 0), (2100, 512, 512, 0),
                                      (700, 1024, 896, 128), (2100, 2048, 512, 0), (4000, 1024, 512, 0)])
def test_matmul_swiglu_equals_unfused_sequence(agemm, fmt, M, F, K, S):
    """GEMM with the SwiGLU in its epilogue (gate / up weight rows interleaved) against the unfused sequence on
    the same quantized operands: projection, then silu and multiply in bf16 (torch-ROCm, the pinned reference
    of tests/test_gpu_swiglu.py); outputs and the tensor scale must be the same bits.  Row counts cover the
    128x64, 128x128, 256x128 and 256x256 tiles (the last two as eight waves for MXFP4) and ragged last tiles."""
    import torch.nn.functional as Fn
    g = torch.Generator().manual_seed(M + F)
    x = recipes.activations(M, K, seed=9000 + M, outlier_frac=0.01, outlier_gain=40.0).cuda()
    idx = torch.randperm(K, generator=g).to(torch.int16).cuda()
    wg = recipes.weights(F, K, seed=9100, std=0.05).cuda()
    wu = recipes.weights(F, K, seed=9101, std=0.05).cuda()
    gx = agemm.tensor_scale(x) if fmt == "NVFP4" else None
    a, sfa = agemm.reorder_quantize_x(x, idx, S, fmt=fmt, global_scale=gx)
    w_cat = torch.cat([wg, wu])
    gw = recipes.tensor_scale(w_cat.cpu(), fmt)
    b_cat, sfb_cat = agemm.reorder_quantize_w(w_cat, idx, S, fmt=fmt, global_scale=gw)
    b_il, sfb_il = agemm.reorder_quantize_w(agemm.interleave_gate_up(wg, wu), idx, S, fmt=fmt, global_scale=gw)
    scale = (gx, gw) if fmt == "NVFP4" else 1.0
    print(f"matmul_swiglu {fmt} M={M} F={F} K={K} S={S}", flush=True)
    h = agemm.matmul(a, b_cat, sfa, sfb_cat, scale, fmt=fmt)
    want = Fn.silu(h[:, :F]) * h[:, F:]
    got, ts = agemm.matmul_swiglu(a, b_il, sfa, sfb_il, scale, fmt=fmt, tensor_scale=True)
    assert got.shape == (M, F)
    assert torch.equal(got, want), float((got.float() - want.float()).abs().max())
    want_ts = want.abs().max().float() / torch.full((), 2688.0, device="cuda")
    assert float(ts) == float(want_ts if float(want_ts) != 0 else 1.0)


@pytest.mark.parametrize("fmt", FMTS)
@pytest.mark.parametrize("counts", [[5, 0, 170, 1, 300, 0, 64, 9], [2500, 2100]])
def test_grouped_matmul_swiglu_equals_unfused_sequence(agemm, fmt, counts):
    import torch.nn.functional as Fn
    F, K, S = 256, 512, 128
    T, E = sum(counts), len(counts)
    g = torch.Generator().manual_seed(77)
    x = recipes.activations(T, K, seed=9200, outlier_frac=0.01, outlier_gain=40.0).cuda()
    seg = segments(counts).cuda()
    idx = torch.stack([torch.randperm(K, generator=g).to(torch.int16) for _ in range(E)]).cuda()
    gs = agemm.grouped_tensor_scale(x, seg) if fmt == "NVFP4" else None
    a, sfa = agemm.grouped_reorder_quantize_x(x, seg, idx, S, fmt=fmt, global_scales=gs)
    cat, il, gws = [], [], []
    for e in range(E):
        wg = recipes.weights(F, K, seed=9300 + e, std=0.05 * (1 + e)).cuda()
        wu = recipes.weights(F, K, seed=9400 + e, std=0.05).cuda()
        gw = recipes.tensor_scale(torch.cat([wg, wu]).cpu(), fmt)
        cat.append(agemm.reorder_quantize_w(torch.cat([wg, wu]), idx[e], S, fmt=fmt, global_scale=gw))
        il.append(agemm.reorder_quantize_w(agemm.interleave_gate_up(wg, wu), idx[e], S, fmt=fmt, global_scale=gw))
        gws.append(gw)
    gw_d = torch.tensor(gws, dtype=torch.float32).cuda() if fmt == "NVFP4" else None
    stack = lambda pairs: (torch.stack([p[0] for p in pairs]), torch.cat([p[1] for p in pairs]))
    print(f"grouped matmul_swiglu {fmt}", flush=True)
    h = agemm.grouped_matmul(a, *stack(cat)[:1], sfa, stack(cat)[1], seg, gs, gw_d, fmt=fmt)
    want = Fn.silu(h[:, :F]) * h[:, F:]
    got, ts = agemm.grouped_matmul_swiglu(a, stack(il)[0], sfa, stack(il)[1], seg, gs, gw_d, fmt=fmt, tensor_scale=True)
    assert torch.equal(got, want)
    segc = seg.cpu()
    for e in range(E):
        rows = want[segc[e]:segc[e + 1]]
        w = float(rows.abs().max().float() / torch.full((), 2688.0, device="cuda")) if rows.numel() else 0.0
        assert float(ts[e]) == (w if w != 0.0 else 1.0), e


def test_forced_kernel_unknown_to_the_format_is_ignored():
    """ARCQ_GEMM_KERNEL names a tile kernel by number; NVFP4 has no 256x128 eight-wave kernel (82).  The fused
    SwiGLU GEMM must then take a kernel it has, not fall through to the direct kernel, which writes all N
    output columns.  The knob is read once per process: a child process with it set."""
    import os
    import subprocess
    import sys
    code = r"""
import sys, torch
sys.path.insert(0, 'tests')
import recipes
import torch.nn.functional as Fn
from arcquant_amd import agemm
M, F, K, S = 300, 256, 512, 128
x = recipes.activations(M, K, seed=1).cuda()
idx = torch.randperm(K, generator=torch.Generator().manual_seed(3)).to(torch.int16).cuda()
wg = recipes.weights(F, K, seed=2, std=0.05).cuda(); wu = recipes.weights(F, K, seed=4, std=0.05).cuda()
for fmt in ("NVFP4", "MXFP4"):
    a, sfa = agemm.reorder_quantize_x(x, idx, S, fmt=fmt)
    b_cat, sfb_cat = agemm.reorder_quantize_w(torch.cat([wg, wu]), idx, S, fmt=fmt)
    b_il, sfb_il = agemm.reorder_quantize_w(agemm.interleave_gate_up(wg, wu), idx, S, fmt=fmt)
    h = agemm.matmul(a, b_cat, sfa, sfb_cat, 1.0, fmt=fmt)
    got = agemm.matmul_swiglu(a, b_il, sfa, sfb_il, 1.0, fmt=fmt)
    torch.cuda.synchronize()
    assert torch.equal(got, Fn.silu(h[:, :F]) * h[:, F:]), fmt
print("OK")
"""
    env = dict(os.environ, ARCQ_GEMM_KERNEL="82")
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([sys.executable, "-c", code], cwd=root, env=env, capture_output=True, text=True, timeout=300)
    assert r.returncode == 0 and "OK" in r.stdout, r.stdout[-2000:] + r.stderr[-2000:]


@pytest.mark.parametrize("T,E,k,dtype", [(4096, 8, 2, torch.bfloat16), (16384, 8, 2, torch.bfloat16), (16385, 8, 2, torch.bfloat16),
                                         (70001, 8, 2, torch.bfloat16), (40000, 64, 6, torch.float32), (300, 8, 2, torch.float32), (1000, 16, 4, torch.bfloat16),
                                         (1, 8, 2, torch.bfloat16), (777, 64, 8, torch.float32), (50, 5, 2, torch.bfloat16),
                                         (513, 3, 3, torch.float32)])
def test_moe_route_matches_torch(agemm, T, E, k, dtype):
    """Softmax / top-k / normalised weights and the expert-sorted bookkeeping against torch's own operators
    (model/qMixtralLayer.py:441-452 and what its loop over experts derives).  bf16 logits tie often; the library
    takes the lower expert number among equals, which a stable descending sort reproduces."""
    import torch.nn.functional as Fn
    g = torch.Generator().manual_seed(T + E)
    logits = (torch.randn(T, E, generator=g) * 2.0).to(dtype).cuda()
    sel, w, seg, position, tok, ws = agemm.moe_route(logits, k)
    p = Fn.softmax(logits, dim=1, dtype=torch.float)
    vals, idx = torch.sort(p, dim=1, descending=True, stable=True)
    want_sel, want_v = idx[:, :k], vals[:, :k]
    assert torch.equal(sel.long(), want_sel)
    want_w = (want_v / want_v.sum(dim=-1, keepdim=True)).to(torch.bfloat16)
    if k == 2:
        assert torch.equal(w, want_w)                      # same arithmetic as torch: same bits
    else:                                                  # torch's sum over k > 2 values has its own order
        assert float((w.float() - want_w.float()).abs().max()) <= 2.0 ** -8
    flat = sel.long().reshape(-1)
    order = torch.argsort(flat, stable=True)
    assert torch.equal(tok.long(), order // k)
    assert torch.equal(ws, w.reshape(-1)[order])
    want_seg = torch.zeros(E + 1, dtype=torch.int64, device="cuda")
    want_seg[1:] = torch.cumsum(torch.bincount(flat, minlength=E), 0)
    assert torch.equal(seg.long(), want_seg)
    want_pos = torch.empty_like(order)
    want_pos[order] = torch.arange(order.numel(), device="cuda")
    assert torch.equal(position, want_pos)


def test_moe_route_without_tokens(agemm):
    sel, w, seg, position, tok, ws = agemm.moe_route(torch.empty((0, 8), dtype=torch.bfloat16, device="cuda"), 2)
    assert sel.shape == (0, 2) and position.numel() == 0 and tok.numel() == 0
    assert torch.equal(seg.cpu(), torch.zeros(9, dtype=torch.int32))


def test_moe_route_with_non_finite_logits(agemm):
    """A NaN logit, a +inf logit or a row of -inf makes every probability of that row NaN (torch's softmax
    does the same).  The routing must stay a routing: every choice an expert number, every pair counted in the
    segments and given a row of its own, and only the affected tokens' weights NaN."""
    T, E, k = 200, 8, 2
    g = torch.Generator().manual_seed(12)
    logits = (torch.randn(T, E, generator=g) * 2.0).to(torch.bfloat16)
    bad = [3, 64, 65, 199]
    logits[3, 5] = float("nan")
    logits[64, 0] = float("inf")
    logits[65] = float("-inf")
    logits[199, 7] = float("nan")
    logits[199, 1] = float("inf")
    sel, w, seg, position, tok, ws = agemm.moe_route(logits.cuda(), k)
    torch.cuda.synchronize()
    sel, w, seg, position, tok = sel.cpu(), w.cpu(), seg.cpu(), position.cpu(), tok.cpu()
    assert int(sel.min()) >= 0 and int(sel.max()) < E
    assert all(len(set(r.tolist())) == k for r in sel)                 # a token never takes an expert twice
    assert int(seg[E]) == T * k and int(seg[0]) == 0
    assert torch.equal(seg[1:] - seg[:-1], torch.bincount(sel.reshape(-1).long(), minlength=E).int())
    assert torch.equal(torch.sort(position).values, torch.arange(T * k))          # a permutation of the pairs
    assert torch.equal(tok.long(), torch.argsort(sel.reshape(-1).long(), stable=True) // k)
    nan_rows = torch.isnan(w.float()).any(1).nonzero().flatten().tolist()
    assert nan_rows == bad
    # NaN ranks above every number and equals go to the lower expert: all-NaN rows take experts 0 and 1
    assert all(sel[t].tolist() == [0, 1] for t in bad)
    # the other tokens are routed as torch routes them
    import torch.nn.functional as Fn
    ok = torch.tensor([t for t in range(T) if t not in bad])
    p = Fn.softmax(logits[ok].float(), dim=1)
    vals, order = torch.sort(p, dim=1, descending=True, stable=True)
    assert torch.equal(sel[ok].long(), order[:, :k])


def test_mixtral_block_with_non_finite_logits():
    """the whole block on such logits: finite outputs for every token but the affected ones"""
    from arcquant_amd import layers
    hidden, ffn, E = 512, 1024, 8
    blk = layers.build_mixtral_block(hidden=hidden, ffn=ffn, num_experts=E, select_num=128, quant_type="NVFP4", seed=3)
    g = torch.Generator().manual_seed(13)
    x = torch.randn(1, 96, hidden, generator=g).to(torch.bfloat16).cuda()
    logits = (torch.randn(96, E, generator=g) * 2.0).to(torch.bfloat16)
    logits[7, 2] = float("nan")
    logits[40] = float("-inf")
    logits[95, 3] = float("inf")
    y, _ = blk(x, router_logits=logits.cuda())
    torch.cuda.synchronize()
    nan_tokens = torch.isnan(y[0].float()).any(1).nonzero().flatten().tolist()
    assert nan_tokens == [7, 40, 95]
    clean = torch.tensor([t for t in range(96) if t not in (7, 40, 95)]).cuda()
    logits2 = logits.clone()
    logits2[[7, 40, 95]] = 0.0
    y2, _ = blk(x, router_logits=logits2.cuda())
    # NVFP4's per-expert tensor scales see the same activations either way unless an affected token is an expert's
    # maximum; the clean tokens' outputs stay finite and close to the run without the bad logits
    assert bool(torch.isfinite(y[0][clean].float()).all())
    assert rel_fro(y[0][clean].float(), y2[0][clean].float()) < 5e-2
