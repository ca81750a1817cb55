"""Layer-level callers (arcquant_amd.layers) on the GPU against the reference's fake-quant flow
restated with the torch oracle on the CPU: same quantizers (bit-exact, see test_gpu_quantize.py),
so what remains is GEMM accumulation order and bf16 roundings between ops.  Tolerances are
relative Frobenius errors, written at each comparison."""
import pytest
import torch
import torch.nn as nn
import torch.nn.functional as F

import recipes

pytestmark = pytest.mark.gpu
FMTS = ["NVFP4", "MXFP4"]


@pytest.fixture(scope="module")
def layers():
    assert torch.cuda.is_available(), "these tests need the MI355X"
    from arcquant_amd import layers as m
    return m


@pytest.fixture(scope="module")
def fq():
    from oracle import fakequant_torch as m
    return m


def rel_fro(got, want):
    got, want = got.double().cpu(), want.double().cpu()
    return float((got - want).norm() / want.norm())


def ref_quant_x(fq, x, idx, S, fmt, scale=None):
    """values of the activation quantizer (model/quantize.py:314-343) with the real-kernel callers'
    tensor scale max|x|/2688 (model/qLlamaLayer.py:74); fp32 [M, K+S], already multiplied back"""
    if scale is None:
        scale = x.abs().max().float() / 2688.0 if fmt == "NVFP4" else torch.tensor(1.0)
    x32 = x[:, idx.long()].float() / scale
    q = fq.blockwise(x32, fmt)
    if S == 0:
        return q * scale
    err = x32 - q
    return torch.cat([q, fq.blockwise(err[:, -S:], fmt)], dim=1) * scale


def ref_quant_w(fq, w, idx, S, fmt):
    scale = w.max().float() / 2688.0 if fmt == "NVFP4" else torch.tensor(1.0)
    w32 = w[:, idx.long()].float() / scale
    q = fq.blockwise(w32, fmt)
    if S:
        q = torch.cat([q, fq.blockwise(w32[:, -S:], fmt)], dim=1)
    return q * scale


def ref_linear(fq, x, w, idx, S, fmt, bias=None, x_scale=None):
    y = ref_quant_x(fq, x, idx, S, fmt, x_scale) @ ref_quant_w(fq, w, idx, S, fmt).T
    y = y.to(torch.bfloat16)
    return y if bias is None else y + bias


@pytest.mark.parametrize("fmt", FMTS)
@pytest.mark.parametrize("bias", [False, True])
def test_qlinear_matches_fake_quant_flow(layers, fq, fmt, bias):
    M, N, K, S = 48, 320, 512, 64
    x = recipes.activations(M, K, seed=21)
    w = recipes.weights(N, K, seed=22)
    idx = recipes.reorder_index(x)
    lin = nn.Linear(K, N, bias=bias, device="cuda", dtype=torch.bfloat16)
    lin.weight.data.copy_(w)
    b = None
    if bias:
        b = (torch.randn(N, generator=torch.Generator().manual_seed(1)) * 0.1).to(torch.bfloat16)
        lin.bias.data.copy_(b)
    ql = layers.QLinearLayer(lin, S, idx, quant_type=fmt)
    tup = layers.quantize_tokens(x.cuda().view(4, 12, K), idx.cuda(), S, fmt)
    assert len(tup) == 5 and tup[3:] == (4, 12)
    y = ql(tup)
    assert y.shape == (4, 12, N) and y.dtype == torch.bfloat16
    want = ref_linear(fq, x, w, idx, S, fmt, b)
    assert rel_fro(y.reshape(M, N), want) < 5e-3        # bf16 output rounding + accumulation order
    # ragged form: bsz None -> [q_len, N] (model/qLinearLayer.py:78-80)
    y2 = ql(layers.quantize_tokens(x.cuda(), idx.cuda(), S, fmt))
    assert y2.shape == (M, N) and torch.equal(y2, y.reshape(M, N))


@pytest.mark.parametrize("fmt", FMTS)
def test_decoder_layer_matches_fake_quant_flow(layers, fq, fmt):
    hidden, inter, nh, nkv, S, eps = 256, 512, 4, 2, 64, 1e-5
    bsz, q_len = 2, 24
    layer = layers.LlamaDecoderLayer(hidden, inter, nh, nkv, eps=eps, select_num=S, select_num_down=S,
                                     quant_type=fmt, seed=4)
    g = torch.Generator().manual_seed(8)
    x = torch.randn(bsz, q_len, hidden, generator=g).to(torch.bfloat16)
    y = layer(x.cuda())
    assert y.shape == x.shape

    # the same flow on the CPU with the torch oracle
    W = {k: v.weight.data.cpu() for k, v in layer.linears.items()}
    g1, g2 = layer.input_layernorm.weight.cpu(), layer.post_attention_layernorm.weight.cpu()
    ih, ii = torch.arange(hidden), torch.arange(inter)
    one = torch.tensor(1.0)
    d = hidden // nh

    def attn(h2d):
        qkv = ref_linear(fq, fq.hf_rmsnorm(h2d, g1, eps), W["qkv"], ih, S, fmt, x_scale=one)
        q = qkv[:, :nh * d].view(bsz, q_len, nh, d).transpose(1, 2)
        k = qkv[:, nh * d:(nh + nkv) * d].view(bsz, q_len, nkv, d).transpose(1, 2)
        v = qkv[:, (nh + nkv) * d:].view(bsz, q_len, nkv, d).transpose(1, 2)
        q, k = layers.rotary_pos_emb(q, k, 0)
        k, v = k.repeat_interleave(nh // nkv, 1), v.repeat_interleave(nh // nkv, 1)
        o = F.scaled_dot_product_attention(q.float(), k.float(), v.float(), is_causal=True).to(torch.bfloat16)
        o = o.transpose(1, 2).reshape(bsz * q_len, hidden)
        return ref_linear(fq, o, W["o"], ih, S, fmt)

    x2 = x.view(-1, hidden)
    h = x2 + attn(x2)
    gu = ref_linear(fq, fq.hf_rmsnorm(h, g2, eps), W["gate_up"], ih, S, fmt, x_scale=one)
    t = F.silu(gu[:, :inter]) * gu[:, inter:]
    want = h + ref_linear(fq, t, W["down"], ii, S, fmt)
    # bf16 attention on the GPU vs fp32 here, and codes that flip where an intermediate differs by a
    # bf16 ulp: a few 1e-3 each; the quantization error itself (vs the bf16 layer) is ~1e-1
    assert rel_fro(y.view(-1, hidden), want) < 2e-2

    # decode step against the same layer run as a longer prefill: KV cache path
    kc = torch.zeros(bsz, nkv, 64, d, dtype=torch.bfloat16, device="cuda")
    vc = torch.zeros_like(kc)
    layer(x.cuda()[:, :q_len - 1], (kc, vc), 0)
    y_last = layer(x.cuda()[:, q_len - 1:], (kc, vc), q_len - 1)
    # NVFP4's tensor scale is taken over whatever batch is quantized, so the two runs differ by
    # quantization noise for NVFP4; MXFP4 has none and must agree to rounding
    tol = 0.15 if fmt == "NVFP4" else 2e-2
    assert rel_fro(y_last[:, 0], y[:, -1]) < tol


@pytest.mark.parametrize("fmt", FMTS)
@pytest.mark.parametrize("tokens", [(2, 24), (1, 1), (3, 100)])
def test_llama_mlp_fused_swiglu_equals_separate_pass(layers, fmt, tokens):
    """LlamaMLP with the SwiGLU formed in the gate_up GEMM's epilogue (interleaved weight rows) and with the
    separate SwiGLU -> quantize pass over [gate | up] (the default): the same bits, residual included"""
    hidden, inter, S = 384, 768, 128
    g = torch.Generator().manual_seed(61)
    gate_up = nn.Linear(hidden, 2 * inter, bias=False, device="cuda", dtype=torch.bfloat16)
    down = nn.Linear(inter, hidden, bias=False, device="cuda", dtype=torch.bfloat16)
    gate_up.weight.data.copy_((torch.randn(2 * inter, hidden, generator=g) * 0.05).to(torch.bfloat16))
    down.weight.data.copy_((torch.randn(hidden, inter, generator=g) * 0.05).to(torch.bfloat16))
    i_in = torch.randperm(hidden, generator=g).to(torch.int16).cuda()
    i_down = torch.randperm(inter, generator=g).to(torch.int16).cuda()
    fused = layers.LlamaMLP(gate_up, down, S, S, i_in, i_down, quant_type=fmt, interleave=True)
    plain = layers.LlamaMLP(gate_up, down, S, S, i_in, i_down, quant_type=fmt)
    assert fused.interleaved and not plain.interleaved
    x = torch.randn(*tokens, hidden, generator=g).to(torch.bfloat16).cuda()
    res = torch.randn(*tokens, hidden, generator=g).to(torch.bfloat16).cuda()
    tup = layers.quantize_tokens(x, i_in, S, fmt)
    print(f"llama mlp fused swiglu {fmt} tokens={tokens}", flush=True)
    assert torch.equal(fused(tup), plain(tup))
    assert torch.equal(fused(tup, residual=res), plain(tup, residual=res))


@pytest.mark.parametrize("fmt", FMTS)
@pytest.mark.parametrize("grouped,interleave", [(True, True), (True, False), (False, True), (False, False)])
def test_mixtral_block_matches_reference_loop(layers, fq, oracle, fmt, grouped, interleave):
    """The MoE block, as grouped launches over all experts and as the per-expert loop, against the
    reference's loop (model/qMixtralLayer.py:441-471) on the CPU; every expert has its own channel orders."""
    hidden, ffn, E, S = 384, 512, 4, 128
    tokens = 96
    g = torch.Generator().manual_seed(9)
    indices = [(torch.randperm(hidden, generator=g).to(torch.int16).cuda(),
                torch.randperm(ffn, generator=g).to(torch.int16).cuda()) for _ in range(E)]
    block = layers.build_mixtral_block(hidden, ffn, E, 2, S, fmt, indices=indices, seed=5, grouped=grouped,
                                       interleave=interleave)
    assert block.grouped == grouped and block.experts[0].interleaved == interleave
    x = torch.randn(1, tokens, hidden, generator=g).to(torch.bfloat16)
    logits = torch.randn(tokens, E, generator=g)
    logits[:, 3] -= 100.0                                   # an expert that receives no token
    print(f"mixtral block {fmt} grouped={grouped} interleave={interleave}", flush=True)
    y, _ = block(x.cuda(), router_logits=logits.cuda())
    assert y.shape == x.shape

    # model/qMixtralLayer.py:441-471 on the CPU; expert weights = w13 / w2 of the block as the CPU oracle dequantizes them
    def dq(lin):
        n = lin.W.shape[0]
        v = oracle.dequantize(lin.W.cpu().numpy(), lin.scale_w.cpu().numpy().reshape(n, -1), fmt)
        return torch.from_numpy(v) * lin.scale.cpu().float()
    w = F.softmax(logits, dim=1, dtype=torch.float)
    w, sel = torch.topk(w, 2, dim=-1)
    w = (w / w.sum(dim=-1, keepdim=True)).to(torch.bfloat16)
    want = torch.zeros(tokens, hidden, dtype=torch.bfloat16)
    x2 = x.view(tokens, hidden)
    for e in range(E):
        slot, top_x = torch.where((sel == e).T)
        if top_x.numel() == 0:
            continue
        ex = block.experts[e]
        ih, ii = indices[e][0].cpu(), indices[e][1].cpu()
        w13 = dq(ex.w13)
        if ex.interleaved:                                  # rows w1_0, w3_0, w1_1, ... -> [w1 | w3]
            w13 = torch.cat([w13[0::2], w13[1::2]])
        w2 = dq(ex.w2)
        cur = x2[top_x]
        hcur = (ref_quant_x(fq, cur, ih, S, fmt) @ w13.T).to(torch.bfloat16)
        t = F.silu(hcur[:, :ffn]) * hcur[:, ffn:]
        out = (ref_quant_x(fq, t, ii, S, fmt) @ w2.T).to(torch.bfloat16)
        want.index_add_(0, top_x, out * w[top_x, slot, None])
    assert rel_fro(y.view(tokens, hidden), want) < 2e-2
    assert float(y.abs().sum()) > 0


def test_mixtral_block_grouped_equals_loop_at_benchmark_size(layers):
    """Benchmark configuration 5: 8 experts, top-2, hidden 4096, intermediate 14336, 4096 tokens routed with
    a Zipf(1.1) skew over the experts, per-expert channel orders from the per-expert channel maxima,
    select_num 128, NVFP4.  The grouped launches against the per-expert loop of the same block (same
    quantized weights): the quantizers are bit-identical, the GEMMs differ in tile shape only."""
    hidden, ffn, E, S, tokens, fmt = 4096, 14336, 8, 128, 4096, "NVFP4"
    g = torch.Generator().manual_seed(55)
    x = recipes.activations(tokens, hidden, seed=5, outlier_frac=0.01, outlier_gain=40.0)
    zipf = 1.0 / torch.arange(1, E + 1, dtype=torch.float32) ** 1.1
    logits = torch.log(zipf)[None, :] + torch.randn(tokens, E, generator=g)
    sel = torch.topk(torch.softmax(logits, 1), 2, dim=-1).indices
    indices = []
    for e in range(E):
        mine = x[(sel == e).any(1)]
        i_in = recipes.reorder_index(mine if mine.numel() else x).cuda()
        indices.append((i_in, torch.randperm(ffn, generator=g).to(torch.int16).cuda()))
    block = layers.build_mixtral_block(hidden, ffn, E, 2, S, fmt, indices=indices, seed=5, grouped=True)
    assert block.grouped
    xc, lc = x.cuda().view(1, tokens, hidden), logits.cuda()
    print("mixtral block at configuration 5 size: grouped", flush=True)
    y_grouped, _ = block(xc, router_logits=lc)
    torch.cuda.synchronize()
    block.grouped = False
    print("mixtral block at configuration 5 size: per-expert loop", flush=True)
    y_loop, _ = block(xc, router_logits=lc)
    torch.cuda.synchronize()
    counts = torch.bincount(sel.reshape(-1), minlength=E).tolist()
    assert max(counts) > 3 * min(counts)                     # the skew is there
    assert rel_fro(y_grouped, y_loop) < 5e-3                 # bf16 roundings of differently ordered fp32 sums
    assert float(y_loop.abs().sum()) > 0


@pytest.mark.parametrize("fmt", FMTS)
def test_mixtral_block_replays_from_a_graph(layers, fmt):
    """The grouped block reads nothing back to the host, so it can be captured: every replay (new tokens and
    router logits copied into the captured inputs, eager work and a synchronisation between replays) gives
    what the eager call gives on the same inputs."""
    hidden, ffn, E, S, tokens = 384, 512, 4, 128, 96
    g = torch.Generator().manual_seed(19)
    block = layers.build_mixtral_block(hidden, ffn, E, 2, S, fmt, seed=7, grouped=True)
    x_in = torch.zeros(1, tokens, hidden, dtype=torch.bfloat16, device="cuda")
    l_in = torch.zeros(tokens, E, dtype=torch.float32, device="cuda")

    def fresh():
        return (torch.randn(1, tokens, hidden, generator=g).to(torch.bfloat16).cuda(),
                torch.randn(tokens, E, generator=g).cuda())

    x0, l0 = fresh()
    x_in.copy_(x0), l_in.copy_(l0)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):                      # warm-up on the capture stream: allocations happen here
        for _ in range(2):
            block(x_in, router_logits=l_in)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    print(f"mixtral block graph capture {fmt}", flush=True)
    with torch.cuda.graph(graph):
        y_out, _ = block(x_in, router_logits=l_in)
    for rep in range(3):
        x1, l1 = fresh()
        want, _ = block(x1, router_logits=l1)          # eager, between the replays
        torch.cuda.synchronize()
        x_in.copy_(x1), l_in.copy_(l1)
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(y_out, want), rep


@pytest.mark.parametrize("fmt", FMTS)
def test_graphed_decode_step_matches_eager(layers, fmt):
    """A decode step over the INT4 paged KV cache replayed from a captured HIP graph gives what the
    eager step gives, on every replay, with eager work and synchronisation between replays, across a
    page boundary (page size 16, lengths 14 -> 19)."""
    from arcquant_amd.kv_cache import MultiLayerPagedKVCache4Bit
    hidden, inter, nh, nkv, S, batch, page = 512, 1024, 4, 2, 64, 3, 16
    layer = layers.LlamaDecoderLayer(hidden, inter, nh, nkv, select_num=S, select_num_down=S, quant_type=fmt, seed=12)
    g = torch.Generator().manual_seed(13)
    prompt = torch.randn(batch, 14, hidden, generator=g).to(torch.bfloat16).cuda()
    caches = [MultiLayerPagedKVCache4Bit(batch, page, 64, "cuda", 1, nkv, 128, dtype=torch.bfloat16) for _ in range(2)]
    for c in caches:
        layer(prompt, c, 0)
    eager_cache, graph_cache = caches
    step = layers.GraphedDecodeStep(layer, graph_cache, batch, hidden)
    assert graph_cache.lengths == [14] * batch                      # capture left the cache where it was
    for i in range(5):
        x = torch.randn(batch, 1, hidden, generator=g).to(torch.bfloat16).cuda()
        print(f"graphed decode {fmt} step {i}", flush=True)
        want = layer(x, eager_cache, eager_cache.lengths[0])        # eager: position = current length
        torch.cuda.synchronize()
        got = step(x).clone()
        torch.cuda.synchronize()
        assert graph_cache.lengths == eager_cache.lengths
        assert torch.equal(got, want), float((got.float() - want.float()).abs().max())
    assert torch.equal(graph_cache.pages, eager_cache.pages) and torch.equal(graph_cache.scales, eager_cache.scales)


def test_graphed_decode_steps_of_two_layers_share_one_cache(layers):
    """Two decoder layers over one two-layer INT4 cache, one graphed step per layer: the cache advances
    once per token (by the first layer's step), and every replay gives what the eager layers give."""
    from arcquant_amd.kv_cache import MultiLayerPagedKVCache4Bit
    fmt, hidden, inter, nh, nkv, S, batch, page = "MXFP4", 512, 1024, 4, 2, 64, 3, 16
    model = [layers.LlamaDecoderLayer(hidden, inter, nh, nkv, select_num=S, select_num_down=S, quant_type=fmt, seed=20 + i)
             for i in range(2)]
    g = torch.Generator().manual_seed(21)
    prompt = torch.randn(batch, 15, hidden, generator=g).to(torch.bfloat16).cuda()
    caches = [MultiLayerPagedKVCache4Bit(batch, page, 64, "cuda", 2, nkv, 128, dtype=torch.bfloat16) for _ in range(2)]
    for c in caches:
        h = prompt
        for i, layer in enumerate(model):
            h = layer(h, c, 0, i)
    eager_cache, graph_cache = caches
    steps = [layers.GraphedDecodeStep(layer, graph_cache, batch, hidden, layer_idx=i) for i, layer in enumerate(model)]
    assert graph_cache.lengths == [15] * batch
    for t in range(4):                                              # lengths 15 -> 19: crosses a page boundary
        x = torch.randn(batch, 1, hidden, generator=g).to(torch.bfloat16).cuda()
        print(f"two-layer graphed decode, token {t}", flush=True)
        pos = eager_cache.lengths[0]
        want = x
        for i, layer in enumerate(model):
            want = layer(want, eager_cache, pos, i)
        torch.cuda.synchronize()
        got = x
        for st in steps:
            got = st(got)
        got = got.clone()
        torch.cuda.synchronize()
        assert graph_cache.lengths == eager_cache.lengths == [16 + t] * batch
        assert torch.equal(got, want), float((got.float() - want.float()).abs().max())
    assert torch.equal(graph_cache.pages, eager_cache.pages) and torch.equal(graph_cache.scales, eager_cache.scales)


def test_chunked_prefill_is_causal(layers):
    """q_len > 1 behind cached tokens over the bf16 (k, v) cache: the second chunk's outputs equal the
    same rows of one full causal prefill (MXFP4: no tensor scale, so the two runs quantize alike)."""
    hidden, inter, nh, nkv, S = 512, 1024, 4, 2, 64
    layer = layers.LlamaDecoderLayer(hidden, inter, nh, nkv, select_num=S, select_num_down=S, quant_type="MXFP4", seed=31)
    g = torch.Generator().manual_seed(32)
    x = torch.randn(2, 24, hidden, generator=g).to(torch.bfloat16).cuda()
    full = layer(x)
    kv = (torch.zeros(2, nkv, 32, 128, dtype=torch.bfloat16, device="cuda"),
          torch.zeros(2, nkv, 32, 128, dtype=torch.bfloat16, device="cuda"))
    first = layer(x[:, :16].contiguous(), kv, 0)
    second = layer(x[:, 16:].contiguous(), kv, 16)
    assert rel_fro(first, full[:, :16]) < 2e-2
    assert rel_fro(second, full[:, 16:]) < 2e-2


@pytest.mark.parametrize("fmt", FMTS)
def test_decoder_layer_from_calibration_files(layers, fq, oracle, fmt, tmp_path):
    """The reference's way of building a layer (model/qLlamaLayer.py:88-262): calibration dicts in its
    file format (reorder_indices.py:88-97), keyed 'layers.{i}.{block}.{proj}.input', loaded from disk and
    handed to the constructors with the layer's own nn.Linear modules.  q / k / v / gate / up stay
    separate, each with the NVFP4 tensor scale of its own weight: their weight codes and scale bytes are
    compared bit for bit with the oracle's per-projection quantizer, the layer output with the
    fake-quant flow on the CPU."""
    from arcquant_amd import calibration as cal
    hidden, inter, nh, nkv, eps, li = 256, 512, 4, 2, 1e-5, 3
    bsz, q_len = 2, 24
    d = hidden // nh
    g = torch.Generator().manual_seed(41)
    shapes = {"q_proj": (nh * d, hidden), "k_proj": (nkv * d, hidden), "v_proj": (nkv * d, hidden),
              "o_proj": (hidden, hidden), "gate_proj": (inter, hidden), "up_proj": (inter, hidden),
              "down_proj": (hidden, inter)}
    gain = {"q_proj": 1.0, "k_proj": 3.0, "v_proj": 0.5, "o_proj": 1.0, "gate_proj": 2.0, "up_proj": 0.7, "down_proj": 1.0}
    W = {k: (torch.randn(*s, generator=g) * 0.02 * gain[k]).to(torch.bfloat16) for k, s in shapes.items()}
    g1 = (torch.rand(hidden, generator=g) + 0.5).to(torch.bfloat16)
    g2 = (torch.rand(hidden, generator=g) + 0.5).to(torch.bfloat16)
    x = torch.randn(bsz, q_len, hidden, generator=g)
    x[..., 7] *= 20.0
    x = x.to(torch.bfloat16)

    # calibration statistics: per-channel max |activation| of each linear's input on a calibration batch
    # (utilize.py:39-45); here random statistics per input, written and read back in the reference's format
    stat = {"attn": torch.rand(hidden, generator=g), "o": torch.rand(hidden, generator=g),
            "mlp": torch.rand(hidden, generator=g), "down": torch.rand(inter, generator=g)}
    block_of = {"q_proj": ("self_attn", "attn", 64), "k_proj": ("self_attn", "attn", 64), "v_proj": ("self_attn", "attn", 64),
                "o_proj": ("self_attn", "o", 128), "gate_proj": ("mlp", "mlp", 64), "up_proj": ("mlp", "mlp", 64),
                "down_proj": ("mlp", "down", 192)}
    ri, sn = {}, {}
    for proj, (block, st, sel) in block_of.items():
        key = cal.NAME_TEMPLATE.format(li, block, proj)
        ri[key] = cal.reorder_index_from_stat(stat[st])
        sn[key] = sel
    cal.save_reorder_index(tmp_path / "reorder_index.pt", ri)
    cal.save_select_num(tmp_path / "select_num.pt", sn)
    ri, sn = cal.load_reorder_index(tmp_path / "reorder_index.pt"), cal.load_select_num(tmp_path / "select_num.pt")

    lin = {}
    for k, (n_out, n_in) in shapes.items():
        lin[k] = nn.Linear(n_in, n_out, bias=False, device="cuda", dtype=torch.bfloat16)
        lin[k].weight.data.copy_(W[k])
    print(f"calibrated decoder layer {fmt}", flush=True)
    layer = layers.QLlamaDecoderLayer(lin, (g1.cuda(), g2.cuda()), eps, nh, nkv, sn, ri, li, quant_type=fmt)
    with pytest.raises(KeyError):
        layers.QLlamaDecoderLayer(lin, (g1.cuda(), g2.cuda()), eps, nh, nkv, sn, ri, li + 1, quant_type=fmt)

    # weight codes / scales of every projection = the oracle's quantizer with that projection's own tensor scale
    mods = {"q_proj": layer.self_attn.q_proj, "k_proj": layer.self_attn.k_proj, "v_proj": layer.self_attn.v_proj,
            "o_proj": layer.self_attn.o_proj, "gate_proj": layer.mlp.gate_proj, "up_proj": layer.mlp.up_proj,
            "down_proj": layer.mlp.down_proj}
    idx_of = {}
    for proj, (block, st, sel) in block_of.items():
        idx = ri[cal.NAME_TEMPLATE.format(li, block, proj)].to(torch.int16)
        idx_of[proj] = (idx, sel)
        gw = recipes.tensor_scale(W[proj], fmt)
        want = oracle.quantize_w(W[proj], idx, sel, fmt, gw)
        m = mods[proj]
        assert (m.W.cpu().numpy() == want["codes"]).all(), proj
        assert (m.scale_w.cpu().numpy().reshape(want["scales"].shape) == want["scales"]).all(), proj
        assert float(m.scale) == pytest.approx(gw, rel=1e-7)
    if fmt == "NVFP4":
        assert len({float(mods[p].scale) for p in ("q_proj", "k_proj", "v_proj")}) == 3

    y = layer(x.cuda())
    assert y.shape == x.shape

    def lin_ref(t, proj):
        idx, sel = idx_of[proj]
        return ref_linear(fq, t, W[proj], idx, sel, fmt)

    x2 = x.view(-1, hidden)
    n1 = fq.hf_rmsnorm(x2, g1, eps)
    qkv = torch.cat([lin_ref(n1, p) for p in ("q_proj", "k_proj", "v_proj")], dim=1)
    q = qkv[:, :nh * d].view(bsz, q_len, nh, d).transpose(1, 2)
    k = qkv[:, nh * d:(nh + nkv) * d].view(bsz, q_len, nkv, d).transpose(1, 2)
    v = qkv[:, (nh + nkv) * d:].view(bsz, q_len, nkv, d).transpose(1, 2)
    q, k = layers.rotary_pos_emb(q, k, 0)
    k, v = k.repeat_interleave(nh // nkv, 1), v.repeat_interleave(nh // nkv, 1)
    o = F.scaled_dot_product_attention(q.float(), k.float(), v.float(), is_causal=True).to(torch.bfloat16)
    h = x2 + lin_ref(o.transpose(1, 2).reshape(bsz * q_len, hidden), "o_proj")
    n2 = fq.hf_rmsnorm(h, g2, eps)
    t = F.silu(lin_ref(n2, "gate_proj")) * lin_ref(n2, "up_proj")
    want = h + lin_ref(t, "down_proj")
    assert rel_fro(y.view(-1, hidden), want) < 2e-2       # as test_decoder_layer_matches_fake_quant_flow

    # the fused norm -> quantize form of the same layer (tensor scale 1) stays within quantization noise of it
    fused = layers.QLlamaDecoderLayer(lin, (g1.cuda(), g2.cuda()), eps, nh, nkv, sn, ri, li, quant_type=fmt,
                                      fuse_norm=True)
    assert rel_fro(fused(x.cuda()), y) < 0.1


def c_ref_linear(oracle, x, w, idx, S, fmt, bias=None):
    """one ARC linear of the fake-quant flow through the C oracle (model/quantize.py:287-343, model/qLinearLayer.py:65-81):
    activations with the callers' tensor scale max|x| / 2688, weights with the signed max / 2688, fp32 product of the
    dequantized operands, bf16 output, bias behind it"""
    import numpy as np
    gx = float(x.abs().max().float() / torch.tensor(2688.0)) if fmt == "NVFP4" else 1.0
    gw = recipes.tensor_scale(w, fmt)
    a = oracle.quantize_x(x, idx, S, fmt, gx, want_dq=True)["dq"]
    b = oracle.quantize_w(w, idx, S, fmt, gw, want_dq=True)["dq"]
    y = (torch.from_numpy(a) @ torch.from_numpy(b).T * np.float32(gx * gw)).to(torch.bfloat16)
    return y if bias is None else y + bias


@pytest.mark.parametrize("fmt", FMTS)
def test_qwen_decoder_layer_at_its_geometry(layers, fq, oracle, fmt, tmp_path):
    """Qwen2.5-7B's decoder layer (model/qQwenLayer.py:88-176, 227-249, 374-391): hidden 3584, 28 query and 4 KV
    heads of 128, q / k / v with bias, intermediate 18944 -- the down projection's input is wider than 16384
    channels and takes the four-units-per-thread quantizers.  Built from calibration files; 48 tokens against the
    fake-quant flow on the CPU (C oracle quantizers, fp32 products)."""
    from arcquant_amd import calibration as cal
    hidden, inter, nh, nkv, eps, li = 3584, 18944, 28, 4, 1e-6, 0
    bsz, q_len, d = 2, 24, 128
    g = torch.Generator().manual_seed(71)
    shapes = {"q_proj": (nh * d, hidden), "k_proj": (nkv * d, hidden), "v_proj": (nkv * d, hidden),
              "o_proj": (hidden, hidden), "gate_proj": (inter, hidden), "up_proj": (inter, hidden),
              "down_proj": (hidden, inter)}
    W = {k: (torch.randn(*s, generator=g) * 0.02).to(torch.bfloat16) for k, s in shapes.items()}
    B = {k: (torch.randn(shapes[k][0], generator=g) * 0.2).to(torch.bfloat16) for k in ("q_proj", "k_proj", "v_proj")}
    g1 = (torch.rand(hidden, generator=g) + 0.5).to(torch.bfloat16)
    g2 = (torch.rand(hidden, generator=g) + 0.5).to(torch.bfloat16)
    x = torch.randn(bsz, q_len, hidden, generator=g)
    x[..., 11] *= 20.0
    x = x.to(torch.bfloat16)
    stat = {"attn": torch.rand(hidden, generator=g), "o": torch.rand(hidden, generator=g),
            "mlp": torch.rand(hidden, generator=g), "down": torch.rand(inter, generator=g)}
    block_of = {"q_proj": ("self_attn", "attn", 128), "k_proj": ("self_attn", "attn", 128), "v_proj": ("self_attn", "attn", 128),
                "o_proj": ("self_attn", "o", 128), "gate_proj": ("mlp", "mlp", 128), "up_proj": ("mlp", "mlp", 128),
                "down_proj": ("mlp", "down", 256)}
    ri, sn = {}, {}
    for proj, (block, st, sel) in block_of.items():
        key = cal.NAME_TEMPLATE.format(li, block, proj)
        ri[key] = cal.reorder_index_from_stat(stat[st])
        sn[key] = sel
    cal.save_reorder_index(tmp_path / "reorder_index.pt", ri)
    cal.save_select_num(tmp_path / "select_num.pt", sn)
    ri, sn = cal.load_reorder_index(tmp_path / "reorder_index.pt"), cal.load_select_num(tmp_path / "select_num.pt")
    lin = {}
    for k, (n_out, n_in) in shapes.items():
        lin[k] = nn.Linear(n_in, n_out, bias=k in B, device="cuda", dtype=torch.bfloat16)
        lin[k].weight.data.copy_(W[k])
        if k in B:
            lin[k].bias.data.copy_(B[k])
    print(f"Qwen2.5-7B decoder layer {fmt}", flush=True)
    layer = layers.QQwen2DecoderLayer(lin, (g1.cuda(), g2.cuda()), eps, nh, nkv, sn, ri, li, quant_type=fmt)
    assert isinstance(layer.self_attn, layers.QQwen2Attention) and isinstance(layer.mlp, layers.QQwen2MLP)
    assert layer.self_attn.q_proj.bias is not None and layer.self_attn.o_proj.bias is None
    # the wide projection's weights: codes and scale bytes against the oracle
    idx_d = ri[cal.NAME_TEMPLATE.format(li, "mlp", "down_proj")].to(torch.int16)
    want = oracle.quantize_w(W["down_proj"], idx_d, 256, fmt, recipes.tensor_scale(W["down_proj"], fmt))
    assert (layer.mlp.down_proj.W.cpu().numpy() == want["codes"]).all()
    assert (layer.mlp.down_proj.scale_w.cpu().numpy().reshape(want["scales"].shape) == want["scales"]).all()

    y = layer(x.cuda())
    torch.cuda.synchronize()
    assert y.shape == x.shape

    def lin_ref(t, proj):
        block, st, sel = block_of[proj]
        idx = ri[cal.NAME_TEMPLATE.format(li, block, proj)].to(torch.int16)
        return c_ref_linear(oracle, t, W[proj], idx, sel, fmt, B.get(proj))

    x2 = x.view(-1, hidden)
    n1 = fq.hf_rmsnorm(x2, g1, eps)
    qkv = torch.cat([lin_ref(n1, p) for p in ("q_proj", "k_proj", "v_proj")], dim=1)
    q = qkv[:, :nh * d].view(bsz, q_len, nh, d).transpose(1, 2)
    k = qkv[:, nh * d:(nh + nkv) * d].view(bsz, q_len, nkv, d).transpose(1, 2)
    v = qkv[:, (nh + nkv) * d:].view(bsz, q_len, nkv, d).transpose(1, 2)
    q, k = layers.rotary_pos_emb(q, k, 0)
    k, v = k.repeat_interleave(nh // nkv, 1), v.repeat_interleave(nh // nkv, 1)
    o = F.scaled_dot_product_attention(q.float(), k.float(), v.float(), is_causal=True).to(torch.bfloat16)
    h = x2 + lin_ref(o.transpose(1, 2).reshape(bsz * q_len, hidden), "o_proj")
    n2 = fq.hf_rmsnorm(h, g2, eps)
    t = F.silu(lin_ref(n2, "gate_proj")) * lin_ref(n2, "up_proj")
    want = h + lin_ref(t, "down_proj")
    # Block by block, each fed the reference's input: a 4-bit layer turns a 1 % difference of its input (here the
    # bf16 attention against the fp32 one, then requantized) into a different set of codes, i.e. into its own
    # quantization noise, so the end-to-end figure says little about the operators
    a, m = layer.self_attn, layer.mlp
    xc = x.cuda()
    n1g = layer.input_layernorm(xc)
    assert torch.equal(n1g.view(-1, hidden).cpu(), n1)
    tq = layers.quantize_tokens(n1g, a.q_reorder_index, a.q_proj.select_num, fmt)
    assert rel_fro(a.qkv_proj(tq).view(-1, qkv.shape[1]), qkv) < 5e-3          # three projections with their biases
    assert rel_fro(a(tq, None, 0, li, residual=xc).view(-1, hidden), h) < 2e-2   # bf16 SDPA, o_proj on its output
    hc = h.cuda().view(bsz, q_len, hidden)
    tq2 = layers.quantize_tokens(layer.post_attention_layernorm(hc), m.up_reorder_index, m.up_proj.select_num, fmt)
    assert rel_fro(m(tq2, residual=hc).view(-1, hidden), want) < 5e-3          # gate / up, SwiGLU over 18944 channels, down
    assert rel_fro(y.view(-1, hidden), want) < 0.25                            # the whole layer: within quantization noise


@pytest.mark.parametrize("fmt", FMTS)
@pytest.mark.parametrize("grouped", [True, False])
def test_mixtral_block_from_calibration_files(layers, oracle, fmt, grouped, tmp_path):
    """The reference's way of building the MoE block (model/qMixtralLayer.py:400-420, 488-508): calibration dicts
    keyed 'layers.{i}.block_sparse_moe.experts.{e}.w{1,2,3}.input' written and read in its file format, every
    expert's w1 / w3 / w2 a QLinearLayer of its own (weight codes and scale bytes bit for bit the oracle's, each
    with the tensor scale of its own weight); the block's output against the reference's loop over experts with
    the C oracle's quantizers on the CPU (model/qMixtralLayer.py:441-471, 523-543)."""
    from arcquant_amd import calibration as cal
    hidden, ffn, E, li, tokens = 384, 512, 4, 5, 96
    g = torch.Generator().manual_seed(81)
    ri, sn, Wt = {}, {}, []
    for e in range(E):
        i_in = cal.reorder_index_from_stat(torch.rand(hidden, generator=g))
        i_w2 = cal.reorder_index_from_stat(torch.rand(ffn, generator=g))
        for proj, idx, sel in (("w1", i_in, 128), ("w3", i_in, 128), ("w2", i_w2, 128)):
            ri[cal.MOE_NAME_TEMPLATE.format(li, e, proj)] = idx
            sn[cal.MOE_NAME_TEMPLATE.format(li, e, proj)] = sel
        Wt.append({"w1": (torch.randn(ffn, hidden, generator=g) * 0.05 * (1 + e)).to(torch.bfloat16),
                   "w3": (torch.randn(ffn, hidden, generator=g) * 0.02).to(torch.bfloat16),
                   "w2": (torch.randn(hidden, ffn, generator=g) * 0.03).to(torch.bfloat16)})
    cal.save_reorder_index(tmp_path / "ri.pt", ri)
    cal.save_select_num(tmp_path / "sn.pt", sn)
    ri, sn = cal.load_reorder_index(tmp_path / "ri.pt"), cal.load_select_num(tmp_path / "sn.pt")

    def linear(w):
        m = nn.Linear(w.shape[1], w.shape[0], bias=False, device="cuda", dtype=torch.bfloat16)
        m.weight.data.copy_(w)
        return m
    gate = nn.Linear(hidden, E, bias=False, device="cuda", dtype=torch.bfloat16)
    experts = [(linear(w["w1"]), linear(w["w3"]), linear(w["w2"])) for w in Wt]
    print(f"calibrated mixtral block {fmt} grouped={grouped}", flush=True)
    block = layers.QMixtralSparseMoeBlock(gate, experts, sn, ri, li, quant_type=fmt, grouped=grouped)
    assert block.grouped == grouped
    with pytest.raises(KeyError):
        layers.QMixtralSparseMoeBlock(gate, experts, sn, ri, li + 1, quant_type=fmt)
    for e, ex in enumerate(block.experts):
        for proj in ("w1", "w3", "w2"):
            key = cal.MOE_NAME_TEMPLATE.format(li, e, proj)
            gw = recipes.tensor_scale(Wt[e][proj], fmt)
            want = oracle.quantize_w(Wt[e][proj], ri[key].to(torch.int16), sn[key], fmt, gw)
            m = getattr(ex, proj)
            assert (m.W.cpu().numpy() == want["codes"]).all(), (e, proj)
            assert (m.scale_w.cpu().numpy().reshape(want["scales"].shape) == want["scales"]).all(), (e, proj)
            assert float(m.scale) == pytest.approx(gw, rel=1e-7)
    if fmt == "NVFP4":
        assert float(block.experts[1].w1.scale) != float(block.experts[1].w3.scale)

    x = torch.randn(1, tokens, hidden, generator=g).to(torch.bfloat16)
    logits = torch.randn(tokens, E, generator=g)
    logits[:, 2] -= 100.0                                   # an expert that receives no token
    y, _ = block(x.cuda(), router_logits=logits.cuda())
    torch.cuda.synchronize()

    w = F.softmax(logits, dim=1, dtype=torch.float)
    w, sel = torch.topk(w, 2, dim=-1)
    w = (w / w.sum(dim=-1, keepdim=True)).to(torch.bfloat16)
    want = torch.zeros(tokens, hidden, dtype=torch.bfloat16)
    x2 = x.view(tokens, hidden)
    for e in range(E):
        slot, top_x = torch.where((sel == e).T)
        if top_x.numel() == 0:
            continue
        k1, k2 = cal.MOE_NAME_TEMPLATE.format(li, e, "w1"), cal.MOE_NAME_TEMPLATE.format(li, e, "w2")
        cur = x2[top_x]
        h1 = c_ref_linear(oracle, cur, Wt[e]["w1"], ri[k1].to(torch.int16), sn[k1], fmt)
        h3 = c_ref_linear(oracle, cur, Wt[e]["w3"], ri[k1].to(torch.int16), sn[k1], fmt)
        out = c_ref_linear(oracle, F.silu(h1) * h3, Wt[e]["w2"], ri[k2].to(torch.int16), sn[k2], fmt)
        want.index_add_(0, top_x, out * w[top_x, slot, None])
    assert rel_fro(y.view(tokens, hidden), want) < 2e-2
    # w3's entry must agree with w1's: both projections read one quantized input (model/qMixtralLayer.py:530-535)
    bad = dict(ri)
    bad[cal.MOE_NAME_TEMPLATE.format(li, 0, "w3")] = torch.flip(ri[cal.MOE_NAME_TEMPLATE.format(li, 0, "w3")], [0])
    with pytest.raises(ValueError):
        layers.QMixtralSparseMoeBlock(gate, experts, sn, bad, li, quant_type=fmt)
