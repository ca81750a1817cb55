#!/usr/bin/env python3
"""Benchmark of the ARC quantized-linear hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--quick] [--headline-only] [--no-cpu]

Prints ONE JSON line.  A "step" is one launch of the fused RMSNorm + reorder + quantize kernel
over one batch of synthetic activations already resident in HBM: M=4096 tokens, hidden 4096,
select_num=256, NVFP4, eps=1e-5, global scale 1 (benchmark configuration 2 at its largest M).
Inputs rotate over enough distinct buffers that the working set exceeds the 256 MB Infinity
Cache, so the rate is an HBM rate, not a cache rate.

  value          algorithmic GB/s over the timed region (wall clock around K launches)
  roofline       the same kernel against the 8 TB/s HBM peak, from HIP events around each launch
  cpu_baseline   the reference's fake-quant arithmetic (torch restatement, oracle/fakequant_torch.py)
                 timed on this box's host cores on a bounded sample of the same workload
  quantize       benchmark configuration 2 in full: fused norm at M in {1, 16, 256, 4096}, select_num in
                 {64, 256}, both formats, plus the plain quantizers at M = 4096
  gemm           benchmark configuration 3 in full: ARC FP4 GEMM at the four Llama-3-8B projection shapes
                 x M in {1, 16, 128, 512, 2048, 4096}, both formats, next to torch's bf16 GEMM of the same
                 (M, N, K'), each with its fraction of the MFMA peak
  layers         benchmark configurations 4 and 5: a decoder layer (prefill 8 x 2048, decode batch 64) and a
                 Mixtral MoE block, reorder indices from channel maxima, next to the same layer in bf16
Everything but the headline step sits outside the timed region.  --quick drops the layer rows and half of
the GEMM rows; --headline-only (for counter runs) keeps the headline kernel and the copy kernels only.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))

HBM_PEAK_GBS = 8000.0            # MI355X HBM3E, published
MFMA_PEAK_TFLOPS = {"MXFP4": 10100.0, "NVFP4": 2500.0, "bf16": 2500.0}   # dense fp4 / bf16 (NVFP4 runs on bf16 MFMA)

H, M_TOKENS, SELECT, EPS = 4096, 4096, 256, 1e-5
FMT = "NVFP4"
# HBM bytes per launch of the headline kernel come from rocprofv3 --pmc FETCH_SIZE and WRITE_SIZE (two
# runs), each scaled by what the same counter reads for arcq_stream_probe moving a known number of bytes.
# The summary of those runs under profiles/ carries the figure on a line of its own together with the
# kernel and the workload it was measured on; it is taken from there, and only for that workload.
TRAFFIC_PROFILE = os.path.join(ROOT, "profiles", "rmsnorm_quantize_nvfp4_4096x4096_hbm_traffic.md")


def measured_traffic(workload_key):
    """(bytes per launch, kernel, source file) from the committed counter summary, or (None, None, None)
    when it is absent or covers another workload"""
    import re
    try:
        text = open(TRAFFIC_PROFILE).read()
    except OSError:
        return None, None, None
    m = re.search(r"^traffic_bytes_per_launch\s*=\s*(\d+)\s*;\s*kernel\s*=\s*(.+?)\s*;\s*workload\s*=\s*(.+?)\s*$", text, re.M)
    if not m or m.group(3) != workload_key:
        return None, None, None
    return int(m.group(1)), m.group(2), os.path.relpath(TRAFFIC_PROFILE, ROOT)


def quant_bytes(M, K, S, fmt, fused_norm):
    """algorithmic bytes of one quantize launch: bf16 rows in, codes + scale bytes out, index
    (and gamma) once"""
    G = 16 if fmt == "NVFP4" else 32
    per_row = 2 * K + (K + S) // 2 + (K + S) // G
    return M * per_row + 2 * K + (2 * K if fused_norm else 0)


def gemm_flops(M, N, Kp):
    return 2.0 * M * N * Kp


def event_times_ms(fn, n, torch):
    """per-launch durations from HIP events recorded on the launch stream"""
    evs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(n)]
    for i, (a, b) in enumerate(evs):
        a.record()
        fn(i)
        b.record()
    torch.cuda.synchronize()
    return [a.elapsed_time(b) for a, b in evs]


def loop_time_ms(fn, n, torch):
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    a.record()
    for i in range(n):
        fn(i)
    b.record()
    torch.cuda.synchronize()
    return a.elapsed_time(b) / n


def cpu_baseline(torch, sample_rows):
    """reference fake-quant path on the host: HF RMSNorm -> gather -> fake_reorder_quantize_x"""
    import recipes
    from oracle import fakequant_torch as fq

    threads = os.cpu_count() or 1
    threads = min(threads, int(os.environ.get("OMP_NUM_THREADS", threads)))
    torch.set_num_threads(threads)
    x = recipes.activations(sample_rows, H, seed=2, outlier_frac=0.005, outlier_gain=50.0)
    gam = recipes.gamma(H, seed=7)
    idx = recipes.reorder_index(fq.hf_rmsnorm(x, gam, EPS)).long()
    best, total, runs = float("inf"), 0.0, 0
    while runs < 3 or (total < 10.0 and runs < 40):       # about 10 s of CPU work, at least 3 runs
        t0 = time.perf_counter()
        y = fq.hf_rmsnorm(x, gam, EPS)
        fq.fake_quantize_x(torch.index_select(y, 1, idx), SELECT, FMT)
        dt = time.perf_counter() - t0
        best, total, runs = min(best, dt), total + dt, runs + 1
    gbs = quant_bytes(sample_rows, H, SELECT, FMT, True) / best / 1e9
    return {"value": round(gbs, 4), "unit": "GB/s", "cores": threads, "kind": "port",
            "sample": f"{sample_rows} of {M_TOKENS} rows of the same workload (torch restatement of "
                      f"model/quantize.py fake_reorder_quantize_x after HF RMSNorm), best of {runs} runs, {best:.3f} s each"}


def mfma_sustained(torch, iters=4000):
    """What the matrix pipe sustains in a register-only loop (no loads, LDS or barriers) on all 256 CUs, by
    instruction and by operand data: the chip lowers its clock under the multipliers' switching power, so the
    ceiling for real operands is well below the data-sheet peak that roofline fractions are quoted against."""
    import ctypes
    from arcquant_amd import _lib
    P = _lib.probe_lib()
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    g = torch.Generator().manual_seed(11)
    rnd = torch.randint(-2 ** 31, 2 ** 31 - 1, (4096,), generator=g, dtype=torch.int64).to(torch.int32)
    # fp16 values as the NVFP4 decode produces them: an FP4 magnitude times (1 + m/8) * 2^e, random signs
    mags = torch.tensor([0, .5, 1, 1.5, 2, 3, 4, 6])[torch.randint(0, 8, (8192,), generator=g)]
    vals = mags * (1 + torch.randint(0, 8, (8192,), generator=g) / 8.0) * torch.pow(2.0, torch.randint(-3, 3, (8192,), generator=g).float())
    vals = (vals * (torch.randint(0, 2, (8192,), generator=g) * 2 - 1)).to(torch.float16)
    gauss = torch.randn(8192, generator=g).to(torch.bfloat16)
    data = {"zeros": torch.zeros(4096, dtype=torch.int32), "random bits": rnd,
            "decoded FP4 x E4M3 as fp16": vals.view(torch.int32), "N(0,1) as bf16": gauss.view(torch.int32)}
    out = torch.empty(256 * 512, dtype=torch.float32, device="cuda")
    rows = []
    for kind, name, kinds_of_data in ((0, "v_mfma_scale_f32_32x32x64_f8f6f4 (FP4, E8M0 scales)", ("zeros", "random bits")),
                                      (1, "v_mfma_f32_32x32x16_f16", ("zeros", "random bits", "decoded FP4 x E4M3 as fp16")),
                                      (2, "v_mfma_f32_32x32x16_bf16", ("zeros", "random bits", "N(0,1) as bf16"))):
        for dname in kinds_of_data:
            src = data[dname].cuda()
            for wps in (1, 2):
                P.arcq_mfma_rate_probe(kind, wps, 50, src.data_ptr(), out.data_ptr(), stream)
                torch.cuda.synchronize()
                a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                a.record()
                P.arcq_mfma_rate_probe(kind, wps, iters, src.data_ptr(), out.data_ptr(), stream)
                b.record()
                torch.cuda.synchronize()
                ms = a.elapsed_time(b)
                rows.append({"instruction": name, "operands": dname, "waves_per_simd": wps,
                             "tflops": round(P.arcq_mfma_rate_probe_flops(kind, wps, iters) / ms / 1e9, 1)})
    return rows


def gemm_rows(torch, agemm, shapes, Ms, fmts, iters=40):
    """ARC GEMM through the C ABI on preallocated outputs.  The quantized weights rotate over enough
    copies (> 300 MB) that every launch streams them from HBM, as a model's layers do; the bf16
    comparison rotates the same way.  For M <= 64 the bound is the weight stream, reported as GB/s."""
    import ctypes
    import recipes
    from arcquant_amd import _lib
    L = _lib.lib()
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    fid = {"NVFP4": 0, "MXFP4": 1}
    rows = []
    for (N, K) in shapes:
        S = 256
        Kp = K + S
        w = recipes.weights(N, K, seed=3).cuda()
        idx = torch.arange(K, dtype=torch.int16, device="cuda")
        wq = {}
        for f in fmts:
            b, sfb = agemm.reorder_quantize_w(w, idx, S, fmt=f, global_scale=recipes.tensor_scale(w.cpu(), f))
            ncopy = max(2, int(3.2e8 // (b.numel() + sfb.numel())) + 1)
            wq[f] = [(b.clone(), sfb.clone()) for _ in range(ncopy)]
        nb = max(2, int(3.2e8 // (N * Kp * 2)) + 1)
        wbs = [torch.randn(N, Kp, device="cuda", dtype=torch.bfloat16) for _ in range(nb)]
        for M in Ms:
            x = recipes.activations(M, K, seed=1).cuda()
            row = {"N": N, "K": K, "Kp": Kp, "M": M}
            c = torch.empty(M, N, dtype=torch.bfloat16, device="cuda")
            for f in fmts:
                a, sfa = agemm.reorder_quantize_x(x, idx, S, fmt=f, global_scale=recipes.tensor_scale(x.cpu(), f))
                ws = wq[f]

                def fn(i, a=a, sfa=sfa, ws=ws, f=f):
                    b, sfb = ws[i % len(ws)]
                    L.arcq_matmul(a.data_ptr(), sfa.data_ptr(), b.data_ptr(), sfb.data_ptr(), M, N, Kp, fid[f], 1.0,
                                  None, None, c.data_ptr(), stream)
                for i in range(5):
                    fn(i)
                ms = loop_time_ms(fn, iters, torch)
                row[f] = {"us": round(ms * 1e3, 2), "tflops": round(gemm_flops(M, N, Kp) / ms / 1e9, 1),
                          "frac_of_mfma_peak": round(gemm_flops(M, N, Kp) / ms / 1e9 / MFMA_PEAK_TFLOPS[f], 4)}
                if M <= 64:
                    wbytes = ws[0][0].numel() + ws[0][1].numel()
                    row[f]["weight_stream_GB/s"] = round(wbytes / ms / 1e6, 1)
                    row[f]["frac_hbm"] = round(wbytes / ms / 1e6 / HBM_PEAK_GBS, 4)
            xa = torch.randn(M, Kp, device="cuda", dtype=torch.bfloat16)
            fn = lambda i: torch.matmul(xa, wbs[i % nb].t(), out=c)
            for i in range(5):
                fn(i)
            ms = loop_time_ms(fn, iters, torch)
            row["bf16_torch"] = {"us": round(ms * 1e3, 2), "tflops": round(gemm_flops(M, N, Kp) / ms / 1e9, 1),
                                 "frac_of_mfma_peak": round(gemm_flops(M, N, Kp) / ms / 1e9 / MFMA_PEAK_TFLOPS["bf16"], 4)}
            for f in fmts:
                row[f]["vs_bf16"] = round(row["bf16_torch"]["us"] / row[f]["us"], 2)
            rows.append(row)
            print("[bench] gemm", json.dumps(row), file=sys.stderr, flush=True)
        del wq, wbs
        torch.cuda.empty_cache()
    return rows


def layer_rows(torch, iters=10):
    """Benchmark configurations 4 and 5 through arcquant_amd.layers, next to the same layer in bf16
    (torch: hipBLASLt GEMMs, the same SDPA).  One decoder layer of Llama-3-8B geometry (hidden 4096,
    32 query / 8 KV heads of 128, SwiGLU 14336, fused qkv and gate_up), prefill 8 x 2048 tokens and a
    decode step of batch 64 over a 2048-token KV cache; one Mixtral MoE block (8 experts, top-2,
    4096 tokens, expert popularity Zipf(1.1)).  Reorder indices are the ascending order of the per-channel
    maxima of each linear's input, taken from one bf16 pass over the same activations."""
    import torch.nn.functional as F
    import recipes
    from arcquant_amd import layers
    rows = []
    hidden, inter, nh, nkv, eps = 4096, 14336, 32, 8, 1e-5
    d = hidden // nh
    g = torch.Generator().manual_seed(4)

    def hidden_states(b, s):
        x = torch.randn(b, s, hidden, generator=g)
        ch = torch.randperm(hidden, generator=g)[:41]
        x[..., ch] *= 40.0
        return x.to(torch.bfloat16).cuda()

    def timed(fn):
        for _ in range(3):
            fn()
        return loop_time_ms(lambda i: fn(), iters, torch)

    def rms(x, w):
        h = x.float()
        h = h * torch.rsqrt(h.pow(2).mean(-1, keepdim=True) + eps)
        return w * h.to(x.dtype)

    def channel_order(t):
        return torch.argsort(t.reshape(-1, t.shape[-1]).float().abs().amax(0), stable=True).to(torch.int16)

    def bf16_layer(W, g1, g2, x, kv=None, past=0, taps=None):
        b, s, _ = x.shape
        n1 = rms(x, g1)
        qkv = F.linear(n1, W["qkv"])
        q = qkv[..., :nh * d].view(b, s, nh, d).transpose(1, 2)
        k = qkv[..., nh * d:(nh + nkv) * d].view(b, s, nkv, d).transpose(1, 2)
        v = qkv[..., (nh + nkv) * d:].view(b, s, nkv, d).transpose(1, 2)
        q, k = layers.rotary_pos_emb(q, k, past)
        if kv is not None:
            kv[0][:, :, past:past + s] = k
            kv[1][:, :, past:past + s] = v
            k, v = kv[0][:, :, :past + s], kv[1][:, :, :past + s]
        o = F.scaled_dot_product_attention(q, k, v, is_causal=(s > 1 and past == 0), enable_gqa=True)
        o = o.transpose(1, 2).reshape(b, s, hidden)
        h = x + F.linear(o, W["o"])
        n2 = rms(h, g2)
        gu = F.linear(n2, W["gate_up"])
        t = F.silu(gu[..., :inter]) * gu[..., inter:]
        if taps is not None:
            taps.update(attn_in=channel_order(n1), o_in=channel_order(o), mlp_in=channel_order(n2), down_in=channel_order(t))
        return h + F.linear(t, W["down"])

    for fmt in ("MXFP4", "NVFP4"):
        # the layer is built twice: once with identity orders to get at its weights, which one bf16 pass turns
        # into the channel orders (the calibration the reference runs offline), then with those orders
        x = hidden_states(8, 2048)
        probe = layers.LlamaDecoderLayer(hidden, inter, nh, nkv, eps=eps, select_num=256, select_num_down=256,
                                         quant_type=fmt, seed=4)
        W = {k: v.weight.data for k, v in probe.linears.items()}
        g1, g2 = probe.input_layernorm.weight, probe.post_attention_layernorm.weight
        taps = {}
        bf16_layer(W, g1, g2, x[:2], taps=taps)
        del probe
        layer = layers.LlamaDecoderLayer(hidden, inter, nh, nkv, eps=eps, select_num=256, select_num_down=256,
                                         quant_type=fmt, seed=4, indices={k: v.cuda() for k, v in taps.items()})
        W = {k: v.weight.data for k, v in layer.linears.items()}
        g1, g2 = layer.input_layernorm.weight, layer.post_attention_layernorm.weight

        ms_arc = timed(lambda: layer(x))
        ms_bf = timed(lambda: bf16_layer(W, g1, g2, x))
        rows.append({"config": "decoder layer prefill 8x2048", "fmt": fmt, "arc_ms": round(ms_arc, 3),
                     "bf16_ms": round(ms_bf, 3), "speedup": round(ms_bf / ms_arc, 2),
                     "tokens_per_s": round(8 * 2048 / ms_arc * 1e3)})
        print("[bench] layer", json.dumps(rows[-1]), file=sys.stderr, flush=True)
        del x
        kvlen = 2048
        kv = (torch.randn(64, nkv, kvlen + 8, d, device="cuda", dtype=torch.bfloat16),
              torch.randn(64, nkv, kvlen + 8, d, device="cuda", dtype=torch.bfloat16))
        x = hidden_states(64, 1)
        ms_arc = timed(lambda: layer(x, kv, kvlen))
        ms_bf = timed(lambda: bf16_layer(W, g1, g2, x, kv, kvlen))
        # the bf16 step as a HIP graph too, so that a graphed ARC step below is compared like with like
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for _ in range(3):
                bf16_layer(W, g1, g2, x, kv, kvlen)
        torch.cuda.current_stream().wait_stream(side)
        bf_graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(bf_graph, stream=side):
            bf16_layer(W, g1, g2, x, kv, kvlen)
        ms_bf_graph = timed(bf_graph.replay)
        rows.append({"config": f"decoder layer decode batch 64, KV length {kvlen}, bf16 KV cache + SDPA, eager", "fmt": fmt,
                     "arc_ms": round(ms_arc, 3), "bf16_ms": round(ms_bf, 3), "speedup": round(ms_bf / ms_arc, 2),
                     "tokens_per_s": round(64 / ms_arc * 1e3)})
        print("[bench] layer", json.dumps(rows[-1]), file=sys.stderr, flush=True)
        # the same decode step over an INT4 paged KV cache (decode attention on the quantized pages)
        from arcquant_amd.kv_cache import MultiLayerPagedKVCache4Bit
        cache = MultiLayerPagedKVCache4Bit(64, 16, kvlen + 64, "cuda", 1, nkv, d, dtype=torch.bfloat16)
        cache.update(kv[0][:, :, :kvlen].transpose(1, 2).contiguous(), kv[1][:, :, :kvlen].transpose(1, 2).contiguous(), 0)

        def paged_step():
            cache.lengths = [kvlen] * 64          # keep the length fixed across timed repetitions
            cache._specs["last_page_offset"].fill_(kvlen % 16 or 16)
            return layer(x, cache, kvlen)
        ms_i4 = timed(paged_step)
        rows.append({"config": f"decoder layer decode batch 64, KV length {kvlen}, INT4 paged KV cache, eager", "fmt": fmt,
                     "arc_ms": round(ms_i4, 3), "bf16_ms": round(ms_bf, 3), "speedup": round(ms_bf / ms_i4, 2),
                     "tokens_per_s": round(64 / ms_i4 * 1e3)})
        print("[bench] layer", json.dumps(rows[-1]), file=sys.stderr, flush=True)
        # ... and the whole step replayed from a captured HIP graph (the KV length grows by one per
        # replay, as in generation: 2048 -> ~2060 over the timed repetitions), against the graphed bf16 step
        cache2 = MultiLayerPagedKVCache4Bit(64, 16, kvlen + 256, "cuda", 1, nkv, d, dtype=torch.bfloat16)
        cache2.update(kv[0][:, :, :kvlen].transpose(1, 2).contiguous(), kv[1][:, :, :kvlen].transpose(1, 2).contiguous(), 0)
        step = layers.GraphedDecodeStep(layer, cache2, 64, hidden)
        step.x.copy_(x)                       # the layer's input sits in the graph's input buffer, as the
        ms_g = timed(lambda: step(step.x))    # previous layer's output would; the bf16 layer reads x in place too
        rows.append({"config": f"decoder layer decode batch 64, KV length {kvlen}+, both steps as HIP graphs "
                               f"(ARC: INT4 paged KV cache; bf16: bf16 KV cache + SDPA)",
                     "fmt": fmt, "arc_ms": round(ms_g, 3), "bf16_ms": round(ms_bf_graph, 3),
                     "speedup": round(ms_bf_graph / ms_g, 2), "tokens_per_s": round(64 / ms_g * 1e3)})
        print("[bench] layer", json.dumps(rows[-1]), file=sys.stderr, flush=True)
        del layer, W, kv, x, cache, cache2, step, bf_graph
        torch.cuda.empty_cache()

    # Mixtral block (benchmark configuration 5: NVFP4; MXFP4 beside it), select_num 128, per-expert channel
    # orders from the per-expert channel maxima of the routed tokens
    E, ffn, tokens = 8, 14336, 4096
    g = torch.Generator().manual_seed(5)
    xcpu = recipes.activations(tokens, hidden, seed=5, outlier_frac=0.01, outlier_gain=40.0)
    x = xcpu.cuda().view(1, tokens, hidden)
    bias = torch.log(1.0 / torch.arange(1, E + 1).float() ** 1.1)
    logits_cpu = torch.randn(tokens, E, generator=g) + bias
    logits = logits_cpu.cuda()
    sel = torch.topk(F.softmax(logits_cpu, dim=1), 2, dim=-1)[1]
    indices = []
    for e in range(E):
        mine = xcpu[(sel == e).any(1)]
        indices.append((recipes.reorder_index(mine if mine.numel() else xcpu).cuda(),
                        torch.randperm(ffn, generator=g).to(torch.int16).cuda()))
    moe_ms = {}
    for fmt in ("NVFP4", "MXFP4"):
        block = layers.build_mixtral_block(hidden, ffn, E, 2, 128, fmt, indices=indices, seed=5)
        grouped = timed(lambda: block(x, router_logits=logits))
        block.grouped = False
        moe_ms[fmt] = (grouped, timed(lambda: block(x, router_logits=logits)))
        del block
        torch.cuda.empty_cache()
    # the same block in bf16 on dequantised-size weights (random: only the time matters)
    w13 = [torch.randn(2 * ffn, hidden, device="cuda", dtype=torch.bfloat16) * 0.02 for _ in range(E)]
    w2 = [torch.randn(hidden, ffn, device="cuda", dtype=torch.bfloat16) * 0.02 for _ in range(E)]

    def bf16_moe():
        xf = x.view(tokens, hidden)
        w = F.softmax(logits, dim=1, dtype=torch.float)
        w, sel = torch.topk(w, 2, dim=-1)
        w = (w / w.sum(dim=-1, keepdim=True)).to(xf.dtype)
        flat = sel.reshape(-1)
        order = torch.argsort(flat, stable=True)
        tok = order // 2
        counts = torch.bincount(flat, minlength=E).tolist()
        xs, ws = xf.index_select(0, tok), w.reshape(-1).index_select(0, order)
        out = torch.zeros_like(xf)
        beg = 0
        for e, n in enumerate(counts):
            if n:
                h = F.linear(xs[beg:beg + n], w13[e])
                y = F.linear(F.silu(h[:, :ffn]) * h[:, ffn:], w2[e]) * ws[beg:beg + n, None]
                out.index_add_(0, tok[beg:beg + n], y)
                beg += n
        return out

    ms_bf = timed(bf16_moe)
    counts = torch.bincount(sel.reshape(-1), minlength=E).tolist()
    for fmt, (ms_arc, ms_loop) in moe_ms.items():
        rows.append({"config": "Mixtral MoE block, 4096 tokens, 8 experts top-2, grouped launches", "fmt": fmt,
                     "arc_ms": round(ms_arc, 3), "arc_per_expert_loop_ms": round(ms_loop, 3),
                     "bf16_ms": round(ms_bf, 3), "speedup": round(ms_bf / ms_arc, 2), "tokens_per_expert": counts,
                     "tokens_per_s": round(tokens / ms_arc * 1e3)})
        print("[bench] layer", json.dumps(rows[-1]), file=sys.stderr, flush=True)
    return rows


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--quick", action="store_true", help="no layer rows, two GEMM shapes")
    ap.add_argument("--headline-only", action="store_true",
                    help="the headline kernel and the copy kernels only (what a counter run should see)")
    ap.add_argument("--gemm-table", action="store_true", help="(kept for older command lines: the full table is the default)")
    ap.add_argument("--layers", action="store_true", help="(kept for older command lines: the layer rows are the default)")
    ap.add_argument("--no-gemm", action="store_true")
    ap.add_argument("--no-quantize-table", action="store_true")
    ap.add_argument("--gemm-shapes", default="", help="NxK[,NxK...]: restrict the GEMM rows to these shapes (counter runs)")
    ap.add_argument("--gemm-ms", default="", help="M[,M...]: restrict the GEMM rows to these M")
    ap.add_argument("--no-layers", action="store_true")
    ap.add_argument("--no-cpu", action="store_true", help="skip the host-CPU baseline leg")
    ap.add_argument("--mfma-probe", action="store_true", help="only the register-only matrix-pipe rates (one JSON line of its own)")
    ap.add_argument("--cpu-rows", type=int, default=M_TOKENS)
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on ONE GPU; every GPU box of this run has one and nothing here shards "
              "across devices (rows of every quantizer and GEMM are independent: shard M, no exchange). "
              "Use --gpus 1.", file=sys.stderr)
        sys.exit(2)

    import ctypes

    import torch
    import recipes
    from arcquant_amd import _lib, agemm

    assert torch.cuda.is_available(), "bench.py needs the MI355X"
    torch.cuda.set_device(0)
    if args.mfma_probe:
        print(json.dumps({"mfma_sustained": mfma_sustained(torch)}), flush=True)
        return
    L = _lib.lib()
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)   # launches and events share this stream

    # ---------------- workload: distinct input buffers beyond the Infinity Cache ----------------
    bytes_per_launch = quant_bytes(M_TOKENS, H, SELECT, FMT, True)
    nbuf = max(2, int(1.2e9 // bytes_per_launch))          # ~1.2 GB of rotating traffic
    base = recipes.activations(M_TOKENS, H, seed=2, outlier_frac=0.005, outlier_gain=50.0)
    gam = recipes.gamma(H, seed=7).cuda()
    idx = recipes.reorder_index(base).cuda()               # ascending per-channel maxima, as the reference calibrates
    xs = [base.cuda() if i == 0 else (base.cuda().roll(i, 0)) for i in range(nbuf)]
    fid = {"NVFP4": 0, "MXFP4": 1}

    def outputs(fmt, S, rows=M_TOKENS):
        return (torch.empty(L.arcq_codes_bytes(rows, H, S), dtype=torch.uint8, device="cuda"),
                torch.empty(L.arcq_scales_bytes(rows, H, S, fid[fmt]), dtype=torch.uint8, device="cuda"))

    outs = [outputs(FMT, SELECT) for _ in range(nbuf)]
    torch.cuda.synchronize()

    # one step = one call of the C-ABI entry point on buffers that already exist (the Python op
    # surface adds two torch.empty per call, more host time than the kernel itself)
    def step(i):
        q, sf = outs[i % nbuf]
        rc = L.arcq_rmsnorm_quantize_x(xs[i % nbuf].data_ptr(), gam.data_ptr(), EPS, M_TOKENS, H, idx.data_ptr(), SELECT,
                                       fid[FMT], 1.0, None, q.data_ptr(), sf.data_ptr(), stream)
        assert rc == 0, rc

    for i in range(args.warmup):
        step(i)
    torch.cuda.synchronize()
    ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    ev0.record()
    for i in range(args.steps):
        step(i)
    ev1.record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    ms_per_step = wall / args.steps * 1e3
    value = bytes_per_launch / (ms_per_step * 1e-3) / 1e9

    # ---------------- roofline of the dominant kernel: HIP events over the same timed region ----------------
    kern_ms = ev0.elapsed_time(ev1) / args.steps           # launches are queued back to back: GPU time per launch
    achieved = bytes_per_launch / (kern_ms * 1e-3) / 1e9
    # the box's own streaming ceiling for this read:write mix: plain copy kernels moving the same bytes, in every
    # launch shape the library has (loads in flight per thread, non-temporal, resident / one-round grids, LDS-direct)
    b_in = M_TOKENS * H * 2
    b_out = ((bytes_per_launch - b_in) // 16) * 16
    sdst = [torch.empty(b_out, dtype=torch.uint8, device="cuda") for _ in range(nbuf)]
    probes = {}
    P = _lib.probe_lib()                                   # measurement-only library of plain copy kernels
    for variant in range(P.arcq_stream_probe_variants()):
        def probe(i, variant=variant):
            P.arcq_stream_probe_variant(xs[i % nbuf].data_ptr(), sdst[i % nbuf].data_ptr(), b_in, b_out, variant, stream)
        for i in range(10):
            probe(i)
        probes[variant] = loop_time_ms(probe, 100, torch)
    best_variant = min(probes, key=probes.get)
    probe_ms = probes[best_variant]
    ceiling = (b_in + b_out) / probe_ms / 1e6
    workload_key = f"fused-norm {FMT} M={M_TOKENS} K={H} S={SELECT}"
    traffic, traffic_kernel, traffic_source = measured_traffic(workload_key)
    roofline = {"bound": "hbm", "kernel": "quantize_rows_wave_kernel<NVFP4, RMSNORM, K/1024 = 4>", "achieved": round(achieved, 1),
                "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBS, 4), "traffic": traffic,
                "traffic_source": traffic_source, "traffic_kernel": traffic_kernel,
                "bytes_per_launch": bytes_per_launch, "avg_launch_us": round(kern_ms * 1e3, 2),
                "streaming_copy_same_bytes": {"us": round(probe_ms * 1e3, 2), "GB/s": round(ceiling, 1),
                                              "frac_of_peak": round(ceiling / HBM_PEAK_GBS, 4), "variant": best_variant,
                                              "all_variants_us": {str(k): round(v * 1e3, 2) for k, v in probes.items()}},
                "frac_of_streaming_copy": round(probe_ms / kern_ms, 4),
                "note": "algorithmic bytes / (HIP-event time over the timed region / launches); "
                        "streaming_copy_same_bytes is the fastest of the library's plain copy kernels moving the same "
                        "bytes on this box (a 44 MB launch cannot reach the peak: the copy shows what one can); "
                        "traffic = HBM bytes per launch from rocprofv3 FETCH_SIZE + WRITE_SIZE (traffic_source)"}

    out = {
        "metric": "ARC FP4 GEMM TFLOPS + quantize GB/s at Llama-3-8B shapes, M=1..4096",
        "value": round(value, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 5), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": f"fused RMSNorm+reorder+quantize, {FMT}, M={M_TOKENS}, hidden={H}, "
                               f"select_num={SELECT}, eps={EPS}, global_scale=1 (benchmark config 2); one step = one "
                               f"C-ABI call; value = algorithmic bytes / wall time; inputs rotate over {nbuf} "
                               f"buffers ({nbuf * bytes_per_launch / 1e9:.2f} GB) to defeat the 256 MB Infinity Cache"},
        "roofline": roofline,
    }
    if args.headline_only:
        print(json.dumps(out), flush=True)
        return

    # ---------------- benchmark configuration 2 in full, and the plain quantizers (reported, not the headline) ----------------
    def time_quant(fn, rows, reps):
        for i in range(5):
            fn(i)
        return loop_time_ms(fn, reps, torch)

    quant = []
    # the NVFP4 tensor scale the reference's callers compute: max|x| / (448 * 6) (model/qLlamaLayer.py:74)
    gs_dev = (xs[0].abs().max().float() / 2688.0).reshape(())
    for fmt in (() if args.no_quantize_table else ("NVFP4", "MXFP4")):
        for S in (64, 256):
            for rows in (1, 16, 256, 4096):
                q, sf = outputs(fmt, S, rows)
                fn = lambda i, fmt=fmt, S=S, q=q, sf=sf, rows=rows: L.arcq_rmsnorm_quantize_x(
                    xs[i % nbuf].data_ptr(), gam.data_ptr(), EPS, rows, H, idx.data_ptr(), S, fid[fmt], 1.0, None,
                    q.data_ptr(), sf.data_ptr(), stream)
                ms = time_quant(fn, rows, 100)
                b = quant_bytes(rows, H, S, fmt, True)
                quant.append({"op": "rmsnorm_quantize_x", "fmt": fmt, "select_num": S, "M": rows, "us": round(ms * 1e3, 2),
                              "GB/s": round(b / ms / 1e6, 1), "frac_hbm": round(b / ms / 1e6 / HBM_PEAK_GBS, 4)})
    for fmt, S, kind in (() if args.no_quantize_table else
                         (("NVFP4", 256, "x_unit"), ("MXFP4", 256, "x_unit"), ("NVFP4", 256, "x_scaled"))):
        q, sf = outputs(fmt, S)
        dgs = ctypes.c_void_p(gs_dev.data_ptr()) if kind == "x_scaled" else None
        fn = lambda i, fmt=fmt, S=S, q=q, sf=sf, dgs=dgs: L.arcq_reorder_quantize_x(
            xs[i % nbuf].data_ptr(), M_TOKENS, H, idx.data_ptr(), S, fid[fmt], 1.0, dgs, q.data_ptr(), sf.data_ptr(),
            stream)
        ms = time_quant(fn, M_TOKENS, 100)
        b = quant_bytes(M_TOKENS, H, S, fmt, False)
        name = {"x_unit": "reorder_quantize_x (tensor scale 1)", "x_scaled": "reorder_quantize_x (tensor scale max|x|/2688 on the device)"}[kind]
        quant.append({"op": name, "fmt": fmt, "select_num": S, "M": M_TOKENS, "us": round(ms * 1e3, 2),
                      "GB/s": round(b / ms / 1e6, 1), "frac_hbm": round(b / ms / 1e6 / HBM_PEAK_GBS, 4)})
    if not args.no_quantize_table:
        # what an NVFP4 linear's input costs in full (model/qLlamaLayer.py:73-77: the tensor scale, then the
        # quantizer): arcq_tensor_scale + arcq_reorder_quantize_x with the scale read on the device, as one row
        q, sf = outputs("NVFP4", SELECT)
        sc = torch.empty((), dtype=torch.float32, device="cuda")

        def scale_then_quantize(i):
            L.arcq_tensor_scale(xs[i % nbuf].data_ptr(), None, H, M_TOKENS, H, 2688.0, sc.data_ptr(), stream)
            L.arcq_reorder_quantize_x(xs[i % nbuf].data_ptr(), M_TOKENS, H, idx.data_ptr(), SELECT, fid["NVFP4"], 1.0,
                                      ctypes.c_void_p(sc.data_ptr()), q.data_ptr(), sf.data_ptr(), stream)
        ms_both = time_quant(scale_then_quantize, M_TOKENS, 100)
        ms_scale = time_quant(lambda i: L.arcq_tensor_scale(xs[i % nbuf].data_ptr(), None, H, M_TOKENS, H, 2688.0,
                                                            sc.data_ptr(), stream), M_TOKENS, 100)
        b = quant_bytes(M_TOKENS, H, SELECT, "NVFP4", False) + 2 * M_TOKENS * H      # the tensor is read twice
        quant.append({"op": "tensor_scale + reorder_quantize_x (two launches)", "fmt": "NVFP4", "select_num": SELECT, "M": M_TOKENS,
                      "us": round(ms_both * 1e3, 2), "tensor_scale_us": round(ms_scale * 1e3, 2),
                      "GB/s": round(b / ms_both / 1e6, 1), "frac_hbm": round(b / ms_both / 1e6 / HBM_PEAK_GBS, 4)})
        # the same as ONE launch (arcq_reorder_quantize_x_absmax: rows stay in LDS while the workgroups exchange maxima)
        ms_one = time_quant(lambda i: L.arcq_reorder_quantize_x_absmax(
            xs[i % nbuf].data_ptr(), M_TOKENS, H, idx.data_ptr(), SELECT, fid["NVFP4"], 2688.0, sc.data_ptr(), q.data_ptr(),
            sf.data_ptr(), stream), M_TOKENS, 100)
        b1 = quant_bytes(M_TOKENS, H, SELECT, "NVFP4", False)
        quant.append({"op": "tensor scale and reorder_quantize_x in one launch", "fmt": "NVFP4", "select_num": SELECT, "M": M_TOKENS,
                      "us": round(ms_one * 1e3, 2), "GB/s": round(b1 / ms_one / 1e6, 1),
                      "frac_hbm": round(b1 / ms_one / 1e6 / HBM_PEAK_GBS, 4)})
        # the fused norm at the prefill size of benchmark configuration 4 (16384 rows, rotating inputs): the rate
        # without the ramp of a 13 us launch
        M4 = 16384
        x4 = [torch.cat([xs[(4 * j + k) % nbuf] for k in range(4)]) for j in range(max(2, nbuf // 4))]
        for fmt in ("NVFP4", "MXFP4"):
            q4, sf4 = outputs(fmt, SELECT, M4)
            fn = lambda i, fmt=fmt, q4=q4, sf4=sf4: L.arcq_rmsnorm_quantize_x(
                x4[i % len(x4)].data_ptr(), gam.data_ptr(), EPS, M4, H, idx.data_ptr(), SELECT, fid[fmt], 1.0, None,
                q4.data_ptr(), sf4.data_ptr(), stream)
            ms = time_quant(fn, M4, 50)
            b = quant_bytes(M4, H, SELECT, fmt, True)
            quant.append({"op": "rmsnorm_quantize_x", "fmt": fmt, "select_num": SELECT, "M": M4, "us": round(ms * 1e3, 2),
                          "GB/s": round(b / ms / 1e6, 1), "frac_hbm": round(b / ms / 1e6 / HBM_PEAK_GBS, 4)})
        del x4
        torch.cuda.empty_cache()
    # long rows: the down projection's input at Llama-3-8B width (14336) and at the reference's widest dedicated
    # shape (28672, kernels/src/down.cu:71-233), 4096 rows each, tensor scale 1; rate per byte side by side
    if not args.no_quantize_table:
        for K in (14336, 28672):
            nb = max(2, int(7e8 // (M_TOKENS * K * 2)))
            xw = [recipes.activations(M_TOKENS, K, seed=20 + i).cuda() for i in range(2)]
            xw += [xw[i % 2].roll(i, 0) for i in range(2, nb)]
            iw = recipes.reorder_index(xw[0].cpu()).cuda()
            for fmt in ("NVFP4", "MXFP4"):
                q = torch.empty(L.arcq_codes_bytes(M_TOKENS, K, SELECT), dtype=torch.uint8, device="cuda")
                sf = torch.empty(L.arcq_scales_bytes(M_TOKENS, K, SELECT, fid[fmt]), dtype=torch.uint8, device="cuda")
                fn = lambda i, fmt=fmt, q=q, sf=sf, K=K: L.arcq_reorder_quantize_x(
                    xw[i % nb].data_ptr(), M_TOKENS, K, iw.data_ptr(), SELECT, fid[fmt], 1.0, None, q.data_ptr(), sf.data_ptr(), stream)
                ms = time_quant(fn, M_TOKENS, 50)
                b = quant_bytes(M_TOKENS, K, SELECT, fmt, False)
                quant.append({"op": "reorder_quantize_x (tensor scale 1)", "fmt": fmt, "select_num": SELECT, "M": M_TOKENS, "K": K,
                              "us": round(ms * 1e3, 2), "GB/s": round(b / ms / 1e6, 1), "frac_hbm": round(b / ms / 1e6 / HBM_PEAK_GBS, 4)})
            del xw
            torch.cuda.empty_cache()
    out["quantize"] = quant
    del xs[1:], outs[1:], sdst[1:]
    torch.cuda.empty_cache()

    if not args.no_gemm:
        shapes = [(6144, 4096), (28672, 4096)] if args.quick else [(6144, 4096), (4096, 4096), (28672, 4096), (4096, 14336)]
        Ms = [1, 16, 128, 512, 2048, 4096]                  # benchmark configuration 3
        if args.gemm_shapes:
            shapes = [tuple(int(v) for v in t.split("x")) for t in args.gemm_shapes.split(",")]
        if args.gemm_ms:
            Ms = [int(v) for v in args.gemm_ms.split(",")]
        out["gemm"] = gemm_rows(torch, agemm, shapes, Ms, ["MXFP4", "NVFP4"])
        out["gemm_peaks_tflops"] = MFMA_PEAK_TFLOPS
    if not (args.quick or args.no_layers):
        out["layers"] = layer_rows(torch)
    if not args.quick:
        out["mfma_sustained"] = mfma_sustained(torch)
        # MoE routing (arcq_moe_route: two launches, three beyond 16384 tokens) by token count, 8 experts, top-2
        route = []
        for T in (4096, 16384, 32768, 65536):
            lg = torch.randn(T, 8, device="cuda").to(torch.bfloat16)
            for _ in range(3):
                agemm.moe_route(lg, 2)
            ms = loop_time_ms(lambda i: agemm.moe_route(lg, 2), 20, torch)
            route.append({"tokens": T, "us": round(ms * 1e3, 1)})
        out["moe_route"] = route

    if not args.no_cpu:
        out["cpu_baseline"] = cpu_baseline(torch, args.cpu_rows)

    print(json.dumps(out), flush=True)


if __name__ == "__main__":
    main()
