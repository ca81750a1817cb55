"""GPU parity of the three quantizers against the CPU oracle: packed codes and scale bytes must be
bit-identical.  Calls go through the Python op surface, i.e. through the C ABI of libarcq_hip.so."""
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


def dev(t):
    return t.cuda()


def compare(tag, got_codes, got_scales, want):
    gc = got_codes.cpu().numpy()
    gs = got_scales.cpu().numpy().reshape(want["scales"].shape)
    bad_c = int((gc != want["codes"]).sum())
    bad_s = int((gs != want["scales"]).sum())
    assert gc.shape == want["codes"].shape
    assert bad_s == 0, f"{tag}: {bad_s} of {gs.size} scale bytes differ; first at {np.argwhere(gs != want['scales'])[:3]}"
    assert bad_c == 0, f"{tag}: {bad_c} of {gc.size} code bytes differ; first at {np.argwhere(gc != want['codes'])[:3]}"


@pytest.mark.parametrize("fmt", FMTS)
@pytest.mark.parametrize("M,K,S", [(1, 4096, 64), (16, 4096, 256), (33, 4096, 0), (256, 4096, 128), (7, 64, 64),
                                   (5, 14336, 256), (3, 28672, 512), (130, 2048, 2048), (4, 3584, 128)])
def test_reorder_quantize_x(agemm, oracle, fmt, M, K, S):
    x = recipes.activations(M, K, seed=1000 + M + K + S)
    idx = recipes.reorder_index(x)
    gs = recipes.tensor_scale(x, fmt)
    want = oracle.quantize_x(x, idx, S, fmt, gs)
    print(f"reorder_quantize_x {fmt} M={M} K={K} S={S} gscale={gs}", flush=True)
    q, sf = agemm.reorder_quantize_x(dev(x), dev(idx), S, fmt=fmt, global_scale=gs)
    compare("host scale", q, sf, want)
    # same thing with the tensor scale read on the device
    q, sf = agemm.reorder_quantize_x(dev(x), dev(idx), S, fmt=fmt,
                                     global_scale=torch.tensor(gs, dtype=torch.float32).cuda())
    compare("device scale", q, sf, want)


@pytest.mark.parametrize("fmt", FMTS)
@pytest.mark.parametrize("N,K,S", [(64, 4096, 128), (9, 14336, 256), (257, 512, 64), (16, 4096, 0)])
def test_reorder_quantize_w(agemm, oracle, fmt, N, K, S):
    w = recipes.weights(N, K, seed=2000 + N + K + S)
    idx = recipes.reorder_index(recipes.activations(32, K, seed=5))
    gs = recipes.tensor_scale(w, fmt)
    want = oracle.quantize_w(w, idx, S, fmt, gs)
    print(f"reorder_quantize_w {fmt} N={N} K={K} S={S}", flush=True)
    q, sf = agemm.reorder_quantize_w(dev(w), dev(idx), S, fmt=fmt, global_scale=gs)
    compare("w", q, sf, want)


@pytest.mark.parametrize("fmt", FMTS)
@pytest.mark.parametrize("M,K,S", [(1, 4096, 64), (1, 4096, 256), (16, 4096, 64), (16, 4096, 256), (256, 4096, 64),
                                   (256, 4096, 256), (19, 8192, 256), (6, 2048, 0)])
def test_rmsnorm_quantize_x(agemm, oracle, fmt, M, K, S):
    x = recipes.activations(M, K, seed=3000 + M + K + S, outlier_frac=0.005, outlier_gain=50.0)
    if M > 2:
        x[2] = 0                                                     # a padding token
    gam = recipes.gamma(K, seed=7)
    eps = 1e-5
    normed = oracle.rmsnorm_quantize_x(x, gam, eps, None, 0, fmt, want_normed=True)["normed"]
    idx = recipes.reorder_index(torch.from_numpy(normed.astype(np.int16)).view(torch.bfloat16))
    want = oracle.rmsnorm_quantize_x(x, gam, eps, idx, S, fmt, 1.0)
    print(f"rmsnorm_quantize_x {fmt} M={M} K={K} S={S}", flush=True)
    q, sf = agemm.rmsnorm_quantize_x(dev(x), dev(gam), eps, dev(idx), S, fmt=fmt)
    compare("rmsnorm", q, sf, want)


@pytest.mark.parametrize("fmt", FMTS)
def test_rmsnorm_quantize_x_benchmark_size(agemm, oracle, fmt):
    """The benchmark's launch (4096 x 4096, select_num 256) against the oracle, every row, and the same
    bits from every one of a series of back-to-back launches."""
    M, K, S = 4096, 4096, 256
    x = recipes.activations(M, K, seed=515, outlier_frac=0.005, outlier_gain=50.0)
    gam = recipes.gamma(K, seed=8)
    idx = recipes.reorder_index(x)
    want = oracle.rmsnorm_quantize_x(x, gam, 1e-5, idx, S, fmt, 1.0)
    print(f"rmsnorm_quantize_x {fmt} M={M} K={K} S={S}", flush=True)
    xd, gd, idxd = dev(x), dev(gam), dev(idx)
    q, sf = agemm.rmsnorm_quantize_x(xd, gd, 1e-5, idxd, S, fmt=fmt)
    compare("rmsnorm 4096x4096", q, sf, want)
    outs = [agemm.rmsnorm_quantize_x(xd, gd, 1e-5, idxd, S, fmt=fmt) for _ in range(12)]
    for q2, sf2 in outs:
        assert torch.equal(q2, q) and torch.equal(sf2, sf)


@pytest.mark.parametrize("fmt", FMTS)
def test_edge_values(agemm, oracle, fmt):
    """zeros, ties, tiny and huge blocks, negative-only blocks, bf16 subnormals."""
    M, K = 8, 256
    g = torch.Generator().manual_seed(9)
    x = torch.randn(M, K, generator=g)
    x[0] = 0.0
    x[1, :64] = torch.tensor([0.25, -0.25, 0.75, -0.75, 1.25, -1.25, 1.75, -1.75, 2.5, -2.5, 3.5, -3.5, 5, -5, 6,
                              -6] * 4)                               # exact ties under scale 1
    x[2] *= 1e-4
    x[3] *= 1e4
    x[4] = -x[4].abs()
    x[5, ::2] = 0
    x[6] = torch.ldexp(torch.ones(K), torch.randint(-30, 8, (K,), generator=g).float())   # powers of two
    x[7, :32] = 1e-39                                                                       # bf16 subnormal range
    x = x.to(torch.bfloat16)
    idx = torch.arange(K).to(torch.int16)
    for S in (0, 64):
        for gs in ((1.0, 0.0371) if fmt == "NVFP4" else (1.0,)):
            want = oracle.quantize_x(x, idx, S, fmt, gs)
            q, sf = agemm.reorder_quantize_x(dev(x), dev(idx), S, fmt=fmt, global_scale=gs)
            compare(f"edge S={S} gs={gs}", q, sf, want)


@pytest.mark.parametrize("fmt", FMTS)
@pytest.mark.parametrize("gs", [0.5, -0.0371, 3e-25, 7e22, 1.0000001, 2688.0])
def test_unusual_tensor_scales(agemm, oracle, fmt, gs):
    """tensor scales that are powers of two (every tie of the grid is hit exactly), negative (the
    reference takes a signed max, model/quantize.py:318), or far outside the usual range (quotients
    that underflow or overflow), for both formats, activations and weights"""
    if fmt == "NVFP4" and gs == 3e-25:
        # NVFP4 block scales stop at 448, so x/gs/448 ~ 1e22 here, where the reference's 15-way argmin
        # (model/quantize.py:14-22) sees 15 equal distances and returns -6 for either sign: outside
        # the domain |x/s| <= 2^24 on which nearest-value rounding is defined
        pytest.skip("quotients beyond 2^24 are outside the reference's own domain")
    M, K, S = 24, 512, 128
    x = recipes.activations(M, K, seed=4242)
    x[1, :64] = torch.tensor([0.25, -0.25, 0.75, -0.75, 1.25, -1.25, 1.75, -1.75, 2.5, -2.5, 3.5, -3.5, 5, -5, 6,
                              -6] * 4).to(torch.bfloat16) * 0.5
    x[2] = 0
    x[3, 5] = 1e-39
    idx = recipes.reorder_index(x)
    print(f"unusual scale {fmt} gs={gs}", flush=True)
    want = oracle.quantize_x(x, idx, S, fmt, gs)
    q, sf = agemm.reorder_quantize_x(dev(x), dev(idx), S, fmt=fmt, global_scale=gs)
    compare(f"x gs={gs}", q, sf, want)
    want = oracle.quantize_w(x, idx, S, fmt, gs)
    q, sf = agemm.reorder_quantize_w(dev(x), dev(idx), S, fmt=fmt,
                                     global_scale=torch.tensor(gs, dtype=torch.float32).cuda())
    compare(f"w gs={gs}", q, sf, want)


def test_large_shape_properties(agemm, oracle):
    """Benchmark-size input (4096 x 4096, S=256): full comparison for NVFP4 with a tensor scale and,
    for both formats, properties that need no oracle: the first K codes do not depend on S, and
    decode(main) + decode(tail) is closer to x than decode(main) on the selected channels."""
    M, K, S = 4096, 4096, 256
    x = recipes.activations(M, K, seed=1)
    idx = recipes.reorder_index(x)
    xd, idxd = dev(x), dev(idx)
    gs = recipes.nvfp4_tensor_scale(x)
    want = oracle.quantize_x(x, idx, S, "NVFP4", gs)
    q, sf = agemm.reorder_quantize_x(xd, idxd, S, fmt="NVFP4", global_scale=gs)
    compare("4096x4096 NVFP4", q, sf, want)
    for fmt in FMTS:
        g = gs if fmt == "NVFP4" else 1.0
        qs, sfs = agemm.reorder_quantize_x(xd, idxd, S, fmt=fmt, global_scale=g)
        q0, sf0 = agemm.reorder_quantize_x(xd, idxd, 0, fmt=fmt, global_scale=g)
        assert torch.equal(qs[:, :K // 2], q0)
        G = 16 if fmt == "NVFP4" else 32
        assert torch.equal(sfs.view(M, -1)[:, :K // G], sf0.view(M, -1))
        dq = agemm.dequantize(qs, sfs, fmt=fmt)
        xr = xd[:, idxd.long()].float() / g
        e_main = (xr[:, K - S:] - dq[:, K - S:K]).abs().mean()
        e_arc = (xr[:, K - S:] - dq[:, K - S:K] - dq[:, K:]).abs().mean()
        assert e_arc < 0.25 * e_main


@pytest.mark.parametrize("fmt", FMTS)
@pytest.mark.parametrize("M,K,S", [(3072, 4096, 256), (4096, 4096, 64), (3073, 4096, 0), (3500, 4096, 1536),
                                   (3100, 4096, 4096), (3100, 1024, 128), (3330, 2048, 2048), (3200, 3072, 192),
                                   (5000, 2048, 64), (9000, 1024, 64)])
def test_many_rows_unit_scale(agemm, oracle, fmt, M, K, S):
    """Three thousand rows and more of a hidden size up to 4096 with tensor scale 1: the fused norm takes
    the wave-per-row kernel there (a wave owns whole rows, one LDS slot per wave refilled in turn); ragged
    row counts, one to three rows per wave, residual blocks in one or in several of a lane's units
    (select_num up to K), K = 3072 (mean by division, not by scaling).  The plain quantizer of the same
    launches is compared as well."""
    x = recipes.activations(M, K, seed=5000 + M + K + S, outlier_frac=0.005, outlier_gain=50.0)
    x[M // 3] = 0
    idx = recipes.reorder_index(x)
    print(f"many rows {fmt} M={M} K={K} S={S}", flush=True)
    want = oracle.quantize_x(x, idx, S, fmt, 1.0)
    q, sf = agemm.reorder_quantize_x(dev(x), dev(idx), S, fmt=fmt)
    compare("plain", q, sf, want)
    gam = recipes.gamma(K, seed=8)
    want = oracle.rmsnorm_quantize_x(x, gam, 1e-5, idx, S, fmt, 1.0)
    q, sf = agemm.rmsnorm_quantize_x(dev(x), dev(gam), 1e-5, dev(idx), S, fmt=fmt)
    compare("fused norm", q, sf, want)


@pytest.mark.parametrize("M,K,S", [(12, 512, 64), (300, 4096, 256), (7, 14336, 128)])
def test_dequantize_matches_oracle(agemm, oracle, M, K, S):
    x = recipes.activations(M, K, seed=77 + M)
    idx = recipes.reorder_index(x)
    for fmt in FMTS:
        gs = recipes.tensor_scale(x, fmt)
        want = oracle.quantize_x(x, idx, S, fmt, gs, want_dq=True)
        q, sf = agemm.reorder_quantize_x(dev(x), dev(idx), S, fmt=fmt, global_scale=gs)
        assert np.array_equal(agemm.dequantize(q, sf, fmt=fmt).cpu().numpy(), want["dq"])


def test_errors(agemm):
    x = dev(recipes.activations(4, 4096, seed=1))
    idx = dev(torch.arange(4096).to(torch.int16))
    with pytest.raises(RuntimeError):
        agemm.reorder_quantize_x(x.float(), idx, 0)                 # dtype
    with pytest.raises(RuntimeError):
        agemm.reorder_quantize_x(x[:, :4000], idx[:4000], 0)        # non-contiguous / bad K
    with pytest.raises(RuntimeError):
        agemm.reorder_quantize_x(x, idx, 24)                        # select_num alignment
    with pytest.raises(RuntimeError):
        agemm.reorder_quantize_x(x, idx.int(), 0)                   # index dtype
    with pytest.raises(RuntimeError):
        agemm.reorder_quantize_x(x.cpu(), idx, 0)                   # device
    with pytest.raises(RuntimeError):
        agemm.reorder_quantize_x(x, idx, 0, fmt="INT4")
    bad = idx.clone()
    bad[3] = bad[4]
    with pytest.raises(RuntimeError):
        agemm.check_index(bad)
    agemm.check_index(idx)
    q, sf = agemm.reorder_quantize_x(x[:0], idx, 64)               # empty input
    assert q.shape == (0, (4096 + 64) // 2) and sf.numel() == 0


@pytest.mark.parametrize("M,K", [(1, 64), (5, 4096), (64, 14336), (2048, 4096), (300, 1000)])
def test_tensor_scale_matches_torch(agemm, M, K):
    """NVFP4 tensor scale in one launch (max|x| / 2688, model/qLlamaLayer.py:73-77) against torch's
    abs().max() and an IEEE division; repeated calls reuse the library's two-word workspace, which must
    come back clean; an all-zero tensor gets 1; strided rows are read in place."""
    g = torch.Generator().manual_seed(100 + M)
    x = (torch.randn(M, K + 8, generator=g) * 3).to(torch.bfloat16)
    x[M // 2, K // 3] = -777.0                                   # the maximum is a negative element
    x[:, K:] = 1e4                                               # outside the view: must not be read
    xd = x.cuda()
    view = xd[:, :K]
    want = view.abs().max().float() / torch.full((), 2688.0, device="cuda")
    print(f"tensor scale M={M} K={K}", flush=True)
    for _ in range(3):
        got = agemm.tensor_scale(view)
        assert got.dtype == torch.float32 and got.dim() == 0
        assert float(got) == float(want)
    assert float(agemm.tensor_scale(torch.zeros(M, K, dtype=torch.bfloat16, device="cuda"))) == 1.0
    assert float(agemm.tensor_scale(view.contiguous(), 6.0)) == float(view.abs().max().float() / torch.full((), 6.0, device="cuda"))


@pytest.mark.parametrize("seed", [3, 11])
def test_quantizers_random_shapes(agemm, oracle, seed):
    """Thirty random (operator, format, rows, K, select_num, tensor scale) problems per seed around the row
    counts and widths where the dispatch changes kernels: codes and scale bytes bit for bit against the oracle."""
    import random
    rnd = random.Random(seed)
    done = 0
    while done < 30:
        fmt = rnd.choice(FMTS)
        G = 16 if fmt == "NVFP4" else 32
        mode = rnd.choice(["x", "w", "norm", "norm", "x"])
        M = rnd.choice([1, 2, 3, 15, 16, 17, 64, 100, 255, 256, 257, 1000, 3071, 3072, 3073, 4096, 5000])
        K = rnd.choice([32, 64, 96, 128, 512, 1024, 2048, 3072, 3584, 4096, 5120, 8192, 14336])
        S = min(rnd.choice([0, G, 64, 128, 256, 512]), K)
        if M * K > 13_000_000:
            continue
        x = recipes.activations(M, K, seed=seed * 100 + done, outlier_frac=0.01, outlier_gain=50.0)
        idx = recipes.reorder_index(x)
        gs = rnd.choice([1.0, recipes.tensor_scale(x, fmt)])
        print(f"random quantizer {done}: {mode} {fmt} M={M} K={K} S={S} gscale={gs}", flush=True)
        if mode == "x":
            want = oracle.quantize_x(x, idx, S, fmt, gs)
            q, sf = agemm.reorder_quantize_x(dev(x), dev(idx), S, fmt=fmt, global_scale=gs)
        elif mode == "w":
            want = oracle.quantize_w(x, idx, S, fmt, gs)
            q, sf = agemm.reorder_quantize_w(dev(x), dev(idx), S, fmt=fmt, global_scale=gs)
        else:
            gamma = (1.0 + 0.1 * torch.randn(K, generator=torch.Generator().manual_seed(done))).to(torch.bfloat16)
            want = oracle.rmsnorm_quantize_x(x, gamma, 1e-5, idx, S, fmt, gs)
            q, sf = agemm.rmsnorm_quantize_x(dev(x), dev(gamma), 1e-5, dev(idx), S, fmt=fmt, global_scale=gs)
        compare(f"{mode} {fmt} M={M} K={K} S={S}", q, sf, want)
        done += 1


@pytest.mark.parametrize("fmt", FMTS)
@pytest.mark.parametrize("M,K,S", [(300, 18944, 256), (257, 27648, 512), (256, 28672, 128), (40, 32736, 64), (3, 16416, 0),
                                   (700, 28672, 1024)])
def test_rows_of_more_than_16384_channels(agemm, oracle, fmt, M, K, S):
    """The reference's dedicated wide shapes (K = 18944: kernels/src/reorder.cu:380-555; 27648 and 28672:
    kernels/src/down.cu:71-233; dispatch kernels/src/bindings.cpp:141-160) and the longest row an int16 index
    allows: four units per thread.  Activations with tensor scale 1 and with the NVFP4 tensor scale (host value
    and device scalar), weights; every row against the oracle."""
    x = recipes.activations(M, K, seed=6000 + M + K)
    x[M // 2] = 0
    idx = recipes.reorder_index(x)
    print(f"wide rows {fmt} M={M} K={K} S={S}", flush=True)
    for gs in ((1.0, recipes.nvfp4_tensor_scale(x)) if fmt == "NVFP4" else (1.0, 0.5)):
        want = oracle.quantize_x(x, idx, S, fmt, gs)
        q, sf = agemm.reorder_quantize_x(dev(x), dev(idx), S, fmt=fmt, global_scale=gs)
        compare(f"x, tensor scale {gs}", q, sf, want)
        q, sf = agemm.reorder_quantize_x(dev(x), dev(idx), S, fmt=fmt, global_scale=torch.tensor(gs, dtype=torch.float32).cuda())
        compare(f"x, tensor scale {gs} on the device", q, sf, want)
    w = recipes.weights(M, K, seed=6001 + M)
    gw = recipes.tensor_scale(w, fmt)
    want = oracle.quantize_w(w, idx, S, fmt, gw)
    q, sf = agemm.reorder_quantize_w(dev(w), dev(idx), S, fmt=fmt, global_scale=gw)
    compare("w", q, sf, want)


def absmax_scale(x) -> float:
    """max|x| / 2688 by an IEEE fp32 division (model/qLlamaLayer.py:73-77), 1 for an all-zero tensor"""
    m = x.abs().max().float() / torch.full((), 2688.0)
    return float(m) if float(m) != 0.0 else 1.0


@pytest.mark.parametrize("M,K,S", [(4096, 4096, 256), (1, 4096, 256), (100, 2048, 128), (1000, 3072, 64), (37, 1024, 0),
                                   (16, 4096, 4096), (4097, 4096, 256), (9, 8192, 128), (33, 1056, 32)])
def test_scale_and_quantize_in_one_call(agemm, oracle, M, K, S):
    """reorder_quantize_x(global_scale="absmax"): the scale is torch's abs().max() / 2688 by an IEEE division, codes
    and scale bytes are the oracle's under that scale -- for tensors that take the one-launch kernel (rows stay in
    LDS while the workgroups exchange maxima) and for those that fall back to two launches (more than 4096 rows,
    other row lengths).  Called three times in a row on one stream: the exchange leaves nothing behind."""
    x = recipes.activations(M, K, seed=7000 + M + K + S)
    x[M // 2, K // 3] = -913.0                                   # the maximum is a negative element of one row
    idx = recipes.reorder_index(x)
    gs = absmax_scale(x)
    want = oracle.quantize_x(x, idx, S, "NVFP4", gs)
    xd, idxd = dev(x), dev(idx)
    print(f"scale + quantize M={M} K={K} S={S} gscale={gs}", flush=True)
    for _ in range(3):
        q, sf, scale = agemm.reorder_quantize_x(xd, idxd, S, fmt="NVFP4", global_scale="absmax")
        assert scale.dtype == torch.float32 and scale.dim() == 0 and float(scale) == gs
        compare("absmax", q, sf, want)


def test_scale_and_quantize_special_tensors(agemm, oracle):
    """All zeros -> scale 1; launches of different sizes one after the other on one stream; MXFP4 (no tensor scale
    in the format: the call still returns max / 2688 and quantizes under it, as the two separate calls do)."""
    K, S = 4096, 128
    idx = dev(recipes.reorder_index(recipes.activations(8, K, seed=1)))
    z = torch.zeros(48, K, dtype=torch.bfloat16, device="cuda")
    q, sf, scale = agemm.reorder_quantize_x(z, idx, S, fmt="NVFP4", global_scale="absmax")
    assert float(scale) == 1.0 and int(q.max()) == 0
    q, sf, scale = agemm.reorder_quantize_x(z[:0], idx, S, fmt="NVFP4", global_scale="absmax")   # no rows at all
    assert q.shape == (0, (K + S) // 2) and sf.numel() == 0 and float(scale) == 1.0
    for M in (4096, 17, 2048, 1, 300):
        x = recipes.activations(M, K, seed=M)
        gs = absmax_scale(x)
        want = oracle.quantize_x(x, idx.cpu(), S, "NVFP4", gs)
        print(f"scale + quantize, sizes in turn: M={M}", flush=True)
        q, sf, scale = agemm.reorder_quantize_x(dev(x), idx, S, fmt="NVFP4", global_scale="absmax")
        assert float(scale) == gs
        compare(f"M={M}", q, sf, want)
    x = recipes.activations(64, K, seed=5)
    q, sf, scale = agemm.reorder_quantize_x(dev(x), idx, S, fmt="MXFP4", global_scale="absmax")
    q2, sf2 = agemm.reorder_quantize_x(dev(x), idx, S, fmt="MXFP4", global_scale=scale)
    assert float(scale) == absmax_scale(x) and torch.equal(q, q2) and torch.equal(sf, sf2)


def test_scale_and_quantize_in_a_graph(agemm, oracle):
    """The one-launch kernel takes nothing from the host that changes from launch to launch, so a captured launch can
    be replayed: three replays with other input values each time, eager launches of another size in between."""
    M, K, S = 512, 4096, 256
    idx = dev(recipes.reorder_index(recipes.activations(8, K, seed=2)))
    xs = [recipes.activations(M, K, seed=40 + i) * (1.0 + i) for i in range(3)]
    buf = dev(xs[0]).clone()
    stream = torch.cuda.Stream()
    with torch.cuda.stream(stream):
        agemm.prepare_stream()
        agemm.reorder_quantize_x(buf, idx, S, fmt="NVFP4", global_scale="absmax")   # warm-up outside the capture
        stream.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=stream):
            q, sf, scale = agemm.reorder_quantize_x(buf, idx, S, fmt="NVFP4", global_scale="absmax")
        for i, x in enumerate(xs):
            buf.copy_(dev(x))
            graph.replay()
            stream.synchronize()
            gs = absmax_scale(x)
            print(f"graph replay {i} gscale={gs}", flush=True)
            assert float(scale) == gs
            compare(f"replay {i}", q, sf, oracle.quantize_x(x, idx.cpu(), S, "NVFP4", gs))
            other = recipes.activations(33, K, seed=90 + i)
            q2, sf2, s2 = agemm.reorder_quantize_x(dev(other), idx, S, fmt="NVFP4", global_scale="absmax")
            stream.synchronize()
            assert float(s2) == absmax_scale(other)


_ALONE = r"""
import sys, torch
sys.path.insert(0, sys.argv[1])
import recipes
from arcquant_amd import agemm
for M, K, S in ((4096, 4096, 256), (50, 2048, 64), (4096, 4096, 256)):
    x = recipes.activations(M, K, seed=M + K).cuda()
    idx = recipes.reorder_index(x.cpu()).cuda()
    print("alone", M, K, S, flush=True)
    q, sf, scale = agemm.reorder_quantize_x(x, idx, S, fmt="NVFP4", global_scale="absmax")
    g = agemm.tensor_scale(x)
    q2, sf2 = agemm.reorder_quantize_x(x, idx, S, fmt="NVFP4", global_scale=g)
    torch.cuda.synchronize()
    assert float(scale) == float(g) and torch.equal(q, q2) and torch.equal(sf, sf2), (M, K, S)
print("ALONE-OK")
"""


def test_scale_and_quantize_when_the_workgroups_do_not_meet(agemm):
    """A workgroup that does not hear from the others in time takes the tensor's maximum by itself.  With a waiting
    time of zero (ARCQ_RESIDENT_SPIN_US=0, read when the library is first used: hence a process of its own) every
    workgroup does so unless the others happen to be done already; results equal the two separate calls'."""
    import os
    import subprocess
    import sys
    here = os.path.dirname(os.path.abspath(__file__))
    env = dict(os.environ, ARCQ_RESIDENT_SPIN_US="0", PYTHONPATH=os.path.dirname(here) + os.pathsep + os.environ.get("PYTHONPATH", ""))
    out = subprocess.run([sys.executable, "-c", _ALONE, here], env=env, capture_output=True, text=True, timeout=300)
    print(out.stdout[-2000:], out.stderr[-2000:], flush=True)
    assert out.returncode == 0 and "ALONE-OK" in out.stdout
