"""GPU parity of the augmented-K FP4 GEMM: within 1e-2 relative Frobenius error of
dequantize-then-matmul in fp32/fp64 (the stated tolerance; bf16 output rounding alone is
~2e-3), on seeded inputs quantized by the GPU quantizers (themselves bit-exact, see
test_gpu_quantize.py)."""
import numpy as np
import pytest
import torch

import recipes

pytestmark = pytest.mark.gpu
FMTS = ["NVFP4", "MXFP4"]
TOL = 1e-2


@pytest.fixture(scope="module")
def agemm():
    assert torch.cuda.is_available(), "these tests need the MI355X"
    from arcquant_amd import agemm as m
    return m


def rel_fro(got, want):
    got, want = got.double(), want.double()
    return float((got - want).norm() / want.norm())


def oracle_dq(oracle, codes, sf, fmt):
    """fp32 values of codes + scale bytes from the CPU oracle's dequantizer, back on the GPU (the
    library's own dequantizer stays out of the GEMM checks)"""
    c = codes.cpu().numpy()
    return torch.from_numpy(oracle.dequantize(c, sf.cpu().numpy().reshape(c.shape[0], -1), fmt)).cuda()


def quantized_pair(agemm, M, N, K, S, fmt, seed):
    x = recipes.activations(M, K, seed=seed)
    w = recipes.weights(N, K, seed=seed + 1)
    idx = recipes.reorder_index(x)
    gx, gw = recipes.tensor_scale(x, fmt), recipes.tensor_scale(w, fmt)
    xd, wd, idxd = x.cuda(), w.cuda(), idx.cuda()
    a, sfa = agemm.reorder_quantize_x(xd, idxd, S, fmt=fmt, global_scale=gx)
    b, sfb = agemm.reorder_quantize_w(wd, idxd, S, fmt=fmt, global_scale=gw)
    return (x, w, idx, gx, gw), (a, sfa, b, sfb)


@pytest.mark.parametrize("fmt", FMTS)
@pytest.mark.parametrize("M,N,K,S", [(1, 128, 256, 64), (16, 256, 512, 0), (37, 200, 1024, 128), (128, 128, 4096, 256),
                                     (130, 384, 448, 64)])
def test_matmul_vs_oracle_fp64(agemm, oracle, fmt, M, N, K, S):
    (x, w, idx, gx, gw), (a, sfa, b, sfb) = quantized_pair(agemm, M, N, K, S, fmt, seed=40 + M + N)
    print(f"matmul {fmt} M={M} N={N} K={K} S={S}", flush=True)
    y = agemm.matmul(a, b, sfa, sfb, gx * gw)
    assert y.shape == (M, N) and y.dtype == torch.bfloat16
    G = 16 if fmt == "NVFP4" else 32
    want = oracle.matmul(a.cpu().numpy(), sfa.cpu().numpy().reshape(M, -1), b.cpu().numpy(),
                         sfb.cpu().numpy().reshape(N, -1), fmt, alpha=gx * gw)
    assert sfa.numel() == M * (K + S) // G
    err = rel_fro(y.cpu().float(), torch.from_numpy(want))
    assert err < TOL, err
    # elementwise: bf16 rounding of an fp32-accumulated sum
    assert torch.allclose(y.cpu().float(), torch.from_numpy(want), rtol=2 ** -7, atol=1e-3 * float(np.abs(want).max()))


@pytest.mark.parametrize("fmt", FMTS)
def test_matmul_scale_argument_forms(agemm, fmt):
    (x, w, idx, gx, gw), (a, sfa, b, sfb) = quantized_pair(agemm, 48, 256, 512, 64, fmt, seed=5)
    y0 = agemm.matmul(a, b, sfa, sfb, gx * gw)
    y1 = agemm.matmul(a, b, sfa, sfb, torch.tensor(gx * gw))                       # CPU tensor, like .item()
    y2 = agemm.matmul(a, b, sfa, sfb, torch.tensor(gx * gw, device="cuda"))        # device scalar, no sync
    y3 = agemm.matmul(a, b, sfa, sfb, (torch.tensor(gx, device="cuda"), torch.tensor(gw, device="cuda")))
    assert torch.equal(y0, y1)
    for y in (y2, y3):
        assert rel_fro(y.float(), y0.float()) < 1e-2 and torch.allclose(y.float(), y0.float(), rtol=2 ** -6, atol=0)
    with pytest.raises(RuntimeError):
        agemm.matmul(a, b[:, :-32], sfa, sfb, 1.0)
    with pytest.raises(RuntimeError):
        agemm.matmul(a.float(), b, sfa, sfb, 1.0)


@pytest.mark.parametrize("fmt", FMTS)
def test_identity_weights_recover_activations(agemm, oracle, fmt):
    """W = I on the reordered channels: Y = d * (dq(x) main + residual) with d = dq(1.0) (1.0 for
    MXFP4, 1.03125 for NVFP4 whose 1/6 block scale rounds to 0.171875): at most two exact
    products per output, so the fp32 sum is exact and the bf16 result is determined."""
    M, K, S = 64, 256, 64
    x = recipes.activations(M, K, seed=12)
    idx = torch.arange(K).to(torch.int16)
    w = torch.eye(K).to(torch.bfloat16)
    a, sfa = agemm.reorder_quantize_x(x.cuda(), idx.cuda(), S, fmt=fmt)
    b, sfb = agemm.reorder_quantize_w(w.cuda(), idx.cuda(), S, fmt=fmt)
    y = agemm.matmul(a, b, sfa, sfb, 1.0).cpu().float()
    dq = oracle.quantize_x(x, idx, S, fmt, 1.0, want_dq=True)["dq"].astype(np.float64)
    d = {"NVFP4": 1.03125, "MXFP4": 1.0}[fmt]
    assert np.all(np.diag(oracle.quantize_w(w, idx, 0, fmt, 1.0, want_dq=True)["dq"]) == d)
    folded = dq[:, :K].copy()
    folded[:, K - S:] += dq[:, K:]
    want = torch.from_numpy(folded * d).to(torch.bfloat16).float()
    assert torch.equal(y, want)


@pytest.mark.parametrize("fmt", FMTS)
@pytest.mark.parametrize("M,N,K,S", [(512, 4096, 4096, 256), (2048, 6144, 4096, 256), (256, 4096, 14336, 256),
                                     (512, 6144, 1024, 128), (448, 6200, 768, 256), (128, 28672, 1024, 256),
                                     (100, 4096, 4096, 256), (384, 4100, 8192, 128)])
def test_matmul_llama_shapes_vs_torch_fp32(agemm, oracle, fmt, M, N, K, S):
    """Benchmark shapes, and shapes of one round of workgroups (at most 256 tiles of 128x64 or 128x128, also
    ragged and with K' % 256 == 128, and K cut into slices for a few hundred rows): compare with torch's
    fp32 matmul on the GPU of the operands as the CPU oracle dequantizes them."""
    (x, w, idx, gx, gw), (a, sfa, b, sfb) = quantized_pair(agemm, M, N, K, S, fmt, seed=3)
    print(f"matmul {fmt} M={M} N={N} K={K} S={S}", flush=True)
    y = agemm.matmul(a, b, sfa, sfb, gx * gw)
    prev = torch.backends.cuda.matmul.allow_tf32
    torch.backends.cuda.matmul.allow_tf32 = False
    try:
        want = (oracle_dq(oracle, a, sfa, fmt) @ oracle_dq(oracle, b, sfb, fmt).T) * (gx * gw)
    finally:
        torch.backends.cuda.matmul.allow_tf32 = prev
    err = rel_fro(y.float(), want)
    assert err < TOL, err
    # and the whole scheme tracks the unquantized product
    y_true = x.cuda().float() @ w.cuda().float().T
    assert rel_fro(y.float(), y_true) < 0.2


@pytest.mark.parametrize("fmt", FMTS)
@pytest.mark.parametrize("M", [1, 5, 16, 17, 32, 48, 64])
@pytest.mark.parametrize("N,K,S", [(6144, 4096, 256), (202, 384, 0), (4100, 1024, 128), (4100, 8192, 128),
                                   (8324, 1024, 256), (8450, 768, 256), (16500, 1024, 128)])
def test_matmul_decode_batches(agemm, oracle, fmt, M, N, K, S):
    """M <= 64 (decode batches) at a benchmark shape and at shapes whose N is not a multiple of the
    16-row strips or of the 4-wide stores: against torch's fp32 matmul of the dequantized operands,
    and, row by row, against the same call on a 128-row batch that contains these rows (another
    kernel computes that one).  The long-K shape and the wider batches of the benchmark shape take the
    split-K path (partial tiles in a workspace, added by a second launch): a repeated call must give
    the same bits.  The two wide shapes take the 128x64 tiles with a ragged last workgroup, one of them
    with N % 4 != 0."""
    (x, w, idx, gx, gw), (a, sfa, b, sfb) = quantized_pair(agemm, 128, N, K, S, fmt, seed=11)
    print(f"matmul decode {fmt} M={M} N={N} K={K} S={S}", flush=True)
    a_m = a[:M].contiguous()
    sfa_m = sfa.view(128, -1)[:M].contiguous().view(-1)
    y = agemm.matmul(a_m, b, sfa_m, sfb, gx * gw)
    assert y.shape == (M, N)
    assert torch.equal(y, agemm.matmul(a_m, b, sfa_m, sfb, gx * gw))
    prev = torch.backends.cuda.matmul.allow_tf32
    torch.backends.cuda.matmul.allow_tf32 = False
    try:
        want = (oracle_dq(oracle, a_m, sfa_m, fmt) @ oracle_dq(oracle, b, sfb, fmt).T) * (gx * gw)
    finally:
        torch.backends.cuda.matmul.allow_tf32 = prev
    assert rel_fro(y.float(), want) < TOL
    y_big = agemm.matmul(a, b, sfa, sfb, gx * gw)[:M]
    # same operands, fp32 accumulation in another order, one bf16 rounding each
    assert rel_fro(y.float(), y_big.float()) < 4e-3


@pytest.mark.parametrize("fmt", FMTS)
@pytest.mark.parametrize("M,N,K,S", [
    (1, 4096, 4096, 256),      # skinny, eight waves
    (48, 6144, 4096, 256),     # split-K: the second launch adds
    (64, 4100, 8192, 128),     # split-K with a ragged last tile
    (33, 28672, 1024, 128),    # tiled 128x64
    (40, 8324, 1024, 256),     # tiled 128x64, ragged last workgroup
    (300, 1000, 2048, 128),    # tiled, ragged M and N: transposed epilogue and the per-element one
    (512, 6144, 1024, 128),    # one round of 128x128 tiles
    (200, 4096, 8448, 256),    # a few hundred rows, long K: slices
    (1100, 1024, 1024, 0),     # 256x256 tiles (MXFP4 cost model may take smaller ones) with a ragged M
    (130, 384, 448, 64),       # K' % 128 != 0: direct kernels
    (5, 202, 384, 0),          # N % 4 != 0: scalar stores
])
def test_matmul_with_residual_equals_separate_add(agemm, fmt, M, N, K, S):
    """arcq_matmul_add through every epilogue: the same bits as matmul(...) + residual in bf16."""
    (x, w, idx, gx, gw), (a, sfa, b, sfb) = quantized_pair(agemm, M, N, K, S, fmt, seed=90 + M)
    g = torch.Generator().manual_seed(M * 7 + N)
    r = (torch.randn(M, N, generator=g) * 0.7).to(torch.bfloat16).cuda()
    print(f"matmul + residual {fmt} M={M} N={N} K={K} S={S}", flush=True)
    y = agemm.matmul(a, b, sfa, sfb, gx * gw)
    z = agemm.matmul(a, b, sfa, sfb, gx * gw, residual=r)
    assert torch.equal(z, y + r)
    with pytest.raises(RuntimeError):
        agemm.matmul(a, b, sfa, sfb, gx * gw, residual=r[:, :-1].contiguous())


def oracle_dq(oracle, q, sf, fmt):
    """fp32 values of quantized rows from the CPU oracle's dequantizer, on the GPU"""
    rows = q.shape[0]
    return torch.from_numpy(oracle.dequantize(q.cpu().numpy(), sf.cpu().numpy().reshape(rows, -1), fmt)).cuda()


def test_matmul_operand_of_more_than_4_gib(agemm, oracle):
    """An activation operand of 4.35 GB (2 000 000 rows of K' = 4352): the eight-wave MXFP4 kernels address rows
    with 32-bit byte offsets, so the dispatch must hand this one to the kernels with 64-bit addresses.  Random
    codes and scale bytes near 2^0; first, middle and last rows against the product of the operands as the CPU
    oracle dequantizes them."""
    M, N, Kp = 2_000_000, 512, 4352
    g = torch.Generator(device="cuda").manual_seed(1)
    a = torch.randint(0, 256, (M, Kp // 2), dtype=torch.uint8, device="cuda", generator=g)
    b = torch.randint(0, 256, (N, Kp // 2), dtype=torch.uint8, device="cuda", generator=g)
    sfa = torch.randint(124, 130, (M * (Kp // 32),), dtype=torch.uint8, device="cuda", generator=g)
    sfb = torch.randint(124, 130, (N * (Kp // 32),), dtype=torch.uint8, device="cuda", generator=g)
    assert a.numel() >= 1 << 32
    print(f"matmul MXFP4 M={M} N={N} K'={Kp}: operand of {a.numel()} bytes", flush=True)
    c = agemm.matmul(a, b, sfa, sfb, 1.0, fmt="MXFP4")
    db = oracle_dq(oracle, b, sfb, "MXFP4")
    prev = torch.backends.cuda.matmul.allow_tf32
    torch.backends.cuda.matmul.allow_tf32 = False
    for r0 in (0, M // 2 + 3, 1_999_000, M - 64):
        da = oracle_dq(oracle, a[r0:r0 + 64], sfa.view(M, -1)[r0:r0 + 64], "MXFP4")
        want = da @ db.T
        err = float((c[r0:r0 + 64].float() - want).norm() / want.norm())
        assert err < 5e-3, (r0, err)
    torch.backends.cuda.matmul.allow_tf32 = prev
    del a, c
    torch.cuda.empty_cache()


@pytest.mark.parametrize("seed", [1, 7])
def test_matmul_random_shapes(agemm, oracle, seed):
    """Forty random (format, M, N, K, select_num) problems per seed, sizes around the tile edges of every
    kernel the dispatch knows: quantize both operands, multiply, compare the whole output with the fp32 product
    of the operands as the CPU oracle dequantizes them (the rounding of the bf16 output bounds the error)."""
    import random
    rnd = random.Random(seed)
    done = 0
    while done < 40:
        fmt = rnd.choice(FMTS)
        M = rnd.choice([1, 2, 7, 16, 17, 31, 32, 33, 63, 64, 65, 100, 127, 128, 129, 200, 255, 256, 257, 300, 511, 512, 513, 700,
                        1000, 1024, 1500, 2048, 2100, 3000])
        N = rnd.choice([8, 16, 24, 64, 100, 128, 136, 200, 256, 264, 500, 512, 520, 1000, 1024, 2048, 2056, 4096, 4104, 6144,
                        8192, 8200, 16384, 28672])
        K = rnd.choice([64, 128, 192, 256, 320, 384, 448, 512, 640, 768, 896, 1024, 1152, 2048, 3072, 4096])
        S = min(rnd.choice([0, 64, 128, 256]), K)
        if M * N > 12_000_000 or N * K > 60_000_000:
            continue
        x = recipes.activations(M, K, seed=seed * 1000 + done, outlier_frac=0.01, outlier_gain=30.0).cuda()
        w = recipes.weights(N, K, seed=seed * 2000 + done).cuda()
        idx = torch.randperm(K, generator=torch.Generator().manual_seed(done)).to(torch.int16).cuda()
        print(f"random shape {done}: {fmt} M={M} N={N} K={K} S={S}", flush=True)
        a, sfa = agemm.reorder_quantize_x(x, idx, S, fmt=fmt)
        b, sfb = agemm.reorder_quantize_w(w, idx, S, fmt=fmt)
        y = agemm.matmul(a, b, sfa, sfb, 1.0, fmt=fmt)
        want = oracle_dq(oracle, a, sfa, fmt) @ oracle_dq(oracle, b, sfb, fmt).T
        err = float((y.float() - want).norm() / max(1e-20, float(want.norm())))
        assert err < 6e-3, (fmt, M, N, K, S, err)
        done += 1
