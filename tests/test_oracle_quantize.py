"""Pins the oracle's row-level routines (CPU only): quantize_x / quantize_w /
rmsnorm_quantize_x / dequantize / matmul.

Checks: the reference's own end-to-end outputs (golden file), the torch
restatement op for op, and structural facts that a slip would break (tail =
Q(residual) for activations, tail = verbatim copy for weights, idempotence,
per-band error bounds, S=0 reduces to the plain block quantizer, matmul against
numpy on dequantised values).
"""
import numpy as np
import pytest
import torch

from oracle import fakequant_torch as fq

FMTS = ["NVFP4", "MXFP4"]


def bits_to_bf16(a):
    return torch.from_numpy(a.astype(np.int16)).view(torch.bfloat16)


def bf16_round(a):
    return torch.from_numpy(np.ascontiguousarray(a, np.float32)).to(torch.bfloat16)


def make_x(M, K, seed, outlier_frac=0.01, outlier_gain=40.0):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(M, K, generator=g)
    n_out = max(1, round(outlier_frac * K))
    x[:, torch.randperm(K, generator=g)[:n_out]] *= outlier_gain
    return x.to(torch.bfloat16)


def channel_order(x):
    return torch.argsort(x.float().abs().amax(0), stable=True).to(torch.int16)


@pytest.mark.parametrize("fmt", FMTS)
def test_golden_end_to_end_x(oracle, golden, fmt):
    x = bits_to_bf16(golden["x_bits"])
    # the reference returns its tensor scale rounded to bf16; the fp32 one it divides by is max(x)/2688
    gs = float(fq.tensor_scale(x, fmt))
    assert float(torch.tensor(gs).to(torch.bfloat16)) == float(golden[f"{fmt}_x_scale"])
    K = x.shape[1]
    for S, key in ((64, "x_out_bits"), (0, "x0_out_bits")):
        r = oracle.quantize_x(x, None, S, fmt, gs, want_dq=True)
        # the reference returns bf16(q*s*scale) when S > 0 and bf16(q*s) when S == 0
        # (quantize.py:333-335 has no multiply): compare bit patterns
        got = torch.from_numpy(r["dq"])
        got = (got * torch.tensor(gs) if S else got).to(torch.bfloat16)
        want = bits_to_bf16(golden[f"{fmt}_{key}"])
        assert got.shape == want.shape == (x.shape[0], K + S)
        assert torch.equal(got.view(torch.int16), want.view(torch.int16))
        # codes/scales decode to exactly those values
        assert np.array_equal(oracle.dequantize(r["codes"], r["scales"], fmt), r["dq"])


@pytest.mark.parametrize("fmt", FMTS)
def test_golden_end_to_end_w(oracle, golden, fmt):
    w = bits_to_bf16(golden["w_bits"])
    gs = float(fq.tensor_scale(w, fmt))
    assert float(torch.tensor(gs).to(torch.bfloat16)) == float(golden[f"{fmt}_w_scale"])
    r = oracle.quantize_w(w, None, 64, fmt, gs, want_dq=True)
    got = torch.from_numpy(r["dq"]).to(torch.bfloat16)          # not multiplied back by scale
    assert torch.equal(got.view(torch.int16), bits_to_bf16(golden[f"{fmt}_w_out_bits"]).view(torch.int16))


@pytest.mark.parametrize("fmt", FMTS)
def test_golden_block_values(oracle, golden, fmt):
    # fp32 outputs of quantize_{nv,mx}fp4_tensor before any bf16 cast
    x = bf16_round(golden[f"{fmt}_block_in"])
    r = oracle.quantize_x(x, None, 0, fmt, 1.0, want_dq=True)
    assert np.array_equal(r["dq"], golden[f"{fmt}_block_out"])


@pytest.mark.parametrize("fmt", FMTS)
@pytest.mark.parametrize("M,K,S", [(5, 256, 64), (3, 512, 0), (2, 1024, 128), (4, 128, 128)])
def test_c_oracle_equals_torch_restatement(oracle, fmt, M, K, S):
    x = make_x(M, K, seed=K + S)
    x[0, :32] = 0
    idx = channel_order(x)
    gs = float(fq.tensor_scale(x, fmt))
    r = oracle.quantize_x(x, idx, S, fmt, gs, want_dq=True)
    codes, sb, q = fq.quantize_x_detailed(x, idx, S, fmt, gs)
    assert np.array_equal(r["codes"], codes)
    assert np.array_equal(r["scales"], sb)
    assert np.array_equal(r["dq"], q.numpy())
    # weights
    w = (make_x(M, K, seed=7 * K + S, outlier_gain=3.0).float() * 0.02).to(torch.bfloat16)
    gw = float(fq.tensor_scale(w, fmt))
    rw = oracle.quantize_w(w, idx, S, fmt, gw, want_dq=True)
    cw, sw, qw = fq.quantize_w_detailed(w, idx, S, fmt, gw)
    assert np.array_equal(rw["codes"], cw) and np.array_equal(rw["scales"], sw)
    assert np.array_equal(rw["dq"], qw.numpy())


@pytest.mark.parametrize("fmt", FMTS)
def test_torch_restatement_public_functions_match_golden(golden, fmt):
    # the functions bench.py times as the CPU baseline reproduce the reference's outputs
    x = bits_to_bf16(golden["x_bits"])
    w = bits_to_bf16(golden["w_bits"])
    qx, _, sx = fq.fake_quantize_x(x, 64, fmt)
    qw, _, sw = fq.fake_quantize_w(w, 64, fmt)
    assert torch.equal(qx.view(torch.int16), bits_to_bf16(golden[f"{fmt}_x_out_bits"]).view(torch.int16))
    assert torch.equal(qw.view(torch.int16), bits_to_bf16(golden[f"{fmt}_w_out_bits"]).view(torch.int16))
    assert float(sx) == float(bf16_round(golden[f"{fmt}_x_scale"].reshape(1))[0])


@pytest.mark.parametrize("fmt", FMTS)
def test_structure_of_augmented_k(oracle, fmt):
    M, K, S = 6, 512, 128
    G = oracle.group_size(fmt)
    x = make_x(M, K, seed=11)
    idx = channel_order(x)
    gs = 0.037 if fmt == "NVFP4" else 1.0
    full = oracle.quantize_x(x, idx, S, fmt, gs, want_dq=True)
    plain = oracle.quantize_x(x, idx, 0, fmt, gs, want_dq=True)
    # first K outputs do not depend on S
    assert np.array_equal(full["codes"][:, :K // 2], plain["codes"])
    assert np.array_equal(full["scales"][:, :K // G], plain["scales"])
    # tail = block quantizer applied to the fp32 residual of the last S reordered channels:
    # feed the residual through the fp32 block path of the torch restatement
    xr = torch.index_select(x, 1, idx.long()).float() / torch.tensor(gs)
    resid = xr[:, K - S:] - torch.from_numpy(plain["dq"][:, K - S:])
    q_tail, pos, s_tail = fq.blockwise(resid.contiguous(), fmt, detail=True)
    assert np.array_equal(full["dq"][:, K:], q_tail.numpy())
    assert np.array_equal(full["codes"][:, K // 2:], fq.pack_positions(pos))
    # ARC's point: main + tail is closer to x than main alone on the selected channels
    e0 = (xr[:, K - S:] - torch.from_numpy(plain["dq"][:, K - S:])).abs().mean()
    e1 = (xr[:, K - S:] - torch.from_numpy(full["dq"][:, K - S:K] + full["dq"][:, K:])).abs().mean()
    assert e1 < 0.25 * e0
    # weights: tail is a verbatim copy of the last S/G blocks
    w = make_x(M, K, seed=12)
    rw = oracle.quantize_w(w, idx, S, fmt, gs)
    assert np.array_equal(rw["codes"][:, K // 2:], rw["codes"][:, (K - S) // 2:K // 2])
    assert np.array_equal(rw["scales"][:, K // G:], rw["scales"][:, (K - S) // G:K // G])


@pytest.mark.parametrize("fmt", FMTS)
def test_idempotent_and_error_bands(oracle, fmt):
    x = make_x(16, 512, seed=5)
    G = oracle.group_size(fmt)
    r = oracle.quantize_x(x, None, 0, fmt, 1.0, want_dq=True)
    dq = r["dq"]
    s = np.repeat(oracle.scale_values(r["scales"], fmt), G, axis=1)
    xv = x.float().numpy()
    n = np.abs(dq / s)
    # half the local grid spacing, in units of the block scale
    half = np.where(n < 2, 0.25, np.where(n < 4, 0.5, 1.0))
    inside = np.abs(xv) <= 6 * s                      # RNE'd UE4M3 scales may leave amax slightly above 6s
    assert np.all(np.abs(xv - dq)[inside] <= (half * s)[inside] * (1 + 1e-6))
    assert np.all(np.abs(xv - dq) <= 1.0 * s * (1 + 1e-6) + (~inside) * np.abs(xv) * 0.07)
    # values that already sit on the grid survive a second pass unchanged (they are exact in bf16:
    # <= 6 significant bits)
    again = oracle.quantize_x(torch.from_numpy(dq).to(torch.bfloat16), None, 0, fmt, 1.0, want_dq=True)
    assert np.array_equal(again["dq"], dq)


def test_identity_index_equals_none_and_gather(oracle):
    x = make_x(4, 256, seed=9)
    idx = channel_order(x)
    a = oracle.quantize_x(x, idx, 64, "NVFP4", 0.05)
    b = oracle.quantize_x(torch.index_select(x, 1, idx.long()), None, 64, "NVFP4", 0.05)
    c = oracle.quantize_x(torch.index_select(x, 1, idx.long()), torch.arange(256).to(torch.int16), 64, "NVFP4", 0.05)
    for k in ("codes", "scales"):
        assert np.array_equal(a[k], b[k]) and np.array_equal(a[k], c[k])


def test_shape_errors(oracle):
    x = make_x(2, 80, seed=1)
    with pytest.raises(ValueError):
        oracle.quantize_x(x, None, 0, "MXFP4")       # K not a multiple of the block size
    x = make_x(2, 128, seed=1)
    with pytest.raises(ValueError):
        oracle.quantize_x(x, None, 48, "MXFP4")      # S not a multiple of 32
    with pytest.raises(ValueError):
        oracle.quantize_x(x, None, 256, "NVFP4")     # S > K


@pytest.mark.parametrize("fmt", FMTS)
def test_rmsnorm_quantize(oracle, fmt):
    M, K, S, eps = 7, 512, 64, 1e-5
    g = torch.Generator().manual_seed(3)
    x = make_x(M, K, seed=4, outlier_frac=0.005, outlier_gain=50.0)
    x[2] = 0                                              # an all-zero token
    gamma = (torch.rand(K, generator=g) + 0.5).to(torch.bfloat16)
    ref_norm = fq.hf_rmsnorm(x, gamma, eps)
    idx = channel_order(ref_norm)
    r = oracle.rmsnorm_quantize_x(x, gamma, eps, idx, S, fmt, 1.0, want_dq=True, want_normed=True)
    normed = bits_to_bf16(r["normed"])
    # (1) the normalisation step against torch's own fp32 reduction: same formula, a different
    #     summation order -> equal up to rare 1-ulp bf16 flips.  Not bitwise; match rate only.
    same = (normed.view(torch.int16) == ref_norm.view(torch.int16)).float().mean().item()
    assert same > 0.995
    assert torch.allclose(normed.float(), ref_norm.float(), rtol=2 ** -7, atol=0)
    # (2) everything after the normalisation is quantize_x on the normalised tensor, bit for bit
    q = oracle.quantize_x(normed, idx, S, fmt, 1.0, want_dq=True)
    for k in ("codes", "scales", "dq"):
        assert np.array_equal(r[k], q[k])
    # (3) closed form for one row, in float64 from scratch
    row = x[1].double()
    rstd = 1.0 / np.sqrt(np.float32(np.float32((row * row).sum().item() / K) + np.float32(eps)))
    h = (x[1].float() * torch.tensor(np.float32(rstd))).to(torch.bfloat16)
    o = (gamma.float() * h.float()).to(torch.bfloat16)
    assert torch.equal(o.view(torch.int16), normed[1].view(torch.int16))


def test_rmsnorm_closed_form_every_row(oracle):
    """The normalisation step at the benchmark's hidden size, every row of a 64 x 4096 case, from scratch
    in exact arithmetic: the sum of squares of bf16 values as an integer sum (python ints cannot
    round), mean and 1/sqrt rounded to fp32 where benchmarks/modeling_arc.py:237-242 rounds them, the
    two bf16 roundings of h and gamma * h.  A dropped term, a wrong divisor (K vs K-1), eps added in
    the wrong place or a single rounding instead of two each fail it."""
    from fractions import Fraction
    M, K, eps = 64, 4096, 1e-5
    x = make_x(M, K, seed=41, outlier_frac=0.005, outlier_gain=50.0)
    x[5] = 0
    x[6] *= 1e-3
    x[7] *= 300.0
    g = torch.Generator().manual_seed(42)
    gamma = (torch.rand(K, generator=g) + 0.5).to(torch.bfloat16)
    r = oracle.rmsnorm_quantize_x(x, gamma, eps, None, 0, "NVFP4", 1.0, want_normed=True)
    normed = bits_to_bf16(r["normed"])
    xd = x.double().numpy()
    for m in range(M):
        # every bf16 is an integer multiple of 2^-133: exact integer sum of squares
        ints = [int(v * 2.0 ** 133) for v in xd[m]]
        assert all(float(i) * 2.0 ** -133 == v for i, v in zip(ints[:8], xd[m][:8]))
        mean = Fraction(sum(i * i for i in ints), K) / Fraction(2) ** 266
        var = np.float32(float(mean))                               # Fraction -> fp64 -> fp32 ...
        for nb in (np.nextafter(var, np.float32(np.inf)), np.nextafter(var, np.float32(-np.inf))):
            # ... is the correctly rounded fp32: no neighbour is closer to the exact mean
            assert abs(Fraction(float(var)) - mean) < abs(Fraction(float(nb)) - mean) or mean == 0
        a = np.float32(var + np.float32(eps))
        rstd = np.float32(1.0) / np.sqrt(a, dtype=np.float32)
        h = (x[m].float() * torch.tensor(rstd)).to(torch.bfloat16)
        o = (gamma.float() * h.float()).to(torch.bfloat16)
        assert torch.equal(o.view(torch.int16), normed[m].view(torch.int16)), m


@pytest.mark.parametrize("fmt", FMTS)
def test_matmul_oracle(oracle, fmt):
    M, N, K, S = 9, 11, 256, 64
    x = make_x(M, K, seed=21)
    w = (make_x(N, K, seed=22, outlier_gain=2.0).float() * 0.02).to(torch.bfloat16)
    idx = channel_order(x)
    gx, gw = float(fq.tensor_scale(x, fmt)), float(fq.tensor_scale(w, fmt))
    a = oracle.quantize_x(x, idx, S, fmt, gx, want_dq=True)
    b = oracle.quantize_w(w, idx, S, fmt, gw, want_dq=True)
    y = oracle.matmul(a["codes"], a["scales"], b["codes"], b["scales"], fmt, alpha=gx * gw)
    want = (a["dq"].astype(np.float64) @ b["dq"].astype(np.float64).T) * (np.float32(gx * gw))
    assert np.allclose(y, want, rtol=1e-6, atol=1e-9)
    # the ARC identity: augmented product = sum over K of (x_hat + r_hat) * w_hat on the selected channels
    xa, wb = a["dq"].astype(np.float64), b["dq"].astype(np.float64)
    folded = xa[:, :K].copy()
    folded[:, K - S:] += xa[:, K:]
    assert np.allclose(want, (folded @ wb[:, :K].T) * np.float32(gx * gw), rtol=1e-9)
    # and it is the reference's F.linear on fake-quantised tensors, up to its bf16 casts
    y_fake = fq.fake_linear(x, w, idx, S, fmt).float().numpy()
    rel = np.linalg.norm(y - y_fake) / np.linalg.norm(y_fake)
    assert rel < 1e-2, rel
    # sanity on the whole scheme: close to the unquantised product, closer with S than without
    y_true = (x.float() @ w.float().T).numpy()
    a0 = oracle.quantize_x(x, idx, 0, fmt, gx)
    b0 = oracle.quantize_w(w, idx, 0, fmt, gw)
    y0 = oracle.matmul(a0["codes"], a0["scales"], b0["codes"], b0["scales"], fmt, alpha=gx * gw)
    err_s = np.linalg.norm(y - y_true) / np.linalg.norm(y_true)
    err_0 = np.linalg.norm(y0 - y_true) / np.linalg.norm(y_true)
    assert err_s < err_0 < 0.3
