"""Pins the oracle's three scalar quantizers (CPU only).

Each is checked three ways: against vectors the reference's own functions
produced (tests/golden/refquant_golden.npz), against the torch restatement
running the reference's sequence of torch ops, and against a closed form or
known-answer table that a plausible slip (wrong tie direction, missing
subnormal floor, off-by-one exponent) would break.
"""
import numpy as np
import torch

from oracle import fakequant_torch as fq


def f32_neighbours(center, width):
    bits = np.asarray(center, np.float32).view(np.int32)[:, None] + np.arange(-width, width + 1, dtype=np.int32)
    return bits.reshape(-1).view(np.float32)


# ------------------------------------------------------------------ e2m1

def test_e2m1_tie_table(oracle):
    # what argmin-first-index on the ascending grid implies: ties go to the LOWER value
    n = np.array([0.25, -0.25, 0.75, -0.75, 1.25, -1.25, 1.75, -1.75, 2.5, -2.5, 3.5, -3.5, 5.0, -5.0], np.float32)
    want = np.array([0.0, -0.5, 0.5, -1.0, 1.0, -1.5, 1.5, -2.0, 2.0, -3.0, 3.0, -4.0, 4.0, -6.0], np.float32)
    val, code = oracle.e2m1(n)
    assert np.array_equal(val, want)
    # sign<<3 | magnitude index
    assert code.tolist() == [0x0, 0x9, 0x1, 0xA, 0x2, 0xB, 0x3, 0xC, 0x4, 0xD, 0x5, 0xE, 0x6, 0xF]


def test_e2m1_zero_and_saturation(oracle):
    # (beyond |n| ~ 2^25 the reference's fp32 differences all round to the same number and its
    # argmin degenerates; block scales keep |n| < 7 unless the tensor scale is absurd, so the path
    # is defined, here and in the kernels, for |n| <= 2^24)
    val, code = oracle.e2m1(np.array([0.0, -0.0, 1e-30, -1e-30, 6.0, 7.0, 1e6, -6.0, -100.0, 0.2499999, -0.2499999],
                                     np.float32))
    assert code.tolist() == [0, 0, 0, 0, 7, 7, 7, 0xF, 0xF, 0, 0]
    assert not np.signbit(val[:4]).any()


def test_e2m1_closed_form_sweep(oracle):
    # nearest grid value; tie -> lower.  Built from exact midpoints, independent of the argmin code.
    rng = np.random.default_rng(1)
    ties = np.array([0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5.0], np.float32)
    n = np.concatenate([rng.uniform(-7, 7, 200000).astype(np.float32), f32_neighbours(ties, 3),
                        -f32_neighbours(ties, 3)])
    mags = np.array([0, .5, 1, 1.5, 2, 3, 4, 6], np.float32)
    a = np.abs(n)
    up = (a[:, None] > ties[None, :]).sum(1)        # positive: strictly above a midpoint moves up
    upn = (a[:, None] >= ties[None, :]).sum(1)      # negative: at the midpoint already moves away from zero
    mi = np.where(n < 0, upn, up)
    want = np.where(n < 0, -mags[mi], mags[mi])
    val, code = oracle.e2m1(n)
    assert np.array_equal(val, want.astype(np.float32))
    assert np.array_equal(code, np.where((n < 0) & (mi > 0), 8 + mi, mi).astype(np.uint8))


def test_e2m1_golden_and_torch(oracle, golden):
    val, _ = oracle.e2m1(golden["e2m1_in"])
    assert np.array_equal(val, golden["e2m1_out"])
    tv, _ = fq.nearest_e2m1(torch.from_numpy(golden["e2m1_in"]))
    assert np.array_equal(tv.numpy(), golden["e2m1_out"])


# ------------------------------------------------------------------ ue4m3

def ue4m3_closed_form(t):
    """RNE to 1+3 mantissa bits on [2e-3, 448], no subnormals (exact integer arithmetic)."""
    t = np.clip(np.asarray(t, np.float32), np.float32(2e-3), np.float32(448.0)).astype(np.float64)
    m, e = np.frexp(t)               # t = m * 2^e, m in [0.5, 1)
    sig = m * 16                     # in [8, 16)
    r = np.round(sig)                # np.round is half-to-even, like torch.round
    return (r * np.ldexp(1.0, e - 4)).astype(np.float32)


def test_ue4m3_closed_form(oracle):
    rng = np.random.default_rng(2)
    t = np.exp2(rng.uniform(-12, 10, 300000)).astype(np.float32)
    # every tie between adjacent 4-bit significands in every binade, and their neighbours
    ties = np.concatenate([np.ldexp(np.arange(8.5, 16.5, 1.0) / 8, e) for e in range(-10, 9)]).astype(np.float32)
    t = np.concatenate([t, f32_neighbours(ties, 2), np.array([0, 1e-9, 2e-3, 0.0019531, 448, 449, 1e6], np.float32)])
    t = np.abs(t)
    val, byte = oracle.ue4m3(t)
    assert np.array_equal(val, ue4m3_closed_form(t))
    assert np.array_equal(oracle.scale_values(byte, "NVFP4"), val)
    assert val.min() == np.float32(2.0 ** -9) and val.max() == np.float32(448.0)


def test_ue4m3_known_answers(oracle):
    t = np.array([1e-9, 2e-3, 2.0 ** -9, 2.0 ** -6, 1.0, 1.0625, 1.0626, 1.1875, 1.9375, 1.94, 447, 448, 1000],
                 np.float32)
    want = np.array([2.0 ** -9, 2.0 ** -9, 2.0 ** -9, 2.0 ** -6, 1.0, 1.0, 1.125, 1.25, 2.0, 2.0, 448, 448, 448],
                    np.float32)
    val, byte = oracle.ue4m3(t)
    assert np.array_equal(val, want)
    # byte = standard E4M3 byte + 16 wherever a standard byte exists (value >= 2^-6)
    assert byte[0] == 0 and byte[3] == 0x08 + 16     # 2^-6 is E4M3 0x08
    assert byte[4] == (9 << 3) and byte[-1] == ((17 << 3) | 6)


def test_ue4m3_golden_and_torch(oracle, golden):
    val, _ = oracle.ue4m3(golden["scale_in"])
    assert np.array_equal(val, golden["ue4m3_out"])
    assert np.array_equal(fq.round_ue4m3(torch.from_numpy(golden["scale_in"])).numpy(), golden["ue4m3_out"])


# ------------------------------------------------------------------ ue8m0

def test_ue8m0_closed_form_away_from_powers(oracle):
    # where the +1e-9 is negligible (t >= 2^-12) and t is not within 1e-4 of a power of two,
    # the result is the plain ceiling power of two
    rng = np.random.default_rng(3)
    t = np.exp2(rng.uniform(-12, 20, 300000)).astype(np.float32)
    m, e = np.frexp(t.astype(np.float64))
    keep = (m > 0.5 + 1e-4) & (m < 1 - 1e-4)
    val, byte = oracle.ue8m0(t[keep])
    assert np.array_equal(val, np.ldexp(1.0, e[keep]).astype(np.float32))
    assert np.array_equal(byte.astype(np.int32) - 127, e[keep])


def test_ue8m0_powers_of_two(oracle):
    # 2^k -> 2^k for k >= -7; the +1e-9 pushes 2^k one binade up from k = -8 down
    k = np.arange(-27, 11)
    val, byte = oracle.ue8m0(np.ldexp(1.0, k).astype(np.float32))
    want = np.where(k >= -7, k, k + 1)
    assert np.array_equal(byte.astype(np.int32) - 127, want), (k, byte.astype(np.int32) - 127)
    # the all-zero block: amax/6 == 0 is replaced by 1e-9 -> 2e-9 -> 2^-28
    assert oracle.ue8m0(np.array([1e-9], np.float32))[1][0] == 127 - 28


def test_ue8m0_golden_and_torch(oracle, golden):
    val, byte = oracle.ue8m0(golden["scale_in"])
    assert np.array_equal(val, golden["ue8m0_out"])
    assert np.array_equal(oracle.scale_values(byte, "MXFP4"), val)
    assert np.array_equal(fq.round_ue8m0(torch.from_numpy(golden["scale_in"])).numpy(), golden["ue8m0_out"])


def test_ue8m0_every_binade_edge_vs_torch(oracle):
    # all 2^k, k=-40..20, with 200 fp32 neighbours each side: the C oracle's correctly
    # rounded log2 and torch.log2 must agree on ceil() everywhere
    t = f32_neighbours(np.ldexp(1.0, np.arange(-40, 21)).astype(np.float32), 200)
    val, _ = oracle.ue8m0(t)
    assert np.array_equal(val, fq.round_ue8m0(torch.from_numpy(t.copy())).numpy())
    v4, _ = oracle.ue4m3(t)
    assert np.array_equal(v4, fq.round_ue4m3(torch.from_numpy(t.copy())).numpy())
