"""CPU sweeps of the kernels' scalar arithmetic (arcquant_amd/csrc/arcq_math.h compiled by g++)
against the oracle.  What the GPU executes per element is this same source, so a closed form
that is wrong anywhere on these sweeps would be wrong in the kernels too."""
import ctypes
import os

import numpy as np
import pytest

import oracle as arcq_oracle


@pytest.fixture(scope="module")
def hm():
    path = arcq_oracle.build_hostmath()
    L = ctypes.CDLL(path)
    vp, i = ctypes.c_void_p, ctypes.c_int
    for n in ("arcq_host_ue4m3", "arcq_host_ue8m0", "arcq_host_e2m1"):
        getattr(L, n).argtypes = [vp, i, vp, vp]
    L.arcq_host_scale_values.argtypes = [vp, i, i, vp]
    return L


def run(fn, a):
    a = np.ascontiguousarray(a, np.float32)
    val = np.empty_like(a)
    byte = np.empty(a.shape, np.uint8)
    fn(a.ctypes.data, a.size, val.ctypes.data, byte.ctypes.data)
    return val, byte


def f32_neighbours(center, width):
    bits = np.asarray(center, np.float32).view(np.int32)[:, None] + np.arange(-width, width + 1, dtype=np.int32)
    return bits.reshape(-1).view(np.float32)


def scale_inputs(seed):
    rng = np.random.default_rng(seed)
    pows = np.ldexp(1.0, np.arange(-60, 60)).astype(np.float32)
    return np.concatenate([
        f32_neighbours(pows, 300),                                  # every binade edge, +-300 ulps
        np.exp2(rng.uniform(-40, 12, 400000)).astype(np.float32),   # log-uniform
        # amax/6 of bf16-valued amax: what main blocks actually produce
        (np.arange(0x0080, 0x7f80, dtype=np.uint32) << 16).view(np.float32) / np.float32(6.0),
        np.array([0.0, 1e-9, 2e-3, 448.0, 1e30], np.float32),
    ]).astype(np.float32)


def test_ue4m3_matches_oracle(hm, oracle):
    t = np.abs(scale_inputs(1))
    t = t[np.isfinite(t)]
    val, byte = run(hm.arcq_host_ue4m3, t)
    ov, ob = oracle.ue4m3(t)
    assert np.array_equal(val, ov) and np.array_equal(byte, ob)


def test_ue8m0_matches_oracle(hm, oracle):
    t = np.abs(scale_inputs(2))
    t = t[np.isfinite(t) & (t < 1e30)]
    val, byte = run(hm.arcq_host_ue8m0, t)
    ov, ob = oracle.ue8m0(np.where(t == 0, np.float32(1e-9), t))     # the caller's 0 -> 1e-9 is folded in
    assert np.array_equal(byte, ob)
    assert np.array_equal(val, ov)


def test_e2m1_matches_oracle(hm, oracle):
    rng = np.random.default_rng(3)
    ties = np.array([0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5.0, 0.5, 1, 1.5, 2, 3, 4, 6], np.float32)
    n = np.concatenate([rng.uniform(-8, 8, 500000).astype(np.float32), f32_neighbours(ties, 4),
                        -f32_neighbours(ties, 4), np.array([0.0, -0.0, 1e-38, -1e-38, 1e-45, -1e-45, 100, -100,
                                                            2.0 ** 24, -2.0 ** 24], np.float32)])
    val, code = run(hm.arcq_host_e2m1, n)
    ov, oc = oracle.e2m1(n)
    assert np.array_equal(code, oc)
    assert np.array_equal(val, ov) and not np.signbit(val[code == 0]).any()


def test_scale_byte_decoders(hm, oracle):
    for fmt, rng_ in ((0, range(0, 143)), (1, range(1, 255))):
        b = np.array(list(rng_), np.uint8)
        val = np.empty(b.shape, np.float32)
        hm.arcq_host_scale_values(b.ctypes.data, b.size, fmt, val.ctypes.data)
        assert np.array_equal(val, oracle.scale_values(b, fmt))


@pytest.mark.parametrize("fmt", [0, 1])
@pytest.mark.parametrize("residual", [0, 1])
def test_coarse_fast_encode_is_exact(hm, fmt, residual):
    """approximate quotient + 2^-13 nudge + hardware RNE == the reference's exact-quotient argmin,
    for every bf16 value x every block scale (x perturbed reciprocals), main blocks and residuals"""
    hm.arcq_host_check_coarse.restype = ctypes.c_longlong
    hm.arcq_host_check_coarse.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.POINTER(ctypes.c_longlong)]
    n = ctypes.c_longlong(0)
    bad = hm.arcq_host_check_coarse(fmt, residual, ctypes.byref(n))
    assert n.value > 1_000_000, n.value
    assert bad == 0, f"{bad} of {n.value} disagree"


def test_div6_coarse_is_exact(hm):
    assert hm.arcq_host_check_div6() == 0


def test_div6_any_is_exact(hm):
    """a/6 as three fused operations equals the IEEE quotient for every fp32 significand"""
    hm.arcq_host_check_div6_any.restype = ctypes.c_long
    assert hm.arcq_host_check_div6_any() == 0


def test_bf16_by_tensor_scale_division_is_exact(hm):
    """x/g (model/quantize.py:330) as q + (x - g*q)*rg for every bf16 significand of x and every
    fp32 significand of g, both signs"""
    hm.arcq_host_check_div_bf16.restype = ctypes.c_long
    hm.arcq_host_check_div_bf16.argtypes = [ctypes.c_int]
    assert hm.arcq_host_check_div_bf16(1) == 0


@pytest.mark.parametrize("fmt", [0, 1])
def test_two_sided_encode_is_exact(hm, fmt):
    """the encode used for tensor scales != 1 (two hardware conversions; e2m1_resolve where they
    differ) gives the reference's code for random operands and for +-200 ulp around every decision
    point, every scale, reciprocal off by -1/0/+1 ulp; the two conversions agree almost always"""
    hm.arcq_host_check_two_sided.restype = ctypes.c_longlong
    hm.arcq_host_check_two_sided.argtypes = [ctypes.c_int, ctypes.c_long, ctypes.POINTER(ctypes.c_longlong),
                                             ctypes.POINTER(ctypes.c_longlong)]
    acc, cnt = ctypes.c_longlong(), ctypes.c_longlong()
    bad = hm.arcq_host_check_two_sided(fmt, 500_000, ctypes.byref(acc), ctypes.byref(cnt))
    assert bad == 0
    assert cnt.value > 50_000_000
    assert acc.value / cnt.value > 0.999


def test_rstd_from_hardware_estimates_is_exact(hm):
    """1/sqrt(var + eps) of the fused RMSNorm kernel: sqrt and reciprocal rebuilt from 1-ulp estimates
    equal 1.0f / sqrtf(a) (two roundings) on a dense stretch of fp32 and across the exponent range"""
    hm.arcq_host_check_rstd.restype = ctypes.c_long
    hm.arcq_host_check_rstd.argtypes = [ctypes.c_long]
    assert hm.arcq_host_check_rstd(40_000_000) == 0


@pytest.mark.parametrize("fmt", [0, 1])
def test_scaled_encode_without_per_element_division_is_exact(hm, fmt):
    """the encode of units outside the residual range under an NVFP4 tensor scale: one division per unit (the
    maximum), codes from x * RN(rg * r) * (1 +- 2^-20), e2m1_resolve on RN(x/g) where the two conversions differ --
    against the reference's code of RN(RN(x/g) / s) for every bf16 x in reach of every block scale, tensor scales
    max / 2688 for every bf16 significand of the maximum and pseudo-random ones, reciprocal off by -1/0/+1 ulp"""
    hm.arcq_host_check_scaled_direct.restype = ctypes.c_longlong
    hm.arcq_host_check_scaled_direct.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.POINTER(ctypes.c_longlong),
                                                 ctypes.POINTER(ctypes.c_longlong)]
    acc, cnt = ctypes.c_longlong(), ctypes.c_longlong()
    bad = hm.arcq_host_check_scaled_direct(fmt, 1500, ctypes.byref(acc), ctypes.byref(cnt))
    assert bad == 0, f"{bad} of {cnt.value}"
    assert cnt.value > 250_000_000
    assert acc.value / cnt.value > 0.99
