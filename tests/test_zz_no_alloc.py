"""arcq_matmul_noalloc (the entry point that allocates nothing: split-K partial tiles in a fixed array
of the code object) through the C ABI against arcq_matmul on the same operands: identical bits, on
two calls in a row, the second with a smaller problem (the array keeps the first call's contents).
Shapes are ones whose plan cuts K into slices, i.e. that use the scratch array at all."""
import ctypes

import pytest
import torch

import recipes

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def L():
    assert torch.cuda.is_available(), "these tests need the MI355X"
    from arcquant_amd import _lib
    return _lib.lib()


def operands(agemm, M, N, K, S, fmt, seed):
    x = recipes.activations(M, K, seed=seed)
    w = recipes.weights(N, K, seed=seed + 1)
    idx = recipes.reorder_index(x).cuda()
    a, sfa = agemm.reorder_quantize_x(x.cuda(), idx, S, fmt=fmt)
    b, sfb = agemm.reorder_quantize_w(w.cuda(), idx, S, fmt=fmt)
    return a, sfa, b, sfb


def call(fn, ops, M, N, Kp, fid):
    a, sfa, b, sfb = ops
    c = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device="cuda")
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    rc = fn(a.data_ptr(), sfa.data_ptr(), b.data_ptr(), sfb.data_ptr(), M, N, Kp, fid, 0.5, None, None, c.data_ptr(), stream)
    return rc, c


@pytest.mark.parametrize("fmt,fid", [("MXFP4", 1), ("NVFP4", 0)])
def test_noalloc_matches_matmul_twice(L, fmt, fid):
    from arcquant_amd import agemm
    limit = L.arcq_matmul_noalloc_limit()
    # down projection of Llama-3-8B at decode batch 64 (8 slices of K: exactly the 8 MiB array), then a
    # smaller problem on the same array: 24 rows, N = 4096, shorter K
    first, second = (64, 4096, 14336, 256), (24, 4096, 8192, 128)
    for M, N, K, S in (first, second):
        need = L.arcq_matmul_scratch_bytes(M, N, K + S, fid)
        assert 0 < need <= limit, (need, limit)                    # these shapes do use the array
        print(f"noalloc {fmt} M={M} N={N} K'={K + S} scratch={need}", flush=True)
        ops = operands(agemm, M, N, K, S, fmt, seed=M)
        rc0, want = call(L.arcq_matmul, ops, M, N, K + S, fid)
        rc1, got = call(L.arcq_matmul_noalloc, ops, M, N, K + S, fid)
        torch.cuda.synchronize()
        assert rc0 == 0 and rc1 == 0
        assert not torch.isnan(got.float()).any()
        assert torch.equal(got, want)


def test_noalloc_without_scratch_and_beyond_the_limit(L):
    from arcquant_amd import agemm
    # a problem whose plan needs no scratch runs the same kernel as arcq_matmul
    M, N, K, S = 16, 4096, 4096, 256
    assert L.arcq_matmul_scratch_bytes(M, N, K + S, 1) == 0
    ops = operands(agemm, M, N, K, S, "MXFP4", seed=3)
    rc0, want = call(L.arcq_matmul, ops, M, N, K + S, 1)
    rc1, got = call(L.arcq_matmul_noalloc, ops, M, N, K + S, 1)
    torch.cuda.synchronize()
    assert rc0 == 0 and rc1 == 0 and torch.equal(got, want)
    # NVFP4 down projection at 512 rows: two slices of 512 x 4096 fp32 = 16 MiB, beyond the array -> refused,
    # nothing launched (MXFP4 does not cut K there: its plan needs no scratch)
    M, N, Kp = 512, 4096, 14592
    assert L.arcq_matmul_scratch_bytes(M, N, Kp, 1) == 0
    assert L.arcq_matmul_scratch_bytes(M, N, Kp, 0) > L.arcq_matmul_noalloc_limit()
    ok = ctypes.c_void_p(0x1000)                                   # never dereferenced: the call returns first
    assert L.arcq_matmul_noalloc(ok, ok, ok, ok, M, N, Kp, 0, 1.0, None, None, ok, None) == 7
    assert b"scratch" in L.arcq_status_string(7)


def test_noalloc_allocates_nothing(L):
    """What the entry point is named for: on a stream the library has never seen (no scratch buffers of its
    own), a call whose plan cuts K leaves the device's free memory where it was -- arcq_matmul on such a stream
    takes 32 MiB for its partial tiles -- and a released stream starts from nothing again."""
    from arcquant_amd import agemm
    M, N, K, S, fid = 64, 4096, 14336, 256, 1
    ops = operands(agemm, M, N, K, S, "MXFP4", seed=5)
    rc, want = call(L.arcq_matmul, ops, M, N, K + S, fid)            # kernels loaded, torch's pools warm
    assert rc == 0
    torch.cuda.synchronize()
    fresh = torch.cuda.Stream()
    c = torch.empty((M, N), dtype=torch.bfloat16, device="cuda")
    a, sfa, b, sfb = ops
    handle = ctypes.c_void_p(fresh.cuda_stream)
    fresh.wait_stream(torch.cuda.current_stream())
    torch.cuda.synchronize()
    free0 = torch.cuda.mem_get_info()[0]
    rc = L.arcq_matmul_noalloc(a.data_ptr(), sfa.data_ptr(), b.data_ptr(), sfb.data_ptr(), M, N, K + S, fid, 0.5, None, None,
                               c.data_ptr(), handle)
    torch.cuda.synchronize()
    free1 = torch.cuda.mem_get_info()[0]
    assert rc == 0 and torch.equal(c, want)
    assert free0 - free1 < (1 << 20), (free0, free1)
    # the allocating entry point on the same stream does take its buffer, and arcq_release_stream gives it back
    rc = L.arcq_matmul(a.data_ptr(), sfa.data_ptr(), b.data_ptr(), sfb.data_ptr(), M, N, K + S, fid, 0.5, None, None,
                       c.data_ptr(), handle)
    torch.cuda.synchronize()
    free2 = torch.cuda.mem_get_info()[0]
    assert rc == 0 and torch.equal(c, want)
    assert free1 - free2 >= (32 << 20) - (1 << 20), (free1, free2)
    assert L.arcq_release_stream(handle) == 0
    free3 = torch.cuda.mem_get_info()[0]
    assert free3 - free2 >= (32 << 20) - (1 << 20), (free2, free3)
    assert L.arcq_release_stream(handle) == 0                         # nothing left: still fine
