"""CPU-only checks of the C-ABI library: it loads, exports every symbol include/arcq.h declares,
sizes buffers as documented and rejects bad arguments before touching a GPU."""
import ctypes
import os
import re

import pytest

from arcquant_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols(header="arcq.h"):
    text = open(os.path.join(ROOT, "include", header)).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(arcq_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    L = _lib.lib()
    names = declared_symbols()
    assert {"arcq_reorder_quantize_x", "arcq_reorder_quantize_w", "arcq_rmsnorm_quantize_x", "arcq_matmul"} <= set(
        names)
    for n in names:
        assert hasattr(L, n), f"{n} is declared in include/arcq.h but not exported"
    assert L.arcq_version() >= 100


def test_buffer_sizes():
    L = _lib.lib()
    assert L.arcq_group_size(0) == 16 and L.arcq_group_size(1) == 32 and L.arcq_group_size(7) == 0
    assert L.arcq_codes_bytes(2048, 4096, 128) == 2048 * 4224 // 2
    assert L.arcq_scales_bytes(2048, 4096, 128, 0) == 2048 * 4224 // 16
    assert L.arcq_scales_bytes(2048, 4096, 128, 1) == 2048 * 4224 // 32
    assert L.arcq_scales_bytes(1, 64, 0, 9) == 0


@pytest.mark.parametrize("K,S,fmt,want", [
    (4096, 128, 2, 3),      # unknown format
    (4100, 0, 0, 2),        # K not a multiple of 32
    (16, 0, 0, 2),          # K too small
    (32768, 0, 0, 2),       # beyond int16 indices
    (4096, 8, 0, 2),        # select_num not a multiple of the block
    (4096, 48, 1, 2),       # ... of 32 for MXFP4
    (4096, 8192, 0, 2),     # select_num > K
])
def test_argument_errors_need_no_gpu(K, S, fmt, want):
    L = _lib.lib()
    dummy = ctypes.c_void_p(0x1000)
    for fn in (L.arcq_reorder_quantize_x, L.arcq_reorder_quantize_w):
        assert fn(dummy, 4, K, dummy, S, fmt, 1.0, None, dummy, dummy, None) == want
    assert L.arcq_rmsnorm_quantize_x(dummy, dummy, 1e-5, 4, K, dummy, S, fmt, 1.0, None, dummy, dummy, None) == want
    assert L.arcq_reorder_quantize_x_absmax(dummy, 4, K, dummy, S, fmt, 2688.0, dummy, dummy, dummy, None) == want


def test_null_alignment_and_matmul_errors():
    L = _lib.lib()
    ok, odd = ctypes.c_void_p(0x1000), ctypes.c_void_p(0x1004)
    assert L.arcq_reorder_quantize_x(None, 4, 4096, ok, 0, 0, 1.0, None, ok, ok, None) == 1
    assert L.arcq_reorder_quantize_x(odd, 4, 4096, ok, 0, 0, 1.0, None, ok, ok, None) == 4
    assert L.arcq_reorder_quantize_x(ok, 0, 4096, ok, 0, 0, 1.0, None, ok, ok, None) == 0   # zero rows: nothing to do
    absmax = L.arcq_reorder_quantize_x_absmax                                                # scale + quantizer as one call
    assert absmax(ok, 4, 4096, ok, 0, 0, 2688.0, None, ok, ok, None) == 1                    # nowhere to put the scale
    assert absmax(None, 4, 4096, ok, 0, 0, 2688.0, ok, ok, ok, None) == 1
    assert absmax(odd, 4, 4096, ok, 0, 0, 2688.0, ok, ok, ok, None) == 4
    assert absmax(ok, 4, 4096, ok, 0, 0, 0.0, ok, ok, ok, None) == 2                         # divisor must be positive
    assert L.arcq_matmul(ok, ok, ok, ok, 4, 4, 100, 0, 1.0, None, None, ok, None) == 2       # K' % 64
    assert L.arcq_matmul(ok, ok, ok, ok, 4, 4, 128, 5, 1.0, None, None, ok, None) == 3
    assert L.arcq_matmul(ok, None, ok, ok, 4, 4, 128, 0, 1.0, None, None, ok, None) == 1
    assert L.arcq_matmul(ok, ok, ok, ok, 0, 4, 128, 0, 1.0, None, None, ok, None) == 0
    assert b"16-byte" in L.arcq_status_string(4)


def test_grouped_entry_points_reject_bad_arguments():
    """the MoE entry points check shapes, pointers and alignment before any launch"""
    L = _lib.lib()
    ok, odd = ctypes.c_void_p(0x1000), ctypes.c_void_p(0x1004)
    gq = L.arcq_grouped_reorder_quantize_x
    assert gq(ok, 8, 4096, ok, 0, ok, 128, 0, None, ok, ok, None) == 2          # no segment
    assert gq(ok, 8, 4100, ok, 2, ok, 128, 0, None, ok, ok, None) == 2          # K % 32
    assert gq(ok, 8, 4096, ok, 2, ok, 8, 0, None, ok, ok, None) == 2            # select_num % 16
    assert gq(ok, 8, 4096, ok, 2, ok, 128, 7, None, ok, ok, None) == 3          # format
    assert gq(ok, 8, 4096, None, 2, ok, 128, 0, None, ok, ok, None) == 1        # no offsets
    assert gq(odd, 8, 4096, ok, 2, ok, 128, 0, None, ok, ok, None) == 4
    assert gq(ok, 0, 4096, ok, 2, ok, 128, 0, None, ok, ok, None) == 0          # no rows: nothing to do
    gs = L.arcq_grouped_swiglu_quantize_x
    assert gs(ok, ok, 4000, 8, 4096, ok, 2, ok, 128, 0, None, ok, ok, None) == 2  # row stride below K
    assert gs(ok, None, 8192, 8, 4096, ok, 2, ok, 128, 0, None, ok, ok, None) == 1
    ts = L.arcq_grouped_tensor_scale
    assert ts(ok, None, 4096, 8, 4096, ok, 0, 2688.0, ok, None) == 2
    assert ts(ok, None, 4096, 8, 4096, ok, 2, 0.0, ok, None) == 2
    assert ts(ok, None, 4096, 8, 4096, ok, 2, 2688.0, None, None) == 1
    gm = L.arcq_grouped_matmul
    assert gm(ok, ok, ok, ok, ok, 2, 8, 256, 448, 1, 1.0, None, None, None, ok, None) == 2    # K' % 128
    assert gm(ok, ok, ok, ok, ok, 2, 8, 256, 384, 1, 1.0, None, None, None, ok, None) == 2    # K' < 512
    assert gm(ok, ok, ok, ok, ok, 0, 8, 256, 512, 1, 1.0, None, None, None, ok, None) == 2    # no segment
    assert gm(ok, ok, ok, ok, None, 2, 8, 256, 512, 1, 1.0, None, None, None, ok, None) == 1
    assert gm(ok, odd, ok, ok, ok, 2, 8, 256, 512, 1, 1.0, None, None, None, ok, None) == 4   # scale bytes unaligned
    assert gm(ok, ok, ok, ok, ok, 2, 0, 256, 512, 1, 1.0, None, None, None, ok, None) == 0
    sw = L.arcq_grouped_matmul_swiglu
    assert sw(ok, ok, ok, ok, ok, 2, 8, 250, 512, 1, 1.0, None, None, ok, None, None) == 2    # N % 16
    assert L.arcq_matmul_swiglu(ok, ok, ok, ok, 8, 256, 448, 1, 1.0, None, None, ok, None, None) == 2
    assert L.arcq_scales_from_absmax(None, 4, 2688.0, None) == 1
    assert L.arcq_scales_from_absmax(ok, 4, -1.0, None) == 2
    mc = L.arcq_moe_combine
    assert mc(ok, ok, ok, 8, 4100, 2, 16, ok, None) == 2                                      # H % 8
    assert mc(ok, ok, ok, 8, 4096, 9, 72, ok, None) == 2                                      # top_k > 8
    assert mc(ok, None, ok, 8, 4096, 2, 16, ok, None) == 1
    assert mc(ok, ok, ok, 0, 4096, 2, 0, ok, None) == 0
    mr = L.arcq_moe_route
    assert L.arcq_moe_route_workspace_bytes(4096, 8) == 64 * 8 * 4
    assert mr(ok, 0, 16, 65, 2, ok, ok, ok, ok, ok, ok, ok, 1 << 20, None) == 2               # more than 64 experts
    assert mr(ok, 0, 16, 8, 9, ok, ok, ok, ok, ok, ok, ok, 1 << 20, None) == 2                # top_k > 8
    assert mr(ok, 0, 16, 4, 5, ok, ok, ok, ok, ok, ok, ok, 1 << 20, None) == 2                # top_k > experts
    assert mr(None, 0, 16, 8, 2, ok, ok, ok, ok, ok, ok, ok, 1 << 20, None) == 1
    assert mr(ok, 0, 4096, 8, 2, ok, ok, ok, ok, ok, ok, ok, 16, None) == 7                   # workspace too small
    P = _lib.probe_lib()                 # the measurement-only library (include/arcq_probe.h)
    assert P.arcq_stream_probe_variants() >= 2
    assert P.arcq_stream_probe_variant(ok, ok, 1024, 512, 99, None) == 2


def test_decode_batches_fit_the_no_alloc_array():
    """arcq_matmul and arcq_matmul_noalloc share one planner: every decode batch (M <= 64) of the Llama-3-8B
    projection shapes must get a plan whose split-K partial tiles fit the fixed array, in both formats"""
    L = _lib.lib()
    limit = L.arcq_matmul_noalloc_limit()
    assert limit == 8 << 20
    for fmt in (0, 1):
        for N, K in ((6144, 4096), (4096, 4096), (28672, 4096), (4096, 14336)):
            for S in (64, 128, 256):
                for M in range(1, 65):
                    need = L.arcq_matmul_scratch_bytes(M, N, K + S, fmt)
                    assert need <= limit, (fmt, M, N, K + S, need)


def test_release_stream_without_buffers_needs_no_gpu_work():
    assert hasattr(_lib.lib(), "arcq_release_stream")


def test_probe_library_is_separate_from_the_product_library():
    """the copy kernels used for measurement live in their own library with their own header"""
    P, L = _lib.probe_lib(), _lib.lib()
    names = declared_symbols("arcq_probe.h")
    assert names == ["arcq_mfma_rate_probe", "arcq_mfma_rate_probe_flops", "arcq_stream_probe", "arcq_stream_probe_variant",
                     "arcq_stream_probe_variants"]
    assert P.arcq_mfma_rate_probe(3, 1, 10, ctypes.c_void_p(0x1000), ctypes.c_void_p(0x1000), None) == 2
    assert P.arcq_mfma_rate_probe_flops(0, 2, 1) == 256.0 * 4 * 2 * 4 * 8 * 2.0 * 32 * 32 * 64
    assert P.arcq_mfma_rate_probe_flops(1, 1, 3) == 256.0 * 4 * 1 * 3 * 4 * 8 * 2.0 * 32 * 32 * 16
    for n in names:
        assert hasattr(P, n) and not hasattr(L, n)
