"""Fused act_fn(gate) * up -> quantize against the unfused sequence the reference's layers run
(model/qLlamaLayer.py:432-439): torch's bf16 SiLU and multiply, then the (bit-exact) activation
quantizer.  The SiLU goes through the exponential of the platform's math library, so two checks:
  * on the GPU, torch's own silu * up feeds the same quantizer: codes and scales must be identical
    (same exp implementation, same formula x / (1 + exp(-x)));
  * against the CPU oracle (torch CPU silu, C oracle quantizer) at most 1e-3 of the code bytes and
    of the scale bytes may differ: a last-bit difference between two exp implementations can move
    a bf16 rounding.  Parity of the activation step is unpinned beyond that (no reference vectors)."""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

import recipes

pytestmark = pytest.mark.gpu
FMTS = ["NVFP4", "MXFP4"]


@pytest.fixture(scope="module")
def agemm():
    assert torch.cuda.is_available(), "these tests need the MI355X"
    from arcquant_amd import agemm as m
    return m


def inputs(M, K, seed):
    g = torch.Generator().manual_seed(seed)
    gu = (torch.randn(M, 2 * K, generator=g) * 1.5).to(torch.bfloat16)
    gu[:, :7] *= 8.0                      # a few large gates (saturated SiLU) and large products
    if M > 1:
        gu[1] = 0
    return gu


@pytest.mark.parametrize("fmt", FMTS)
@pytest.mark.parametrize("M,K,S", [(1, 512, 64), (33, 1024, 128), (16, 14336, 256), (130, 2048, 0), (70, 18944, 256),
                                   (33, 28672, 512)])
def test_fused_equals_unfused_on_gpu(agemm, oracle, fmt, M, K, S):
    gu = inputs(M, K, seed=70 + M)
    gud = gu.cuda()
    gate, up = gud[:, :K], gud[:, K:]                  # strided views of the fused projection output
    t = F.silu(gate) * up
    idx = recipes.reorder_index(t.cpu())
    idxd = idx.cuda()
    print(f"swiglu {fmt} M={M} K={K} S={S}", flush=True)
    # tensor scale 1
    q0, s0 = agemm.reorder_quantize_x(t.contiguous(), idxd, S, fmt=fmt)
    q1, s1 = agemm.swiglu_quantize_x(gate, up, idxd, S, fmt=fmt)
    assert torch.equal(q0, q1) and torch.equal(s0, s1)
    # NVFP4 tensor scale from the fused absmax pass
    q2, s2, scale = agemm.swiglu_quantize_x(gate, up, idxd, S, fmt=fmt, global_scale="absmax")
    want_scale = t.abs().max().float() / torch.full((), 2688.0, device="cuda")
    assert float(scale) == float(want_scale)
    q3, s3 = agemm.reorder_quantize_x(t.contiguous(), idxd, S, fmt=fmt, global_scale=want_scale)
    assert torch.equal(q2, q3) and torch.equal(s2, s3)
    # contiguous separate tensors give the same result as the strided views
    q4, s4 = agemm.swiglu_quantize_x(gate.contiguous(), up.contiguous(), idxd, S, fmt=fmt)
    assert torch.equal(q4, q1) and torch.equal(s4, s1)

    # CPU oracle: torch CPU silu * up, then the C oracle quantizer
    t_cpu = F.silu(gu[:, :K]) * gu[:, K:]
    want = oracle.quantize_x(t_cpu, idx, S, fmt, 1.0)
    dc = float((q1.cpu().numpy() != want["codes"]).mean())
    ds = float((s1.cpu().numpy().reshape(want["scales"].shape) != want["scales"]).mean())
    assert dc <= 1e-3 and ds <= 1e-3, (dc, ds)


def test_infinite_gate_leaves_its_neighbour_alone(agemm):
    """The kernels form the products of a pair of elements with a dot instruction whose unused term is
    (other half) * 0: an infinite activation would turn its neighbour's product into NaN there.  Waves that
    hold a non-finite activation multiply the unpacked halves instead, as torch's elementwise silu * up does:
    max |t| of an eight-element row around such a pair is the infinity itself, not NaN."""
    import ctypes
    from arcquant_amd import _lib
    L = _lib.lib()
    inf = float("inf")
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    for gate in ([inf, 2.0, 1, 1, 1, 1, 1, 1], [2.0, inf, 1, 1, 1, 1, 1, 1], [1, 1, 1, 1, 1, 1, 3.0, inf]):
        g = torch.tensor(gate, dtype=torch.bfloat16, device="cuda")
        u = torch.full((8,), 0.5, dtype=torch.bfloat16, device="cuda")
        want = (F.silu(g) * u).abs().float()
        assert int(torch.isinf(want).sum()) == 1 and not bool(torch.isnan(want).any())     # torch: one inf, no NaN
        out = torch.zeros((), dtype=torch.float32, device="cuda")
        assert L.arcq_tensor_scale(g.data_ptr(), u.data_ptr(), 8, 1, 8, 1.0, out.data_ptr(), stream) == 0
        torch.cuda.synchronize()
        assert float(out) == inf, (gate, float(out))          # a NaN neighbour would win the maximum (its bits are larger)
    # and the finite neighbour's value is what it is without the infinity beside it
    g = torch.tensor([0.0, 2.0, 0, 0, 0, 0, 0, 0], dtype=torch.bfloat16, device="cuda")
    u = torch.full((8,), 0.5, dtype=torch.bfloat16, device="cuda")
    out = torch.zeros((), dtype=torch.float32, device="cuda")
    assert L.arcq_tensor_scale(g.data_ptr(), u.data_ptr(), 8, 1, 8, 1.0, out.data_ptr(), stream) == 0
    assert float(out) == float((F.silu(g) * u).abs().max())


def test_errors(agemm):
    g = torch.zeros(4, 64, dtype=torch.bfloat16, device="cuda")
    idx = torch.arange(64, dtype=torch.int16, device="cuda")
    with pytest.raises(RuntimeError):
        agemm.swiglu_quantize_x(g, g[:, :32], idx, 0)
    with pytest.raises(RuntimeError):
        agemm.swiglu_quantize_x(g.float(), g.float(), idx, 0)
    with pytest.raises(RuntimeError):
        agemm.swiglu_quantize_x(g, g, idx, 16, fmt="MXFP4")     # select_num not a multiple of 32


def test_silu_of_every_bf16_value(agemm):
    """The SiLU inside the fused kernels against torch's own bf16 silu on the GPU for all 65536 bf16
    inputs: arcq_tensor_scale over a tensor of eight copies of g with up = 1 and divisor 1 returns
    |silu(g)| itself.  Finite inputs here; test_infinite_gate_leaves_its_neighbour_alone covers the others."""
    import ctypes
    from arcquant_amd import _lib
    L = _lib.lib()
    bits = torch.arange(65536, dtype=torch.int32)
    g = (bits << 16).view(torch.float32).to(torch.bfloat16)          # exact: the low half is zero
    finite = torch.isfinite(g.float())
    gate = g.cuda()[:, None].repeat(1, 8).contiguous()               # [65536, 8]
    up = torch.ones(8, dtype=torch.bfloat16, device="cuda")
    out = torch.zeros(65536, dtype=torch.float32, device="cuda")
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    print("silu over all bf16 values", flush=True)
    base_g, base_o = gate.data_ptr(), out.data_ptr()
    for i in range(65536):
        if not bool(finite[i]):
            continue
        rc = L.arcq_tensor_scale(base_g + 16 * i, up.data_ptr(), 8, 1, 8, 1.0, base_o + 4 * i, stream)
        assert rc == 0
    torch.cuda.synchronize()
    want = F.silu(g.cuda()).abs().float()
    want = torch.where(want == 0, torch.ones_like(want), want)       # the entry point maps an all-zero tensor to 1
    got, want = out.cpu()[finite], want.cpu()[finite]
    bad = (got != want).nonzero().flatten()
    assert bad.numel() == 0, [(hex(int(bits[finite][j])), float(got[j]), float(want[j])) for j in bad[:8]]
