"""INT4 paged KV cache on the GPU: the fused quantize + append against the torch restatement of
model/kv_cache.py:23-37 (codes and (scale, zero) pairs bit-exact), the pre-quantized store, and the
decode attention against fp64 softmax attention over the dequantized cache.  Attention tolerance:
relative Frobenius error of the fp16 / bf16 output <= 1e-3 / 5e-3 (the output rounding alone is
3e-4 / 2e-3; the kernel accumulates in fp32)."""
import pytest
import torch

pytestmark = pytest.mark.gpu
DTYPES = [torch.float16, torch.bfloat16]


@pytest.fixture(scope="module")
def kvc():
    assert torch.cuda.is_available(), "these tests need the MI355X"
    from arcquant_amd import kv_cache as m
    return m


@pytest.fixture(scope="module")
def ref():
    from oracle import kvcache_torch as m
    return m


def make_table(lengths, page_size, batch):
    """pages of sequence b: b, b + batch, ... (model/kv_cache.py:293-296)"""
    cnt = [(n + page_size - 1) // page_size for n in lengths]
    indptr, indices, last = [0], [], []
    for b, (n, c) in enumerate(zip(lengths, cnt)):
        indptr.append(indptr[-1] + c)
        indices += [j * batch + b for j in range(c)]
        off = n % page_size
        last.append(page_size if (n and off == 0) else off)
    t = lambda x: torch.tensor(x, dtype=torch.int32)
    return t(indptr), t(indices), t(last), max(cnt) if cnt else 0


def rel_fro(got, want):
    got, want = got.double().cpu(), want.double().cpu()
    return float((got - want).norm() / want.norm())


@pytest.mark.parametrize("dtype", DTYPES)
def test_quantize_append_is_bit_exact(kvc, ref, dtype):
    batch, heads, page_size, layers, layer = 3, 2, 16, 2, 1
    lengths = [37, 16, 5]                                   # ragged prefill, page boundary, short
    g = torch.Generator().manual_seed(3)
    total = sum(lengths)
    k = (torch.randn(total, heads, 128, generator=g) * 2).to(dtype)
    v = torch.randn(total, heads, 128, generator=g).to(dtype)
    k[3] = 0.25                                             # constant row: max - min below the clamp
    v[4, 0, :64] = 0
    indptr, indices, last, maxc = make_table(lengths, page_size, batch)
    pages = torch.zeros((maxc + 1) * batch, layers, 2, heads, page_size, 64, dtype=torch.uint8, device="cuda")
    params = torch.zeros((maxc + 1) * batch, layers, 2, heads, page_size, 2, dtype=dtype, device="cuda")
    seq = torch.tensor([0, 37, 53, 58], dtype=torch.int32)
    print(f"kv append {dtype}", flush=True)
    kvc.quantize_append(pages, params, indptr.cuda(), indices.cuda(), last.cuda(), k.cuda(), v.cuda(), layer,
                        seqlen_indptr=seq.cuda())
    # one more token per sequence (crosses a page boundary for sequence 1: 16 -> 17)
    lengths2 = [n + 1 for n in lengths]
    indptr2, indices2, last2, _ = make_table(lengths2, page_size, batch)
    k1 = torch.randn(batch, heads, 128, generator=g).to(dtype)
    v1 = torch.randn(batch, heads, 128, generator=g).to(dtype)
    kvc.quantize_append(pages, params, indptr2.cuda(), indices2.cuda(), last2.cuda(), k1.cuda(), v1.cuda(), layer)

    pc, sc = pages.cpu(), params.cpu()
    assert int(pc[:, 0].sum()) == 0 and float(sc[:, 0].abs().sum()) == 0          # the other layer is untouched
    for b in range(batch):
        (kc, kp), (vc, vp) = ref.gather_sequence(pc, sc, indptr2, indices2, last2, layer, b)
        lo = int(seq[b])
        kb = torch.cat([k[lo:lo + lengths[b]], k1[b:b + 1]])
        vb = torch.cat([v[lo:lo + lengths[b]], v1[b:b + 1]])
        for codes, par, x in ((kc, kp, kb), (vc, vp, vb)):
            q, s, z = ref.asym_quantize_and_pack_i4(x)
            assert torch.equal(codes, ref.unpack(q))
            assert torch.equal(par[..., 0], s[..., 0].double()) and torch.equal(par[..., 1], z[..., 0].double())


def test_store_prequantized_rows(kvc, ref):
    batch, heads, page_size = 2, 4, 8
    lengths = [9, 8]
    g = torch.Generator().manual_seed(4)
    x = torch.randn(sum(lengths), heads, 128, generator=g).half()
    kq, ks, kz = ref.asym_quantize_and_pack_i4(x)
    vq, vs, vz = ref.asym_quantize_and_pack_i4(-x)
    kp, vp = torch.cat([ks, kz], -1), torch.cat([vs, vz], -1)
    indptr, indices, last, maxc = make_table(lengths, page_size, batch)
    pages = torch.zeros(maxc * batch, 1, 2, heads, page_size, 64, dtype=torch.uint8, device="cuda")
    params = torch.zeros(maxc * batch, 1, 2, heads, page_size, 2, dtype=torch.float16, device="cuda")
    seq = torch.tensor([0, 9, 17], dtype=torch.int32).cuda()
    kvc.init_kv_i4(pages, params, indptr.cuda(), indices.cuda(), last.cuda(), kq.cuda(), vq.cuda(), kp.cuda(), vp.cuda(),
                   seq, 0)
    for b, lo in enumerate((0, 9)):
        (kc, kpar), (vc, vpar) = ref.gather_sequence(pages.cpu(), params.cpu(), indptr, indices, last, 0, b)
        assert torch.equal(kc, ref.unpack(kq[lo:lo + lengths[b]]))
        assert torch.equal(vc, ref.unpack(vq[lo:lo + lengths[b]]))
        assert torch.equal(kpar, kp[lo:lo + lengths[b]].double()) and torch.equal(vpar, vp[lo:lo + lengths[b]].double())


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("page_size", [16, 8, 32])          # 8: the VALU kernel; multiples of 16: the MFMA kernel
@pytest.mark.parametrize("q_heads,kv_heads", [(4, 4), (8, 4), (32, 8)])
def test_decode_attention(kvc, ref, dtype, q_heads, kv_heads, page_size):
    batch, layers, layer = 4, 2, 0
    lengths = [1, 16, 77, 260]
    g = torch.Generator().manual_seed(5)
    total = sum(lengths)
    k = (torch.randn(total, kv_heads, 128, generator=g) * 1.5).to(dtype)
    v = torch.randn(total, kv_heads, 128, generator=g).to(dtype)
    q = torch.randn(batch, q_heads, 128, generator=g).to(dtype)
    indptr, indices, last, maxc = make_table(lengths, page_size, batch)
    pages = torch.zeros(maxc * batch, layers, 2, kv_heads, page_size, 64, dtype=torch.uint8, device="cuda")
    params = torch.full((maxc * batch, layers, 2, kv_heads, page_size, 2), float("nan"), dtype=dtype, device="cuda")
    offs = [0]                                               # unused rows hold NaN: they must not leak into results
    for n in lengths:
        offs.append(offs[-1] + n)
    print(f"kv decode {dtype} heads {q_heads}/{kv_heads} page {page_size}", flush=True)
    kvc.quantize_append(pages, params, indptr.cuda(), indices.cuda(), last.cuda(), k.cuda(), v.cuda(), layer,
                        seqlen_indptr=torch.tensor(offs, dtype=torch.int32).cuda())
    o = torch.empty_like(q).cuda()
    kvc.batch_decode_i4(o, q.cuda(), pages, params, indptr.cuda(), indices.cuda(), last.cuda(), layer)
    want = ref.decode_attention(q, pages.cpu(), params.cpu(), indptr, indices, last, layer)
    tol = 1e-3 if dtype == torch.float16 else 5e-3
    assert rel_fro(o, want) < tol
    # a one-token sequence returns that token's dequantized value row
    (kc, kp), (vc, vp) = ref.gather_sequence(pages.cpu(), params.cpu(), indptr, indices, last, layer, 0)
    v0 = vc.double() * vp[..., :1] - vp[..., 1:]
    assert rel_fro(o[0, 0], v0[0, 0]) < tol


def test_cache_container_flow(kvc, ref):
    """prefill + three decode steps through MultiLayerPagedKVCache4Bit on two layers"""
    batch, heads, q_heads, layers, page_size = 2, 2, 4, 2, 16
    dtype = torch.bfloat16
    cache = kvc.MultiLayerPagedKVCache4Bit(batch, page_size, 64, "cuda", layers, heads, 128, dtype=dtype)
    g = torch.Generator().manual_seed(6)
    hist = {l: [] for l in range(layers)}
    for step, t in enumerate((30, 1, 1, 1)):
        for l in range(layers):
            k = torch.randn(batch, t, heads, 128, generator=g).to(dtype)
            v = torch.randn(batch, t, heads, 128, generator=g).to(dtype)
            hist[l].append((k, v))
            r = cache.update(k.cuda(), v.cuda(), l)
            if step == 0:
                assert isinstance(r, tuple)
                continue
            q = torch.randn(batch, 1, q_heads, 128, generator=g).to(dtype)
            out = r(q.cuda())
            assert out.shape == (batch, 1, q_heads, 128)
            kall = torch.cat([a for a, _ in hist[l]], dim=1)
            vall = torch.cat([b for _, b in hist[l]], dim=1)
            kq, ks, kz = ref.asym_quantize_and_pack_i4(kall)
            vq, vs, vz = ref.asym_quantize_and_pack_i4(vall)
            kd = ref.unpack(kq).double() * ks.double() - kz.double()
            vd = ref.unpack(vq).double() * vs.double() - vz.double()
            gsz = q_heads // heads
            want = torch.zeros(batch, q_heads, 128, dtype=torch.float64)
            for b in range(batch):
                for h in range(q_heads):
                    s = (kd[b, :, h // gsz] @ q[b, 0, h].double()) * 128 ** -0.5
                    want[b, h] = torch.softmax(s, 0) @ vd[b, :, h // gsz]
            assert rel_fro(out[:, 0], want) < 5e-3
    assert cache.get_seq_length() == 33


@pytest.mark.parametrize("dtype", DTYPES)
def test_rope_quantize_append_is_bit_exact(kvc, ref, dtype):
    """The fused decode-step launch against the same step done with torch on the CPU: rotary embedding
    (model/qLlamaLayer.py:30-64, every op rounded to the dtype), then the quantizer restatement.
    Rotated queries, codes and (scale, zero) pairs must be identical; rows are strided as a slice of
    a wider projection output would be."""
    batch, nh, nkv, page_size, layers, layer = 3, 4, 2, 16, 2, 1
    lengths = [17, 32, 5]                                   # lengths AFTER the append: new page, page end, short
    g = torch.Generator().manual_seed(11)
    width = (nh + 2 * nkv) * 128
    wide = (torch.randn(batch, width + 64, generator=g) * 1.5).to(dtype)
    qkv = wide[:, :width]
    positions = torch.tensor([n - 1 for n in lengths], dtype=torch.int32)
    positions[2] = 40                                       # a position that differs from the length (padded prompt)
    cos_t, sin_t = kvc.rope_tables(64, 128, dtype, "cuda")
    indptr, indices, last, maxc = make_table(lengths, page_size, batch)
    pages = torch.zeros(maxc * batch, layers, 2, nkv, page_size, 64, dtype=torch.uint8, device="cuda")
    params = torch.zeros(maxc * batch, layers, 2, nkv, page_size, 2, dtype=dtype, device="cuda")
    print(f"rope + kv append {dtype}", flush=True)
    q_rot = kvc.rope_quantize_append(wide.cuda()[:, :width], nh, cos_t, sin_t, positions.cuda(), pages, params,
                                     indptr.cuda(), indices.cuda(), last.cuda(), layer)
    torch.cuda.synchronize()

    # the same on the CPU, op by op
    q = qkv[:, :nh * 128].view(batch, nh, 128)
    k = qkv[:, nh * 128:(nh + nkv) * 128].view(batch, nkv, 128)
    v = qkv[:, (nh + nkv) * 128:].view(batch, nkv, 128)
    cos = torch.cat([cos_t.cpu(), cos_t.cpu()], dim=-1)[positions.long()][:, None]     # [batch, 1, 128]
    sin = torch.cat([sin_t.cpu(), sin_t.cpu()], dim=-1)[positions.long()][:, None]
    rot = lambda x: torch.cat((-x[..., 64:], x[..., :64]), dim=-1)
    q_want = q * cos + rot(q) * sin
    k_rot = k * cos + rot(k) * sin
    assert torch.equal(q_rot.cpu(), q_want)
    pc, sc = pages.cpu(), params.cpu()
    assert int(pc[:, 0].sum()) == 0
    for b in range(batch):
        (kc, kp), (vc, vp) = ref.gather_sequence(pc, sc, indptr, indices, last, layer, b)
        for codes, par, x in ((kc, kp, k_rot[b:b + 1]), (vc, vp, v[b:b + 1])):
            qq, s, z = ref.asym_quantize_and_pack_i4(x)
            assert torch.equal(codes[-1:], ref.unpack(qq))
            assert torch.equal(par[-1:, :, 0], s[..., 0].double()) and torch.equal(par[-1:, :, 1], z[..., 0].double())
            assert int(codes[:-1].sum()) == 0                # earlier slots untouched


def test_decode_attention_many_sequences(kvc, ref):
    """Enough (sequence, KV head) pairs that the kernel takes every sequence whole (one workgroup per
    pair, no split ranges, no merge launch); the small batches above take the split path.  One sequence
    is empty: its output is zero."""
    batch, q_heads, kv_heads, page_size, dtype = 40, 32, 8, 16, torch.bfloat16
    g = torch.Generator().manual_seed(17)
    lengths = [int(n) for n in torch.randint(1, 90, (batch,), generator=g)]
    lengths[7] = 0
    total = sum(lengths)
    k = torch.randn(total, kv_heads, 128, generator=g).to(dtype)
    v = torch.randn(total, kv_heads, 128, generator=g).to(dtype)
    q = torch.randn(batch, q_heads, 128, generator=g).to(dtype)
    indptr, indices, last, maxc = make_table(lengths, page_size, batch)
    pages = torch.zeros(maxc * batch, 1, 2, kv_heads, page_size, 64, dtype=torch.uint8, device="cuda")
    params = torch.full((maxc * batch, 1, 2, kv_heads, page_size, 2), float("nan"), dtype=dtype, device="cuda")
    offs = [0]
    for n in lengths:
        offs.append(offs[-1] + n)
    print("kv decode, 40 sequences x 8 KV heads", flush=True)
    kvc.quantize_append(pages, params, indptr.cuda(), indices.cuda(), last.cuda(), k.cuda(), v.cuda(), 0,
                        seqlen_indptr=torch.tensor(offs, dtype=torch.int32).cuda(), max_new_tokens=max(lengths))
    o = torch.full_like(q, 7.0).cuda()
    kvc.batch_decode_i4(o, q.cuda(), pages, params, indptr.cuda(), indices.cuda(), last.cuda(), 0)
    want = ref.decode_attention(q, pages.cpu(), params.cpu(), indptr, indices, last, 0)
    keep = [b for b in range(batch) if b != 7]
    assert rel_fro(o[keep], want[keep]) < 5e-3
    assert float(o[7].abs().sum()) == 0.0


def test_decode_attention_long_sequence_whole(kvc, ref):
    """256 (sequence, KV head) pairs, so every sequence is taken whole by one workgroup, and one of them
    long enough (8200 tokens, more than 64 chunks per wave) that the kernel fetches its page numbers in
    more than one block while chunks are in flight."""
    batch, q_heads, kv_heads, page_size, dtype = 64, 8, 4, 16, torch.bfloat16
    g = torch.Generator().manual_seed(29)
    lengths = [int(n) for n in torch.randint(1, 60, (batch,), generator=g)]
    lengths[3] = 8200
    total = sum(lengths)
    k = torch.randn(total, kv_heads, 128, generator=g).to(dtype)
    v = torch.randn(total, kv_heads, 128, generator=g).to(dtype)
    q = torch.randn(batch, q_heads, 128, generator=g).to(dtype)
    indptr, indices, last, maxc = make_table(lengths, page_size, batch)
    pages = torch.zeros(maxc * batch, 1, 2, kv_heads, page_size, 64, dtype=torch.uint8, device="cuda")
    params = torch.full((maxc * batch, 1, 2, kv_heads, page_size, 2), float("nan"), dtype=dtype, device="cuda")
    offs = [0]
    for n in lengths:
        offs.append(offs[-1] + n)
    print("kv decode, 64 sequences x 4 KV heads, one of 8200 tokens", flush=True)
    kvc.quantize_append(pages, params, indptr.cuda(), indices.cuda(), last.cuda(), k.cuda(), v.cuda(), 0,
                        seqlen_indptr=torch.tensor(offs, dtype=torch.int32).cuda(), max_new_tokens=max(lengths))
    o = torch.full_like(q, 7.0).cuda()
    kvc.batch_decode_i4(o, q.cuda(), pages, params, indptr.cuda(), indices.cuda(), last.cuda(), 0)
    want = ref.decode_attention(q, pages.cpu(), params.cpu(), indptr, indices, last, 0)
    assert rel_fro(o, want) < 5e-3
    assert rel_fro(o[3], want[3]) < 5e-3


@pytest.mark.parametrize("dtype", DTYPES)
def test_rope_rows_match_torch(kvc, dtype):
    """The one-pass rotary embedding of a prompt against torch's q * cos + rotate_half(q) * sin on the
    CPU (every op rounded to the dtype): bit-identical, for strided projection rows and a start offset."""
    seqs, q_len, nh, nkv, pos0 = 3, 21, 4, 2, 5
    g = torch.Generator().manual_seed(23)
    width = (nh + 2 * nkv) * 128
    wide = (torch.randn(seqs * q_len, width + 8, generator=g) * 2).to(dtype)
    cos_t, sin_t = kvc.rope_tables(64, 128, dtype, "cuda")
    print(f"rope rows {dtype}", flush=True)
    q_rot, k_rot = kvc.rope(wide.cuda()[:, :width], q_len, pos0, nh, nkv, cos_t, sin_t)
    torch.cuda.synchronize()
    pos = (pos0 + torch.arange(seqs * q_len) % q_len).long()
    cos = torch.cat([cos_t.cpu(), cos_t.cpu()], dim=-1)[pos][:, None]
    sin = torch.cat([sin_t.cpu(), sin_t.cpu()], dim=-1)[pos][:, None]
    rot = lambda x: torch.cat((-x[..., 64:], x[..., :64]), dim=-1)
    q = wide[:, :nh * 128].view(-1, nh, 128)
    k = wide[:, nh * 128:(nh + nkv) * 128].view(-1, nkv, 128)
    assert torch.equal(q_rot.cpu(), q * cos + rot(q) * sin)
    assert torch.equal(k_rot.cpu(), k * cos + rot(k) * sin)


@pytest.mark.parametrize("name,dtype", [("f16", torch.float16), ("bf16", torch.bfloat16)])
def test_quantize_append_matches_reference_vectors(kvc, ref, name, dtype):
    """the fused quantize + append on the inputs of the reference-written vectors
    (tests/golden/refkv_golden.npz, from model/kv_cache.py:21-37): codes, scales and zeros as the
    reference's own function returned them"""
    import os
    import numpy as np
    gold = dict(np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "refkv_golden.npz"),
                        allow_pickle=False))
    x = torch.from_numpy(gold[f"{name}_x_bits"]).view(dtype)           # [12 tokens, 8 heads, 128]
    tokens, heads, _ = x.shape
    page_size = 4
    indptr, indices, last, maxc = make_table([tokens], page_size, 1)
    pages = torch.zeros(maxc, 1, 2, heads, page_size, 64, dtype=torch.uint8, device="cuda")
    params = torch.zeros(maxc, 1, 2, heads, page_size, 2, dtype=dtype, device="cuda")
    seq = torch.tensor([0, tokens], dtype=torch.int32).cuda()
    print(f"kv append, reference vectors, {name}", flush=True)
    kvc.quantize_append(pages, params, indptr.cuda(), indices.cuda(), last.cuda(), x.cuda(), x.flip(0).contiguous().cuda(), 0,
                        seqlen_indptr=seq)
    (kc, kp), (vc, vp) = ref.gather_sequence(pages.cpu(), params.cpu(), indptr, indices, last, 0, 0)
    want_q = ref.unpack(torch.from_numpy(gold[f"{name}_q"]))
    want_s = torch.from_numpy(gold[f"{name}_scale_bits"]).view(dtype).double()[..., 0]
    want_z = torch.from_numpy(gold[f"{name}_zero_bits"]).view(dtype).double()[..., 0]
    assert torch.equal(kc, want_q) and torch.equal(vc, want_q.flip(0))
    assert torch.equal(kp[..., 0], want_s) and torch.equal(kp[..., 1], want_z)
    assert torch.equal(vp[..., 0], want_s.flip(0)) and torch.equal(vp[..., 1], want_z.flip(0))


def test_inconsistent_page_table_stores_nothing(kvc):
    """a sequence whose table has no page (or no room for its new tokens) must not be written anywhere:
    the kernels skip such rows instead of indexing the page list out of range"""
    heads, page_size = 2, 16
    pages = torch.zeros(4, 1, 2, heads, page_size, 64, dtype=torch.uint8, device="cuda")
    params = torch.zeros(4, 1, 2, heads, page_size, 2, dtype=torch.float16, device="cuda")
    k = torch.randn(2, heads, 128).half().cuda()
    # sequence 0 has no pages at all; sequence 1 owns page 2 and holds one token after the append
    indptr = torch.tensor([0, 0, 1], dtype=torch.int32).cuda()
    indices = torch.tensor([2], dtype=torch.int32).cuda()
    last = torch.tensor([0, 1], dtype=torch.int32).cuda()
    kvc.quantize_append(pages, params, indptr, indices, last, k, k, 0)
    torch.cuda.synchronize()
    assert int(pages[[0, 1, 3]].sum()) == 0 and float(params[[0, 1, 3]].abs().sum()) == 0
    assert int(pages[2, 0, :, :, 0].sum()) > 0 and int(pages[2, 0, :, :, 1:].sum()) == 0
    # the pre-quantized store takes the same table; three new tokens for a sequence that holds one: skipped rows
    q = torch.full((4, heads, 64), 0x77, dtype=torch.uint8, device="cuda")
    par = torch.ones(4, heads, 2, dtype=torch.float16, device="cuda")
    pages.zero_()
    seq = torch.tensor([0, 1, 4], dtype=torch.int32).cuda()
    kvc.init_kv_i4(pages, params, indptr, indices, last, q, q, par, par, seq, 0)
    torch.cuda.synchronize()
    assert int(pages[[0, 1, 3]].sum()) == 0
    assert int(pages[2, 0, :, :, 1:].sum()) == 0                       # only slot 0 (the token that fits) is written


def test_agemm_module_exports_the_kv_operators():
    """the reference reaches the KV operators through its extension module (kernels/src/bindings.cpp:576-578,
    model/kv_cache.py:49-80): the drop-in module carries the same three names"""
    from arcquant_amd import agemm, kv_cache
    for name in ("init_kv_i4", "append_kv_i4", "batch_decode_i4"):
        assert getattr(agemm, name) is getattr(kv_cache, name)
    ns = {}
    exec("from arcquant_amd.agemm import *", ns)
    assert {"matmul", "reorder_quantize_x", "reorder_quantize_w", "rmsnorm_quantize_x", "init_kv_i4", "append_kv_i4",
            "batch_decode_i4"} <= set(ns)
