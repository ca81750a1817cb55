"""The torch restatement of the reference's INT4 KV-cache quantizer (oracle/kvcache_torch.py) against
vectors written by the reference's own scripted function (tests/golden/make_golden_kv.py from
model/kv_cache.py:21-37), fp16 and bf16: packed codes, scales and zeros must be identical bits."""
import os

import numpy as np
import pytest
import torch

from oracle import kvcache_torch as kvt

ROOT = os.path.dirname(os.path.abspath(__file__))


@pytest.fixture(scope="module")
def golden_kv():
    return dict(np.load(os.path.join(ROOT, "golden", "refkv_golden.npz"), allow_pickle=False))


@pytest.mark.parametrize("name,dtype", [("f16", torch.float16), ("bf16", torch.bfloat16)])
def test_asym_quantize_and_pack_i4_matches_reference_vectors(golden_kv, name, dtype):
    x = torch.from_numpy(golden_kv[f"{name}_x_bits"]).view(dtype)
    q, scale, zero = kvt.asym_quantize_and_pack_i4(x)
    assert q.dtype == torch.uint8 and scale.dtype == dtype and zero.dtype == dtype
    assert np.array_equal(q.numpy(), golden_kv[f"{name}_q"])
    assert np.array_equal(scale.view(torch.int16).numpy(), golden_kv[f"{name}_scale_bits"])
    assert np.array_equal(zero.view(torch.int16).numpy(), golden_kv[f"{name}_zero_bits"])
    # the vectors hold what they were built to hold: a constant row (range 0 -> the 1e-5 clamp), ties
    flat = x.reshape(-1, 128)
    const = (flat.amax(-1) == flat.amin(-1)).nonzero().flatten()
    assert const.numel() >= 3
    floor = torch.tensor(1e-5).to(dtype) / 15
    assert torch.all(scale.reshape(-1)[const] == floor)
    # the inverse (model/kv_cache.py:39-43): n * scale - zero in the cache dtype
    dq = (kvt.unpack(q) * scale - zero).to(dtype)
    assert np.array_equal(dq.view(torch.int16).numpy(), golden_kv[f"{name}_dq_bits"])
