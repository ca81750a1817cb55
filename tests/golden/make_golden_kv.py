"""Writes tests/golden/refkv_golden.npz from the reference's own INT4 KV-cache quantizer.

Run once, in the development container only (the reference checkout does not exist on the GPU
box):  python tests/golden/make_golden_kv.py

asym_quantize_and_pack_i4 (model/kv_cache.py:21-37) is wrapped in torch.jit.script and what it
returns hinges on how torch rounds each intermediate in fp16 / bf16, which no closed form pins.
The module is loaded by file path; its top-level ``import agemm`` (the CUDA extension, absent here)
is satisfied by an empty placeholder module, since the quantizer does not touch it.  Only inputs
and outputs are stored -- no reference source.

Vectors: rows of 128 values, fp16 and bf16, ~N(0,1) and scaled by 1e-3 / 30, rows with a constant
value (range 0 -> the 1e-5 clamp), rows with one outlier, rows of zeros, and rows built to land on
rounding ties of (x + zero) / scale.  The function is called three times per input (the scripted
function's first calls are profiling runs); all calls must agree.
"""
import importlib.util
import os
import sys
import types

import numpy as np
import torch

REF = "/root/reference/model/kv_cache.py"
OUT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "refkv_golden.npz")


def load_reference():
    sys.modules.setdefault("agemm", types.ModuleType("agemm"))
    spec = importlib.util.spec_from_file_location("ref_kv_cache", REF)
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def rows(dtype, g):
    x = torch.randn(96, 128, generator=g)
    x[16:32] *= 1e-3
    x[32:48] *= 30.0
    x[48] = 0.0
    x[49] = 1.5
    x[50] = -2.25
    x[51] = 3e-6
    x[52, 7] = 200.0
    x[53, 100] = -150.0
    x[54] = torch.arange(128).float() / 127.0 * 15.0           # quotients on the integers and halves
    x[55] = torch.arange(128).float() / 254.0 * 15.0 - 3.0
    x[56] = (torch.arange(128) % 31).float() * 0.5
    x[57, :64] = 1.0
    x[57, 64:] = 1.0 + 2 ** -7
    return x.to(dtype).reshape(12, 8, 128)                       # [tokens, heads, 128]


def main():
    rk = load_reference()
    g = torch.Generator().manual_seed(20240702)
    out = {}
    for name, dtype in (("f16", torch.float16), ("bf16", torch.bfloat16)):
        x = rows(dtype, g)
        res = [rk.asym_quantize_and_pack_i4(x.clone()) for _ in range(3)]
        for q, s, z in res[1:]:
            assert torch.equal(q, res[0][0]) and torch.equal(s, res[0][1]) and torch.equal(z, res[0][2])
        q, s, z = res[0]
        assert q.dtype == torch.uint8 and s.dtype == dtype and z.dtype == dtype, (q.dtype, s.dtype, z.dtype)
        out[f"{name}_x_bits"] = x.view(torch.int16).numpy()
        out[f"{name}_q"] = q.numpy()
        out[f"{name}_scale_bits"] = s.view(torch.int16).numpy()
        out[f"{name}_zero_bits"] = z.view(torch.int16).numpy()
        # and the inverse the reference pairs with it (model/kv_cache.py:39-43)
        out[f"{name}_dq_bits"] = rk.unpack_i4_and_asym_dequantize(q, s, z).to(dtype).view(torch.int16).numpy()
    np.savez_compressed(OUT, **out)
    print("wrote", OUT, os.path.getsize(OUT), "bytes")


if __name__ == "__main__":
    main()
