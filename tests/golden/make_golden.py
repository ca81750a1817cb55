"""Writes tests/golden/refquant_golden.npz from the reference's own fake quantizer.

Run once, in the development container only (the reference checkout does not
exist on the GPU box):  python tests/golden/make_golden.py

The reference's model/quantize.py is loaded by file path; its top-level
``import agemm`` (the CUDA extension, absent here) is satisfied by an empty
placeholder module because none of the value-domain functions used below touch
it.  Only inputs and outputs are stored -- no reference source.

Vectors captured (inputs are generated here, seeded):
  * quantize_e2m1 on every tie point, its fp32 neighbours, and a sweep;
  * quantize_ue4m3 / quantize_ue8m0 on every power of two 2^-40..2^10, the 64
    fp32 values either side of each, and a log-uniform sweep (these two depend
    on torch.log2's rounding, which no closed form pins);
  * fake_reorder_quantize_x / _w end to end on 8x256 bf16 inputs with outlier
    channels, select_num 64, NVFP4 and MXFP4.
"""
import importlib.util
import os
import sys
import types

import numpy as np
import torch

REF = "/root/reference/model/quantize.py"
OUT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "refquant_golden.npz")


def load_reference():
    sys.modules.setdefault("agemm", types.ModuleType("agemm"))
    spec = importlib.util.spec_from_file_location("ref_quantize", REF)
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def neighbours(center: np.ndarray, width: int) -> np.ndarray:
    bits = center.astype(np.float32).view(np.int32)[:, None] + np.arange(-width, width + 1, dtype=np.int32)[None, :]
    return bits.reshape(-1).view(np.float32)


def main():
    rq = load_reference()
    g = torch.Generator().manual_seed(20240611)
    out = {}

    ties = np.array([0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5.0, 6.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0], np.float32)
    e2_in = np.concatenate([neighbours(ties, 2), -neighbours(ties, 2), np.array([0.0, -0.0, 7.5, -7.5, 1e-30, -1e-30],
                           np.float32), (torch.rand(4096, generator=g) * 14 - 7).numpy()]).astype(np.float32)
    out["e2m1_in"] = e2_in
    out["e2m1_out"] = rq.quantize_e2m1(torch.from_numpy(e2_in)).numpy()

    pows = np.ldexp(1.0, np.arange(-40, 11)).astype(np.float32)
    sweep = np.exp2(torch.rand(8192, generator=g).numpy() * 50 - 40).astype(np.float32)
    sc_in = np.concatenate([neighbours(pows, 64), sweep, np.array([1e-9, 2e-3, 448.0, 500.0, 1e-12], np.float32)])
    sc_in = sc_in[np.isfinite(sc_in) & (sc_in > 0)].astype(np.float32)
    out["scale_in"] = sc_in
    out["ue4m3_out"] = rq.quantize_ue4m3(torch.from_numpy(sc_in)).numpy()
    out["ue8m0_out"] = rq.quantize_ue8m0(torch.from_numpy(sc_in)).numpy()

    M, K, S = 8, 256, 64
    x = torch.randn(M, K, generator=g)
    x[:, torch.randperm(K, generator=g)[:6]] *= 40
    x[3, :32] = 0.0                      # an all-zero block
    x[5, 64:96] *= 1e-3                  # a tiny block
    x = x.to(torch.bfloat16)
    w = (torch.randn(M, K, generator=g) * 0.02).to(torch.bfloat16)
    out["x_bits"] = x.view(torch.int16).numpy()
    out["w_bits"] = w.view(torch.int16).numpy()
    ar = torch.arange(K)
    for fmt in ("NVFP4", "MXFP4"):
        qx, _, sx = rq.fake_reorder_quantize_x(x, ar, S, dtype=fmt)
        qw, _, sw = rq.fake_reorder_quantize_w(w, ar, S, dtype=fmt)
        qx0, _, _ = rq.fake_reorder_quantize_x(x, ar, 0, dtype=fmt)
        out[f"{fmt}_x_out_bits"] = qx.view(torch.int16).numpy()
        out[f"{fmt}_x0_out_bits"] = qx0.view(torch.int16).numpy()
        out[f"{fmt}_x_scale"] = sx.float().numpy()
        out[f"{fmt}_w_out_bits"] = qw.view(torch.int16).numpy()
        out[f"{fmt}_w_scale"] = sw.float().numpy()
        # block-level values before the bf16 cast, straight from the tensor quantizers
        fn = rq.quantize_nvfp4_tensor if fmt == "NVFP4" else rq.quantize_mxfp4_tensor
        out[f"{fmt}_block_in"] = x.float().numpy()
        out[f"{fmt}_block_out"] = fn(x.float()).numpy()
    np.savez_compressed(OUT, **out)
    print("wrote", OUT, os.path.getsize(OUT), "bytes")


if __name__ == "__main__":
    main()
