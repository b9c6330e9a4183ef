"""Writes tests/golden/quant_golden.npz: input/output vectors of the REFERENCE per-block INT8 quantiser.

Runs, in this container only, the reference's own ``per_block_int8``
(/root/reference/backends/_enflame/ops/sage_attention/quant_per_block.py:49-101) on CPU tensors through
Triton's CPU interpreter (TRITON_INTERPRET=1, which evaluates the kernel body with NumPy), because the
reference's tests hold no golden vectors for the quantiser: nothing else in the reference fixes the
exact integers (in particular IEEE division versus multiplication by a reciprocal).  Only the vectors
are committed; the reference source never leaves /root/reference.

Usage (from the repo root):  TRITON_INTERPRET=1 python tests/golden/make_quant_golden.py
"""
import os
import sys

os.environ.setdefault("TRITON_INTERPRET", "1")
os.environ.setdefault("PYTHONDONTWRITEBYTECODE", "1")
sys.dont_write_bytecode = True   # importing the reference must not write a __pycache__ into its (read-only) tree

import numpy as np
import torch

REF_DIR = "/root/reference/backends/_enflame/ops/sage_attention"
sys.path.insert(0, REF_DIR)
from quant_per_block import per_block_int8  # noqa: E402  (the reference implementation)


def bits16(t: torch.Tensor) -> np.ndarray:
    return t.contiguous().view(torch.int16).numpy().copy()


def main():
    g = torch.Generator().manual_seed(2026)
    cases = []
    specs = [
        # name, dtype, layout, B, Hq, Hkv, Lq, Lk, D, BLKQ, BLKK, use_km, sm_scale
        ("f16_hnd_128", torch.float16, "HND", 1, 2, 1, 128, 128, 64, 128, 64, False, None),
        ("bf16_nhd_tail", torch.bfloat16, "NHD", 1, 2, 2, 129, 70, 128, 128, 64, True, None),
        ("bf16_hnd_blk64_128", torch.bfloat16, "HND", 2, 2, 1, 200, 264, 128, 64, 128, True, 0.1),
        ("f16_hnd_ties", torch.float16, "HND", 1, 1, 1, 128, 64, 64, 128, 64, False, 1.0 / 1.44269504),
    ]
    out = {}
    for name, dtype, layout, B, Hq, Hkv, Lq, Lk, D, BLKQ, BLKK, use_km, sm in specs:
        shape = (lambda H, L: (B, H, L, D) if layout == "HND" else (B, L, H, D))
        q = torch.randn(shape(Hq, Lq), generator=g).to(dtype)
        k = torch.randn(shape(Hkv, Lk), generator=g).to(dtype)
        if name.endswith("ties"):
            # values whose quotient by the scale lands on exact .5 ties: tile max 127 -> scale 1
            q = (torch.randint(-253, 254, shape(Hq, Lq), generator=g).float() * 0.5).to(dtype)
            q.view(-1)[0] = 127.0
            k = (torch.randint(-253, 254, shape(Hkv, Lk), generator=g).float() * 0.5).to(dtype)
            k.view(-1)[5] = -127.0
        km = None
        if use_km:
            km = k.float().mean(dim=2 if layout == "HND" else 1, keepdim=True).to(dtype)
        qi, qs, ki, ks = per_block_int8(q, k, km=km, BLKQ=BLKQ, BLKK=BLKK, sm_scale=sm, tensor_layout=layout)
        out[f"{name}.q"] = bits16(q)
        out[f"{name}.k"] = bits16(k)
        if km is not None:
            out[f"{name}.km"] = bits16(km)
        out[f"{name}.qi"] = qi.numpy().copy()
        out[f"{name}.qs"] = qs.numpy().copy()
        out[f"{name}.ki"] = ki.numpy().copy()
        out[f"{name}.ks"] = ks.numpy().copy()
        out[f"{name}.meta"] = np.array([0 if dtype == torch.float16 else 1, 0 if layout == "HND" else 1, BLKQ, BLKK,
                                        -1.0 if sm is None else sm], dtype=np.float64)
        cases.append(name)
    out["cases"] = np.array(cases)
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "quant_golden.npz")
    np.savez_compressed(path, **out)
    print("wrote", path, "cases:", cases)


if __name__ == "__main__":
    main()
