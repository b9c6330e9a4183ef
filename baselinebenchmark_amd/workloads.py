"""Synthetic inputs of the five benchmark configurations (seeded, generated on the CPU or directly on
the device) and their effective operation counts.

Effective ops = 4 * B * Hq * Sq * Skv * D * (1/2 if causal), the reference's own convention
(backends/_enflame/benchmarks/sage_attention_native_benchmark.py:447-455,
 backends/_hygon/benchmarks/benchmark_sageattention_hygon.py:70-71) with the usual half for causal.
"""
from __future__ import annotations

from dataclasses import dataclass, field

import torch

SEED = 2026

CONFIGS = {
    # name: B, Hq, Hkv, S, D, dtype, layout, causal, BLKQ, BLKK, pv, k_offset_std, outlier_frac
    "c0": dict(B=1, Hq=8, Hkv=8, S=1024, D=64, dtype=torch.float16, layout="HND", causal=False, BLKQ=128, BLKK=128,
               pv="fp16", k_offset_std=0.0, outliers=0.0),
    "c1": dict(B=4, Hq=32, Hkv=32, S=4096, D=128, dtype=torch.bfloat16, layout="HND", causal=True, BLKQ=128, BLKK=64,
               pv="fp16", k_offset_std=2.0, outliers=0.0),
    "c2": dict(B=2, Hq=32, Hkv=32, S=16384, D=128, dtype=torch.bfloat16, layout="HND", causal=True, BLKQ=64, BLKK=128,
               pv="fp8", k_offset_std=2.0, outliers=0.0),
    "c3": dict(B=1, Hq=24, Hkv=24, S=32760, D=128, dtype=torch.bfloat16, layout="NHD", causal=False, BLKQ=128, BLKK=64,
               pv="fp8", k_offset_std=0.0, outliers=0.01),
}
VARLEN_C4 = dict(nseq=16, lo=512, hi=32768, Hq=32, Hkv=8, D=128, dtype=torch.bfloat16, causal=True, BLKQ=128, BLKK=64,
                 pv="fp8")


@dataclass
class Workload:
    name: str
    q: torch.Tensor
    k: torch.Tensor
    v: torch.Tensor
    layout: str
    causal: bool
    kwargs: dict
    ops: float
    desc: str
    cu_seqlens: torch.Tensor | None = None
    max_seqlen: int = 0
    extra: dict = field(default_factory=dict)


def effective_ops(B, Hq, Sq, Skv, D, causal) -> float:
    return 4.0 * B * Hq * Sq * Skv * D * (0.5 if causal else 1.0)


def _shape(layout, B, H, S, D):
    return (B, H, S, D) if layout == "HND" else (B, S, H, D)


def make(name: str, device="cuda", heads: int | None = None, batch: int | None = None) -> Workload:
    """Builds config ``name`` ("c0".."c4").  ``heads``/``batch`` shrink the problem (CPU baseline samples)."""
    if name == "c4":
        return make_varlen(device=device)
    c = dict(CONFIGS[name])
    if heads is not None:
        c["Hq"] = c["Hkv"] = heads
    if batch is not None:
        c["B"] = batch
    g = torch.Generator(device=device).manual_seed(SEED)
    B, Hq, Hkv, S, D, layout, dtype = c["B"], c["Hq"], c["Hkv"], c["S"], c["D"], c["layout"], c["dtype"]

    def rnd(H):
        return torch.randn(_shape(layout, B, H, S, D), generator=g, device=device, dtype=torch.float32)

    q, k, v = rnd(Hq), rnd(Hkv), rnd(Hkv)
    if c["k_offset_std"]:
        off = torch.randn(_shape(layout, 1, Hkv, 1, D), generator=g, device=device, dtype=torch.float32) * c["k_offset_std"]
        k = k + off
    if c["outliers"]:
        n = max(1, int(Hq * D * c["outliers"]))
        pairs = torch.randperm(Hq * D, generator=g, device=device)[:n]
        for t in (q, k, v):
            flat = t.view(B, S, Hq * D) if layout == "NHD" else t.transpose(1, 2).reshape(B, S, Hq * D)
            flat[:, :, pairs] *= 20.0
            if layout == "HND":
                t.copy_(flat.view(B, S, Hq, D).transpose(1, 2))
    q, k, v = q.to(dtype), k.to(dtype), v.to(dtype)
    kwargs = dict(tensor_layout=layout, is_causal=c["causal"], pv_mode=c["pv"], BLKQ=c["BLKQ"], BLKK=c["BLKK"], smooth_k=True)
    desc = (f"{name}: B{B} Hq{Hq} Hkv{Hkv} S{S} D{D} {str(dtype).replace('torch.', '')} {layout} "
            f"{'causal' if c['causal'] else 'non-causal'} Qblk{c['BLKQ']} Kblk{c['BLKK']} PV-{c['pv']}")
    return Workload(name, q, k, v, layout, c["causal"], kwargs, effective_ops(B, Hq, S, S, D, c["causal"]), desc)


def make_varlen(device="cuda", nseq: int | None = None) -> Workload:
    c = dict(VARLEN_C4)
    if nseq is not None:
        c["nseq"] = nseq
    g = torch.Generator().manual_seed(SEED)
    lens = torch.randint(c["lo"], c["hi"] + 1, (c["nseq"],), generator=g)
    cu = torch.zeros(c["nseq"] + 1, dtype=torch.int32)
    cu[1:] = torch.cumsum(lens, 0)
    T = int(cu[-1])
    gd = torch.Generator(device=device).manual_seed(SEED)
    q = torch.randn((T, c["Hq"], c["D"]), generator=gd, device=device, dtype=torch.float32).to(c["dtype"])
    k = torch.randn((T, c["Hkv"], c["D"]), generator=gd, device=device, dtype=torch.float32).to(c["dtype"])
    v = torch.randn((T, c["Hkv"], c["D"]), generator=gd, device=device, dtype=torch.float32).to(c["dtype"])
    ops = float(sum(4.0 * c["Hq"] * int(L) * int(L) * c["D"] * 0.5 for L in lens))
    kwargs = dict(is_causal=True, pv_mode=c["pv"], BLKQ=c["BLKQ"], BLKK=c["BLKK"], smooth_k=True)
    desc = f"c4: {c['nseq']} packed seqs L in [{c['lo']},{c['hi']}] (total {T}) Hq{c['Hq']} Hkv{c['Hkv']} D{c['D']} bf16 causal PV-fp8"
    return Workload("c4", q, k, v, "NHD", True, kwargs, ops, desc, cu_seqlens=cu.to(device), max_seqlen=int(lens.max()),
                    extra=dict(lens=[int(x) for x in lens]))
