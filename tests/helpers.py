"""Shared helpers of the test-suite: seeded inputs in the reference's test style and golden decoding."""
import numpy as np
import torch


def shape4(layout, B, H, L, D):
    return (B, H, L, D) if layout == "HND" else (B, L, H, D)


def randn(layout, B, H, L, D, dtype, gen, offset_std=0.0):
    x = torch.randn(shape4(layout, B, H, L, D), generator=gen)
    if offset_std:
        off = torch.randn(shape4(layout, B, H, 1, D), generator=gen) * offset_std
        x = x + off
    return x.to(dtype)


def golden_case(g, name):
    meta = g[f"{name}.meta"]
    dtype = torch.float16 if meta[0] == 0 else torch.bfloat16
    layout = "HND" if meta[1] == 0 else "NHD"
    d = dict(dtype=dtype, layout=layout, BLKQ=int(meta[2]), BLKK=int(meta[3]), sm_scale=None if meta[4] < 0 else float(meta[4]))
    d["q"] = torch.from_numpy(g[f"{name}.q"].copy()).view(dtype)
    d["k"] = torch.from_numpy(g[f"{name}.k"].copy()).view(dtype)
    d["km"] = torch.from_numpy(g[f"{name}.km"].copy()).view(dtype) if f"{name}.km" in g else None
    for key in ("qi", "qs", "ki", "ks"):
        d[key] = torch.from_numpy(g[f"{name}.{key}"].copy())
    return d
