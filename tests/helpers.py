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


def sageattn_cabi(q, k, v, out, *, layout="HND", is_causal=False, pv="fp16", BLKQ=128, BLKK=64, smooth_k=True, sm_scale=None,
                  static=False, lse=None, workspace=None):
    """sage_sageattn / sage_sageattn_static straight through ctypes, with the tensors' own strides (any view whose last
    axis is contiguous), bypassing the Python shim's contiguity checks.  Returns the C return code."""
    import ctypes
    from baselinebenchmark_amd import _cabi

    lib = _cabi.lib()

    def lay(t):
        if layout == "HND":
            return t.shape[0], t.shape[1], t.shape[2], t.shape[3], t.stride(0), t.stride(1), t.stride(2)
        return t.shape[0], t.shape[2], t.shape[1], t.shape[3], t.stride(0), t.stride(2), t.stride(1)

    B, Hq, Sq, D, qsb, qsh, qsn = lay(q)
    _, Hkv, Skv, _, ksb, ksh, ksn = lay(k)
    _, _, _, _, vsb, vsh, vsn = lay(v)
    _, _, _, _, osb, osh, osn = lay(out)
    pvm = _cabi.PV_FP8 if pv == "fp8" else _cabi.PV_FP16
    dt = _cabi.DT_BF16 if q.dtype == torch.bfloat16 else _cabi.DT_F16
    P = lambda t: ctypes.c_void_p(0 if t is None else t.data_ptr())
    stream = ctypes.c_void_p(torch.cuda.current_stream(q.device).cuda_stream)
    tail = (B, Hq, Hkv, Sq, Skv, D, qsb, qsh, qsn, ksb, ksh, ksn, vsb, vsh, vsn, osb, osh, osn, dt, BLKQ, BLKK,
            float(D ** -0.5 if sm_scale is None else sm_scale), int(is_causal), int(smooth_k), pvm, None, None, 0, 0, stream)
    if static:
        return lib.sage_sageattn_static(P(q), P(k), P(v), P(out), P(lse), *tail)
    nbytes = lib.sage_sageattn_workspace_bytes(B, Hq, Hkv, Sq, Skv, D, BLKQ, BLKK, pvm, 0, 0, 0)
    ws = workspace if workspace is not None else torch.empty(max(nbytes, 256), device=q.device, dtype=torch.uint8)
    return lib.sage_sageattn(P(q), P(k), P(v), P(out), P(lse), P(ws), ws.numel(), *tail)


def check_rows_fp8(got, q_rows, k1, v1, r0, blkq, blkk, causal, out_dtype):
    """Rows r0 .. r0 + T of ONE (batch, head) of a long FP8 P.V problem against the oracle, host cost O(T * S):
    got [T, D] (the library's output rows), q_rows [T, D], k1 / v1 [S, D] raw operands of that head (K smoothed with its
    own mean, per-block INT8 by the oracle's quantiser, V per-channel e4m3).  Returns the metrics against
    (a) the exact-softmax formula on the same quantised operands, (b) the kernel's arithmetic model, (c) FP32 SDPA on
    the raw operands."""
    from oracle import attention as oa
    from oracle import fp8_model as fm
    from oracle import quant as oq
    T, S = q_rows.shape[0], k1.shape[0]
    q4, k4, v4 = q_rows[None, None].cpu(), k1[None, None].cpu(), v1[None, None].cpu()
    qi, qs, ki, ks = oq.per_block_int8(q4, k4, km=oq.k_mean(k4), BLKQ=blkq, BLKK=blkk)
    v8, vsc = oq.quant_v_fp8(v4)
    vis = (torch.arange(S)[None, :] <= torch.arange(r0, r0 + T)[:, None])[None, None] if causal else None
    ref, _ = oa.sage_reference(qi, ki, v8, qs, ks, "HND", blkq, blkk, attn_mask=vis, v_scale=vsc)
    model, _ = fm.fp8_attention_model(qi, ki, v4, qs, ks, "HND", blkq, blkk, is_causal=causal, row_offset=r0)
    logits = (q4.double() @ k4.double().transpose(-1, -2)) * (q4.shape[-1] ** -0.5)
    if causal:
        logits = logits.masked_fill(~vis, -float("inf"))
    sdpa = torch.softmax(logits, dim=-1) @ v4.double()
    g = got.detach().cpu().float()[None, None]
    return oa.metrics(g, ref), oa.metrics(g, model), oa.metrics(g, sdpa.float())
