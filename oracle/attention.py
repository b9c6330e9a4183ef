"""CPU restatement of the reference's SageAttention forward math (test infrastructure only).

``sage_reference`` is the formula the reference's own tests check their kernels against:
  backends/_hygon/test/sageattention/test_sageattention_hip.py:8-28   (with masks and LSE)
  backends/_enflame/test/test_sage_attention_native.py:62-81
  backends/_enflame/benchmarks/sage_attention_native_benchmark.py:276-292
i.e. softmax(ln2 * (Qi8*qs)(Ki8*ks)^T [+ mask]) @ V in floating point, scales expanded with
repeat_interleave over their block, KV heads expanded for GQA, LSE in base 2.
Causal masking, varlen packing and FP8 V are not in the reference (parity unpinned there);
they are defined here in the obvious way and pinned in tests against
torch.nn.functional.scaled_dot_product_attention and per-sequence loops.
"""
from __future__ import annotations

import math

import torch
import torch.nn.functional as F

LN2 = math.log(2.0)


def _hnd(x: torch.Tensor, layout: str) -> torch.Tensor:
    if layout == "HND":
        return x
    if layout == "NHD":
        return x.transpose(1, 2)
    raise ValueError(f"tensor_layout {layout!r} is not supported")


def expand_scale(scale: torch.Tensor, block: int, length: int) -> torch.Tensor:
    """test_sageattention_hip.py:8-9."""
    return scale.repeat_interleave(block, dim=-1)[..., :length, None]


def expand_scale_interleaved(scale: torch.Tensor, block: int, groups: int, length: int) -> torch.Tensor:
    """Interleaved scales per block: eight -> row n takes scale[(n // block) * 8 + n % 8]; four -> scale[(n // block) * 4 +
    (n % 8) // 2]."""
    n = torch.arange(length)
    g = n % 8 if groups == 8 else (n % 8) // 2
    return scale[..., (n // block) * groups + g, None]


def sage_reference(q_int8, k_int8, v, q_scale, k_scale, tensor_layout="HND", BLKQ=128, BLKK=64,
                   is_causal=False, attn_mask=None, v_scale=None, dtype=torch.float64, q_interleave=1, k_interleave=1):
    """Attention on already-quantised operands.  Returns (out [layout of q], lse2 [B,Hq,Sq]).

    * v may be fp16/bf16/fp32, or float8_e4m3fn together with ``v_scale`` [B,Hkv,D]
      (dequantised as fp8 * scale).
    * causal mask is top-left aligned (key j visible to query i iff j <= i), which is
      torch SDPA's ``is_causal=True`` convention.
    * rows with no visible key give out = 0 and lse = -inf.
    * ``q_interleave`` = 8 / ``k_interleave`` = 4: q_scale / k_scale hold eight / four interleaved scales per block
      (oracle.quant.quant_per_block_int8).
    """
    q = _hnd(q_int8, tensor_layout).cpu().to(dtype)
    k = _hnd(k_int8, tensor_layout).cpu().to(dtype)
    vv = _hnd(v, tensor_layout).cpu().to(torch.float32).to(dtype)
    if v_scale is not None:
        vv = vv * v_scale.cpu().to(dtype)[:, :, None, :]
    sq, skv = q.shape[-2], k.shape[-2]
    q = q * (expand_scale(q_scale.cpu().to(dtype), BLKQ, sq) if q_interleave == 1 else
             expand_scale_interleaved(q_scale.cpu().to(dtype), BLKQ, q_interleave, sq))
    k = k * (expand_scale(k_scale.cpu().to(dtype), BLKK, skv) if k_interleave == 1 else
             expand_scale_interleaved(k_scale.cpu().to(dtype), BLKK, k_interleave, skv))
    group = q.shape[1] // k.shape[1]
    k = k.repeat_interleave(group, dim=1)
    vv = vv.repeat_interleave(group, dim=1)
    logits = torch.matmul(q, k.transpose(-1, -2))
    if attn_mask is not None:
        m = attn_mask.cpu()
        logits = logits.masked_fill(~m, -float("inf")) if m.dtype == torch.bool else logits + m.to(dtype)
    if is_causal:
        i = torch.arange(sq)[:, None]
        j = torch.arange(skv)[None, :]
        logits = logits.masked_fill(j > i, -float("inf"))
    nat = logits * LN2
    lse = torch.logsumexp(nat, dim=-1)
    probs = torch.exp(nat - torch.where(torch.isfinite(lse), lse, torch.zeros_like(lse))[..., None])
    probs = torch.where(torch.isfinite(lse)[..., None], probs, torch.zeros_like(probs))
    out = torch.matmul(probs, vv)
    out = _hnd(out, tensor_layout) if tensor_layout == "NHD" else out
    return out.contiguous(), lse / LN2


def sdpa_fp32(q, k, v, tensor_layout="HND", is_causal=False, sm_scale=None, dtype=torch.float32):
    """Plain scaled-dot-product attention on the un-quantised inputs (the second oracle the
    north-star tolerance is stated against); GQA by head repetition."""
    qq = _hnd(q, tensor_layout).cpu().to(dtype)
    kk = _hnd(k, tensor_layout).cpu().to(dtype)
    vv = _hnd(v, tensor_layout).cpu().to(dtype)
    group = qq.shape[1] // kk.shape[1]
    if group > 1:
        kk = kk.repeat_interleave(group, dim=1)
        vv = vv.repeat_interleave(group, dim=1)
    out = F.scaled_dot_product_attention(qq, kk, vv, is_causal=is_causal, scale=sm_scale)
    out = _hnd(out, tensor_layout) if tensor_layout == "NHD" else out
    return out.contiguous()


def sdpa_fp32_varlen(q, k, v, cu_seqlens_q, cu_seqlens_k, is_causal=False, sm_scale=None):
    """Packed [T,H,D] inputs: loop over sequences, each through sdpa_fp32 (NHD)."""
    out = torch.empty(q.shape, dtype=torch.float32)
    cq = [int(x) for x in cu_seqlens_q]
    ck = [int(x) for x in cu_seqlens_k]
    for i in range(len(cq) - 1):
        o = sdpa_fp32(q[cq[i]:cq[i + 1]].unsqueeze(0), k[ck[i]:ck[i + 1]].unsqueeze(0),
                      v[ck[i]:ck[i + 1]].unsqueeze(0), "NHD", is_causal, sm_scale)
        out[cq[i]:cq[i + 1]] = o[0]
    return out


def metrics(actual: torch.Tensor, expected: torch.Tensor) -> dict:
    """backends/_mthreads/benchmarks/sage_attention_benchmark_compare.py:324-339 plus the
    relative RMSE of test_sageattention_hip.py:52-53."""
    a = actual.detach().cpu().double().flatten()
    e = expected.detach().cpu().double().flatten()
    d = a - e
    return {
        "finite": bool(torch.isfinite(a).all()),
        "cosine": F.cosine_similarity(a, e, dim=0).item(),
        "relative_l1": (d.abs().sum() / (a.abs().sum() + e.abs().sum() + 1e-8)).item(),
        "rmse": d.square().mean().sqrt().item(),
        "rel_rmse": (d.square().mean().sqrt() / (e.square().mean().sqrt() + 1e-6)).item(),
        "max_abs": d.abs().max().item(),
    }


def cpu_quantize_sdpa(q, k, v, tensor_layout="HND", is_causal=False, sm_scale=None, BLKQ=128, BLKK=64,
                      smooth_k=True):
    """The reference's CPU-expressible pipeline, used as the timed CPU baseline:
    per-block INT8 quantise (+K smoothing) -> per-block dequantise with ln2 folded into Q
    -> torch SDPA with scale=1.0, i.e. the structure of
    backends/_enflame/ops/sage_attention/attn_qk_int8_per_block_native.py:309-379.
    Vectorised torch ops only (float32), so it runs on all host threads."""
    qh = _hnd(q, tensor_layout).float()
    kh = _hnd(k, tensor_layout).float()
    vh = _hnd(v, tensor_layout).float()
    if smooth_k:
        kh = kh - kh.mean(dim=2, keepdim=True)
    d = qh.shape[-1]
    if sm_scale is None:
        sm_scale = d ** -0.5

    def quant_dequant(x, blk, mult):
        b, h, l, c = x.shape
        nb = (l + blk - 1) // blk
        xp = F.pad(x * mult, (0, 0, 0, nb * blk - l)).reshape(b, h, nb, blk * c)
        scale = (xp.abs().amax(dim=-1, keepdim=True) / 127.0).clamp_min(1e-12)
        z = xp / scale
        z = torch.trunc(z + 0.5 * torch.where(z >= 0, 1.0, -1.0))
        return (z * scale).reshape(b, h, nb * blk, c)[:, :, :l]

    qd = quant_dequant(qh, BLKQ, sm_scale * 1.44269504) * LN2
    kd = quant_dequant(kh, BLKK, 1.0)
    group = qd.shape[1] // kd.shape[1]
    if group > 1:
        kd = kd.repeat_interleave(group, dim=1)
        vh = vh.repeat_interleave(group, dim=1)
    out = F.scaled_dot_product_attention(qd, kd, vh, is_causal=is_causal, scale=1.0)
    return _hnd(out, tensor_layout) if tensor_layout == "NHD" else out
