"""CPU restatement of the reference's SageAttention quantizers (test infrastructure only).

All arithmetic is IEEE binary32 carried out by NumPy (``np.float32`` scalars and arrays;
NumPy's float32 multiply, divide and add are correctly rounded), so this file is the
meaning of "bit-exact" for the HIP quantizer.

Reference lines followed:
  * kernel   backends/_enflame/ops/sage_attention/quant_per_block.py:20-46
  * host     backends/_enflame/ops/sage_attention/quant_per_block.py:49-101
  * guard    backends/_hygon/ops/sageattention/sageattention_triton.py:35
Parity unpinned (not in the reference's code, defined here and pinned against the mathematics in the tests): k_mean,
quant_v_fp8, and the interleaved scales per block of quant_per_block_int8(groups=8 or 4).
"""
from __future__ import annotations

import numpy as np
import torch

LOG2E_REF = 1.44269504  # the literal used by quant_per_block.py:87
SCALE_FLOOR = np.float32(1.0e-12)  # sageattention_triton.py:35
FP8_E4M3_MAX = np.float32(448.0)


def _to_f32(x: torch.Tensor) -> np.ndarray:
    """fp16/bf16/fp32 torch tensor -> float32 ndarray (exact widening)."""
    return x.detach().cpu().to(torch.float32).numpy()


def _round_to_dtype(x32: np.ndarray, dtype: torch.dtype) -> np.ndarray:
    """Round a float32 array to ``dtype`` (RNE) and widen back to float32."""
    t = torch.from_numpy(np.ascontiguousarray(x32)).to(dtype)
    return t.to(torch.float32).numpy()


def quant_tile_int8(x32: np.ndarray, mult) -> tuple[np.ndarray, np.float32]:
    """One [rows, C] tile.  quant_per_block.py:38-46 (+ the 1e-12 floor).

    x = fp32(x) * mult; scale = max|x| / 127; q = trunc(x / scale + 0.5*sgn(x/scale)).
    ``x32`` holds only the valid rows of the tile: masked rows load as 0 and cannot
    raise the maximum (quant_per_block.py:38), and are not stored (:45).
    """
    x = x32.astype(np.float32, copy=False) * np.float32(mult)
    amax = np.float32(np.max(np.abs(x))) if x.size else np.float32(0.0)
    scale = np.maximum(amax / np.float32(127.0), SCALE_FLOOR).astype(np.float32)
    z = x / scale
    z = z + np.float32(0.5) * np.where(z >= 0, np.float32(1.0), np.float32(-1.0)).astype(np.float32)
    q = np.trunc(z).astype(np.int32).astype(np.int8)
    return q, np.float32(scale)


def quant_per_block_int8(x_hnd32: np.ndarray, blk: int, mult, groups: int = 1) -> tuple[np.ndarray, np.ndarray]:
    """[B, H, L, C] float32 -> (int8 [B,H,L,C], float32 scale [B,H,ceil(L/blk)*groups]).

    Vectorised over tiles; identical arithmetic to ``quant_tile_int8``.
    Grid of quant_per_block.py:81 / :91: one program per (block, head, batch).
    ``groups`` = 8: eight interleaved scales per block, scale g for the rows r of the block with r % 8 == g;
    ``groups`` = 4: four, scale t for the rows with (r % 8) // 2 == t (the granularities upstream SageAttention calls
    per-thread for Q and K, with its WARPQ / WARPK = blk).  The reference has no code for them (parity unpinned): they
    are defined here as the same tile arithmetic applied to each row group, and pinned in the tests against a
    row-group loop over ``quant_tile_int8``.
    """
    B, H, L, C = x_hnd32.shape
    nblk = (L + blk - 1) // blk
    pad = nblk * blk - L
    x = x_hnd32.astype(np.float32, copy=False) * np.float32(mult)
    if pad:
        x = np.concatenate([x, np.zeros((B, H, pad, C), np.float32)], axis=2)
    # [.., block, octet of rows, group, rows of the group inside the octet, channel]; one group: the whole block
    per_octet = {1: 1, 8: 1, 4: 2}[groups]
    xt = x.reshape(B, H, nblk, blk // (groups * per_octet), groups, per_octet, C)
    amax = np.max(np.abs(xt), axis=(3, 5, 6)).astype(np.float32)
    scale = np.maximum(amax / np.float32(127.0), SCALE_FLOOR).astype(np.float32)          # [B, H, nblk, groups]
    z = xt / scale[:, :, :, None, :, None, None]
    z = z + np.float32(0.5) * np.where(z >= 0, np.float32(1.0), np.float32(-1.0)).astype(np.float32)
    q = np.trunc(z).astype(np.int32).astype(np.int8).reshape(B, H, nblk * blk, C)[:, :, :L]
    return np.ascontiguousarray(q), np.ascontiguousarray(scale.reshape(B, H, nblk * groups))


def _hnd(x: np.ndarray, layout: str) -> np.ndarray:
    if layout == "HND":
        return x
    if layout == "NHD":
        return x.transpose(0, 2, 1, 3)
    raise ValueError(f"Unknown tensor layout: {layout}")


def q_multiplier(head_dim: int, sm_scale=None) -> np.float32:
    """quant_per_block.py:78-79 and :87: Python-float product, then one rounding to fp32
    when Triton passes the scalar as an fp32 kernel argument."""
    if sm_scale is None:
        sm_scale = head_dim ** -0.5
    return np.float32(float(sm_scale) * LOG2E_REF)


def per_block_int8(q, k, km=None, BLKQ=128, BLKK=64, sm_scale=None, tensor_layout="HND", q_interleave=1, k_interleave=1):
    """Restates per_block_int8 (quant_per_block.py:49-101) on CPU tensors.

    Returns torch CPU tensors (q_int8, q_scale, k_int8, k_scale) with the reference's
    shapes: int8 like q / k, scales [B, H, ceil(L/BLK)] float32 (q_scale [B, H, ceil(L/BLKQ)*8] with
    ``q_interleave=8``, k_scale [B, H, ceil(L/BLKK)*4] with ``k_interleave=4``, see quant_per_block_int8).
    """
    if km is not None:
        k = k - km  # input-dtype subtraction, quant_per_block.py:53-54
    q32 = _hnd(_to_f32(q), tensor_layout)
    k32 = _hnd(_to_f32(k), tensor_layout)
    head_dim = q32.shape[-1]
    qi, qs = quant_per_block_int8(q32, BLKQ, q_multiplier(head_dim, sm_scale), q_interleave)
    ki, ks = quant_per_block_int8(k32, BLKK, np.float32(1.0), k_interleave)
    qi = np.ascontiguousarray(_hnd(qi, tensor_layout)) if tensor_layout == "NHD" else qi
    ki = np.ascontiguousarray(_hnd(ki, tensor_layout)) if tensor_layout == "NHD" else ki
    return (torch.from_numpy(qi), torch.from_numpy(qs), torch.from_numpy(ki), torch.from_numpy(ks))


def k_mean(k: torch.Tensor, tensor_layout="HND") -> torch.Tensor:
    """Per-(batch, kv-head, channel) mean of K over the sequence, in k's dtype.

    NOT in the reference (km is only ever an argument there): parity unpinned.
    Definition used by this build: exact sum accumulated in float64, divided by the
    length in float64, rounded once to float32 and then once to the input dtype.  For
    fp16/bf16 inputs the float64 sum is exact for every realistic dynamic range, which
    makes the value independent of the summation order (the GPU sums in another order).
    Returned with a keep-dim sequence axis so that ``k - km`` broadcasts.
    """
    seq_axis = 2 if tensor_layout == "HND" else 1
    s = k.detach().cpu().to(torch.float64).sum(dim=seq_axis, keepdim=True)
    m32 = (s / float(k.shape[seq_axis])).to(torch.float32)
    return m32.to(k.dtype)


def quant_v_fp8(v: torch.Tensor, tensor_layout="HND"):
    """Per-channel FP8-e4m3fn quantisation of V over the sequence.  Parity unpinned.

    scale[b,h,c] = max(amax_n |v| / 448, 1e-12) (fp32, IEEE divide);
    v8 = RNE_e4m3fn(clamp(fp32(v) / scale, -448, 448)).
    Returns (v_fp8 torch.float8_e4m3fn with v's shape, scale [B, H, C] float32).
    """
    v32 = _hnd(_to_f32(v), tensor_layout)
    amax = np.max(np.abs(v32), axis=2).astype(np.float32)
    scale = np.maximum(amax / FP8_E4M3_MAX, SCALE_FLOOR).astype(np.float32)
    z = np.clip(v32 / scale[:, :, None, :], -FP8_E4M3_MAX, FP8_E4M3_MAX).astype(np.float32)
    z = np.ascontiguousarray(_hnd(z, tensor_layout)) if tensor_layout == "NHD" else z
    v8 = torch.from_numpy(np.ascontiguousarray(z)).to(torch.float8_e4m3fn)
    return v8, torch.from_numpy(scale)


def seq_block_offsets(cu_seqlens, blk: int) -> np.ndarray:
    """Prefix sum of ceil(L_i / blk): where each packed sequence's scale blocks start."""
    cu = np.asarray(cu_seqlens, dtype=np.int64)
    lens = cu[1:] - cu[:-1]
    return np.concatenate([[0], np.cumsum((lens + blk - 1) // blk)]).astype(np.int64)


def per_block_int8_varlen(q, k, cu_seqlens_q, cu_seqlens_k, km=None, BLKQ=128, BLKK=64, sm_scale=None):
    """Packed variant: q [Tq, Hq, D], k [Tk, Hkv, D]; blocks restart at every sequence.

    Not in the reference: parity unpinned; defined as per_block_int8 (quant_per_block.py
    :49-101) applied to each sequence independently.  ``km`` is [nseq, Hkv, D] or None.
    Scales are [H, total_blocks] with sequence i's blocks at seq_block_offsets()[i].
    """
    cuq = np.asarray(cu_seqlens_q, dtype=np.int64)
    cuk = np.asarray(cu_seqlens_k, dtype=np.int64)
    nseq = len(cuq) - 1
    oq, ok = seq_block_offsets(cuq, BLKQ), seq_block_offsets(cuk, BLKK)
    qi = torch.empty(q.shape, dtype=torch.int8)
    ki = torch.empty(k.shape, dtype=torch.int8)
    qs = torch.empty((q.shape[1], int(oq[-1])), dtype=torch.float32)
    ks = torch.empty((k.shape[1], int(ok[-1])), dtype=torch.float32)
    for i in range(nseq):
        qq = q[cuq[i]:cuq[i + 1]].unsqueeze(0)
        kk = k[cuk[i]:cuk[i + 1]].unsqueeze(0)
        kmi = None if km is None else km[i].reshape(1, 1, k.shape[1], k.shape[2])
        a, b, c, d = per_block_int8(qq, kk, km=kmi, BLKQ=BLKQ, BLKK=BLKK, sm_scale=sm_scale, tensor_layout="NHD")
        qi[cuq[i]:cuq[i + 1]] = a[0]
        ki[cuk[i]:cuk[i + 1]] = c[0]
        qs[:, oq[i]:oq[i + 1]] = b[0]
        ks[:, ok[i]:ok[i + 1]] = d[0]
    return qi, qs, ki, ks
