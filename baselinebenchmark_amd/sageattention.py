"""Python entry points of the MI355X SageAttention forward path.

A thin shim over the C ABI (include/sage_mi355x.h): it checks the arguments the way the reference
wrappers do, allocates outputs and scratch with torch, and passes raw pointers, strides and the
current HIP stream.  All arithmetic happens in hand-written gfx950 kernels.

Mirrored reference interfaces (same names, argument meaning and error classes):
  per_block_int8  backends/_enflame/ops/sage_attention/quant_per_block.py:49-101
                  backends/_hygon/ops/sageattention/sageattention_hip.py:37-51
  forward         backends/_hygon/ops/sageattention/sageattention_hip.py:54-74
                  backends/_enflame/ops/sage_attention/attn_qk_int8_per_block_native.py:438-523
  sageattn        call sites backends/_metax/benchmarks/sage_attention/benchmark.py:29 and
                  backends/_mthreads/benchmarks/sage_attention_benchmark_compare.py:300-313
  backend_name    backends/_hygon/ops/sageattention/sageattention_hip.py:77-79
"""
from __future__ import annotations

import ctypes

import torch

from . import _cabi
from ._cabi import DT_BF16, DT_F16, PANEL_ROWS, PV_FP8, PV_FP16, check, lib

__all__ = ["per_block_int8", "forward", "sageattn", "sageattn_varlen", "backend_name", "k_mean", "prepare_v",
           "per_block_int8_varlen", "varlen_plan"]

_LOG2E_REF = 1.44269504  # quant_per_block.py:87


def backend_name() -> str:
    return lib().sage_backend_name().decode()


# ------------------------------------------------------------------------------------------------
# helpers
# ------------------------------------------------------------------------------------------------
def _ptr(t):
    return ctypes.c_void_p(0 if t is None else t.data_ptr())


def _stream(t: torch.Tensor):
    return ctypes.c_void_p(torch.cuda.current_stream(t.device).cuda_stream)


def _dt(dtype: torch.dtype) -> int:
    if dtype == torch.float16:
        return DT_F16
    if dtype == torch.bfloat16:
        return DT_BF16
    raise TypeError(f"dtype {dtype} is not float16 or bfloat16")


def _check_float(name: str, x) -> None:
    """sageattention_hip.py:30-34."""
    if not isinstance(x, torch.Tensor) or not x.is_cuda or x.dtype not in (torch.float16, torch.bfloat16):
        raise TypeError(f"{name} must be a GPU FP16/BF16 tensor")
    if x.ndim != 4 or not x.is_contiguous():
        raise ValueError(f"{name} must be contiguous rank 4")


def _layout(t: torch.Tensor, tensor_layout: str):
    """(B, H, L, D, stride_b, stride_h, stride_n), sageattention_triton.py:132-137."""
    if tensor_layout == "HND":
        return t.shape[0], t.shape[1], t.shape[2], t.shape[3], t.stride(0), t.stride(1), t.stride(2)
    if tensor_layout == "NHD":
        return t.shape[0], t.shape[2], t.shape[1], t.shape[3], t.stride(0), t.stride(2), t.stride(1)
    raise ValueError(f"tensor_layout {tensor_layout!r} is not supported")


def _check_blocks_quant(BLKQ, BLKK):
    for b in (BLKQ, BLKK):
        if b not in (16, 32, 64, 128):
            raise NotImplementedError(f"quantisation block {b} is not supported (16, 32, 64 or 128)")


def _q_mult(head_dim: int, sm_scale) -> float:
    if sm_scale is None:
        sm_scale = head_dim ** -0.5
    return float(sm_scale) * _LOG2E_REF


# ------------------------------------------------------------------------------------------------
# quantisers
# ------------------------------------------------------------------------------------------------
@torch.no_grad()
def k_mean(k: torch.Tensor, tensor_layout: str = "HND") -> torch.Tensor:
    """Per-(batch, kv-head, channel) mean of K over the sequence in k's dtype, shaped to broadcast
    against k ([B,H,1,D] for HND, [B,1,H,D] for NHD): the `km` argument of per_block_int8."""
    _check_float("k", k)
    B, H, L, D, sb, sh, sn = _layout(k, tensor_layout)
    if D not in (64, 128):
        raise NotImplementedError("head_dim must be 64 or 128")
    km = torch.empty((B, H, D), device=k.device, dtype=k.dtype)
    ws_bytes = lib().sage_k_mean_workspace_bytes(B, H, L, D)
    ws = torch.empty(max(ws_bytes, 8), device=k.device, dtype=torch.uint8)
    check(lib().sage_k_mean(_ptr(k), _ptr(km), _ptr(ws), ws_bytes, B, H, L, D, sb, sh, sn, _dt(k.dtype), None, _stream(k)))
    return km.view(B, H, 1, D) if tensor_layout == "HND" else km.view(B, 1, H, D)


BLK_INTERLEAVE8 = 0x100   # SAGE_BLK_INTERLEAVE8 of the C ABI: eight interleaved scales per Q block
BLK_INTERLEAVE4 = 0x200   # SAGE_BLK_INTERLEAVE4: four interleaved scales per K block


def _check_interleave(q_interleave) -> int:
    if q_interleave not in (1, 8):
        raise ValueError("q_interleave must be 1 (one scale per Q block) or 8 (rows r, r+8, ... of a block share a scale)")
    return BLK_INTERLEAVE8 if q_interleave == 8 else 0


def _check_k_interleave(k_interleave, BLKK) -> int:
    if k_interleave not in (1, 4):
        raise ValueError("k_interleave must be 1 (one scale per K block) or 4 (keys n with equal (n % 8) // 2 share a scale)")
    if k_interleave == 4 and BLKK == 16:
        raise NotImplementedError("four interleaved K scales need K blocks of 32, 64 or 128 keys")
    return BLK_INTERLEAVE4 if k_interleave == 4 else 0


def _quant_one(x, km, blk, mult, tensor_layout, groups=1):
    B, H, L, D, sb, sh, sn = _layout(x, tensor_layout)
    out = torch.empty(x.shape, device=x.device, dtype=torch.int8)
    _, _, _, _, osb, osh, osn = _layout(out, tensor_layout)
    scale = torch.empty((B, H, (L + blk - 1) // blk * groups), device=x.device, dtype=torch.float32)
    km_sb = km_sh = 0
    if km is not None:
        if km.dtype != x.dtype or km.device != x.device:
            raise ValueError("km must have k's dtype and device")
        km = km.expand((B, H, 1, D) if tensor_layout == "HND" else (B, 1, H, D))
        if km.stride(-1) != 1 and D > 1:
            km = km.contiguous()
        km_sb, km_sh = (km.stride(0), km.stride(1)) if tensor_layout == "HND" else (km.stride(0), km.stride(2))
    check(lib().sage_quant_int8(_ptr(x), _ptr(out), _ptr(scale), _ptr(km), B, H, L, D, sb, sh, sn, osb, osh, osn,
                                km_sb, km_sh, blk | {1: 0, 8: BLK_INTERLEAVE8, 4: BLK_INTERLEAVE4}[groups], mult, _dt(x.dtype),
                                None, None, 0, _stream(x)))
    return out, scale


@torch.no_grad()
def per_block_int8(q, k, km=None, BLKQ=128, BLKK=64, sm_scale=None, tensor_layout="HND", q_interleave=1, k_interleave=1):
    """Per-block INT8 quantisation of Q and K; returns (q_int8, q_scale, k_int8, k_scale).

    Same contract as quant_per_block.py:49-101: optional ``k - km`` in the input dtype, Q scaled by
    ``sm_scale * 1.44269504`` (default sm_scale = head_dim**-0.5), K by 1, scales [B, H, ceil(L/BLK)].
    ``q_interleave=8`` (no counterpart in the reference's code; the granularity upstream SageAttention calls per-thread,
    with WARPQ = BLKQ): every Q block gets eight scales, scale g for its rows r with r % 8 == g, and q_scale is
    [B, H, ceil(L/BLKQ) * 8]; pass the same keyword to ``forward``.  ``k_interleave=4`` is upstream's per-thread K
    granularity (WARPK = BLKK): four scales per K block, scale t for its keys n with (n % 8) // 2 == t, k_scale
    [B, H, ceil(L/BLKK) * 4].  ``per_block_int8(..., BLKQ=32, BLKK=64, q_interleave=8, k_interleave=4)`` is upstream's
    per_thread_int8 with this reference's quantiser arithmetic.
    """
    _check_float("q", q)
    _check_float("k", k)
    if q.dtype != k.dtype or q.device != k.device:
        raise ValueError("q and k must have the same dtype and device")
    if tensor_layout not in ("HND", "NHD"):
        raise ValueError(f"Unknown tensor layout: {tensor_layout}")
    if q.shape[-1] not in (64, 128):
        raise NotImplementedError("head_dim must be 64 or 128")
    if q.shape[-1] != k.shape[-1]:
        raise ValueError("q and k head dimensions differ")
    _check_blocks_quant(BLKQ, BLKK)
    _check_interleave(q_interleave)
    _check_k_interleave(k_interleave, BLKK)
    q_int8, q_scale = _quant_one(q, None, BLKQ, _q_mult(q.shape[-1], sm_scale), tensor_layout, q_interleave)
    k_int8, k_scale = _quant_one(k, km, BLKK, 1.0, tensor_layout, k_interleave)
    return q_int8, q_scale, k_int8, k_scale


@torch.no_grad()
def prepare_v(v: torch.Tensor, tensor_layout: str = "HND", pv_mode: str = "fp16"):
    """V -> MFMA-ready panels.  Returns (panels uint8 tensor, v_scale [B,H,D] float32 or None)."""
    _check_float("v", v)
    pv = _pv(pv_mode)
    B, H, L, D, sb, sh, sn = _layout(v, tensor_layout)
    if D not in (64, 128):
        raise NotImplementedError("head_dim must be 64 or 128")
    panels = torch.empty(max(lib().sage_v_panel_bytes(B, H, L, D, pv), 16), device=v.device, dtype=torch.uint8)
    v_scale = ws = None
    ws_bytes = 0
    if pv == PV_FP8:
        v_scale = torch.empty((B, H, D), device=v.device, dtype=torch.float32)
        ws_bytes = lib().sage_prep_v_workspace_bytes(B, H, L, D, pv)
        ws = torch.empty(max(ws_bytes, 8), device=v.device, dtype=torch.uint8)
    check(lib().sage_prep_v(_ptr(v), _ptr(panels), _ptr(v_scale), _ptr(ws), ws_bytes, B, H, L, D, sb, sh, sn,
                            _dt(v.dtype), pv, None, None, 0, _stream(v)))
    return panels, v_scale


def _pv(pv_mode) -> int:
    if pv_mode in ("fp16", PV_FP16, torch.float16):
        return PV_FP16
    if pv_mode in ("fp8", PV_FP8, getattr(torch, "float8_e4m3fn", "fp8")):
        return PV_FP8
    raise ValueError(f"pv_mode {pv_mode!r} is not 'fp16' or 'fp8'")


def _mask_args(attn_mask, B, Hq, Sq, Skv, device):
    """Validate an explicit mask and return (tensor kept alive, kind, element strides).

    Boolean masks keep the keys that are True; any other dtype is an additive bias and is read as
    fp32 (sageattention_triton.py:180-186, :92-105).  The mask must be broadcastable to
    [B, Hq, Sq, Skv]; broadcast dimensions are passed with stride 0, nothing is materialised.
    """
    if not isinstance(attn_mask, torch.Tensor):
        raise TypeError("attn_mask must be a tensor")
    if not attn_mask.is_cuda or attn_mask.device != device:
        raise ValueError("attn_mask must be on the same device as q")
    if attn_mask.ndim > 4:
        raise ValueError("attn_mask must have at most 4 dimensions")
    if attn_mask.dtype == torch.bool:
        kind, m = 1, attn_mask
    elif attn_mask.dtype.is_floating_point:
        kind, m = 2, attn_mask if attn_mask.dtype == torch.float32 else attn_mask.float()
    else:
        raise TypeError("attn_mask must be boolean or floating point")
    try:
        m = m.expand(B, Hq, Sq, Skv)
    except RuntimeError as exc:
        raise ValueError(f"attn_mask of shape {tuple(attn_mask.shape)} does not broadcast to {(B, Hq, Sq, Skv)}") from exc
    return m, kind, m.stride()


# ------------------------------------------------------------------------------------------------
# attention on quantised operands
# ------------------------------------------------------------------------------------------------
@torch.no_grad()
def forward(q, k, v, q_scale, k_scale, tensor_layout="HND", attn_mask=None, output_dtype=torch.float16,
            return_lse=False, maxnreg=None, block_m=None, num_warps=None, num_stages=None, backend=None,
            BLKQ=128, BLKK=64, is_causal=False, pv_mode="fp16", q_interleave=1, k_interleave=1):
    """Fused INT8-QK attention on operands produced by per_block_int8; returns (out, lse).

    Signature of sageattention_hip.py:55-56 / attn_qk_int8_per_block_native.py:438-453; the tuning
    keywords (maxnreg, block_m, num_warps, num_stages, backend) are accepted and ignored as in
    sageattention_triton.py:169.  Additions: ``BLKQ``/``BLKK`` name the scale blocks when they are
    not the reference's 128/64, ``is_causal`` and ``pv_mode`` ("fp16" | "fp8").
    ``attn_mask``: boolean (True keeps the key) or additive bias on the base-2 logits, broadcastable
    to [B, Hq, Sq, Skv] (sageattention_triton.py:92-105); not combinable with ``is_causal``.
    ``lse`` is base 2 (sageattention_triton.py:127-129) and an empty tensor unless requested.
    ``q_interleave=8`` / ``k_interleave=4``: q_scale / k_scale hold eight / four interleaved scales per block (see
    per_block_int8).
    """
    qflag = _check_interleave(q_interleave)
    kflag = _check_k_interleave(k_interleave, BLKK)
    for name, t in (("q", q), ("k", k)):
        if not isinstance(t, torch.Tensor) or not t.is_cuda or t.dtype != torch.int8 or not t.is_contiguous():
            raise TypeError(f"{name} must be contiguous GPU INT8")
    _check_float("v", v)
    if q_scale.dtype != torch.float32 or k_scale.dtype != torch.float32:
        raise TypeError("q_scale and k_scale must be FP32")
    if output_dtype not in (torch.float16, torch.bfloat16):
        raise NotImplementedError("output_dtype must be FP16 or BF16")
    if maxnreg is not None and maxnreg <= 0:
        raise ValueError("maxnreg must be positive")
    if attn_mask is not None and is_causal:
        raise NotImplementedError("attn_mask cannot be combined with is_causal")
    if q.ndim != 4 or k.ndim != 4:
        raise ValueError("q, k, and v must be rank-4 tensors")
    B, Hq, Sq, D, qsb, qsh, qsn = _layout(q, tensor_layout)
    Bk, Hkv, Skv, Dk, ksb, ksh, ksn = _layout(k, tensor_layout)
    Bv, Hv, Sv, Dv, _, _, _ = _layout(v, tensor_layout)
    if Dk != D or Dv != D or Sv != Skv or Hv != Hkv or Bk != B or Bv != B:
        raise ValueError("incompatible q/k/v shapes")
    if Hq % Hkv:
        raise ValueError("query heads must be divisible by KV heads")
    if D not in (64, 128):
        raise NotImplementedError("head_dim must be 64 or 128")
    if BLKQ not in (16, 32, 64, 128) or BLKK not in (16, 32, 64, 128):
        raise NotImplementedError("the attention kernel needs Q and K scale blocks of 16, 32, 64 or 128 rows")
    exp_q = (B, Hq, (Sq + BLKQ - 1) // BLKQ * q_interleave)
    exp_k = (B, Hkv, (Skv + BLKK - 1) // BLKK * k_interleave)
    if tuple(q_scale.shape) != exp_q:
        raise ValueError(f"q_scale has shape {tuple(q_scale.shape)}, expected {exp_q}")
    if tuple(k_scale.shape) != exp_k:
        raise ValueError(f"k_scale has shape {tuple(k_scale.shape)}, expected {exp_k}")
    if q_scale.device != q.device or k_scale.device != q.device or k.device != q.device or v.device != q.device:
        raise ValueError("all tensors must be on the same device")
    pv = _pv(pv_mode)
    mask_info = _mask_args(attn_mask, B, Hq, Sq, Skv, q.device) if attn_mask is not None else None
    panels, v_scale = prepare_v(v, tensor_layout, pv)
    out = torch.empty(q.shape, device=q.device, dtype=output_dtype)
    _, _, _, _, osb, osh, osn = _layout(out, tensor_layout)
    lse = torch.empty((B, Hq, Sq), device=q.device, dtype=torch.float32) if return_lse else torch.empty(0, device=q.device)
    if mask_info is not None:
        m, kind, ms = mask_info
        check(lib().sage_attn_fwd_masked(_ptr(q), _ptr(k), _ptr(panels), _ptr(q_scale.contiguous()),
                                         _ptr(k_scale.contiguous()), _ptr(v_scale), _ptr(out),
                                         _ptr(lse if return_lse else None),
                                         B, Hq, Hkv, Sq, Skv, D, qsb, qsh, qsn, ksb, ksh, ksn, osb, osh, osn,
                                         BLKQ | qflag, BLKK | kflag, pv, _dt(output_dtype), _ptr(m), kind, ms[0], ms[1], ms[2], ms[3],
                                         _stream(q)))
        return out, lse
    check(lib().sage_attn_fwd(_ptr(q), _ptr(k), _ptr(panels), _ptr(q_scale.contiguous()), _ptr(k_scale.contiguous()),
                              _ptr(v_scale), _ptr(out), _ptr(lse if return_lse else None),
                              B, Hq, Hkv, Sq, Skv, D, qsb, qsh, qsn, ksb, ksh, ksn, osb, osh, osn,
                              BLKQ | qflag, BLKK | kflag, int(bool(is_causal)), pv, _dt(output_dtype),
                              None, None, None, 0, 0, 0, 0, _stream(q)))
    return out, lse


@torch.no_grad()
def forward_fused_q(q, k, v, k_scale, tensor_layout="HND", sm_scale=None, output_dtype=None, return_lse=False,
                    BLKQ=128, BLKK=64, is_causal=False, pv_mode="fp16", k_interleave=1):
    """forward() for a floating-point ``q`` and an already quantised ``k``: each q-tile is quantised inside the
    attention kernel (bit-identical to per_block_int8 on q followed by forward()).  For callers that keep K
    quantised across calls.  ``k``/``k_scale`` as returned by per_block_int8 (``k_interleave=4``: with four interleaved
    scales per K block); returns (out, lse) like forward()."""
    kflag = _check_k_interleave(k_interleave, BLKK)
    _check_float("q", q)
    _check_float("v", v)
    if not isinstance(k, torch.Tensor) or not k.is_cuda or k.dtype != torch.int8 or not k.is_contiguous():
        raise TypeError("k must be contiguous GPU INT8")
    if k_scale.dtype != torch.float32:
        raise TypeError("k_scale must be FP32")
    output_dtype = q.dtype if output_dtype is None else output_dtype
    if output_dtype not in (torch.float16, torch.bfloat16):
        raise NotImplementedError("output_dtype must be FP16 or BF16")
    B, Hq, Sq, D, qsb, qsh, qsn = _layout(q, tensor_layout)
    Bk, Hkv, Skv, Dk, ksb, ksh, ksn = _layout(k, tensor_layout)
    Bv, Hv, Sv, Dv, _, _, _ = _layout(v, tensor_layout)
    if Dk != D or Dv != D or Sv != Skv or Hv != Hkv or Bk != B or Bv != B:
        raise ValueError("incompatible q/k/v shapes")
    if Hq % Hkv:
        raise ValueError("query heads must be divisible by KV heads")
    if D not in (64, 128):
        raise NotImplementedError("head_dim must be 64 or 128")
    if BLKQ not in (16, 32, 64, 128) or BLKK not in (16, 32, 64, 128):
        raise NotImplementedError("the fused-Q kernel needs Q and K scale blocks of 16, 32, 64 or 128 rows")
    if tuple(k_scale.shape) != (B, Hkv, (Skv + BLKK - 1) // BLKK * k_interleave):
        raise ValueError(f"k_scale has shape {tuple(k_scale.shape)}, expected {(B, Hkv, (Skv + BLKK - 1) // BLKK * k_interleave)}")
    pv = _pv(pv_mode)
    panels, v_scale = prepare_v(v, tensor_layout, pv)
    out = torch.empty(q.shape, device=q.device, dtype=output_dtype)
    _, _, _, _, osb, osh, osn = _layout(out, tensor_layout)
    lse = torch.empty((B, Hq, Sq), device=q.device, dtype=torch.float32) if return_lse else torch.empty(0, device=q.device)
    check(lib().sage_attn_fwd_qfused(_ptr(q), _dt(q.dtype), float(D ** -0.5 if sm_scale is None else sm_scale), _ptr(k),
                                     _ptr(panels), _ptr(k_scale.contiguous()), _ptr(v_scale), _ptr(out),
                                     _ptr(lse if return_lse else None),
                                     B, Hq, Hkv, Sq, Skv, D, qsb, qsh, qsn, ksb, ksh, ksn, osb, osh, osn,
                                     BLKQ, BLKK | kflag, int(bool(is_causal)), pv, _dt(output_dtype), None, None, None, 0, 0, 0,
                                     _stream(q)))
    return out, lse


# ------------------------------------------------------------------------------------------------
# one-call API
# ------------------------------------------------------------------------------------------------
def _apply_recipe(quant_recipe, BLKQ, BLKK, pv_mode):
    """``quant_recipe`` as passed at sage_attention_benchmark_compare.py:93, :300-313 -- (Q rows per scale, K rows
    per scale, V rows per scale with -1 = the whole sequence, V channels per scale): the one V granularity built
    here is (-1, 1), per-channel FP8-e4m3 V (``V=FP8``, :571), so a recipe selects the FP8 P.V path."""
    if quant_recipe is None:
        return BLKQ, BLKK, ("fp16" if pv_mode is None else pv_mode)
    try:
        bq, bk, vrows, vcols = (int(x) for x in quant_recipe)
    except (TypeError, ValueError) as exc:
        raise ValueError(f"quant_recipe must be four integers, got {quant_recipe!r}") from exc
    if (vrows, vcols) != (-1, 1):
        raise NotImplementedError("V is quantised per channel over the whole sequence: quant_recipe[2:] must be (-1, 1)")
    if pv_mode is not None and _pv(pv_mode) != PV_FP8:
        raise ValueError("a quant_recipe quantises V to FP8: pv_mode must be 'fp8' or left unset")
    return bq, bk, "fp8"


@torch.no_grad()
def sageattn(q, k, v, tensor_layout="HND", is_causal=False, sm_scale=None, smooth_k=True, pv_mode=None,
             BLKQ=128, BLKK=64, return_lse=False, qk_quant_dtype="int8", quant_recipe=None, attn_mask=None,
             cu_seqlens_q=None, cu_seqlens_k=None, max_seqlen_q=None, max_seqlen_k=None, q_interleave=1,
             k_interleave=1, **kwargs):
    """Quantise + attend in one call: out = softmax(q k^T * sm_scale [causal | + attn_mask]) v.

    Returns ``out`` (q's shape and dtype), or ``(out, lse)`` with ``return_lse=True`` where lse is
    the natural-log log-sum-exp of ``sm_scale * q k^T (+ mask)`` for the ORIGINAL k: what K smoothing
    removes from the logits is added back (checked as in test_sage_attention_mate.py:171-178).
    ``attn_mask``: boolean (True keeps) or additive in natural-log units, broadcastable to
    [B, Hq, Sq, Skv]; not combinable with ``is_causal``.
    ``quant_recipe`` (the keyword of sage_attention_benchmark_compare.py:300-313): (Q rows, K rows, -1, 1) sets the
    scale blocks and selects per-channel FP8 V, e.g. the external recipe (128, 16, -1, 1); without it ``BLKQ`` /
    ``BLKK`` / ``pv_mode`` ("fp16" by default) apply.
    ``cu_seqlens_q`` / ``cu_seqlens_k`` (int32 [nseq+1] on the device) switch to packed variable-length batches:
    q is then [total_q, Hq, D], k and v [total_k, Hkv, D], ``tensor_layout`` is not consulted, ``max_seqlen_q`` /
    ``max_seqlen_k`` bound the sequence lengths (derived from cu_seqlens, with one host synchronisation, when left
    out), and lse comes back as [Hq, total_q]; see sageattn_varlen, which this call is then identical to.
    ``q_interleave=8`` / ``k_interleave=4``: eight interleaved Q scales / four interleaved K scales per block (see
    per_block_int8); fixed-length batches only.
    """
    if qk_quant_dtype != "int8":
        raise NotImplementedError("only INT8 Q/K quantisation is implemented")
    if kwargs:
        raise TypeError(f"unexpected arguments: {sorted(kwargs)}")
    BLKQ, BLKK, pv_mode = _apply_recipe(quant_recipe, BLKQ, BLKK, pv_mode)
    qflag = _check_interleave(q_interleave)
    kflag = _check_k_interleave(k_interleave, BLKK)
    if cu_seqlens_q is not None or cu_seqlens_k is not None:
        if qflag or kflag:
            raise NotImplementedError("interleaved scales are not supported for packed batches")
        if attn_mask is not None:
            raise NotImplementedError("attn_mask is not supported for packed batches")
        cu_seqlens_k = cu_seqlens_q if cu_seqlens_k is None else cu_seqlens_k
        cu_seqlens_q = cu_seqlens_k if cu_seqlens_q is None else cu_seqlens_q
        _check_cu("cu_seqlens_q", cu_seqlens_q, q.device)
        _check_cu("cu_seqlens_k", cu_seqlens_k, q.device)
        if max_seqlen_q is None:
            max_seqlen_q = int((cu_seqlens_q[1:] - cu_seqlens_q[:-1]).max().item())
        if max_seqlen_k is None:
            max_seqlen_k = int((cu_seqlens_k[1:] - cu_seqlens_k[:-1]).max().item())
        return sageattn_varlen(q, k, v, cu_seqlens_q, cu_seqlens_k, max_seqlen_q, max_seqlen_k, is_causal=is_causal,
                               sm_scale=sm_scale, smooth_k=smooth_k, pv_mode=pv_mode, BLKQ=BLKQ, BLKK=BLKK,
                               return_lse=return_lse)
    if max_seqlen_q is not None or max_seqlen_k is not None:
        raise ValueError("max_seqlen_q / max_seqlen_k only apply together with cu_seqlens_q / cu_seqlens_k")
    for name, t in (("q", q), ("k", k), ("v", v)):
        _check_float(name, t)
    if not (q.dtype == k.dtype == v.dtype) or not (q.device == k.device == v.device):
        raise ValueError("q, k and v must have the same dtype and device")
    B, Hq, Sq, D, qsb, qsh, qsn = _layout(q, tensor_layout)
    Bk, Hkv, Skv, Dk, ksb, ksh, ksn = _layout(k, tensor_layout)
    Bv, Hv, Sv, Dv, vsb, vsh, vsn = _layout(v, tensor_layout)
    if Dk != D or Dv != D or Sv != Skv or Hv != Hkv or Bk != B or Bv != B:
        raise ValueError("incompatible q/k/v shapes")
    if Hq % Hkv:
        raise ValueError("query heads must be divisible by KV heads")
    if D not in (64, 128):
        raise NotImplementedError("head_dim must be 64 or 128")
    if BLKQ not in (16, 32, 64, 128) or BLKK not in (16, 32, 64, 128):
        raise NotImplementedError("the attention kernel needs Q and K scale blocks of 16, 32, 64 or 128 rows")
    pv = _pv(pv_mode)
    out = torch.empty(q.shape, device=q.device, dtype=q.dtype)
    _, _, _, _, osb, osh, osn = _layout(out, tensor_layout)
    lse = torch.empty((B, Hq, Sq), device=q.device, dtype=torch.float32) if return_lse else None
    ws_bytes = lib().sage_sageattn_workspace_bytes_for(B, Hq, Hkv, Sq, Skv, D, BLKQ | qflag, BLKK | kflag, pv, 0, 0, 0,
                                                       int(bool(smooth_k)), int(bool(return_lse)), int(attn_mask is not None))
    ws = torch.empty(max(ws_bytes, 256), device=q.device, dtype=torch.uint8)
    if attn_mask is not None:
        if is_causal:
            raise NotImplementedError("attn_mask cannot be combined with is_causal")
        m, kind, ms = _mask_args(attn_mask, B, Hq, Sq, Skv, q.device)
        check(lib().sage_sageattn_masked(_ptr(q), _ptr(k), _ptr(v), _ptr(out), _ptr(lse), _ptr(ws), ws_bytes,
                                         B, Hq, Hkv, Sq, Skv, D, qsb, qsh, qsn, ksb, ksh, ksn, vsb, vsh, vsn, osb, osh, osn,
                                         _dt(q.dtype), BLKQ | qflag, BLKK | kflag, float(D ** -0.5 if sm_scale is None else sm_scale),
                                         0, int(bool(smooth_k)), pv, None, None, 0, 0,
                                         _ptr(m), kind, ms[0], ms[1], ms[2], ms[3], _stream(q)))
    else:
        check(lib().sage_sageattn(_ptr(q), _ptr(k), _ptr(v), _ptr(out), _ptr(lse), _ptr(ws), ws_bytes,
                                  B, Hq, Hkv, Sq, Skv, D, qsb, qsh, qsn, ksb, ksh, ksn, vsb, vsh, vsn, osb, osh, osn,
                                  _dt(q.dtype), BLKQ | qflag, BLKK | kflag, float(D ** -0.5 if sm_scale is None else sm_scale),
                                  int(bool(is_causal)), int(bool(smooth_k)), pv, None, None, 0, 0, _stream(q)))
    if return_lse:
        return out, lse * 0.6931471805599453
    return out


# ------------------------------------------------------------------------------------------------
# packed variable-length batches
# ------------------------------------------------------------------------------------------------
def _check_packed(name, x):
    if not isinstance(x, torch.Tensor) or not x.is_cuda or x.dtype not in (torch.float16, torch.bfloat16):
        raise TypeError(f"{name} must be a GPU FP16/BF16 tensor")
    if x.ndim != 3 or not x.is_contiguous():
        raise ValueError(f"{name} must be contiguous [total_tokens, heads, head_dim]")


def _check_cu(name, cu, device):
    if not isinstance(cu, torch.Tensor) or cu.dtype != torch.int32 or cu.ndim != 1 or cu.numel() < 2:
        raise TypeError(f"{name} must be a 1-D int32 tensor of length nseq+1")
    if cu.device != device:
        raise ValueError(f"{name} must be on the same device as q")


@torch.no_grad()
def sageattn_varlen(q, k, v, cu_seqlens_q, cu_seqlens_k, max_seqlen_q, max_seqlen_k, is_causal=False, sm_scale=None,
                    smooth_k=True, pv_mode="fp16", BLKQ=128, BLKK=64, return_lse=False):
    """Packed variable-length attention: q [Tq, Hq, D], k/v [Tk, Hkv, D], cu_seqlens int32 [nseq+1]
    on the device.  Quantisation blocks and the K mean restart at every sequence; the (sequence,
    q-tile) work list is built and cost-ordered on the device, so no host synchronisation happens.
    With ``return_lse=True`` returns ``(out, lse)``, lse [Hq, Tq] float32: the natural-log log-sum-exp of
    ``sm_scale * q k^T`` (causal-masked if asked) of every packed row over its own sequence, for the original k
    (what K smoothing removes is added back) -- the quantity a split-KV or ring merge needs."""
    for name, t in (("q", q), ("k", k), ("v", v)):
        _check_packed(name, t)
    _check_cu("cu_seqlens_q", cu_seqlens_q, q.device)
    _check_cu("cu_seqlens_k", cu_seqlens_k, q.device)
    if cu_seqlens_q.numel() != cu_seqlens_k.numel():
        raise ValueError("cu_seqlens_q and cu_seqlens_k must describe the same number of sequences")
    if not (q.dtype == k.dtype == v.dtype) or not (q.device == k.device == v.device):
        raise ValueError("q, k and v must have the same dtype and device")
    Tq, Hq, D = q.shape
    Tk, Hkv, Dk = k.shape
    if Dk != D or tuple(v.shape) != tuple(k.shape):
        raise ValueError("incompatible q/k/v shapes")
    if Hq % Hkv:
        raise ValueError("query heads must be divisible by KV heads")
    if D not in (64, 128):
        raise NotImplementedError("head_dim must be 64 or 128")
    if BLKQ not in (16, 32, 64, 128) or BLKK not in (16, 32, 64, 128):
        raise NotImplementedError("the attention kernel needs Q and K scale blocks of 16, 32, 64 or 128 rows")
    nseq = cu_seqlens_q.numel() - 1
    pv = _pv(pv_mode)
    out = torch.empty_like(q)
    lse = torch.empty((Hq, Tq), device=q.device, dtype=torch.float32) if return_lse else None
    ws_bytes = lib().sage_sageattn_workspace_bytes_for(nseq, Hq, Hkv, int(max_seqlen_q), int(max_seqlen_k), D, BLKQ, BLKK, pv,
                                                       Tq, Tk, 1, int(bool(smooth_k)), int(bool(return_lse)), 0)
    ws = torch.empty(max(ws_bytes, 256), device=q.device, dtype=torch.uint8)
    check(lib().sage_sageattn(_ptr(q), _ptr(k), _ptr(v), _ptr(out), _ptr(lse), _ptr(ws), ws_bytes,
                              nseq, Hq, Hkv, int(max_seqlen_q), int(max_seqlen_k), D,
                              0, q.stride(1), q.stride(0), 0, k.stride(1), k.stride(0), 0, v.stride(1), v.stride(0),
                              0, out.stride(1), out.stride(0),
                              _dt(q.dtype), BLKQ, BLKK, float(D ** -0.5 if sm_scale is None else sm_scale),
                              int(bool(is_causal)), int(bool(smooth_k)), pv,
                              _ptr(cu_seqlens_q), _ptr(cu_seqlens_k), Tq, Tk, _stream(q)))
    if return_lse:
        return out, lse * 0.6931471805599453
    return out


@torch.no_grad()
def varlen_plan(cu_seqlens_q, cu_seqlens_k, total_q, BLKQ=128, BLKK=64, is_causal=False):
    """Runs the device-side scheduler and returns its raw int32 buffer plus the offsets of
    (cu_qblk, cu_kblk, cu_panel, tile_count, tiles) inside it."""
    _check_cu("cu_seqlens_q", cu_seqlens_q, cu_seqlens_q.device)
    nseq = cu_seqlens_q.numel() - 1
    n = lib().sage_varlen_plan_ints(nseq, int(total_q))
    plan = torch.zeros(n, device=cu_seqlens_q.device, dtype=torch.int32)
    offs = (ctypes.c_int64 * 5)()
    lib().sage_varlen_plan_offsets(nseq, int(total_q), offs)
    check(lib().sage_varlen_plan(_ptr(cu_seqlens_q), _ptr(cu_seqlens_k), nseq, int(total_q), BLKQ, BLKK,
                                 int(bool(is_causal)), _ptr(plan), n, _stream(plan)))
    return plan, [int(x) for x in offs]


@torch.no_grad()
def per_block_int8_varlen(q, k, cu_seqlens_q, cu_seqlens_k, max_seqlen_q, max_seqlen_k, km=None, BLKQ=128, BLKK=64,
                          sm_scale=None):
    """Packed per-block INT8 quantiser: blocks restart at each sequence.  Returns
    (q_int8, q_scale [Hq, nblk_bound], k_int8, k_scale [Hkv, nblk_bound], plan, plan_offsets); sequence i's
    blocks start at plan[offs[0] + i] (Q) / plan[offs[1] + i] (K).  ``km`` is [nseq, Hkv, D] or None."""
    _check_packed("q", q)
    _check_packed("k", k)
    _check_blocks_quant(BLKQ, BLKK)
    Tq, Hq, D = q.shape
    Tk, Hkv, _ = k.shape
    nseq = cu_seqlens_q.numel() - 1
    plan, offs = varlen_plan(cu_seqlens_q, cu_seqlens_k, Tq, BLKQ, BLKK)
    qi = torch.empty(q.shape, device=q.device, dtype=torch.int8)
    ki = torch.empty(k.shape, device=k.device, dtype=torch.int8)
    qs_sh, ks_sh = Tq // BLKQ + nseq, Tk // BLKK + nseq
    qs = torch.zeros((Hq, qs_sh), device=q.device, dtype=torch.float32)
    ks = torch.zeros((Hkv, ks_sh), device=q.device, dtype=torch.float32)
    esz = 4
    cu_qblk = ctypes.c_void_p(plan.data_ptr() + offs[0] * esz)
    cu_kblk = ctypes.c_void_p(plan.data_ptr() + offs[1] * esz)
    check(lib().sage_quant_int8(_ptr(q), _ptr(qi), _ptr(qs), None, nseq, Hq, int(max_seqlen_q), D,
                                0, q.stride(1), q.stride(0), 0, qi.stride(1), qi.stride(0), 0, 0,
                                BLKQ, _q_mult(D, sm_scale), _dt(q.dtype), _ptr(cu_seqlens_q), cu_qblk, qs_sh, _stream(q)))
    km_sb = km_sh = 0
    if km is not None:
        km = km.contiguous()
        km_sb, km_sh = km.stride(0), km.stride(1)
    check(lib().sage_quant_int8(_ptr(k), _ptr(ki), _ptr(ks), _ptr(km), nseq, Hkv, int(max_seqlen_k), D,
                                0, k.stride(1), k.stride(0), 0, ki.stride(1), ki.stride(0), km_sb, km_sh,
                                BLKK, 1.0, _dt(k.dtype), _ptr(cu_seqlens_k), cu_kblk, ks_sh, _stream(k)))
    return qi, qs, ki, ks, plan, offs
