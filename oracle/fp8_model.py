"""Arithmetic model of the FP8 P.V attention kernel (test infrastructure only; nothing in the package imports it).

``oracle.attention.sage_reference`` is the reference's formula (exact softmax, unquantised V).  The FP8 P.V path is
not in the reference (parity unpinned there): its result differs from that formula by the quantisation of P and V
to e4m3, which a cosine >= 0.999 gate bounds only loosely.  This file restates what the HIP kernel computes, step
by step and in the kernel's own number formats, so that GPU tests can hold the kernel to the rounding of its
output type instead:

  * V and its per-channel scales as ``oracle.quant.quant_v_fp8`` produces them (the GPU bytes are bit-equal);
  * scores from the INT32 dot products through the kernel's fp32 FMAs (accumulators biased by 1.5 * 2^23);
  * key tiles of 128 and query groups of 32 rows (one wavefront): the reference maximum of a row only moves when
    some row of its group grew by more than tau = 3 over it (lazy rescale), then o and the row sum are scaled by
    exp2(old - new);
  * P = 2^5 * exp2(s - m) rounded to e4m3 (round to nearest even) -- or, for the kernels that need no LSE and no
    explicit mask, the block-scaled "linear-mantissa" code: the keys of a 128-key tile form one block per query row with
    the exponent e = max(ceil(row maximum of the tile - m), -110); the code is 8 * t + 56 - 0.3, t = s - m - e + 8.75,
    rounded to nearest (as the high byte of a 16-bit conversion of (256 * code + 127.5) / 65535) and read as an e4m3
    byte, and the matrix pipe multiplies the block by 2^(e - 8) (its E8M0 scale operand).  There the reference maximum
    moves when a row's tile maximum exceeds it by more than 20;
  * O = sum P8 * V8 and the denominator sum P8 (of the very same rounded values), fp32 accumulation on the GPU,
    float64 here; out = O / den * v_scale;  LSE2 = m + log2(sum of the unrounded p) - 5.

Pinned in tests/test_oracle_fp8_model.py: against brute-force Python loops on tiny shapes, and against
``sage_reference`` on the fp8-dequantised V within the error that rounding P to 3 mantissa bits allows.
"""
from __future__ import annotations

import numpy as np
import torch

from . import quant as oq

BIAS = np.float32(12582912.0)      # 1.5 * 2^23: the INT32 accumulators start from its bit pattern
PSHIFT = np.float32(5.0)
TAU = np.float32(3.0)
CODE_BIAS = np.float32(-0.3)
BLOCK_TOP = np.float32(8.75)       # the block maximum is coded within one binade below 2^8.75 (code <= 126 = 448)
BLOCK_TAU = np.float32(20.0)
BLOCK_MIN_EXP = np.float32(-110.0)
BLOCK_SCALE_BIAS = 119             # E8M0 byte of a block = 119 + e: the matrix pipe applies 2^(e - 8)
M_INIT = np.float32(-1.0e30)
KN = np.float32(256.0) / np.float32(65535.0)                      # code units -> units of the 16-bit conversion
KN8 = np.float32(8.0) * KN
KC = np.float32(np.float32(KN * np.float32(np.float32(56.0) + CODE_BIAS)) + np.float32(127.5) / np.float32(65535.0))
TILE = 128                         # keys per tile
GROUP = 32                         # query rows per wavefront


def _fma32(a, b, c):
    """fp32 fused multiply-add: the product of two fp32 values is exact in float64; one rounding to fp32."""
    return (np.asarray(a, np.float64) * np.asarray(b, np.float64) + np.asarray(c, np.float64)).astype(np.float32)


def decode_e4m3(code: np.ndarray) -> np.ndarray:
    """Value of an e4m3fn byte with the sign bit clear: 8 * (exponent + 7) + mantissa."""
    code = code.astype(np.int64)
    e, m = code >> 3, code & 7
    return np.where(e == 0, m * 2.0 ** -9, np.exp2((e - 7).astype(np.float64)) * (1.0 + m / 8.0))


def linear_code_of(acc: np.ndarray, sc: np.ndarray, k0b: np.ndarray) -> np.ndarray:
    """The kernel's linear-mantissa code of 2^t: y = 8 * t + 56 + CODE_BIAS rounded to nearest, computed the kernel's way
    (baselinebenchmark_amd/csrc/sage_attn_kernel.h, softmax): fp32 FMAs deliver x = (256 * y + 127.5) / 65535, the 16-bit
    conversion gives rne(65535 * x) saturated to [0, 65535], and the code is its high byte.  acc [R, N] biased fp32
    accumulators, sc [R, N] fp32 scale products, k0b [R] the per-row constant of the tile (block_constants)."""
    mul = (KN8 * sc).astype(np.float32)
    c = _fma32(-BIAS, mul, k0b[:, None])
    with np.errstate(invalid="ignore"):
        x = _fma32(acc, mul, c)
        u16 = np.rint(np.clip(x.astype(np.float64), 0.0, 1.0) * 65535.0)
    return np.where(np.isnan(u16), 0.0, np.floor(u16 / 256.0))


def block_constants(bmax: np.ndarray, m_used: np.ndarray):
    """Per row: the block exponent e = max(ceil(bmax - m), -110) and the fma constant of the code, both in fp32 as the
    kernel computes them.  bmax [R] fp32 maxima of the row's scores in the tile (-inf without visible keys), m_used [R]."""
    with np.errstate(invalid="ignore"):
        d = (bmax - m_used).astype(np.float32)
        e = np.maximum(np.ceil(d), BLOCK_MIN_EXP).astype(np.float32)
    k0 = _fma32(KN8, (BLOCK_TOP - m_used).astype(np.float32), KC)
    return e, _fma32(-KN8, e, k0)


def _rne_e4m3(p32: np.ndarray) -> np.ndarray:
    """fp32 -> e4m3fn (round to nearest even) -> float64 value, through torch's CPU cast."""
    t = torch.from_numpy(np.ascontiguousarray(p32, dtype=np.float32)).to(torch.float8_e4m3fn).to(torch.float32)
    return t.numpy().astype(np.float64)


def fp8_attention_model(q_int8, k_int8, v, q_scale, k_scale, tensor_layout="HND", BLKQ=128, BLKK=64, is_causal=False,
                        attn_mask=None, mask_mult=1.0, linear_code=None, want_lse=False, row_offset=0):
    """Returns (out float64 [layout of q], lse2 float64 [B,Hq,Sq] or None).

    ``row_offset``: q_int8 / q_scale hold the query rows row_offset, row_offset + 1, ... of a longer problem (a multiple
    of 32 and of BLKQ, so that wavefront groups and scale blocks keep their places); it only moves the causal diagonal.

    ``linear_code``: None picks what the library picks (the linear-mantissa code when neither a mask nor LSE is
    asked for, exact exp2 + e4m3 rounding otherwise).  ``attn_mask``: bool (True keeps) or additive, already
    expanded to [B,Hq,Sq,Skv]; the additive mask is multiplied by ``mask_mult`` in fp32 as the kernel does.
    """
    hnd = (lambda x: x) if tensor_layout == "HND" else (lambda x: x.transpose(1, 2))
    qi = hnd(q_int8).cpu().numpy().astype(np.float64)
    ki = hnd(k_int8).cpu().numpy().astype(np.float64)
    v8, vsc = oq.quant_v_fp8(v.cpu(), tensor_layout)
    v8 = hnd(v8.to(torch.float32)).numpy().astype(np.float64)
    vsc = vsc.numpy().astype(np.float32)
    qs = q_scale.cpu().numpy().astype(np.float32)
    ks = k_scale.cpu().numpy().astype(np.float32)
    B, Hq, Sq, D = qi.shape
    Hkv, Skv = ki.shape[1], ki.shape[2]
    G = Hq // Hkv
    masked = attn_mask is not None
    if linear_code is None:
        linear_code = not masked and not want_lse
    if masked:
        assert not is_causal and not linear_code
        mask = attn_mask.cpu().numpy()
    out = np.zeros((B, Hq, Sq, D), np.float64)
    lse = np.full((B, Hq, Sq), -np.inf, np.float64)
    rows = np.arange(Sq)
    assert row_offset % GROUP == 0 and row_offset % BLKQ == 0
    rows_abs = rows + row_offset
    ngroups = (Sq + GROUP - 1) // GROUP
    gidx = rows // GROUP
    for b in range(B):
        for hq in range(Hq):
            hk = hq // G
            qrow_scale = qs[b, hq][rows // BLKQ]                                   # [Sq] fp32
            m_used = np.full(Sq, M_INIT, np.float32)
            o = np.zeros((Sq, D), np.float64)
            den = np.zeros(Sq, np.float64)
            lsum = np.zeros(Sq, np.float64)
            for n0 in range(0, Skv, TILE):
                if is_causal and n0 > rows_abs[-1]:
                    break                                    # tiles above the diagonal: skipped, as in the kernel
                n1 = min(n0 + TILE, Skv)
                keys = np.arange(n0, n1)
                sc = (qrow_scale[:, None] * ks[b, hk][keys // BLKK][None, :]).astype(np.float32)   # fp32 product
                acc = (BIAS.astype(np.float64) + qi[b, hq] @ ki[b, hk, n0:n1].T).astype(np.float32)   # exact: |dot| < 2^22
                dead = np.zeros((Sq, n1 - n0), bool)
                if is_causal:
                    dead |= keys[None, :] > rows_abs[:, None]
                if masked:
                    sv = ((acc - BIAS).astype(np.float32) * sc).astype(np.float32)   # bias off first (exact), one rounding
                    mk = mask[b, hq][:, n0:n1]
                    if mk.dtype == np.bool_:
                        dead |= ~mk
                    else:
                        with np.errstate(invalid="ignore"):
                            sv = _fma32(mk.astype(np.float32), np.float32(mask_mult), sv)
                    sv = np.where(dead, -np.inf, sv).astype(np.float32)
                    mloc = sv.max(axis=1)
                else:
                    score = _fma32(acc, sc, (-BIAS * sc).astype(np.float32))
                    mloc = np.where(dead, -np.inf, score).max(axis=1).astype(np.float32)
                # lazy rescale, decided per group of 32 rows
                grew = mloc > (m_used + (BLOCK_TAU if linear_code else TAU)).astype(np.float32)
                trig = np.zeros(ngroups, bool)
                np.logical_or.at(trig, gidx, grew)
                upd = trig[gidx]
                m_new = np.where(upd, np.maximum(m_used, mloc), m_used).astype(np.float32)
                alpha = np.exp2((m_used - m_new).astype(np.float32).astype(np.float64))
                o *= alpha[:, None]
                den *= alpha
                lsum *= alpha
                m_used = m_new
                base = (PSHIFT - m_used).astype(np.float32)                       # [Sq]
                if linear_code:
                    e, k0b = block_constants(mloc, m_used)
                    code = linear_code_of(acc, sc, k0b)
                    code = np.where(dead, 0, code)
                    p8 = decode_e4m3(code) * np.exp2(e.astype(np.float64) - 8.0)[:, None]
                else:
                    if masked:
                        with np.errstate(invalid="ignore"):
                            t = (sv + base[:, None]).astype(np.float32)
                    else:
                        c = _fma32(-BIAS, sc, base[:, None])
                        t = _fma32(acc, sc, c)
                    t = np.where(dead, -np.inf, t).astype(np.float32)
                    p = np.exp2(t.astype(np.float64)).astype(np.float32)
                    lsum += p.astype(np.float64).sum(axis=1)
                    p8 = _rne_e4m3(p)
                o += p8 @ v8[b, hk, n0:n1]
                den += p8.sum(axis=1)
            live = den > 0
            inv = np.where(live, 1.0 / np.where(live, den, 1.0), 0.0)
            out[b, hq] = o * inv[:, None] * vsc[b, hk][None, :].astype(np.float64)
            if want_lse:
                with np.errstate(divide="ignore"):
                    lse[b, hq] = np.where(lsum > 0, m_used.astype(np.float64) + np.log2(np.where(lsum > 0, lsum, 1.0)) - 5.0, -np.inf)
    o_t = torch.from_numpy(out)
    o_t = o_t.transpose(1, 2).contiguous() if tensor_layout == "NHD" else o_t
    return o_t, (torch.from_numpy(lse) if want_lse else None)
