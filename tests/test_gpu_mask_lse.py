"""GPU parity of the explicit-mask variants of the attention kernel and of the LSE that the one-call
pipeline returns, through the C ABI.

Reference behaviour followed:
  * forward(..., attn_mask=bool | additive) and the LSE2 output: sageattention_triton.py:92-105, :127-129,
    checked as test_sageattention_hip.py:40-58 does (mask[..., ::3] = False / -2.0; relative RMSE < 3e-2,
    |LSE2 error| < 3e-2) on its shapes (129 x 70, 4 query heads, 2 KV heads, D = 128).
  * sageattn(..., attn_mask=, smooth_k=True, return_lse=True): test_sage_attention_mate.py:186-208, :467-492
    against softmax(sm_scale * q k^T + mask) and its natural-log logsumexp (:171-178) with
    atol 1.5e-1 / rtol 3e-2 on the LSE (:347-353).
"""
import math

import pytest
import torch

import baselinebenchmark_amd as sa
from oracle import attention as oa
from tests.helpers import randn

pytestmark = [pytest.mark.gpu, pytest.mark.sage_attention]
DEV = "cuda"


def _masks(kind, B, Hq, Sq, Skv, g):
    if kind == "bool_stride3":
        m = torch.ones((B, Hq, Sq, Skv), dtype=torch.bool)
        m[..., ::3] = False
    elif kind == "additive_stride3":
        m = torch.zeros((B, Hq, Sq, Skv))
        m[..., ::3] = -2.0
    elif kind == "bool_random":
        m = torch.rand((B, Hq, Sq, Skv), generator=g) > 0.4
        m[..., 0] = True      # no empty rows here
    elif kind == "additive_random":
        m = torch.randn((B, Hq, Sq, Skv), generator=g)
    elif kind == "additive_neg_inf":
        m = torch.zeros((B, Hq, Sq, Skv))
        m[torch.rand((B, Hq, Sq, Skv), generator=g) < 0.5] = -float("inf")
        m[..., 1] = 0.0
    else:
        raise AssertionError(kind)
    return m


@pytest.mark.parametrize("kind", ["bool_stride3", "additive_stride3", "bool_random", "additive_random", "additive_neg_inf"])
@pytest.mark.parametrize("pv", ["fp16", "fp8"])
@pytest.mark.parametrize("shape", [(1, 4, 2, 129, 70, 128), (2, 2, 1, 300, 391, 64)])
def test_forward_with_mask_matches_reference_formula(kind, pv, shape):
    B, Hq, Hkv, Sq, Skv, D = shape
    g = torch.Generator().manual_seed(2026 + D + Sq + Skv)
    q = randn("HND", B, Hq, Sq, D, torch.float16, g)
    k = randn("HND", B, Hkv, Skv, D, torch.float16, g)
    v = randn("HND", B, Hkv, Skv, D, torch.float16, g)
    mask = _masks(kind, B, Hq, Sq, Skv, g)
    qi, qs, ki, ks = sa.per_block_int8(q.to(DEV), k.to(DEV))
    out, lse = sa.forward(qi, ki, v.to(DEV), qs, ks, attn_mask=mask.to(DEV), return_lse=True, pv_mode=pv)
    torch.cuda.synchronize()
    ref, ref_lse = oa.sage_reference(qi.cpu(), ki.cpu(), v, qs.cpu(), ks.cpu(), "HND", 128, 64, attn_mask=mask)
    m = oa.metrics(out.cpu().float(), ref)
    assert m["finite"]
    if pv == "fp16":
        assert m["rel_rmse"] < 3e-2              # the reference's bound
        assert m["rel_rmse"] < 2e-3              # what this kernel achieves
        assert (lse.cpu().double() - ref_lse).abs().max().item() < 1e-3
    else:
        assert m["cosine"] >= 0.999 and m["rel_rmse"] < 5e-2
        assert (lse.cpu().double() - ref_lse).abs().max().item() < 3e-2


@pytest.mark.parametrize("kind", ["bool_random", "additive_random", "additive_neg_inf"])
@pytest.mark.parametrize("pv", ["fp16", "fp8"])
@pytest.mark.parametrize("gran", [(128, 16, 1), (32, 64, 4), (64, 128, 4), (16, 32, 4)])
@pytest.mark.parametrize("shape", [(1, 4, 2, 129, 70, 128), (2, 2, 1, 300, 391, 64)])
def test_forward_with_mask_and_fine_k_scales(kind, pv, gran, shape):
    """An explicit mask together with K scale blocks of 16 keys (the external (128, 16) recipe) and with four interleaved
    K scales per block: against the formula with the scales expanded key by key.  (No counterpart in the reference,
    whose forward has one K granularity: the masked kernels look the scale of every score up, so only the lookup
    changes.)"""
    B, Hq, Hkv, Sq, Skv, D = shape
    blkq, blkk, ki4 = gran
    g = torch.Generator().manual_seed(77 + D + Sq + blkk + ki4)
    q = randn("HND", B, Hq, Sq, D, torch.float16, g)
    k = randn("HND", B, Hkv, Skv, D, torch.float16, g, offset_std=1.0)
    # keys of very different magnitude inside a block, so that a wrong scale lookup shows
    k = k * (1.0 + 3.0 * (torch.arange(Skv) % 7 == 0).to(k.dtype))[None, None, :, None]
    v = randn("HND", B, Hkv, Skv, D, torch.float16, g)
    mask = _masks(kind, B, Hq, Sq, Skv, g)
    qi, qs, ki, ks = sa.per_block_int8(q.to(DEV), k.to(DEV), BLKQ=blkq, BLKK=blkk, k_interleave=ki4)
    out, lse = sa.forward(qi, ki, v.to(DEV), qs, ks, attn_mask=mask.to(DEV), return_lse=True, pv_mode=pv, BLKQ=blkq, BLKK=blkk,
                          k_interleave=ki4)
    torch.cuda.synchronize()
    ref, ref_lse = oa.sage_reference(qi.cpu(), ki.cpu(), v, qs.cpu(), ks.cpu(), "HND", blkq, blkk, attn_mask=mask, k_interleave=ki4)
    m = oa.metrics(out.cpu().float(), ref)
    assert m["finite"]
    if pv == "fp16":
        assert m["rel_rmse"] < 2e-3
        assert (lse.cpu().double() - ref_lse).abs().max().item() < 1e-3
    else:
        assert m["cosine"] >= 0.999 and m["rel_rmse"] < 5e-2
        assert (lse.cpu().double() - ref_lse).abs().max().item() < 3e-2
    # the one-call pipeline takes the same combination
    full = sa.sageattn(q.to(DEV), k.to(DEV), v.to(DEV), attn_mask=mask.to(DEV), pv_mode=pv, BLKQ=blkq, BLKK=blkk, k_interleave=ki4)
    torch.cuda.synchronize()
    logits = torch.einsum("bhqd,bhkd->bhqk", q.double(), k.double().repeat_interleave(Hq // Hkv, 1)) * D ** -0.5
    logits = logits.masked_fill(~mask, -float("inf")) if mask.dtype == torch.bool else logits + mask.double()
    exact = torch.softmax(logits, -1) @ v.double().repeat_interleave(Hq // Hkv, 1)
    assert oa.metrics(full.cpu().float(), exact)["cosine"] >= 0.999
    # ... and without K smoothing it is the two steps above, bit for bit: the granularity reaches the pipeline's quantiser
    # (boolean masks; an additive mask is in natural-log units there and in base-2 units for forward)
    if mask.dtype == torch.bool:
        plain = sa.sageattn(q.to(DEV), k.to(DEV), v.to(DEV), attn_mask=mask.to(DEV), pv_mode=pv, BLKQ=blkq, BLKK=blkk,
                            k_interleave=ki4, smooth_k=False)
        assert torch.equal(plain, out)


def test_mask_broadcasts_without_being_materialised_and_accepts_half_bias():
    g = torch.Generator().manual_seed(11)
    B, Hq, Hkv, Sq, Skv, D = 2, 4, 2, 200, 333, 64
    q = randn("NHD", B, Hq, Sq, D, torch.bfloat16, g)
    k = randn("NHD", B, Hkv, Skv, D, torch.bfloat16, g)
    v = randn("NHD", B, Hkv, Skv, D, torch.bfloat16, g)
    qi, qs, ki, ks = sa.per_block_int8(q.to(DEV), k.to(DEV), tensor_layout="NHD")
    key_padding = torch.ones((B, 1, 1, Skv), dtype=torch.bool)      # [B, 1, 1, Skv]: strides 0 for heads and rows
    key_padding[0, ..., 250:] = False
    key_padding[1, ..., 100:] = False
    out, _ = sa.forward(qi, ki, v.to(DEV), qs, ks, tensor_layout="NHD", attn_mask=key_padding.to(DEV),
                        output_dtype=torch.bfloat16)
    ref, _ = oa.sage_reference(qi.cpu(), ki.cpu(), v.to(torch.float16), qs.cpu(), ks.cpu(), "NHD", 128, 64,
                               attn_mask=key_padding.expand(B, Hq, Sq, Skv))
    assert oa.metrics(out.cpu().float(), ref)["rel_rmse"] < 1e-2    # bf16 output rounding
    rel_bias = (torch.randn((Sq, Skv), generator=g) * 0.5).to(torch.float16)   # [Sq, Skv] half-precision bias
    out2, _ = sa.forward(qi, ki, v.to(DEV), qs, ks, tensor_layout="NHD", attn_mask=rel_bias.to(DEV))
    ref2, _ = oa.sage_reference(qi.cpu(), ki.cpu(), v.to(torch.float16), qs.cpu(), ks.cpu(), "NHD", 128, 64,
                                attn_mask=rel_bias.float().expand(B, Hq, Sq, Skv))
    assert oa.metrics(out2.cpu().float(), ref2)["rel_rmse"] < 2e-3


def test_rows_without_any_visible_key_give_zero_output_and_minus_inf_lse():
    g = torch.Generator().manual_seed(12)
    q = randn("HND", 1, 2, 70, 64, torch.float16, g)
    k = randn("HND", 1, 2, 150, 64, torch.float16, g)
    v = randn("HND", 1, 2, 150, 64, torch.float16, g)
    mask = torch.ones((1, 2, 70, 150), dtype=torch.bool)
    mask[:, :, 5, :] = False
    mask[:, 1, 33, :] = False
    qi, qs, ki, ks = sa.per_block_int8(q.to(DEV), k.to(DEV))
    out, lse = sa.forward(qi, ki, v.to(DEV), qs, ks, attn_mask=mask.to(DEV), return_lse=True)
    out, lse = out.cpu().float(), lse.cpu()
    assert torch.isfinite(out).all()
    assert out[:, :, 5].abs().max() == 0 and out[:, 1, 33].abs().max() == 0
    assert torch.isinf(lse[:, :, 5]).all() and (lse[:, :, 5] < 0).all() and lse[0, 1, 33] == -float("inf")
    assert torch.isfinite(lse[:, 0, 33]).all()
    ref, _ = oa.sage_reference(qi.cpu(), ki.cpu(), v, qs.cpu(), ks.cpu(), "HND", 128, 64, attn_mask=mask)
    keep = torch.ones(70, dtype=torch.bool); keep[5] = False; keep[33] = False
    assert oa.metrics(out[:, :, keep], ref[:, :, keep])["rel_rmse"] < 2e-3


def test_mask_of_ones_equals_no_mask_bitwise():
    g = torch.Generator().manual_seed(13)
    q = randn("HND", 1, 2, 260, 128, torch.float16, g)
    k = randn("HND", 1, 2, 260, 128, torch.float16, g)
    v = randn("HND", 1, 2, 260, 128, torch.float16, g)
    qi, qs, ki, ks = sa.per_block_int8(q.to(DEV), k.to(DEV))
    a, la = sa.forward(qi, ki, v.to(DEV), qs, ks, return_lse=True)
    b, lb = sa.forward(qi, ki, v.to(DEV), qs, ks, return_lse=True,
                       attn_mask=torch.ones((1, 1, 260, 260), dtype=torch.bool, device=DEV))
    c, lc = sa.forward(qi, ki, v.to(DEV), qs, ks, return_lse=True, attn_mask=torch.zeros((260, 260), device=DEV))
    # the masked variants scale the scores before the maximum instead of after: same values up to fp32 rounding
    assert (a.float() - b.float()).abs().max().item() <= 2e-3 and (a.float() - c.float()).abs().max().item() <= 2e-3
    assert (la - lb).abs().max().item() < 1e-4 and (la - lc).abs().max().item() < 1e-4
    assert torch.equal(b, c) and torch.equal(lb, lc)


@pytest.mark.parametrize("mask_kind", [None, "bool", "additive"])
@pytest.mark.parametrize("pv", ["fp16", "fp8"])
def test_sageattn_lse_is_that_of_the_original_logits_with_k_smoothing(mask_kind, pv):
    # shapes and masks of test_sage_attention_mate.py:467-487, plus a K with a large per-channel offset so
    # that the smoothing correction (q . k_mean) is far larger than the tolerance
    torch.manual_seed(7)
    q = torch.randn((1, 2, 129, 128), dtype=torch.float16)
    k = torch.randn((1, 1, 70, 128), dtype=torch.float16) + (3.0 * torch.randn((1, 1, 1, 128))).to(torch.float16)
    v = torch.randn((1, 1, 70, 128), dtype=torch.float16)
    mask = None
    if mask_kind == "bool":
        mask = torch.ones((1, 2, 129, 70), dtype=torch.bool); mask[..., ::3] = False
    elif mask_kind == "additive":
        mask = torch.zeros((1, 2, 129, 70)); mask[..., ::3] = -2.0
    out, lse = sa.sageattn(q.to(DEV), k.to(DEV), v.to(DEV), smooth_k=True, return_lse=True, pv_mode=pv,
                           attn_mask=None if mask is None else mask.to(DEV))
    scores = torch.matmul(q.double(), k.double().repeat_interleave(2, dim=1).transpose(-1, -2)) * 128 ** -0.5
    if mask is not None:
        scores = scores.masked_fill(~mask, -float("inf")) if mask.dtype == torch.bool else scores + mask.double()
    ref = torch.matmul(torch.softmax(scores, dim=-1), v.double().repeat_interleave(2, dim=1))
    ref_lse = torch.logsumexp(scores, dim=-1)
    m = oa.metrics(out.cpu().float(), ref)
    assert m["cosine"] >= 0.999
    torch.testing.assert_close(lse.cpu().double(), ref_lse, atol=1.5e-1, rtol=3e-2)     # the reference's bound
    assert (lse.cpu().double() - ref_lse).abs().max().item() < 6e-2                     # measured: INT8 noise on the logits
    # without the correction the LSE is off by sm_scale * q . mean(k): make sure the test can see that
    km = k.double().mean(dim=2, keepdim=True).repeat_interleave(2, dim=1)
    shift = (torch.matmul(q.double(), km.transpose(-1, -2)) * 128 ** -0.5).abs().max().item()
    assert shift > 1.0


def test_sageattn_lse_correction_causal_gqa_nhd_bf16():
    g = torch.Generator().manual_seed(21)
    B, Hq, Hkv, S, D = 2, 8, 2, 700, 128
    q = randn("NHD", B, Hq, S, D, torch.bfloat16, g)
    k = (randn("NHD", B, Hkv, S, D, torch.bfloat16, g).float() + 2.0 * torch.randn((B, 1, Hkv, D), generator=g)).to(torch.bfloat16)
    v = randn("NHD", B, Hkv, S, D, torch.bfloat16, g)
    out, lse = sa.sageattn(q.to(DEV), k.to(DEV), v.to(DEV), tensor_layout="NHD", is_causal=True, return_lse=True,
                           pv_mode="fp8", BLKQ=64, BLKK=128)
    qh, kh = q.transpose(1, 2).double(), k.transpose(1, 2).double().repeat_interleave(Hq // Hkv, dim=1)
    scores = torch.matmul(qh, kh.transpose(-1, -2)) * D ** -0.5
    i = torch.arange(S)
    scores = scores.masked_fill(i[None, :] > i[:, None], -float("inf"))
    assert tuple(lse.shape) == (B, Hq, S)
    assert (lse.cpu().double() - torch.logsumexp(scores, dim=-1)).abs().max().item() < 1e-1
    ref = oa.sdpa_fp32(q, k, v, "NHD", True)
    assert oa.metrics(out.cpu().float(), ref)["cosine"] >= 0.999
