"""FP8 P.V kernels against the arithmetic model of oracle/fp8_model.py, through the C ABI.

The other FP8 tests compare with the exact-softmax formula on unquantised V at cosine >= 0.999 -- a bound on the
ALGORITHM (e4m3 P and V).  Here the kernel's own arithmetic is checked: same quantised V, same reference-maximum
walk (tiles of 128 keys, groups of 32 rows, lazy rescale), same fp8 code for P (block-scaled where the library uses
the linear-mantissa code), denominator from the rounded values.  What
is left between kernel and model is the fp32 accumulation order and the rounding of the output type, so the bound is
the output type's: relative RMSE < 6e-4 for fp16 outputs (half an ulp is 2.4e-4 worst case, 1.4e-4 rms) and < 2.5e-3
for bf16 outputs (1.1e-3 rms), |LSE2 error| < 2e-4.
"""
import random

import pytest
import torch

import baselinebenchmark_amd as sa
from oracle import attention as oa
from oracle import fp8_model as fm
from oracle import quant as oq
from tests.helpers import randn

pytestmark = [pytest.mark.gpu, pytest.mark.sage_attention]
DEV = "cuda"


def _bound(dtype):
    return 6e-4 if dtype == torch.float16 else 2.5e-3


def _check(out, model, dtype, what=""):
    m = oa.metrics(out.cpu().float(), model)
    assert m["finite"] and m["rel_rmse"] < _bound(dtype), (what, m)
    return m


@pytest.mark.parametrize("lse", [False, True], ids=["linear-code", "exact-exp2-lse"])
@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("cfg", [("HND", 1, 4, 2, 300, 900, 128, torch.float16, 64, 128),
                                 ("NHD", 2, 2, 2, 513, 513, 64, torch.bfloat16, 128, 64),
                                 ("HND", 1, 2, 1, 700, 2100, 128, torch.bfloat16, 32, 32),
                                 ("HND", 1, 2, 2, 257, 640, 128, torch.float16, 128, 16)])
def test_forward_fp8_matches_the_model(cfg, causal, lse):
    layout, B, Hq, Hkv, Sq, Skv, D, dtype, blkq, blkk = cfg
    g = torch.Generator().manual_seed(hash((Sq, Skv, D)) % (1 << 30))
    q = randn(layout, B, Hq, Sq, D, dtype, g)
    k = randn(layout, B, Hkv, Skv, D, dtype, g)
    v = randn(layout, B, Hkv, Skv, D, dtype, g)
    qi, qs, ki, ks = sa.per_block_int8(q.to(DEV), k.to(DEV), BLKQ=blkq, BLKK=blkk, tensor_layout=layout)
    out, l2 = sa.forward(qi, ki, v.to(DEV), qs, ks, tensor_layout=layout, output_dtype=dtype, return_lse=lse, BLKQ=blkq,
                         BLKK=blkk, is_causal=causal, pv_mode="fp8")
    model, ml = fm.fp8_attention_model(qi.cpu(), ki.cpu(), v, qs.cpu(), ks.cpu(), layout, blkq, blkk, is_causal=causal,
                                       want_lse=lse)
    _check(out, model, dtype, cfg)
    if lse:
        assert (l2.cpu().double() - ml).abs().max().item() < 2e-4


@pytest.mark.parametrize("kind", ["bool", "additive"])
def test_masked_fp8_matches_the_model(kind):
    B, Hq, Hkv, Sq, Skv, D = 2, 4, 2, 200, 391, 128
    g = torch.Generator().manual_seed(99)
    q = randn("HND", B, Hq, Sq, D, torch.float16, g)
    k = randn("HND", B, Hkv, Skv, D, torch.float16, g)
    v = randn("HND", B, Hkv, Skv, D, torch.float16, g)
    mask = torch.rand((B, Hq, Sq, Skv), generator=g) < 0.7 if kind == "bool" else torch.randn((B, Hq, Sq, Skv), generator=g) * 2
    qi, qs, ki, ks = sa.per_block_int8(q.to(DEV), k.to(DEV))
    out, l2 = sa.forward(qi, ki, v.to(DEV), qs, ks, attn_mask=mask.to(DEV), return_lse=True, pv_mode="fp8")
    model, ml = fm.fp8_attention_model(qi.cpu(), ki.cpu(), v, qs.cpu(), ks.cpu(), "HND", 128, 64, attn_mask=mask, want_lse=True)
    _check(out, model, torch.float16, kind)
    assert (l2.cpu().double() - ml).abs().max().item() < 2e-4


def test_single_query_row_with_an_additive_mask():
    """The case a random sweep once scored at cosine 0.99894 against the exact-softmax formula on unquantised V:
    D=128 fp16, one query row, 259 keys, two query heads on one KV head, scale blocks 32/128, additive mask of shape
    (1, 259), FP8 P.V, no LSE.  Two output rows make the cosine against the unquantised formula a noisy statistic (it
    measures the e4m3 rounding of V and P on 2 x 128 numbers); against the model the kernel has to agree to the
    rounding of its output, and numerator and denominator must see the same rounded probabilities."""
    g = torch.Generator().manual_seed(1234)
    for trial in range(8):
        q = randn("HND", 1, 2, 1, 128, torch.float16, g)
        k = randn("HND", 1, 1, 259, 128, torch.float16, g)
        v = randn("HND", 1, 1, 259, 128, torch.float16, g)
        mask = torch.randn((1, 259), generator=g) * 2.0
        qi, qs, ki, ks = sa.per_block_int8(q.to(DEV), k.to(DEV), BLKQ=32, BLKK=128)
        out, _ = sa.forward(qi, ki, v.to(DEV), qs, ks, attn_mask=mask.to(DEV), BLKQ=32, BLKK=128, pv_mode="fp8")
        full = mask.expand(1, 2, 1, 259)
        model, _ = fm.fp8_attention_model(qi.cpu(), ki.cpu(), v, qs.cpu(), ks.cpu(), "HND", 32, 128, attn_mask=full)
        _check(out, model, torch.float16, trial)
        # a constant V row must come back exactly (to output rounding): the denominator is the sum of the rounded P
        vc = v[:, :, :1].expand(-1, -1, 259, -1).contiguous()
        outc, _ = sa.forward(qi, ki, vc.to(DEV), qs, ks, attn_mask=mask.to(DEV), BLKQ=32, BLKK=128, pv_mode="fp8")
        v8, vsc = oq.quant_v_fp8(vc)
        want = (v8.double() * vsc.double()[:, :, None, :])[:, :, :1].expand(1, 2, 1, 128)
        assert torch.allclose(outc.cpu().double(), want, rtol=2 ** -10, atol=1e-6), trial


@pytest.mark.parametrize("binades", [9.5, 11.5, 12.5, 13.5, 15.5, 30.0])
@pytest.mark.parametrize("lse", [False, True], ids=["linear-code", "exact-exp2-lse"])
def test_one_large_key_above_a_flat_tail(binades, lse):
    """An attention sink over a flat tail: key 0 lies `binades` above 8191 equal keys, which together carry most of the
    softmax mass.  Gated on the relative RMSE against the exact-softmax formula (a cosine hardly notices a lost tail).  The
    block-scaled linear code keeps three mantissa bits at any distance; the exact-exponential kernels (LSE wanted) code P
    against the row maximum and lose the tail where e4m3's 18 binades end, which is stated here as their bound."""
    S, D, Sq = 8192, 64, 32
    qi = torch.zeros(1, 1, Sq, D, dtype=torch.int8)
    qi[..., 0] = 100
    ki = torch.zeros(1, 1, S, D, dtype=torch.int8)
    ki[0, 0, 0, 0] = 100
    qs, ks = torch.full((1, 1, 1), binades / 10000.0), torch.ones(1, 1, S // 64)
    v = torch.randn(1, 1, S, D, generator=torch.Generator().manual_seed(3)).to(torch.float16)
    out, _ = sa.forward(qi.to(DEV), ki.to(DEV), v.to(DEV), qs.to(DEV), ks.to(DEV), return_lse=lse, pv_mode="fp8")
    v8, vsc = oq.quant_v_fp8(v)
    ref, _ = oa.sage_reference(qi, ki, v8, qs, ks, "HND", 128, 64, v_scale=vsc)
    model, _ = fm.fp8_attention_model(qi, ki, v, qs, ks, "HND", 128, 64, want_lse=lse)
    _check(out, model, torch.float16, (binades, lse))
    err = oa.metrics(out.cpu().float(), ref)["rel_rmse"]
    if not lse:
        assert err < 0.02, err
    else:
        assert err < (0.06 if binades <= 12.5 else 0.2 if binades <= 15.5 else 1.01), err


def test_one_call_pipeline_fp8_matches_the_model():
    """sageattn (K smoothing, quantisers, fused-Q attention kernel) against oracle quantisers + model."""
    g = torch.Generator().manual_seed(4321)
    B, Hq, Hkv, S, D = 1, 4, 2, 1000, 128
    q = randn("HND", B, Hq, S, D, torch.bfloat16, g)
    k = randn("HND", B, Hkv, S, D, torch.bfloat16, g, offset_std=2.0)
    v = randn("HND", B, Hkv, S, D, torch.bfloat16, g)
    for causal in (False, True):
        out = sa.sageattn(q.to(DEV), k.to(DEV), v.to(DEV), is_causal=causal, pv_mode="fp8", BLKQ=64, BLKK=128)
        qi, qs, ki, ks = oq.per_block_int8(q, k, km=oq.k_mean(k), BLKQ=64, BLKK=128)
        model, _ = fm.fp8_attention_model(qi, ki, v, qs, ks, "HND", 64, 128, is_causal=causal)
        _check(out, model, torch.bfloat16, causal)


def _draw(rng):
    hkv = rng.choice([1, 2])
    return dict(D=rng.choice([64, 128]), dtype=rng.choice([torch.float16, torch.bfloat16]), layout=rng.choice(["HND", "NHD"]),
                B=rng.choice([1, 2]), Hkv=hkv, Hq=hkv * rng.choice([1, 2]),
                Sq=rng.choice([1, 33, 129, 257, 300, 640]), Skv=rng.choice([1, 64, 130, 259, 513, 900, 1500]),
                blkq=rng.choice([16, 32, 64, 128]), blkk=rng.choice([16, 32, 64, 128]), lse=rng.random() < 0.4,
                causal=rng.random() < 0.5, seed=rng.randrange(1 << 30))


@pytest.mark.parametrize("c", [_draw(random.Random(900 + i)) for i in range(24)], ids=[f"case{i}" for i in range(24)])
def test_random_fp8_configurations_match_the_model(c):
    g = torch.Generator().manual_seed(c["seed"])
    q = randn(c["layout"], c["B"], c["Hq"], c["Sq"], c["D"], c["dtype"], g)
    k = randn(c["layout"], c["B"], c["Hkv"], c["Skv"], c["D"], c["dtype"], g)
    v = randn(c["layout"], c["B"], c["Hkv"], c["Skv"], c["D"], c["dtype"], g)
    kw = dict(BLKQ=c["blkq"], BLKK=c["blkk"], tensor_layout=c["layout"])
    qi, qs, ki, ks = sa.per_block_int8(q.to(DEV), k.to(DEV), **kw)
    out, l2 = sa.forward(qi, ki, v.to(DEV), qs, ks, output_dtype=c["dtype"], return_lse=c["lse"], is_causal=c["causal"],
                         pv_mode="fp8", **kw)
    model, ml = fm.fp8_attention_model(qi.cpu(), ki.cpu(), v, qs.cpu(), ks.cpu(), c["layout"], c["blkq"], c["blkk"],
                                       is_causal=c["causal"], want_lse=c["lse"])
    _check(out, model, c["dtype"], c)
    if c["lse"]:
        fin = torch.isfinite(ml)
        assert torch.equal(fin, torch.isfinite(l2.cpu()))
        assert (l2.cpu().double() - ml)[fin].abs().max().item() < 2e-4
