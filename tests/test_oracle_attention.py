"""Pins oracle/attention.py without a GPU: against torch SDPA (a library routine the formula reduces
to), a brute-force triple loop on tiny shapes, and structural invariants of causal masking."""
import math

import pytest
import torch
import torch.nn.functional as F

from oracle import attention as oa
from oracle import quant as oq
from tests.helpers import randn


def _quantised(layout, B, Hq, Hkv, Sq, Skv, D, seed, blkq=128, blkk=64):
    g = torch.Generator().manual_seed(seed)
    q = randn(layout, B, Hq, Sq, D, torch.float16, g)
    k = randn(layout, B, Hkv, Skv, D, torch.float16, g)
    v = randn(layout, B, Hkv, Skv, D, torch.float16, g)
    qi, qs, ki, ks = oq.per_block_int8(q, k, BLKQ=blkq, BLKK=blkk, tensor_layout=layout)
    return q, k, v, qi, qs, ki, ks


@pytest.mark.parametrize("layout", ["HND", "NHD"])
@pytest.mark.parametrize("causal", [False, True])
def test_reference_reduces_to_sdpa_on_dequantised_operands(layout, causal):
    q, k, v, qi, qs, ki, ks = _quantised(layout, 1, 4, 2, 129, 129, 64, 1)
    out, lse = oa.sage_reference(qi, ki, v, qs, ks, layout, is_causal=causal)
    hnd = (lambda t: t if layout == "HND" else t.transpose(1, 2))
    qd = hnd(qi).double() * oa.expand_scale(qs.double(), 128, 129)
    kd = hnd(ki).double() * oa.expand_scale(ks.double(), 64, 129)
    kd, vd = kd.repeat_interleave(2, dim=1), hnd(v).double().repeat_interleave(2, dim=1)
    ref = F.scaled_dot_product_attention(qd, kd, vd, is_causal=causal, scale=math.log(2.0))
    assert torch.allclose(hnd(out), ref, atol=1e-9, rtol=1e-9)


def test_reference_brute_force_tiny():
    q, k, v, qi, qs, ki, ks = _quantised("HND", 1, 2, 1, 5, 7, 64, 2, blkq=128, blkk=64)
    out, lse = oa.sage_reference(qi, ki, v, qs, ks, "HND")
    for h in range(2):
        for i in range(5):
            logits = [sum(int(qi[0, h, i, d]) * int(ki[0, 0, j, d]) for d in range(64)) * float(qs[0, h, 0]) * float(ks[0, 0, 0])
                      for j in range(7)]
            mx = max(logits)
            w = [2.0 ** (l - mx) for l in logits]
            tot = sum(w)
            for d in (0, 17, 63):
                val = sum(w[j] * float(v[0, 0, j, d]) for j in range(7)) / tot
                assert abs(out[0, h, i, d].item() - val) < 1e-9
            assert abs(lse[0, h, i].item() - (mx + math.log2(tot))) < 1e-9


def test_causal_row_depends_only_on_earlier_keys():
    q, k, v, qi, qs, ki, ks = _quantised("HND", 1, 1, 1, 64, 64, 64, 3)
    out, _ = oa.sage_reference(qi, ki, v, qs, ks, "HND", is_causal=True)
    v2 = v.clone()
    v2[0, 0, 40:] += 5.0
    out2, _ = oa.sage_reference(qi, ki, v2, qs, ks, "HND", is_causal=True)
    assert torch.equal(out[0, 0, :40], out2[0, 0, :40])
    assert not torch.equal(out[0, 0, 40:], out2[0, 0, 40:])
    # first row attends to key 0 only
    assert torch.allclose(out[0, 0, 0], v[0, 0, 0].double())


def test_masks_follow_reference_test_semantics():
    # bool / additive masks as in backends/_hygon/test/sageattention/test_sageattention_hip.py:38-45
    q, k, v, qi, qs, ki, ks = _quantised("HND", 1, 4, 2, 129, 70, 128, 4)
    mb = torch.ones((1, 4, 129, 70), dtype=torch.bool)
    mb[..., ::3] = False
    ma = torch.zeros((1, 4, 129, 70))
    ma[..., ::3] = -float("inf")
    o1, l1 = oa.sage_reference(qi, ki, v, qs, ks, "HND", attn_mask=mb)
    o2, l2 = oa.sage_reference(qi, ki, v, qs, ks, "HND", attn_mask=ma)
    assert torch.allclose(o1, o2) and torch.allclose(l1, l2)


def test_k_smoothing_leaves_softmax_unchanged():
    g = torch.Generator().manual_seed(6)
    q = randn("HND", 1, 2, 64, 64, torch.float32, g)
    k = randn("HND", 1, 2, 64, 64, torch.float32, g, offset_std=3.0)
    v = randn("HND", 1, 2, 64, 64, torch.float32, g)
    q, k, v = q.double(), k.double(), v.double()
    a = oa.sdpa_fp32(q, k, v, dtype=torch.float64)
    b = oa.sdpa_fp32(q, k - k.mean(dim=2, keepdim=True), v, dtype=torch.float64)
    assert torch.allclose(a, b, atol=1e-9)


def test_quantised_pipeline_is_close_to_sdpa():
    q, k, v, qi, qs, ki, ks = _quantised("NHD", 2, 4, 4, 200, 200, 128, 7)
    out, _ = oa.sage_reference(qi, ki, v, qs, ks, "NHD", is_causal=True)
    ref = oa.sdpa_fp32(q, k, v, "NHD", is_causal=True)
    m = oa.metrics(out, ref)
    assert m["cosine"] > 0.9995 and m["rmse"] < 0.015  # CLI thresholds of sage_attention_benchmark_compare.py:158-160
    cpu = oa.cpu_quantize_sdpa(q, k, v, "NHD", is_causal=True, smooth_k=False)
    assert oa.metrics(cpu, out)["cosine"] > 0.99999


def test_varlen_sdpa_equals_loop():
    g = torch.Generator().manual_seed(8)
    lens = [5, 33, 64]
    cu = [0, 5, 38, 102]
    q = torch.randn((102, 4, 64), generator=g)
    k = torch.randn((102, 2, 64), generator=g)
    v = torch.randn((102, 2, 64), generator=g)
    out = oa.sdpa_fp32_varlen(q, k, v, cu, cu, is_causal=True)
    o1 = oa.sdpa_fp32(q[5:38].unsqueeze(0), k[5:38].unsqueeze(0), v[5:38].unsqueeze(0), "NHD", True)
    assert torch.equal(out[5:38], o1[0])
