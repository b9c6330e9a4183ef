"""Edge shapes through the C ABI: single rows and keys, sequences shorter than one tile, empty batches,
lengths around the tile and scale-block boundaries.  Every result is checked against the oracle formula on the
same quantised operands (FP16 P.V: relative RMSE < 2e-3, |LSE2 error| < 1e-3; FP8 P.V: cosine >= 0.999)."""
import pytest
import torch

import baselinebenchmark_amd as sa
from oracle import attention as oa
from tests.helpers import randn

pytestmark = [pytest.mark.gpu, pytest.mark.sage_attention]
DEV = "cuda"


@pytest.mark.parametrize("shape", [(1, 1), (1, 1000), (300, 1), (2, 3), (31, 33), (32, 32), (33, 31), (63, 65), (64, 64),
                                   (127, 129), (128, 128), (129, 127), (255, 257), (256, 256), (257, 255), (511, 513)])
@pytest.mark.parametrize("pv", ["fp16", "fp8"])
def test_lengths_around_every_boundary(shape, pv):
    Sq, Skv = shape
    g = torch.Generator().manual_seed(1000 + 7 * Sq + Skv)
    B, Hq, Hkv, D = 1, 2, 1, 64
    q = randn("HND", B, Hq, Sq, D, torch.float16, g)
    k = randn("HND", B, Hkv, Skv, D, torch.float16, g)
    v = randn("HND", B, Hkv, Skv, D, torch.float16, g)
    qi, qs, ki, ks = sa.per_block_int8(q.to(DEV), k.to(DEV))
    out, lse = sa.forward(qi, ki, v.to(DEV), qs, ks, return_lse=True, pv_mode=pv)
    ref, ref_lse = oa.sage_reference(qi.cpu(), ki.cpu(), v, qs.cpu(), ks.cpu(), "HND", 128, 64)
    m = oa.metrics(out.cpu().float(), ref)
    assert m["finite"]
    if pv == "fp16":
        assert m["rel_rmse"] < 2e-3 and (lse.cpu().double() - ref_lse).abs().max().item() < 1e-3
    else:
        assert m["cosine"] >= 0.999


@pytest.mark.parametrize("S", [1, 2, 65, 130, 259])
def test_causal_square_small(S):
    g = torch.Generator().manual_seed(2000 + S)
    q = randn("NHD", 2, 4, S, 128, torch.bfloat16, g)
    k = randn("NHD", 2, 2, S, 128, torch.bfloat16, g)
    v = randn("NHD", 2, 2, S, 128, torch.bfloat16, g)
    out = sa.sageattn(q.to(DEV), k.to(DEV), v.to(DEV), tensor_layout="NHD", is_causal=True)
    ref = oa.sdpa_fp32(q, k, v, "NHD", True)
    assert oa.metrics(out.cpu().float(), ref)["cosine"] >= 0.999
    # the first query sees exactly the first key: its output is V[0] of its KV head (up to fp16 P.V rounding)
    first = out[:, 0].cpu().float()
    expected = v[:, 0].float().repeat_interleave(2, dim=1)
    assert (first - expected).abs().max().item() < 2e-2


def test_empty_batch_and_empty_heads_return_empty_tensors():
    q = torch.empty((0, 4, 128, 64), dtype=torch.float16, device=DEV)
    out = sa.sageattn(q, q, q)
    assert tuple(out.shape) == (0, 4, 128, 64)
    qi, qs, ki, ks = sa.per_block_int8(q, q)
    assert tuple(qi.shape) == (0, 4, 128, 64) and tuple(qs.shape) == (0, 4, 1)
    o, l = sa.forward(qi, ki, q, qs, ks, return_lse=True)
    assert tuple(o.shape) == (0, 4, 128, 64) and tuple(l.shape) == (0, 4, 128)


def test_inputs_are_not_modified_and_results_are_deterministic():
    g = torch.Generator().manual_seed(3000)
    q = randn("HND", 1, 4, 500, 128, torch.bfloat16, g).to(DEV)
    k = randn("HND", 1, 4, 500, 128, torch.bfloat16, g).to(DEV)
    v = randn("HND", 1, 4, 500, 128, torch.bfloat16, g).to(DEV)
    q0, k0, v0 = q.clone(), k.clone(), v.clone()
    a = sa.sageattn(q, k, v, is_causal=True, pv_mode="fp8", BLKQ=64, BLKK=128)
    b = sa.sageattn(q, k, v, is_causal=True, pv_mode="fp8", BLKQ=64, BLKK=128)
    assert torch.equal(q, q0) and torch.equal(k, k0) and torch.equal(v, v0)      # test_official_wheel.py:20-32
    assert torch.equal(a, b)


def test_many_heads_few_rows_exercises_the_head_to_xcd_mapping():
    # 24 = 3 * 8 KV groups: the XCD-aware permutation path; 5 groups: the plain path
    for hkv in (24, 5):
        g = torch.Generator().manual_seed(4000 + hkv)
        q = randn("HND", 1, 2 * hkv, 70, 64, torch.float16, g)
        k = randn("HND", 1, hkv, 90, 64, torch.float16, g)
        v = randn("HND", 1, hkv, 90, 64, torch.float16, g)
        qi, qs, ki, ks = sa.per_block_int8(q.to(DEV), k.to(DEV))
        out, _ = sa.forward(qi, ki, v.to(DEV), qs, ks)
        ref, _ = oa.sage_reference(qi.cpu(), ki.cpu(), v, qs.cpu(), ks.cpu(), "HND", 128, 64)
        assert oa.metrics(out.cpu().float(), ref)["rel_rmse"] < 2e-3
