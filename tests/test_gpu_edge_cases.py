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


@pytest.mark.parametrize("pv", ["fp16", "fp8"])
def test_no_keys_at_all_gives_zeros_and_minus_infinity(pv):
    """Skv == 0 with Sq > 0: every row is a row with no visible key (out = 0, LSE = -inf), and nothing of K, V or their
    scales may be read -- the FP8 V scales in particular are never written in that case."""
    q = torch.randn((2, 4, 77, 128), dtype=torch.float16, device=DEV)
    kv = torch.empty((2, 2, 0, 128), dtype=torch.float16, device=DEV)
    junk = torch.full((1 << 20,), float("nan"), device=DEV)   # poison what the allocator hands out next
    del junk
    out, lse = sa.sageattn(q, kv, kv, pv_mode=pv, return_lse=True)
    assert tuple(out.shape) == tuple(q.shape) and torch.count_nonzero(out).item() == 0
    assert torch.isinf(lse).all() and (lse < 0).all()
    out = sa.sageattn(q, kv, kv, pv_mode=pv)
    assert torch.count_nonzero(out).item() == 0
    qi, qs, ki, ks = sa.per_block_int8(q, kv)
    o2, l2 = sa.forward(qi, ki, kv, qs, ks, return_lse=True, pv_mode=pv)
    assert torch.count_nonzero(o2).item() == 0 and torch.isinf(l2).all()


@pytest.mark.parametrize("pv,causal,lse", [("fp8", True, False), ("fp16", False, True)])
def test_strided_views_of_a_fused_qkv_buffer_through_the_c_abi(pv, causal, lse):
    """q, k and v as slices of one [B, S, 3, H, D] buffer (row stride 3*H*D) and a strided output: the INT8 copies the
    one-call pipeline makes inside its workspace must not inherit those strides.  The workspace is exactly the size
    the library asks for and sits in the middle of a guarded allocation, so a stray write is seen."""
    from baselinebenchmark_amd import _cabi
    from tests.helpers import sageattn_cabi
    B, S, H, D = 2, 300, 4, 128
    g = torch.Generator().manual_seed(31)
    qkv = torch.randn((B, S, 3, H, D), generator=g).to(torch.bfloat16).to(DEV)
    q, k, v = qkv[:, :, 0], qkv[:, :, 1], qkv[:, :, 2]          # NHD views, row stride 3*H*D
    assert not q.is_contiguous()
    obuf = torch.zeros((B, S, 2, H, D), dtype=torch.bfloat16, device=DEV)
    out = obuf[:, :, 1]
    need = _cabi.lib().sage_sageattn_workspace_bytes_for(B, H, H, S, S, D, 64, 128, _cabi.PV_FP8 if pv == "fp8" else _cabi.PV_FP16,
                                                         0, 0, 0, 1, int(lse), 0)   # exactly what THIS call uses
    assert need <= _cabi.lib().sage_sageattn_workspace_bytes(B, H, H, S, S, D, 64, 128, _cabi.PV_FP8 if pv == "fp8" else _cabi.PV_FP16, 0, 0, 0)
    guard = 1 << 16
    buf = torch.full((need + 2 * guard + 256,), 0x5A, dtype=torch.uint8, device=DEV)
    base = (-(buf.data_ptr() + guard)) % 256 + guard
    ws = buf[base:base + need]
    lse_t = torch.empty((B, H, S), dtype=torch.float32, device=DEV) if lse else None
    rc = sageattn_cabi(q, k, v, out, layout="NHD", is_causal=causal, pv=pv, BLKQ=64, BLKK=128, workspace=ws, lse=lse_t)
    assert rc == 0, _cabi.lib().sage_last_error().decode()
    torch.cuda.synchronize()
    assert (buf[:base] == 0x5A).all() and (buf[base + need:] == 0x5A).all()
    assert torch.count_nonzero(obuf[:, :, 0]).item() == 0
    ref = sa.sageattn(q.contiguous(), k.contiguous(), v.contiguous(), tensor_layout="NHD", is_causal=causal, pv_mode=pv,
                      BLKQ=64, BLKK=128, return_lse=lse)
    if lse:
        ref, ref_lse = ref
        assert torch.allclose(lse_t * 0.6931471805599453, ref_lse, rtol=0, atol=1e-6)
    assert torch.equal(out.contiguous().view(torch.int16), ref.view(torch.int16))
