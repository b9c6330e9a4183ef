"""Correctness script of the ``backends/_amd`` bundle: the cases of the other vendors' script
(backends/_hygon/test/sageattention/test_sageattention_hip.py:31-70: HND and NHD, GQA, head_dim 64 and 128, a
129 x 70 problem under a boolean and an additive mask, relative RMSE of the output and maximum LSE error below 3e-2),
run against the fp32 formula on the dequantised operands, plus the one-call ``sageattn`` with both P.V formats.

    python backends/_amd/test/sage_attention/test_sageattention_hip.py        # needs an MI355X
    python -m pytest backends/_amd/test -q                                    # the same cases under pytest

The library's own parity tests (bit-exact quantisers, the attention kernels against a CPU restatement of the
reference's algorithm, golden vectors) are the ``tests/`` folder beside the ``baselinebenchmark_amd`` package.
"""
import math
import sys
from pathlib import Path

import torch

sys.path.insert(0, str(Path(__file__).resolve().parents[2] / "ops"))
from sage_attention import backend_name, forward, per_block_int8, sageattn  # noqa: E402

LN2 = math.log(2.0)


def formula(q, k, v, q_scale, k_scale, layout, mask=None, causal=False):
    """softmax in base 2 over the dequantised logits, as every vendor's script restates it."""
    if layout == "NHD":
        q, k, v = (x.transpose(1, 2) for x in (q, k, v))
    sq, skv = q.shape[-2], k.shape[-2]
    q = q.double() * q_scale.double().repeat_interleave(128, dim=-1)[..., :sq, None]
    k = k.double() * k_scale.double().repeat_interleave(64, dim=-1)[..., :skv, None]
    group = q.shape[1] // k.shape[1]
    k, v = k.repeat_interleave(group, dim=1), v.double().repeat_interleave(group, dim=1)
    logits = q @ k.transpose(-1, -2)
    if mask is not None:
        logits = logits.masked_fill(~mask, -math.inf) if mask.dtype == torch.bool else logits + mask.double()
    if causal:
        logits = logits.masked_fill(torch.ones(sq, skv, dtype=torch.bool, device=q.device).triu(1), -math.inf)
    out = torch.softmax(logits * LN2, dim=-1) @ v
    lse = torch.logsumexp(logits * LN2, dim=-1) / LN2
    return (out.transpose(1, 2) if layout == "NHD" else out), lse


def rel_rmse(got, want):
    return ((got.double() - want).square().mean().sqrt() / (want.square().mean().sqrt() + 1e-6)).item()


def make_inputs(case, seed):
    """Seeded N(0,1) operands of one table row, generated on the host (so a case reads the same on any device) in
    the (batch, head, row, channel) order and then laid out as the row asks."""
    gen = torch.Generator().manual_seed(seed)
    dtype = getattr(torch, case["dtype"])
    shapes = {"q": (1, case["q_heads"], case["rows"], case["dim"]), "k": (1, case["kv_heads"], case["keys"], case["dim"]),
              "v": (1, case["kv_heads"], case["keys"], case["dim"])}
    ops = {}
    for name, shape in shapes.items():
        x = torch.randn(shape, generator=gen).to(dtype)
        ops[name] = (x.transpose(1, 2).contiguous() if case["layout"] == "NHD" else x).cuda()
    return ops["q"], ops["k"], ops["v"]


def make_mask(case):
    """Every third key hidden (boolean) or pushed down by two logits (additive): the two mask kinds of ``forward``."""
    if case["mask"] is None:
        return None
    every_third = (torch.arange(case["keys"], device="cuda") % 3 == 0).expand(1, case["q_heads"], case["rows"], case["keys"])
    if case["mask"] == "bool":
        return ~every_third
    return torch.where(every_third, -2.0, 0.0).contiguous()


def run_case(index, case):
    q, k, v = make_inputs(case, seed=9000 + index)
    mask = make_mask(case)
    dtype = q.dtype
    qi, qs, ki, ks = per_block_int8(q, k, tensor_layout=case["layout"])
    out, lse = forward(qi, ki, v, qs, ks, tensor_layout=case["layout"], attn_mask=mask, output_dtype=dtype, return_lse=True)
    want, want_lse = formula(qi, ki, v, qs, ks, case["layout"], mask)
    out_err, lse_err = rel_rmse(out, want), (lse.double() - want_lse).abs().max().item()
    print({**case, "out_rel_rmse": out_err, "lse_max_abs": lse_err})
    assert torch.isfinite(out).all() and torch.isfinite(lse).all(), case
    assert out_err < 3e-2 and lse_err < 3e-2, (case, out_err, lse_err)   # the other vendors' bounds


def run_one_call(pv_mode, dim, causal):
    """sageattn against plain softmax(q k^T / sqrt(d)) v on the unquantised inputs: the end-to-end error budget."""
    torch.manual_seed(7 + dim)
    q = torch.randn((2, 4, 300, dim), device="cuda", dtype=torch.bfloat16)
    k = torch.randn((2, 2, 300, dim), device="cuda", dtype=torch.bfloat16) + 0.5
    v = torch.randn_like(k)
    out = sageattn(q, k, v, is_causal=causal, pv_mode=pv_mode)
    want = torch.nn.functional.scaled_dot_product_attention(q.double(), k.double().repeat_interleave(2, 1),
                                                           v.double().repeat_interleave(2, 1), is_causal=causal)
    err = rel_rmse(out, want)
    cos = torch.nn.functional.cosine_similarity(out.double().flatten(), want.flatten(), dim=0).item()
    print("sageattn pv", pv_mode, "D", dim, "causal", causal, "rel_rmse", err, "cosine", cos)
    assert cos >= 0.999 and err < 5e-2


def _case(layout, kv_heads, dim, rows, keys, mask=None, dtype="float16", q_heads=4):
    return dict(layout=layout, q_heads=q_heads, kv_heads=kv_heads, dim=dim, rows=rows, keys=keys, mask=mask, dtype=dtype)


# The shapes the other vendors' script covers (both layouts, grouped-query heads, both head dimensions, the ragged
# 129 x 70 problem under each mask kind, in fp16 and bf16) and one longer ragged NHD problem.
CASES = [
    _case("HND", 1, 64, 128, 128),
    _case("NHD", 2, 64, 128, 128),
    _case("HND", 2, 128, 129, 70, mask="bool"),
    _case("HND", 2, 128, 129, 70, mask="additive"),
    _case("HND", 2, 128, 129, 70, mask="bool", dtype="bfloat16"),
    _case("NHD", 4, 128, 257, 513),
]
ONE_CALL = [("fp16", 64, False), ("fp16", 128, True), ("fp8", 64, True), ("fp8", 128, False)]


def test_forward_cases():
    for index, case in enumerate(CASES):
        run_case(index, case)


def test_one_call_cases():
    for case in ONE_CALL:
        run_one_call(*case)


if __name__ == "__main__":
    print("SageAttention backend:", backend_name())
    test_forward_cases()
    test_one_call_cases()
    print("SageAttention MI355X correctness: PASS")
