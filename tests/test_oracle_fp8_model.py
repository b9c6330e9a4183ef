"""Pins oracle/fp8_model.py (the arithmetic model of the FP8 P.V kernel) without a GPU, by what the mathematics fixes:
the e4m3 decoder against torch's float8 type, a one-tile closed form written with scalar Python loops and struct-level
fp32 rounding, exact invariants (a constant V comes back exactly; numerator and denominator see the same rounded
probabilities), independence of the tile walk, and closeness to the exact-softmax formula within what rounding P to
three mantissa bits allows."""
import math
import struct

import numpy as np
import pytest
import torch

from oracle import attention as oa
from oracle import fp8_model as fm
from oracle import quant as oq
from tests.helpers import randn


def _f32(x):
    return struct.unpack("f", struct.pack("f", x))[0]


def _quantised(layout, B, Hq, Hkv, Sq, Skv, D, seed, blkq=64, blkk=128, dtype=torch.float16, koff=0.0):
    g = torch.Generator().manual_seed(seed)
    q = randn(layout, B, Hq, Sq, D, dtype, g)
    k = randn(layout, B, Hkv, Skv, D, dtype, g, offset_std=koff)
    v = randn(layout, B, Hkv, Skv, D, dtype, g)
    qi, qs, ki, ks = oq.per_block_int8(q, k, BLKQ=blkq, BLKK=blkk, tensor_layout=layout)
    return q, k, v, qi, qs, ki, ks


def test_decode_matches_torch_float8_for_every_code():
    codes = np.arange(0, 127)
    ref = torch.tensor(codes, dtype=torch.uint8).view(torch.float8_e4m3fn).to(torch.float32).numpy()
    assert np.array_equal(fm.decode_e4m3(codes), ref.astype(np.float64))


def test_linear_code_is_within_a_mantissa_step_of_the_exponential():
    t = np.linspace(-9.0, 8.0, 20001)
    code = np.clip(np.rint(8 * t + 56 - 0.3), 0, 255)
    val = fm.decode_e4m3(code)
    big = t > -6          # normal range of e4m3
    rel = np.abs(val[big] / np.exp2(t[big]) - 1)
    assert rel.max() < 0.125 and np.abs(np.mean(val[big] / np.exp2(t[big])) - 1) < 0.02   # centred by the -0.3
    assert (np.diff(val) >= 0).all()                                                       # monotone


def test_linear_code_by_way_of_the_16_bit_conversion_is_the_code_value_rounded_to_nearest():
    """The kernel reaches the code through a 16-bit conversion and its high byte; away from ties that must be
    rint(8 * t + 56 - 0.3) computed in float64 from the same operands, and next to ties one of the two neighbours."""
    rng = np.random.default_rng(5)
    R, N = 64, 128
    dots = rng.integers(-40000, 40000, size=(R, N))
    acc = (12582912.0 + dots).astype(np.float32)
    sc = np.broadcast_to(rng.uniform(1e-4, 3e-4, size=(R, 1)).astype(np.float32), (R, N))
    base = (5.0 - (dots.max(axis=1) * sc[:, 0].astype(np.float64))).astype(np.float32) + rng.uniform(0, 3, R).astype(np.float32)
    k0 = fm._fma32(fm.KN8, base, fm.KC)                       # the constant of a block with exponent 0
    code = fm.linear_code_of(acc, sc, k0)
    y = 8.0 * (dots * sc.astype(np.float64) + base[:, None].astype(np.float64)) + 56.0 - 0.3
    want = np.clip(np.rint(y), 0, 255)
    near_tie = np.abs(y - np.floor(y) - 0.5) < 0.02
    assert (~near_tie).mean() > 0.9 and want.max() >= 100 and (want == 0).any()
    assert (code[~near_tie] == want[~near_tie]).all()
    assert (np.abs(code - want) <= 1).all()


def _e4m3_value(code):
    return float(torch.tensor([code], dtype=torch.uint8).view(torch.float8_e4m3fn).float())


@pytest.mark.parametrize("linear", [False, True])
def test_one_tile_closed_form_with_scalar_loops(linear):
    """Skv <= 128: one tile, the reference maximum is the row's own maximum, so the model must equal
    sum_j P8_j V8_j / sum_j P8_j * v_scale with P8 computed score by score from the INT32 dot products.  Block-scaled
    codes: the tile is one block per row with the exponent e = max(ceil(row maximum - m), -110) (0 here, the reference
    maximum being the row maximum), the code that of 2^(s - m - e + 8.75), its weight 2^(e - 8)."""
    q, k, v, qi, qs, ki, ks = _quantised("HND", 1, 2, 1, 5, 9, 64, 11)
    out, lse = fm.fp8_attention_model(qi, ki, v, qs, ks, "HND", 64, 128, linear_code=linear, want_lse=not linear)
    v8, vsc = oq.quant_v_fp8(v)
    v8 = v8.float()
    kn = _f32(256.0 / 65535.0)
    kn8 = _f32(8.0 * kn)
    kc = _f32(_f32(kn * _f32(56.0 - 0.3)) + _f32(127.5 / 65535.0))
    for h in range(2):
        for i in range(5):
            sc = _f32(float(qs[0, h, 0]) * float(ks[0, 0, 0]))
            dots = [sum(int(qi[0, h, i, d]) * int(ki[0, 0, j, d]) for d in range(64)) for j in range(9)]
            nb = _f32(-12582912.0 * sc)
            scores = [_f32((12582912.0 + d) * sc + nb) for d in dots]
            m = max(scores)
            base = _f32(5.0 - m)
            p8, praw = [], []
            for j, d in enumerate(dots):
                if linear:
                    e = max(math.ceil(_f32(max(scores) - m)), -110)
                    k0 = _f32(kn8 * _f32(8.75 - m) + kc)
                    k0b = _f32(-kn8 * e + k0)
                    mul = _f32(kn8 * sc)
                    c = _f32(-12582912.0 * mul + k0b)
                    x = _f32((12582912.0 + d) * mul + c)
                    code = int(np.rint(min(max(x, 0.0), 1.0) * 65535.0)) >> 8
                    assert code <= 126
                    p8.append(_e4m3_value(code) * 2.0 ** (e - 8))
                else:
                    c = _f32(-12582912.0 * sc + base)
                    p = _f32(2.0 ** _f32((12582912.0 + d) * sc + c))
                    praw.append(p)
                    p8.append(float(torch.tensor([p]).to(torch.float8_e4m3fn).float()))
            den = sum(p8)
            for ch in (0, 31, 63):
                val = sum(p8[j] * float(v8[0, 0, j, ch]) for j in range(9)) / den * float(vsc[0, 0, ch])
                assert abs(out[0, h, i, ch].item() - val) < 1e-12 * max(1.0, abs(val)) + 1e-12
            if not linear:
                assert abs(lse[0, h, i].item() - (m + math.log2(sum(praw)) - 5.0)) < 1e-9


def test_block_scaled_codes_use_the_top_of_the_range_in_every_tile():
    """The largest score of a row in a tile is coded within one binade below 2^8.75: codes 118 ... 126, never the NaN
    byte, however far the tile lies below (or, within the lazy-rescale margin, above) the reference maximum."""
    rng = np.random.default_rng(6)
    R, N = 64, 128
    dots = rng.integers(-40000, 40000, size=(R, N))
    acc = (12582912.0 + dots).astype(np.float32)
    sc = np.broadcast_to(rng.uniform(1e-4, 3e-4, size=(R, 1)).astype(np.float32), (R, N))
    score = fm._fma32(acc, sc, (-fm.BIAS * sc).astype(np.float32))
    bmax = score.max(axis=1)
    for lag in (-20.0, -3.0, 0.0, 17.5, 60.0, 200.0):                     # reference maximum minus the tile's maximum
        m_used = (bmax + np.float32(lag) + rng.uniform(0, 1, R).astype(np.float32)).astype(np.float32)
        e, k0b = fm.block_constants(bmax, m_used)
        code = fm.linear_code_of(acc, sc, k0b)
        top = code.max(axis=1)
        if lag <= 100:
            assert (e == np.ceil(bmax - m_used)).all()
            assert (top >= 118).all() and (top <= 126).all(), lag
            # the value a code stands for, with its block's factor, is 2^(s - m + 0.75) within a mantissa step
            val = fm.decode_e4m3(code) * np.exp2(e.astype(np.float64) - 8.0)[:, None]
            want = np.exp2(score.astype(np.float64) - m_used[:, None] + 0.75)
            live = code >= 8
            assert live.mean() > 0.3 and (np.abs(val[live] / want[live] - 1) < 0.13).all()
        else:
            assert (e == -110).all() and (code == 0).all()              # 2^-200 of the maximum: flushed, exponent clamped


@pytest.mark.parametrize("binades", [9.5, 11.5, 12.5, 13.5, 15.5, 30.0])
def test_one_large_key_above_a_flat_tail(binades):
    """A single key `binades` above 8191 equal ones (an attention sink over a flat tail): the tail carries most of the
    softmax mass although each of its keys is tiny next to the row maximum.  A code scaled to the row maximum alone
    flushes or mis-codes the tail from about 12 binades on (e4m3 has 18); block-scaled codes keep every tile at the top
    of the range, so only the 127 tail keys that share the large key's tile are lost and the error stays that of three
    mantissa bits at any distance."""
    S, D, Sq = 8192, 64, 32
    qi = torch.zeros(1, 1, Sq, D, dtype=torch.int8)
    qi[..., 0] = 100
    ki = torch.zeros(1, 1, S, D, dtype=torch.int8)
    ki[0, 0, 0, 0] = 100
    qs, ks = torch.full((1, 1, 1), binades / 10000.0), torch.ones(1, 1, S // 64)
    v = torch.randn(1, 1, S, D, generator=torch.Generator().manual_seed(3)).to(torch.bfloat16)
    v8, vsc = oq.quant_v_fp8(v)
    ref, _ = oa.sage_reference(qi, ki, v8, qs, ks, "HND", 128, 64, v_scale=vsc)
    lin, _ = fm.fp8_attention_model(qi, ki, v, qs, ks, "HND", 128, 64, linear_code=True)
    assert oa.metrics(lin, ref)["rel_rmse"] < 0.02


@pytest.mark.parametrize("linear", [False, True])
@pytest.mark.parametrize("causal", [False, True])
def test_a_constant_value_row_comes_back_exactly(linear, causal):
    """If every key carries the same V row, O / l is that row whatever the probabilities are -- provided the
    denominator is the sum of the very values that multiply V.  Several tiles, so the lazy rescale is exercised."""
    q, k, v, qi, qs, ki, ks = _quantised("HND", 1, 2, 2, 150, 700, 64, 12, koff=1.0)
    v = v[:, :, :1].expand(-1, -1, 700, -1).contiguous()
    out, _ = fm.fp8_attention_model(qi, ki, v, qs, ks, "HND", 64, 128, is_causal=causal, linear_code=linear)
    v8, vsc = oq.quant_v_fp8(v)
    want = (v8.double() * vsc.double()[:, :, None, :])[:, :, :1].expand(-1, -1, 150, -1)
    assert torch.allclose(out, want, rtol=1e-12, atol=1e-12)


def test_model_is_close_to_the_exact_softmax_on_the_same_quantised_operands():
    q, k, v, qi, qs, ki, ks = _quantised("NHD", 1, 4, 2, 300, 900, 128, 13, koff=2.0, dtype=torch.bfloat16)
    v8, vsc = oq.quant_v_fp8(v, "NHD")
    ref, ref_lse = oa.sage_reference(qi, ki, v8, qs, ks, "NHD", 64, 128, is_causal=True, v_scale=vsc)
    exact, lse = fm.fp8_attention_model(qi, ki, v, qs, ks, "NHD", 64, 128, is_causal=True, linear_code=False, want_lse=True)
    lin, _ = fm.fp8_attention_model(qi, ki, v, qs, ks, "NHD", 64, 128, is_causal=True, linear_code=True)
    me, ml = oa.metrics(exact, ref), oa.metrics(lin, ref)
    # e4m3 rounding of P: relative error up to 2^-4 per probability, independent from key to key
    assert me["cosine"] > 0.9997 and me["rel_rmse"] < 0.025
    assert ml["cosine"] > 0.9995 and ml["rel_rmse"] < 0.035
    # LSE comes from the unrounded probabilities: only fp32 score rounding separates it from the formula
    assert (lse - ref_lse).abs().max().item() < 2e-3
    sd = oa.sdpa_fp32(q, k - oq.k_mean(k, "NHD"), v, "NHD", True)      # and the north-star gate against plain SDPA
    assert oa.metrics(lin, sd)["cosine"] >= 0.999


def test_masks_and_dead_rows():
    q, k, v, qi, qs, ki, ks = _quantised("HND", 1, 2, 1, 70, 259, 64, 14)
    mb = torch.rand((1, 2, 70, 259), generator=torch.Generator().manual_seed(1)) < 0.6
    mb[0, 1, 5] = False                              # a row with no visible key
    ma = torch.zeros((1, 2, 70, 259))
    ma[~mb] = -float("inf")
    ob, lb = fm.fp8_attention_model(qi, ki, v, qs, ks, "HND", 64, 128, attn_mask=mb, want_lse=True)
    oadd, ladd = fm.fp8_attention_model(qi, ki, v, qs, ks, "HND", 64, 128, attn_mask=ma, want_lse=True)
    assert torch.equal(ob, oadd) and torch.equal(lb, ladd)
    assert torch.count_nonzero(ob[0, 1, 5]).item() == 0 and lb[0, 1, 5].item() == -float("inf")
    v8, vsc = oq.quant_v_fp8(v)
    ref, ref_lse = oa.sage_reference(qi, ki, v8, qs, ks, "HND", 64, 128, attn_mask=mb, v_scale=vsc)
    assert oa.metrics(ob, ref)["cosine"] > 0.9995
    fin = torch.isfinite(ref_lse)
    assert torch.equal(fin, torch.isfinite(lb)) and (lb - ref_lse)[fin].abs().max().item() < 2e-3
