"""Pins the CPU oracle of the INT8 quantiser (oracle/quant.py) without a GPU.

Evidence, in order of independence:
 1. golden vectors produced by the reference's own per_block_int8 under Triton's CPU interpreter
    (tests/golden/make_quant_golden.py) -- bit-exact;
 2. an exact-rational restatement (fractions.Fraction, correctly rounded by construction) of
    quant_per_block.py:38-46 on small tiles -- catches a reciprocal-multiply or a wrong tie rule;
 3. closed-form invariants (arg-max -> +-127, half-step error bound, tail rows ignored).
"""
import math
from fractions import Fraction

import numpy as np
import pytest
import torch

from oracle import quant as oq
from tests.helpers import golden_case, randn


# ---------------------------------------------------------------- 1. golden vectors
def test_oracle_matches_reference_golden(golden):
    for name in golden["cases"]:
        c = golden_case(golden, str(name))
        qi, qs, ki, ks = oq.per_block_int8(c["q"], c["k"], km=c["km"], BLKQ=c["BLKQ"], BLKK=c["BLKK"],
                                           sm_scale=c["sm_scale"], tensor_layout=c["layout"])
        assert torch.equal(qi, c["qi"]), name
        assert torch.equal(ki, c["ki"]), name
        assert torch.equal(qs, c["qs"]), name
        assert torch.equal(ks, c["ks"]), name


# ---------------------------------------------------------------- 2. exact rational restatement
def _rn32(fr: Fraction) -> np.float32:
    """Round an exact rational to the nearest binary32 (ties to even), no intermediate rounding."""
    if fr == 0:
        return np.float32(0.0)
    sign = -1 if fr < 0 else 1
    a = abs(fr)
    e = math.floor(math.log2(a)) if a >= 1 else -math.ceil(-math.log2(float(a)) - 1e-12)
    while Fraction(2) ** e > a:
        e -= 1
    while Fraction(2) ** (e + 1) <= a:
        e += 1
    e = max(e, -126)
    ulp = Fraction(2) ** (e - 23)
    n = a / ulp
    fl = n.numerator // n.denominator
    rem = n - fl
    if rem > Fraction(1, 2) or (rem == Fraction(1, 2) and fl % 2 == 1):
        fl += 1
    return np.float32(sign * float(fl * ulp))


def _tile_rational(x32, mult):
    xs = [_rn32(Fraction(float(v)) * Fraction(float(np.float32(mult)))) for v in x32.ravel()]
    amax = max(abs(float(v)) for v in xs)
    scale = _rn32(Fraction(amax) / 127)
    scale = max(scale, np.float32(1e-12))
    out = []
    for v in xs:
        z = _rn32(Fraction(float(v)) / Fraction(float(scale)))
        z = _rn32(Fraction(float(z)) + (Fraction(1, 2) if z >= 0 else Fraction(-1, 2)))
        out.append(int(math.trunc(float(z))))
    return np.array(out, dtype=np.int64).reshape(x32.shape), scale


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("mult", [1.0, 128 ** -0.5 * 1.44269504, 0.3])
def test_oracle_tile_equals_exact_rational(dtype, mult):
    g = torch.Generator().manual_seed(7)
    x = (torch.randn((24, 16), generator=g) * 3).to(dtype)
    x32 = x.float().numpy()
    q, s = oq.quant_tile_int8(x32, mult)
    qr, sr = _tile_rational(x32, mult)
    assert s == sr
    assert np.array_equal(q.astype(np.int64), qr)


def test_round_half_away_from_zero_ties():
    # tile max 127 -> scale exactly 1 -> quotients are the inputs: k + 0.5 must round away from zero
    x = np.array([[127.0, 0.5, -0.5, 1.5, -1.5, 2.5, -2.5, 126.5, -126.5, 0.0, -0.0, 0.49999997]], np.float32)
    q, s = oq.quant_tile_int8(x, 1.0)
    assert s == np.float32(1.0)
    # the last one is the add-then-truncate artefact the reference has (quant_per_block.py:43-44):
    # 0.49999997 + 0.5 rounds up to 1.0 in binary32, so it quantises to 1, not 0
    assert q.tolist() == [[127, 1, -1, 2, -2, 3, -3, 127, -127, 0, 0, 1]]


# ---------------------------------------------------------------- 3. invariants
@pytest.mark.parametrize("layout", ["HND", "NHD"])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_invariants(layout, dtype):
    g = torch.Generator().manual_seed(11)
    B, H, L, D, blk = 2, 3, 200, 64, 64
    q = randn(layout, B, H, L, D, dtype, g)
    k = randn(layout, B, H, L, D, dtype, g, offset_std=2.0)
    qi, qs, ki, ks = oq.per_block_int8(q, k, BLKQ=blk, BLKK=blk, tensor_layout=layout)
    assert qs.shape == (B, H, math.ceil(L / blk)) and qs.dtype == torch.float32
    for x, xi, xs, mult in ((q, qi, qs, oq.q_multiplier(D)), (k, ki, ks, np.float32(1.0))):
        x32 = (x.float() if layout == "HND" else x.float().transpose(1, 2)).numpy() * np.float32(mult)
        xi_h = (xi if layout == "HND" else xi.transpose(1, 2)).numpy().astype(np.int32)
        assert np.abs(xi_h).max() <= 127
        rows = np.repeat(xs.numpy(), blk, axis=-1)[..., :L, None]
        # half-step bound (+1 ulp of the quotient)
        assert np.all(np.abs(x32 - xi_h * rows) <= rows * (0.5 + 1e-5))
        # the arg-max element of every tile maps to +-127 and scale = amax/127
        for b in range(B):
            for h in range(H):
                for t in range(math.ceil(L / blk)):
                    tile = x32[b, h, t * blk:(t + 1) * blk]
                    ti = xi_h[b, h, t * blk:(t + 1) * blk]
                    i = np.unravel_index(np.argmax(np.abs(tile)), tile.shape)
                    assert abs(ti[i]) == 127
                    assert xs[b, h, t].item() == np.float32(np.abs(tile).max()) / np.float32(127)


def test_tail_rows_do_not_leak_into_scale():
    g = torch.Generator().manual_seed(3)
    x = torch.randn((1, 1, 70, 64), generator=g).half()
    big = torch.cat([x, torch.full((1, 1, 58, 64), 1000.0).half()], dim=2)  # what a padded load would see
    qi, qs, _, _ = oq.per_block_int8(x, x, BLKQ=128, BLKK=64)
    qi2, qs2, _, _ = oq.per_block_int8(big, big, BLKQ=128, BLKK=64)
    assert not torch.equal(qs, qs2[..., :1])  # sanity: the padding would have changed the scale
    assert qi.shape == x.shape and qs.shape == (1, 1, 1)


def test_zero_tile_gets_floor_scale():
    x = torch.zeros((1, 1, 64, 64), dtype=torch.float16)
    qi, qs, ki, ks = oq.per_block_int8(x, x, BLKQ=64, BLKK=64)
    assert torch.all(qi == 0) and torch.all(ki == 0)
    assert qs.item() == np.float32(1e-12) and ks.item() == np.float32(1e-12)


def test_q_multiplier_matches_full_precision_log2e_for_supported_head_dims():
    for d in (64, 128):
        assert oq.q_multiplier(d) == np.float32(d ** -0.5 * 1.4426950408889634)


def test_exhaustive_fp16_values_single_tile():
    # every finite fp16 value once, in tiles of 128x64: vectorised oracle == per-tile oracle
    bits = np.arange(65536, dtype=np.uint16)
    vals = torch.from_numpy(bits.view(np.int16)).view(torch.float16)
    vals = vals[torch.isfinite(vals)]
    n = (vals.numel() // (128 * 64)) * 128 * 64
    x = vals[:n].reshape(1, 1, -1, 64)
    qi, qs, _, _ = oq.per_block_int8(x, x, BLKQ=128, BLKK=128, sm_scale=1.0 / 1.44269504)
    x32 = x.float().numpy()[0, 0]
    for t in range(x32.shape[0] // 128):
        q, s = oq.quant_tile_int8(x32[t * 128:(t + 1) * 128], np.float32(1.0 / 1.44269504 * 1.44269504))
        assert s == qs[0, 0, t].item()
        assert np.array_equal(q, qi[0, 0, t * 128:(t + 1) * 128].numpy())


def test_k_mean_definition():
    # The reference never computes km (it is an argument of per_block_int8), so this is a DEFINITION, not parity: the
    # bound below catches a wrong axis or a missing division, the exact-rational test after it fixes the rounding order.
    g = torch.Generator().manual_seed(5)
    k = randn("NHD", 2, 3, 333, 64, torch.bfloat16, g, offset_std=2.0)
    km = oq.k_mean(k, "NHD")
    assert km.shape == (2, 1, 3, 64) and km.dtype == torch.bfloat16
    ref = k.double().mean(dim=1, keepdim=True)
    assert torch.all((km.double() - ref).abs() <= ref.abs() * 2 ** -8 + 1e-30)


def _round_fraction(x, precision, emin):
    """Round-to-nearest-even of an exact rational to a binary float with `precision` significand bits and minimum
    normal exponent `emin` (subnormals below it), returned as an exact Fraction."""
    from fractions import Fraction
    if x == 0:
        return Fraction(0)
    sign, a = (-1 if x < 0 else 1), abs(x)
    e = a.numerator.bit_length() - a.denominator.bit_length()
    if Fraction(2) ** e > a:
        e -= 1                                   # now 2^e <= a < 2^(e+1)
    ulp = Fraction(2) ** (max(e, emin) - (precision - 1))
    n = a / ulp
    lo = n.numerator // n.denominator
    rem = n - lo
    if rem > Fraction(1, 2) or (rem == Fraction(1, 2) and lo % 2 == 1):
        lo += 1
    return sign * lo * ulp


@pytest.mark.parametrize("dtype,precision,emin", [(torch.float16, 11, -14), (torch.bfloat16, 8, -126)])
def test_k_mean_against_exact_rational_arithmetic(dtype, precision, emin):
    # Definition: mean = exact sum / L, rounded ONCE to binary32 and then once to the input dtype.  Two channels are built
    # so that a plausible other order gives another value (checked at the end), which pins the rounding order and not
    # only the axis:
    #   channel 0: 64 + 64 + 128*h + 125 values of 2^-18 (h = half a step of the dtype at 1.0).  The exact mean lies just
    #     above the half-way point 1 + h and rounds up; a float32 accumulation along the sequence drops every 2^-18
    #     (half an ulp of 128.x is 2^-17), lands on the tie and rounds to even, 1.0.
    #   channel 1: 2 + 2 + 4*h + 2^-38 + zeros ... over L = 4 would do; with L = 128: 64 + 64 + 128*h + 2^-24.  The exact
    #     mean is the half-way point plus 2^-31: binary32 rounds it to the tie, which then goes to even (1.0); rounding
    #     the exact mean directly to the dtype goes up.
    from fractions import Fraction
    g = torch.Generator().manual_seed(11)
    L, C = 128, 12
    h = 2.0 ** -precision
    k = (torch.randn((1, 1, L, C), generator=g) * 3.0 + torch.randn((1, 1, 1, C), generator=g) * 40.0).to(dtype)
    col0 = torch.full((L,), 2.0 ** -18)
    col0[0], col0[1], col0[2] = 64.0, 64.0, 128 * h
    col1 = torch.zeros(L)
    col1[0], col1[1], col1[2], col1[3] = 64.0, 64.0, 128 * h, 2.0 ** -24
    k[0, 0, :, 0], k[0, 0, :, 1] = col0.to(dtype), col1.to(dtype)
    assert torch.equal(k[0, 0, :, 0].double(), col0.double()) and torch.equal(k[0, 0, :, 1].double(), col1.double())
    km = oq.k_mean(k, "HND")
    for c in range(C):
        total = sum(Fraction(float(k[0, 0, n, c])) for n in range(L))       # fp16/bf16 values are exact Fractions
        want = _round_fraction(_round_fraction(total / L, 24, -126), precision, emin)
        assert Fraction(float(km[0, 0, 0, c])) == want, (c, float(km[0, 0, 0, c]), float(want))
    assert float(km[0, 0, 0, 0]) == 1.0 + 2 * h and float(km[0, 0, 0, 1]) == 1.0
    # the other orders, on the same tensor
    acc = torch.zeros((), dtype=torch.float32)
    for n in range(L):
        acc = acc + k[0, 0, n, 0].float()
    assert float((acc / L).to(dtype)) == 1.0                                               # float32 accumulation: the tie
    total1 = sum(Fraction(float(k[0, 0, n, 1])) for n in range(L))
    assert _round_fraction(total1 / L, precision, emin) == Fraction(1) + Fraction(2) * Fraction(h)   # one rounding: up


def test_fp8_value_set_matches_reference_bit_decoder():
    # restates the bit layout of backends/_enflame/ops/hpc_ops_attention/fp8_utils.py:19-38
    bits = torch.arange(256, dtype=torch.int16).to(torch.uint8)
    vals = bits.view(torch.float8_e4m3fn).float()
    for b in range(256):
        s, e, m = b >> 7, (b >> 3) & 15, b & 7
        if e == 15 and m == 7:
            assert math.isnan(vals[b].item())
            continue
        mag = (m / 8.0) * 2.0 ** -6 if e == 0 else (1 + m / 8.0) * 2.0 ** (e - 7)
        assert vals[b].item() == (-mag if s else mag)


def test_quant_v_fp8_roundtrip_error_bound():
    g = torch.Generator().manual_seed(9)
    v = randn("HND", 1, 2, 300, 64, torch.bfloat16, g)
    v8, sc = oq.quant_v_fp8(v, "HND")
    assert v8.dtype == torch.float8_e4m3fn and sc.shape == (1, 2, 64)
    deq = v8.float() * sc[:, :, None, :]
    err = (deq - v.float()).abs()
    assert torch.all(err <= v.float().abs() * 2 ** -4 + sc[:, :, None, :] * 2 ** -9)
    assert torch.all(v8.float().abs().amax(dim=2) == 448.0)


def test_varlen_equals_per_sequence():
    g = torch.Generator().manual_seed(13)
    lens = [70, 129, 256, 1]
    cu = np.concatenate([[0], np.cumsum(lens)])
    q = torch.randn((sum(lens), 2, 64), generator=g).half()
    k = torch.randn((sum(lens), 1, 64), generator=g).half()
    qi, qs, ki, ks = oq.per_block_int8_varlen(q, k, cu, cu, BLKQ=128, BLKK=64)
    offq = oq.seq_block_offsets(cu, 128)
    assert offq.tolist() == [0, 1, 3, 5, 6]
    a, b, c, d = oq.per_block_int8(q[70:199].unsqueeze(0), k[70:199].unsqueeze(0), tensor_layout="NHD")
    assert torch.equal(qi[70:199], a[0]) and torch.equal(qs[:, 1:3], b[0])


def test_interleaved_q_scales_equal_the_tile_quantiser_applied_to_each_row_group():
    """Eight interleaved scales per block (the granularity upstream SageAttention calls per-thread; no code in the
    reference: parity unpinned): by definition the tile arithmetic of quant_per_block.py:38-46 on the rows r of a block
    with r % 8 == g.  The vectorised oracle is pinned against that row-group loop, ragged last block and empty groups
    included, and with one group it is the per-block quantiser."""
    rng = np.random.default_rng(5)
    x = rng.standard_normal((2, 3, 70, 64)).astype(np.float32) * np.float32(3.0)
    x[0, 1, 33] *= np.float32(40.0)                       # an outlier row only raises the scale of its own group
    for blk in (16, 32, 64, 128):
        q1, s1 = oq.quant_per_block_int8(x, blk, 0.3)
        q1b, s1b = oq.quant_per_block_int8(x, blk, 0.3, 1)
        assert np.array_equal(q1, q1b) and np.array_equal(s1, s1b)
        q8, s8 = oq.quant_per_block_int8(x, blk, 0.3, 8)
        nblk = (70 + blk - 1) // blk
        assert s8.shape == (2, 3, nblk * 8) and q8.shape == x.shape
        for b in range(2):
            for h in range(3):
                for t in range(nblk):
                    for g in range(8):
                        rows = [r for r in range(t * blk, min(70, (t + 1) * blk)) if r % 8 == g]
                        if not rows:
                            assert s8[b, h, t * 8 + g] == oq.SCALE_FLOOR
                            continue
                        qq, ss = oq.quant_tile_int8(x[b, h, rows], 0.3)
                        assert ss == s8[b, h, t * 8 + g] and np.array_equal(qq, q8[b, h, rows]), (blk, b, h, t, g)
    _, s8 = oq.quant_per_block_int8(x, 32, 0.3, 8)
    _, s1 = oq.quant_per_block_int8(x, 32, 0.3)
    assert s8[0, 1, 8 + 1] == s1[0, 1, 1] and (s8[0, 1, 8:16] <= s1[0, 1, 1]).all() and s8[0, 1, 8] < 0.2 * s1[0, 1, 1]


def test_four_interleaved_scales_equal_the_tile_quantiser_applied_to_each_key_group():
    """Four interleaved scales per block (scale t for the rows r with (r % 8) // 2 == t: upstream's per-thread K
    granularity; no code in the reference, parity unpinned): the vectorised oracle against the row-group loop."""
    rng = np.random.default_rng(6)
    x = rng.standard_normal((1, 2, 150, 64)).astype(np.float32)
    x[0, 1, 70:72] *= np.float32(50.0)
    for blk in (32, 64, 128):
        q4, s4 = oq.quant_per_block_int8(x, blk, 1.0, 4)
        nblk = (150 + blk - 1) // blk
        assert s4.shape == (1, 2, nblk * 4)
        for h in range(2):
            for t in range(nblk):
                for g in range(4):
                    rows = [r for r in range(t * blk, min(150, (t + 1) * blk)) if (r % 8) // 2 == g]
                    if not rows:
                        assert s4[0, h, t * 4 + g] == oq.SCALE_FLOOR
                        continue
                    qq, ss = oq.quant_tile_int8(x[0, h, rows], 1.0)
                    assert ss == s4[0, h, t * 4 + g] and np.array_equal(qq, q4[0, h, rows]), (blk, h, t, g)
    _, s4 = oq.quant_per_block_int8(x, 64, 1.0, 4)
    _, s1 = oq.quant_per_block_int8(x, 64, 1.0)
    assert s4[0, 1, 4 + 3] == s1[0, 1, 1] and s4[0, 1, 4 + 0] < 0.2 * s1[0, 1, 1]      # rows 70, 71: group 3 of block 1

