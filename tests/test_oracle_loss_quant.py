"""CPU pins for the oracle's integer cross-entropy gradient and float -> int8 quantisers.

The expected values come from tests/golden/ti_loss_kat.json (exact rational arithmetic with explicit float32
rounding, written by tests/golden/make_ti_loss_kat.py without torch or oracle code; the first rows are worked
by hand) and tests/golden/quantize_kat.json (hand-derived).  A wrong constant (47274, the offset 10, 2^15, 2^11),
a missing truncation or a transposed operand changes at least one of them."""
import json
import math
import os
from decimal import Decimal, getcontext
from fractions import Fraction

import numpy as np
import pytest
import torch

from oracle import c_oracle as co
from oracle import niti_oracle as po

HERE = os.path.dirname(os.path.abspath(__file__))


def _load(name):
    with open(os.path.join(HERE, "golden", name)) as f:
        return json.load(f)


def test_ti_loss_known_answers():
    cases = _load("ti_loss_kat.json")["cases"]
    assert len(cases) >= 30
    branches = set()
    for c in cases:
        out = torch.tensor([c["row"]], dtype=torch.int8)
        tgt = torch.tensor([c["target"]])
        want = c["expected"]
        assert po.ti_loss_pre_round(out, c["out_exp"], tgt).tolist()[0] == want, c["name"]
        assert co.ti_loss_pre_round(out, c["out_exp"], tgt).tolist()[0] == want, c["name"]
        branches.add(c["out_exp"] > -7)
        # softmax minus one-hot, scaled by 2^11: the columns add up to about zero, the target is the only negative one
        assert want[c["target"]] <= 0 and all(v >= 0 for i, v in enumerate(want) if i != c["target"])
        assert abs(sum(want)) <= len(want)
    assert branches == {True, False}


def test_ti_loss_hand_rows():
    """The rows that can be followed with pencil and paper, written out here once more."""
    t = lambda row, e, k: po.ti_loss_pre_round(torch.tensor([row], dtype=torch.int8), e, torch.tensor([k])).tolist()[0]
    assert t([0] * 10, -7, 3) == [204, 204, 204, -1835] + [204] * 6
    assert t([1] + [0] * 9, -7, 0) == [-1835] + [204] * 9
    assert t([1] + [0] * 9, -7, 1) == [206, -1837] + [204] * 8
    assert t([5] * 10, 0, 9) == [204] * 9 + [-1835]
    assert t([3] + [1] * 9, 14, 0) == [0] * 10
    assert t([3] + [1] * 9, 14, 2) == [2048, 0, -2048] + [0] * 7


def test_ti_loss_python_and_c_agree_on_random_batches():
    g = torch.Generator().manual_seed(99)
    for e in (-12, -9, -7, -6, -4, -3, -1, 0, 1, 3, 7):
        for spread in (4, 30, 127):
            out = torch.randint(-spread, spread + 1, (64, 10), generator=g, dtype=torch.int8)
            tgt = torch.randint(0, 10, (64,), generator=g)
            a, b = po.ti_loss_pre_round(out, e, tgt), co.ti_loss_pre_round(out, e, tgt)
            assert torch.equal(a, b), (e, spread)
            u = torch.randint(0, 16, (64, 10), generator=g, dtype=torch.int32)
            for dm in ("floor", "trunc"):
                err, ee = po.ti_loss(out, e, tgt, u, dm)
                assert ee == 0 and torch.equal(err, co.sto_shift(a, 4, u, dm == "trunc"))


def test_exp2_contract_is_the_correctly_rounded_power():
    """The fixed double sequence against a 50-digit decimal evaluation rounded once to float32, on integers, on
    arguments of the kind the loss produces (multiples of 2^-15 up to 10) and on random float32 values."""
    getcontext().prec = 50
    g = torch.Generator().manual_seed(5)
    vals = [0.0, 1.0, 2.0, 10.0, 0.5, 0.25, 9.999969482421875, 1.442718505859375]
    vals += [float(v) / 32768.0 for v in torch.randint(0, 327680, (300,), generator=g).tolist()]
    vals += torch.rand(300, generator=g).mul(24).tolist()
    s = torch.tensor(vals, dtype=torch.float32)
    got = po.exp2_contract(s)
    for v, r in zip(s.tolist(), got.tolist()):
        exact = Fraction(Decimal(2) ** Decimal(v))      # v is a float32, exactly representable as a decimal
        want = float(np.float32(float(exact)))          # double rounding is harmless at 50 digits vs 2^-29 spacing
        lo, hi = np.nextafter(np.float32(want), np.float32(0)), np.nextafter(np.float32(want), np.float32(np.inf))
        assert abs(Fraction(r) - exact) <= min(abs(Fraction(float(lo)) - exact), abs(Fraction(float(hi)) - exact)), v
        assert r == want, v
        assert co.exp2_contract(v) == r, v
    assert po.exp2_contract(torch.tensor([3.0, 10.0])).tolist() == [8.0, 1024.0]


def test_float_to_int8_known_answers():
    for c in _load("quantize_kat.json")["float_to_int8"]:
        x = torch.tensor(c["x"], dtype=torch.float32)
        assert x.double().tolist() == c["x"], "inputs must be exact float32 values: " + c["name"]
        q, e = po.float_to_int8(x)
        assert q.tolist() == c["q"] and e == c["exp"], c["name"]
        qc, ec = co.float_to_int8(x)
        assert qc.tolist() == c["q"] and ec == c["exp"], c["name"]


def test_weight_quant_known_answers():
    for c in _load("quantize_kat.json")["weight_quant"]:
        w = torch.tensor(c["w"], dtype=torch.float32)
        q, e = po.weight_quant(w)
        assert q.tolist() == c["q"] and e == c["exp"], c["name"]
        qc, ec = co.weight_quant(w)
        assert qc.tolist() == c["q"] and ec == c["exp"], c["name"]


def test_quantisers_python_and_c_agree_and_respect_their_invariants():
    g = torch.Generator().manual_seed(6)
    for scale in (1e-3, 0.3, 1.0, 2.5, 100.0, 3e4):
        x = torch.randn(4, 3, 9, 7, generator=g) * scale
        q, e = po.float_to_int8(x)
        qc, ec = co.float_to_int8(x)
        assert torch.equal(q, qc) and e == ec
        # the largest magnitude lands in (64, 128]: the range uses the top bit
        assert 64 <= int(q.to(torch.int16).abs().max()) <= 128
        # dequantised values are within half a step of the input (or clamped at the top)
        step = 2.0 ** e
        assert float((q.float() * step - x).abs().max()) <= 1.0 * step
        y, ey = po.quantize_input_nhwc(x)
        assert ey == e and torch.equal(y, q.permute(0, 2, 3, 1)) and y.is_contiguous()
        w, ew = po.weight_quant(x)
        wc, ewc = co.weight_quant(x)
        assert torch.equal(w, wc) and ew == ewc == e
        assert int(w.to(torch.int16).abs().max()) == 127


def test_ceil_log2_of_a_float():
    for r, want in ((1.0, 0), (2.0, 1), (3.0, 2), (4.0, 2), (4.000000476837158, 3), (0.5, -1), (0.75, 0), (0.2, -2),
                    (16.000001907348633, 5), (1e-3, -9), (2.0 ** -20, -20), (65536.0, 16)):
        assert po.ceil_log2_f32(r) == want, r
        assert int(co.lib().nito_ceil_log2_f32(__import__("ctypes").c_float(r))) == want, r
    # against exact integer arithmetic on random float32 values
    g = torch.Generator().manual_seed(7)
    for v in (torch.rand(200, generator=g) * 1000 + 1e-4).tolist():
        f = Fraction(float(np.float32(v)))
        k = po.ceil_log2_f32(v)
        assert Fraction(2) ** (k - 1) < f <= Fraction(2) ** k


def test_float_log2_band_documented():
    """Where the reference's float32 ceil(log2 r) deviates from the exact value: first float32 above 2^k, k >= 4."""
    r = float(np.nextafter(np.float32(16.0), np.float32(32.0)))
    assert po.ceil_log2_f32(r) == 5
    x = torch.tensor([r, 1.0])
    q_exact, e_exact = po.float_to_int8(x, log2_mode="exact")
    assert (q_exact.tolist(), e_exact) == ([64, 4], -2)
    q_f32, e_f32 = po.float_to_int8(x, log2_mode="f32")
    assert (e_f32, q_f32.tolist()) in ((-2, [64, 4]), (-3, [127, 8]))   # a correctly rounded log2f gives the second
    r2 = float(np.nextafter(np.float32(4.0), np.float32(8.0)))           # below 16 there is no such band
    assert po.float_to_int8(torch.tensor([r2]), log2_mode="f32")[1] == po.float_to_int8(torch.tensor([r2]))[1] == -4
