"""Pins the two oracle statements of NITI's integer rounding (ti_torch.py:23-147,366-377):
hand-derived known answers, exhaustive cross-check literal-torch vs closed-form C, and
properties a dropped term / wrong sign would break."""
import numpy as np
import pytest
import torch

from oracle import c_oracle as co
from oracle import niti_oracle as po

MODES = [("floor", False), ("trunc", True)]


def T(v, dt=torch.int32):
    return torch.tensor(v, dtype=dt)


@pytest.mark.parametrize("mode,trunc", MODES)
def test_kat_round_psto_sto(kat, mode, trunc):
    X = T(kat["X"])
    assert po.RoundShift(X, 7, mode).tolist() == kat[f"round_s7_{mode}"]
    assert co.round_shift(X, 7, trunc).tolist() == kat[f"round_s7_{mode}"]
    X1 = T(kat["X_s1"])
    assert po.RoundShift(X1, 1, mode).tolist() == kat[f"round_s1_{mode}"]
    assert co.round_shift(X1, 1, trunc).tolist() == kat[f"round_s1_{mode}"]
    assert po.PstoShift(X, 7, mode).tolist() == kat[f"psto_s7_{mode}"]
    assert co.psto_shift(X, 7, trunc).tolist() == kat[f"psto_s7_{mode}"]
    r20 = torch.arange(-20, 21, dtype=torch.int32)
    assert po.PstoShift(r20, 4, mode).tolist() == kat[f"psto_s4_m20_20_{mode}"]
    assert co.psto_shift(r20, 4, trunc).tolist() == kat[f"psto_s4_m20_20_{mode}"]
    r5 = torch.arange(-5, 6, dtype=torch.int32)
    assert po.PstoShift(r5, 1, mode).tolist() == kat[f"psto_s1_m5_5_{mode}"]
    assert co.psto_shift(r5, 1, trunc).tolist() == kat[f"psto_s1_m5_5_{mode}"]
    u7 = torch.full_like(r20, 7)
    assert po.StoShift(r20, 4, u7, mode).tolist() == kat[f"sto_s4_u7_m20_20_{mode}"]
    assert co.sto_shift(r20, 4, u7, trunc).tolist() == kat[f"sto_s4_u7_m20_20_{mode}"]


def test_kat_bitwidth(kat):
    for r, bw in kat["bitwidth_int"].items():
        assert po.bitwidth_int(int(r)) == bw
        assert co.bitwidth_int(int(r)) == bw
    for r, bw in kat["bitwidth_f32"].items():
        assert po.bitwidth_f32(int(r)) == bw            # literal torch CPU evaluation
        assert po.bitwidth_f32_model(int(r)) == bw      # integer model the HIP path uses


def test_bitwidth_forms_agree_outside_band():
    # the float form equals the integer form for every r < 2^21 ...
    rs = np.unique(np.concatenate([np.arange(0, 70000), 2 ** np.arange(1, 21), 2 ** np.arange(1, 21) + 1,
                                   2 ** np.arange(1, 21) - 1, np.random.default_rng(0).integers(1, 2 ** 21, 20000)]))
    v = torch.from_numpy(rs.astype(np.int64)).float()
    lit = torch.where(v == 0, torch.zeros_like(v), torch.ceil(torch.log2(torch.clamp(v, min=1)))).to(torch.int64).tolist()
    for r, l in zip(rs.tolist(), lit):
        assert po.bitwidth_int(r) == l, r
        assert po.bitwidth_f32_model(r) == l, r
    # ... and the integer model of the float form tracks torch's log2 inside the band
    for k in range(21, 31):
        for d in range(0, 40):
            r = 2 ** k + d
            assert po.bitwidth_f32_model(r) == po.bitwidth_f32(r), (k, d)
            r = 2 ** k - d - 1
            assert po.bitwidth_f32_model(r) == po.bitwidth_f32(r), (k, -d - 1)


@pytest.mark.parametrize("mode,trunc", MODES)
def test_exhaustive_python_vs_c(mode, trunc):
    x = torch.arange(-2 ** 15, 2 ** 15 + 1, dtype=torch.int32)
    g = torch.Generator().manual_seed(7)
    for s in range(1, 13):
        assert torch.equal(po.RoundShift(x, s, mode), co.round_shift(x, s, trunc)), s
        assert torch.equal(po.PstoShift(x, s, mode), co.psto_shift(x, s, trunc)), s
        u = torch.randint(0, 2 ** s, x.shape, generator=g, dtype=torch.int32)
        assert torch.equal(po.StoShift(x, s, u, mode), co.sto_shift(x, s, u, trunc)), s
    # large magnitudes, large shifts
    xl = torch.randint(-2 ** 31 + 1, 2 ** 31 - 1, (200000,), generator=g, dtype=torch.int64).to(torch.int32)
    for s in (13, 17, 20, 24):
        assert torch.equal(po.RoundShift(xl, s, mode), co.round_shift(xl, s, trunc))
        assert torch.equal(po.PstoShift(xl, s, mode), co.psto_shift(xl, s, trunc))
        u = torch.randint(0, 2 ** s, xl.shape, generator=g, dtype=torch.int32)
        assert torch.equal(po.StoShift(xl, s, u, mode), co.sto_shift(xl, s, u, trunc))


def test_round_shift_is_textbook_rounding():
    # floor mode == round-half-up of x / 2^s; trunc mode == round-half-away-from-zero
    x = torch.arange(-5000, 5001, dtype=torch.int32)
    for s in range(1, 9):
        exact = x.double() / 2 ** s
        up = torch.floor(exact + 0.5).clamp(-127, 127).to(torch.int8)
        away = (torch.sign(exact) * torch.floor(exact.abs() + 0.5)).clamp(-127, 127).to(torch.int8)
        assert torch.equal(po.RoundShift(x, s, "floor"), up)
        assert torch.equal(po.RoundShift(x, s, "trunc"), away)


@pytest.mark.parametrize("mode", ["floor", "trunc"])
def test_sto_extremes_and_ranges(mode):
    x = torch.arange(-3000, 3001, dtype=torch.int32)
    for s in (1, 3, 6):
        q = torch.div(x, 2 ** s, rounding_mode=mode)
        rem = (x - q * 2 ** s).abs()
        top = torch.full_like(x, 2 ** s - 1)
        # u = 2^s - 1: never bumps
        assert torch.equal(po.StoShift(x, s, top, mode), q.clamp(-127, 127).to(torch.int8))
        # u = 0: bumps away from zero (sign of x) iff any bit was dropped
        bump = (rem > 0).to(torch.int32) * torch.sign(x)
        assert torch.equal(po.StoShift(x, s, torch.zeros_like(x), mode), (q + bump).clamp(-127, 127).to(torch.int8))
        for f in (po.RoundShift, po.PstoShift):
            y = f(x, s, mode)
            assert int(y.min()) >= -127 and int(y.max()) <= 127
        # non-negative inputs do not depend on the division mode
        pos = x[x >= 0]
        assert torch.equal(po.RoundShift(pos, s, "floor"), po.RoundShift(pos, s, "trunc"))
        assert torch.equal(po.PstoShift(pos, s, "floor"), po.PstoShift(pos, s, "trunc"))


def test_sto_is_unbiased_in_trunc_mode():
    # averaged over all u in [0, 2^s), trunc-mode StoShift reproduces x / 2^s exactly
    s = 4
    x = torch.arange(-200, 201, dtype=torch.int32)
    acc = torch.zeros(x.shape, dtype=torch.float64)
    for u in range(2 ** s):
        acc += po.StoShift(x, s, torch.full_like(x, u), "trunc").double()
    assert torch.allclose(acc / 2 ** s, x.double() / 2 ** s)


@pytest.mark.parametrize("mode,trunc", MODES)
def test_calc_wrappers(mode, trunc):
    g = torch.Generator().manual_seed(3)
    # all-zero tensor: bitwidth 0, plain cast, exponent untouched
    z = torch.zeros(33, dtype=torch.int32)
    y, e = po.act_calc(z, -5, div_mode=mode)
    assert torch.equal(y, z.to(torch.int8)) and e == -5
    y, sft = po.grad_calc(z, 5, div_mode=mode)
    assert torch.equal(y, z.to(torch.int8)) and sft == 0
    # max |x| == 128: bitwidth 7, shift 0, 128 wraps to -128
    w = T([128, -128, 127, 5, -3])
    y, e = po.act_calc(w, 2, div_mode=mode)
    assert y.tolist() == [-128, -128, 127, 5, -3] and e == 2
    yc, sc = co.requant(w, 7, "round", trunc)
    assert yc.tolist() == y.tolist() and sc == 0
    # max |x| == 129: bitwidth 8, shift 1
    w = T([129, -129, 1, -1, 0])
    y, s1 = po.err_calc(w, div_mode=mode)
    assert s1 == 1 and y.tolist() == ([65, -64, 1, 0, 0] if mode == "floor" else [65, -65, 1, -1, 0])
    # grad: bitwidth <= mu keeps the values
    gsmall = T([31, -32, 7])
    y, sft = po.grad_calc(gsmall, 5, div_mode=mode)
    assert y.tolist() == [31, -32, 7] and sft == 0
    # random tensors: python composition == C composition for every method
    for hi in (100, 300, 40000, 3000000):
        x = torch.randint(-hi, hi + 1, (4097,), generator=g, dtype=torch.int32)
        for tgt, fn in ((7, "act"), (5, "grad"), (3, "grad")):
            for method in ("round", "psto", "sto"):
                bw = po.RangeEstimate(x)
                s = max(bw - tgt, 0)
                u = torch.randint(0, 2 ** max(s, 1), x.shape, generator=g, dtype=torch.int32)
                if fn == "act":
                    yp, ep = po.act_calc(x, 0, method, mode, u)
                else:
                    yp, ep = po.grad_calc(x, tgt, method, mode, u)
                yc, sc = co.requant(x, tgt, method, trunc, u)
                assert torch.equal(yp, yc) and ep == sc == s
                if fn == "grad" and s >= 1:
                    assert int(yp.abs().max()) <= 2 ** tgt


def test_weight_update():
    w = T([127, -127, 0, 100, -100, 5], torch.int8)
    g = T([-32, 32, 7, -32, 32, 5], torch.int8)
    exp = [127, -127, -7, 127, -127, 0]
    assert po.weight_update(w, g).tolist() == exp
    assert co.weight_update(w, g).tolist() == exp
    a = torch.arange(-127, 128, dtype=torch.int16)
    ww, gg = torch.meshgrid(a, a, indexing="ij")
    out = po.weight_update(ww.to(torch.int8), gg.to(torch.int8))
    assert torch.equal(out.to(torch.int16), (ww - gg).clamp(-127, 127))
    assert torch.equal(out, co.weight_update(ww.to(torch.int8).contiguous(), gg.to(torch.int8).contiguous()))
    assert int(out.min()) == -127


def test_f32_roundtrip_special_cases():
    x = T([0, 1, -1, 2 ** 24, 2 ** 24 + 1, 2 ** 24 + 3, -(2 ** 24 + 1), -(2 ** 24 + 3), 2 ** 31 - 1, -2 ** 31,
           2 ** 31 - 64, 2 ** 31 - 65, 123456789])
    want = [0, 1, -1, 2 ** 24, 2 ** 24, 2 ** 24 + 4, -(2 ** 24), -(2 ** 24 + 4), 2 ** 31 - 1, -2 ** 31,
            2 ** 31 - 1, 2 ** 31 - 128, 123456792]
    assert po.f32_roundtrip(x).tolist() == want
    assert co.f32_roundtrip(x).tolist() == want
    g = torch.Generator().manual_seed(5)
    small = torch.randint(-2 ** 24, 2 ** 24 + 1, (100000,), generator=g, dtype=torch.int32)
    assert torch.equal(po.f32_roundtrip(small), small)           # identity below 2^24
    big = torch.randint(-2 ** 31, 2 ** 31 - 1, (100000,), generator=g, dtype=torch.int64).to(torch.int32)
    assert torch.equal(po.f32_roundtrip(big), co.f32_roundtrip(big))
