"""Writes tests/golden/ti_loss_kat.json: known answers for the reference's integer cross-entropy gradient
(ti_loss.py:5-36, everything before the final StoShift) derived WITHOUT torch, numpy or anything under oracle/.

Every float32 operation of the reference's sequence is modelled as the exact rational result followed by one
round-to-nearest-even to a 24-bit significand (what IEEE-754 binary32 prescribes for + - * / and for the
int64 -> float32 conversion); ``2 ** s`` is the correctly rounded float32 power, computed from a 60-digit
decimal evaluation.  Integer steps (the int64 sums of truncated values, the quadratic branch) are Python ints.
The first cases are small enough to follow with pencil and paper; their derivations are stored beside them.

Run:  python tests/golden/make_ti_loss_kat.py
"""
import json
import os
import random
from decimal import Decimal, getcontext
from fractions import Fraction

getcontext().prec = 60


def f32(q):
    """Round a rational to the nearest float32 (ties to even); normal range only."""
    q = Fraction(q)
    if q == 0:
        return q
    sign = -1 if q < 0 else 1
    a = abs(q)
    e = 0                       # find e with 2^23 <= a / 2^e < 2^24
    while a / Fraction(2) ** e >= 2 ** 24:
        e += 1
    while a / Fraction(2) ** e < 2 ** 23:
        e -= 1
    assert -126 - 23 <= e <= 127 - 23, "outside the normal float32 range"
    m = a / Fraction(2) ** e
    lo = m.numerator // m.denominator
    rem = m - lo
    if rem > Fraction(1, 2) or (rem == Fraction(1, 2) and lo % 2 == 1):
        lo += 1
    return sign * lo * Fraction(2) ** e


def trunc(q):
    q = Fraction(q)
    n = abs(q.numerator) // q.denominator
    return n if q >= 0 else -n


def pow2_f32(s):
    """Correctly rounded float32 value of 2**s for a rational s >= 0."""
    n = s.numerator // s.denominator
    f = s - n
    frac = Decimal(2) ** (Decimal(f.numerator) / Decimal(f.denominator)) if f != 0 else Decimal(1)
    return f32(Fraction(frac) * 2 ** n)


def pre_round(row, out_exp, target):
    """ti_loss.py:9-34 for one sample; returns (int32 values that StoShift receives, intermediate values)."""
    steps = {}
    if out_exp > -7:
        s = [f32(f32(v * 47274) / 32768) for v in row]                       # :14
        s = [f32(x * 2 ** out_exp) if out_exp >= 0 else f32(x / 2 ** (-out_exp)) for x in s]   # :15-18
        offset = f32(max(s) - 10)                                            # :20-21
        s = [max(f32(x - offset), Fraction(0)) for x in s]                   # :22-23
        g = [f32(pow2_f32(x) - 1) for x in s]                                # :24
        steps["s_minus_offset"] = [float(x) for x in s]
        out_sum = sum(trunc(x) for x in g)                                   # :31 (dtype=int64 truncates each term)
        scaled = [f32(f32(x * 2048) / f32(out_sum)) for x in g]              # :33
    else:
        g = [2 ** (1 - 2 * out_exp) + v * 2 ** (1 - out_exp) + v * v for v in row]   # :28-29, int64
        out_sum = sum(g)                                                     # :31
        scaled = [f32(f32(x * 2048) / f32(out_sum)) for x in g]              # :33 (int64 product, float32 quotient)
    steps["numerators"] = [float(x) for x in g]
    steps["out_sum"] = int(out_sum)
    tsum = sum(trunc(x) for x in scaled)                                     # :34
    steps["scaled"] = [float(x) for x in scaled]
    steps["scaled_int_sum"] = int(tsum)
    scaled[target] = f32(scaled[target] - f32(tsum))                         # :34 (float32 -= int64)
    return [int(trunc(x)) for x in scaled], steps                            # :35 .type(torch.int32)


HAND = [
    dict(name="quadratic branch, all logits zero", out_exp=-7, target=3, row=[0] * 10,
         derivation="each term 2^15 = 32768; sum 327680; 32768*2048/327680 = 204.8 -> truncates to 204; "
                    "sum of truncations 2040; target 204.8 - 2040 = -1835.2 -> -1835"),
    dict(name="quadratic branch, one logit 1, target on it", out_exp=-7, target=0, row=[1] + [0] * 9,
         derivation="terms 32768 + 256 + 1 = 33025 and 32768; sum 327937; 33025*2048/327937 = 206.24.., "
                    "32768*2048/327937 = 204.63..; truncations 206 + 9*204 = 2042; target 206.24 - 2042 = -1835.75.. -> -1835"),
    dict(name="quadratic branch, one logit 1, target elsewhere", out_exp=-7, target=1, row=[1] + [0] * 9,
         derivation="as above; target 204.63.. - 2042 = -1837.36.. -> -1837"),
    dict(name="quadratic branch, exponent -8, logits +-10", out_exp=-8, target=1, row=[10, -10] + [0] * 8,
         derivation="terms 2^17 + 10*2^9 + 100 = 136292, 2^17 - 5120 + 100 = 126052, 131072; sum 1310920"),
    dict(name="base-2 branch, all logits equal", out_exp=0, target=9, row=[5] * 10,
         derivation="s - (max - 10) = 10 for every class; 2^10 - 1 = 1023; sum 10230; 1023*2048/10230 = 204.8 -> 204; "
                    "target 204.8 - 2040 -> -1835"),
    dict(name="base-2 branch, exponent 14 makes s an integer (v * 23637 * 2), one logit above the rest, target on it",
         out_exp=14, target=0, row=[3] + [1] * 9,
         derivation="s = 141822, 47274; offset 141812; differences 10 and < 0 -> 0; 2^10 - 1 = 1023, 2^0 - 1 = 0; "
                    "sum 1023; 1023*2048/1023 = 2048; target 2048 - 2048 = 0"),
    dict(name="same, target elsewhere", out_exp=14, target=2, row=[3] + [1] * 9,
         derivation="as above; target 0 - 2048 = -2048"),
]


def main():
    rnd = random.Random(20240611)
    cases = []
    for h in HAND:
        exp, steps = pre_round(h["row"], h["out_exp"], h["target"])
        cases.append(dict(h, expected=exp, steps=steps))
    # rows whose float32 steps round (not hand-checkable; exact-rational model above)
    for out_exp in (-6, -3, -1, 0, 1, 2, 5):
        for spread in (3, 12, 127):
            row = [rnd.randint(-spread, spread) for _ in range(10)]
            target = rnd.randrange(10)
            exp, steps = pre_round(row, out_exp, target)
            cases.append(dict(name="exact-rational model", out_exp=out_exp, target=target, row=row, expected=exp, steps=steps))
    for out_exp in (-7, -8, -10, -12):
        row = [rnd.randint(-127, 127) for _ in range(10)]
        target = rnd.randrange(10)
        exp, steps = pre_round(row, out_exp, target)
        cases.append(dict(name="exact-rational model, quadratic branch", out_exp=out_exp, target=target, row=row, expected=exp,
                          steps=steps))
    out = dict(_comment="Known answers for ti_loss.py:5-34 (the int32 tensor StoShift receives). Written by make_ti_loss_kat.py "
                        "with exact rational arithmetic and explicit float32 rounding; no torch, no oracle code involved. "
                        "`steps` are intermediate values for checking by hand.",
               cases=cases)
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "ti_loss_kat.json")
    with open(path, "w") as f:
        json.dump(out, f, indent=1)
    print("wrote", path, len(cases), "cases")


if __name__ == "__main__":
    main()
