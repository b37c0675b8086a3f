"""CPU oracle for NITI's int8 hot path -- TEST INFRASTRUCTURE, NOT PRODUCT CODE.

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may import this
module.  The shipped package (niti_amd) never does: its ops fail loudly when the HIP
library is missing instead of falling back to anything in here.

Everything runs on torch CPU tensors / numpy.  Each function restates one function of
the reference (path given relative to the reference checkout) and says which line range
it follows.  Two independent statements exist for the integer rounding helpers:

  * this file: the *literal* torch elementwise sequence the reference executes
    (``//``, ``*``, ``-``, ``torch.where`` ...) evaluated on CPU int32 tensors, with the
    division made explicit (``floor`` = what ``//`` does on torch >= 1.13, ``trunc`` =
    what it did on torch <= 1.12, the version the reference's Dockerfile pins);
  * oracle/niti_oracle.c: closed forms written with shifts and masks.

tests/test_oracle_*.py pins both against hand-checkable known answers, against each
other exhaustively, and against library routines (torch CPU conv2d / _int_mm /
max_pool2d, torch.nn.grad.*), adjoint identities and brute-force loops.

Pin status per function (what fixes the result, besides the source text):
  conv2d_fprop_i32        library routine (F.conv2d int32/fp64) + brute force + invariants
  conv2d_dgrad_i32        reference's own flip/transpose identity + adjoint identity + torch.nn.grad
  conv2d_wgrad_i32        reference's own transpose identity + adjoint identity + torch.nn.grad
  f32_roundtrip           closed form + special cases (2^24+1, 2^24+3, INT32_MAX)
  int8mm                  torch._int_mm + numpy int64 matmul
  bitwidth_int / _f32     known answers r->bw; f32 form checked against torch.log2 on CPU
  RoundShift/StoShift/PstoShift   hand-derived known-answer tables (both division modes)
  act_calc/err_calc/grad_calc     composition + special cases (all-zero, 128 wrap, bw<=mu)
  weight_update           closed form, saturation
  maxpool fwd             F.max_pool2d int8 + brute force
  maxpool bwd             unique maxima: closed form.  TIES: parity unpinned (cuDNN's rule is
                          closed source); rule chosen here = first maximum in (kh,kw) scan
                          order (= torch CPU), "all" kept as a switchable alternative.
  ti_loss                 known answers of tests/golden/ti_loss_kat.json (exact rational arithmetic with
                          explicit float32 rounding, hand-worked rows for both exponent branches) + the
                          plain-C statement.  ``2 ** s`` follows exp2_contract (a fixed sequence of double
                          operations = the correctly rounded float32 power on every tested argument); the
                          reference's own result there depends on its platform's powf by an ulp.
  float_to_int8 / weight_quant   hand-derived known answers (tests/golden/quantize_kat.json: ranges at and
                          next to powers of two, half-way ties, both clamps) + the plain-C statement.
                          ceil(log2 r) is exact arithmetic on the float; the reference's float32 log2
                          rounds to the lower integer for the first float32 values above 2^k, k >= 4.
The reference holds no tests, golden vectors or fixtures for any of these.
"""
from __future__ import annotations

import math
from typing import Optional, Tuple

import numpy as np
import torch
import torch.nn.functional as F

BITWIDTH = 7  # ti_torch.py:458

FLOOR = "floor"
TRUNC = "trunc"


# --------------------------------------------------------------------------------------
# integer division by a power of two, both historical meanings of torch's ``//``
# --------------------------------------------------------------------------------------
def _idiv(x: torch.Tensor, d: int, div_mode: str) -> torch.Tensor:
    if div_mode == FLOOR:
        return torch.div(x, d, rounding_mode="floor")
    if div_mode == TRUNC:
        return torch.div(x, d, rounding_mode="trunc")
    raise ValueError(div_mode)


def int8_clip(x: torch.Tensor, clip_val: int = 127) -> torch.Tensor:
    """ti_torch.py:71-72."""
    return torch.clamp(x, -clip_val, clip_val).to(torch.int8)


def RoundShift(x: torch.Tensor, shift: int, div_mode: str = FLOOR) -> torch.Tensor:
    """ti_torch.py:23-31 (round to nearest by looking at the first dropped bit)."""
    q = _idiv(x, 2 ** shift, div_mode)
    rem = x - q * (2 ** shift)
    bump = _idiv(rem, 2 ** (shift - 1), div_mode)
    return int8_clip(q + bump)


def StoShift(x: torch.Tensor, shift: int, rand: torch.Tensor, div_mode: str = FLOOR) -> torch.Tensor:
    """ti_torch.py:33-46.  ``rand`` replaces the device ``torch.randint(0, 2**shift)`` of
    line 41 so both sides of a parity test consume identical random bits."""
    q = _idiv(x, 2 ** shift, div_mode)
    rem = torch.abs(x - q * (2 ** shift))
    bump = torch.where(rem <= rand.to(x.dtype), torch.zeros_like(x), torch.ones_like(x))
    bump = bump * torch.sign(x)
    return int8_clip(q + bump)


def PstoShift(x: torch.Tensor, shift: int, div_mode: str = FLOOR) -> torch.Tensor:
    """ti_torch.py:48-69 (low half of the dropped bits acts as the random number)."""
    q = _idiv(x, 2 ** shift, div_mode)
    rem = torch.abs(x - q * (2 ** shift))
    half = shift // 2
    hi = _idiv(rem, 2 ** half, div_mode)          # rem >= 0: both modes agree
    lo = rem - hi * (2 ** half)
    if shift % 2 == 1:
        lo = lo * 2
    bump = torch.where(hi <= lo, torch.zeros_like(x), torch.ones_like(x))
    bump = bump * torch.sign(x)
    return int8_clip(q + bump)


ROUND_METHODS = {"round": RoundShift, "sto": StoShift, "psto": PstoShift}


# --------------------------------------------------------------------------------------
# range estimate
# --------------------------------------------------------------------------------------
def bitwidth_int(r: int) -> int:
    """Exact integer form of ceil(log2(r)) for r >= 1, 0 for r == 0:  bit_length(r-1)."""
    r = int(r)
    return 0 if r <= 0 else (r - 1).bit_length()


def bitwidth_f32(r: int) -> int:
    """ti_torch.py:366-377 evaluated literally with torch CPU fp32 ops:
    ``int(ceil(log2(float32(r))))``.  Differs from bitwidth_int only for r slightly above
    a power of two >= 2^21 and for r >= 2^24 (fp32 rounding of r itself)."""
    if int(r) == 0:
        return 0
    v = torch.tensor(int(r), dtype=torch.int64).float()
    return int(torch.ceil(torch.log2(v)))


def bitwidth_f32_model(r: int) -> int:
    """Integer-only model of bitwidth_f32 under a correctly rounded log2f: convert r to fp32
    (round-to-nearest-even), split into 2^e * (1 + j*2^-23); fl(e + log2(1+j*2^-23)) == e
    iff the fraction is below half an ulp of e.  This is what the HIP path implements for
    bitwidth mode "f32"."""
    r = int(r)
    if r == 0:
        return 0
    f = np.float32(r)
    bits = int(np.frombuffer(np.float32(f).tobytes(), dtype=np.uint32)[0])
    e = ((bits >> 23) & 0xFF) - 127
    j = bits & 0x7FFFFF
    if j == 0:
        return e
    if e <= 0:
        return e + 1
    # ulp(e) for e in [2^t, 2^(t+1)) is 2^(t-23); e + log2(m) rounds back down to e iff
    # log2(m) < ulp(e)/2 (log2 of a non-power-of-two rational is irrational: no ties).
    t = e.bit_length() - 1
    half_ulp = 2.0 ** (t - 24)
    return e if (1.0 + j * 2.0 ** -23) < 2.0 ** half_ulp else e + 1   # doubles are ample here


def absmax(x: torch.Tensor) -> int:
    if x.numel() == 0:
        return 0
    return int(torch.max(torch.abs(x.to(torch.int64))))


def RangeEstimate(x: torch.Tensor, bw_mode: str = "int") -> int:
    """ti_torch.py:369-377."""
    r = absmax(x)
    if bw_mode == "int":
        return bitwidth_int(r)
    if bw_mode == "f32":
        return bitwidth_f32(r)
    raise ValueError(bw_mode)


# --------------------------------------------------------------------------------------
# requantisation wrappers
# --------------------------------------------------------------------------------------
def _apply_round(method: str, acc: torch.Tensor, shift: int, div_mode: str, rand):
    if method == "sto":
        return StoShift(acc, shift, rand, div_mode)
    return ROUND_METHODS[method](acc, shift, div_mode)


def _wrap_i8(acc: torch.Tensor) -> torch.Tensor:
    """``int32.type(torch.int8)``: keeps the low byte (128 -> -128)."""
    return acc.to(torch.int32).to(torch.int8)


def act_calc(acc, exp_in, method="round", div_mode=FLOOR, rand=None, bw_mode="int"):
    """ti_torch.py:103-117.  Returns (int8 tensor, exp_out)."""
    shift = RangeEstimate(acc, bw_mode) - BITWIDTH
    if shift > 0:
        return _apply_round(method, acc, shift, div_mode, rand), exp_in + shift
    return _wrap_i8(acc), exp_in


def err_calc(acc, method="round", div_mode=FLOOR, rand=None, bw_mode="int"):
    """ti_torch.py:119-133.  Returns (int8 tensor, shift or 0)."""
    shift = RangeEstimate(acc, bw_mode) - BITWIDTH
    if shift > 0:
        return _apply_round(method, acc, shift, div_mode, rand), shift
    return _wrap_i8(acc), 0


def grad_calc(acc, mu, method="psto", div_mode=FLOOR, rand=None, bw_mode="int"):
    """ti_torch.py:135-147.  Returns (int8 tensor, shift or 0)."""
    bw = RangeEstimate(acc, bw_mode)
    shift = bw - mu
    if bw == 0:
        return torch.zeros(acc.shape, dtype=torch.int8), 0
    if shift < 1:
        return _wrap_i8(acc), 0
    return _apply_round(method, acc, shift, div_mode, rand), shift


def weight_update(w: torch.Tensor, g: torch.Tensor) -> torch.Tensor:
    """ti_torch.py:21: w <- clip(int16(w) - int16(g), +-127)."""
    return int8_clip(w.to(torch.int16) - g.to(torch.int16))


# --------------------------------------------------------------------------------------
# convolution / GEMM (int32 results)
# --------------------------------------------------------------------------------------
def f32_roundtrip(acc: torch.Tensor) -> torch.Tensor:
    """CUTLASS LinearCombinationClamp<int32, 4, int32, float> with alpha=1, beta=0
    (pytorch/cutlass-extension/cutlassconv_kernel.cu:78-85,159 and
    include/cutlass/epilogue/thread/linear_combination_clamp.h:371-389):
    int32 -> fp32 (RNE) -> clamp to [INT32_MIN, INT32_MAX as float] -> round-to-nearest int32
    with saturation."""
    f = acc.to(torch.int64).to(torch.float32)
    d = f.to(torch.float64)
    d = torch.clamp(d, -2147483648.0, 2147483647.0)
    return d.to(torch.int64).clamp(-2147483648, 2147483647).to(torch.int32)


def _nhwc_to_nchw(x):
    return x.permute(0, 3, 1, 2)


def conv2d_fprop_i32(x: torch.Tensor, w: torch.Tensor, stride: int = 1, padding: int = 1,
                     check_overflow: bool = True) -> torch.Tensor:
    """Cross-correlation of NHWC int8 ``x`` with KRSC int8 ``w`` -> NPQK int32
    (cutlassconv_kernel.cu:107-148; index math
    conv2d_fprop_activation_tile_access_iterator_analytic.h:182-211)."""
    xi = _nhwc_to_nchw(x).to(torch.int32).contiguous()
    wi = _nhwc_to_nchw(w).to(torch.int32).contiguous()
    if check_overflow:
        # the MFMA accumulator wraps where the reference's mma.sync saturates: make sure no
        # test input can reach either.  |acc| <= sum |x||w| <= 127*127*R*S*C.
        bound = int(torch.max(torch.abs(xi))) * int(torch.max(torch.abs(wi))) * w.shape[1] * w.shape[2] * w.shape[3] \
            if x.numel() and w.numel() else 0
        assert bound < 2 ** 31, "int32 accumulator could overflow on this input"
    y = F.conv2d(xi, wi, stride=stride, padding=padding)
    return y.permute(0, 2, 3, 1).contiguous()


def conv2d_fprop_loops(x: torch.Tensor, w: torch.Tensor, stride: int = 1, padding: int = 1) -> torch.Tensor:
    """Brute-force definition y[n,p,q,k] = sum_{r,s,c} x[n,p*st-pad+r,q*st-pad+s,c] * w[k,r,s,c]
    in int64 numpy; tiny shapes only."""
    xn = x.numpy().astype(np.int64)
    wn = w.numpy().astype(np.int64)
    N, H, W, C = xn.shape
    K, R, S, _ = wn.shape
    P = (H + 2 * padding - R) // stride + 1
    Q = (W + 2 * padding - S) // stride + 1
    y = np.zeros((N, P, Q, K), dtype=np.int64)
    for n in range(N):
        for p in range(P):
            for q in range(Q):
                for r in range(R):
                    h = p * stride - padding + r
                    if h < 0 or h >= H:
                        continue
                    for s in range(S):
                        ww = q * stride - padding + s
                        if ww < 0 or ww >= W:
                            continue
                        y[n, p, q, :] += wn[:, r, s, :] @ xn[n, h, ww, :]
    return torch.from_numpy(y)


def conv2d_int8(x, w, stride=1, padding=1, f32_epilogue=True):
    """ti_torch.py:178-192 -> sp_conv[_optimized]: zero-pad C to a multiple of 16 (a no-op on
    the result), fprop, then the fp32 round trip of the CUTLASS epilogue."""
    if x.shape[3] % 16 != 0:
        padc = 16 - x.shape[3] % 16
        x = F.pad(x, (0, padc))
        w = F.pad(w, (0, padc))
    y = conv2d_fprop_i32(x, w, stride, padding)
    return f32_roundtrip(y) if f32_epilogue else y


def dgrad_weight(w: torch.Tensor) -> torch.Tensor:
    """ti_torch.py:404: flip the taps and swap in/out channels (KRSC -> CRSK)."""
    return torch.flip(w, [1, 2]).transpose(0, 3).contiguous()


def conv2d_dgrad_i32(err, w, stride=1, padding=1, f32_epilogue=True):
    """ti_torch.py:403-405: dgrad expressed as fprop of the error with flipped/transposed
    weights.  A true dgrad only for stride 1 and 2*padding == R-1."""
    return conv2d_int8(err, dgrad_weight(w), stride, padding, f32_epilogue)


def conv2d_dgrad_def(err, w, H, W, stride=1, padding=1):
    """Definition: dx[n,h,w,c] = sum_{p,q,r,s,k : h=p*st-pad+r, w=q*st-pad+s} err[n,p,q,k] w[k,r,s,c]
    via torch.nn.grad.conv2d_input in fp64 (exact for these magnitudes)."""
    e = _nhwc_to_nchw(err).double().contiguous()
    wi = _nhwc_to_nchw(w).double().contiguous()
    N = err.shape[0]
    C = w.shape[3]
    dx = torch.nn.grad.conv2d_input((N, C, H, W), wi, e, stride=stride, padding=padding)
    return dx.permute(0, 2, 3, 1).contiguous().to(torch.int64)


def conv2d_wgrad_i32(act, err, stride=1, padding=1, f32_epilogue=True):
    """ti_torch.py:430-432: wgrad expressed as fprop on (0,3)-transposed operands; result KRSC
    int32.  dW[k,r,s,c] = sum_{n,p,q} err[n,p,q,k] * act[n,p+r-pad,q+s-pad,c] (stride 1)."""
    at = act.transpose(0, 3).contiguous()
    et = err.transpose(0, 3).contiguous()
    return conv2d_int8(at, et, stride, padding, f32_epilogue).transpose(0, 3).contiguous()


def conv2d_wgrad_def(act, err, R, S, stride=1, padding=1):
    """Definition via torch.nn.grad.conv2d_weight in fp64; KRSC int64."""
    a = _nhwc_to_nchw(act).double().contiguous()
    e = _nhwc_to_nchw(err).double().contiguous()
    K = err.shape[3]
    C = act.shape[3]
    dw = torch.nn.grad.conv2d_weight(a, (K, C, R, S), e, stride=stride, padding=padding)
    return dw.permute(0, 2, 3, 1).contiguous().to(torch.int64)


def conv2d_weight_int8(act, weight_size, err, stride=1, padding=1):
    """ti_torch.py:194-233 (first-layer wgrad through a grouped conv with fp32 partials summed
    over the batch).  Every partial and the total stay below 2^24 for the shapes the
    reference feeds, so the fp32 result equals the integer sum; returned as float32 KRSC."""
    K, R, S, C = weight_size
    dw = conv2d_wgrad_def(act, err, R, S, stride, padding)
    assert int(dw.abs().max()) < 2 ** 24 if dw.numel() else True
    return dw.to(torch.float32)


def int8mm(lhs: torch.Tensor, rhs: torch.Tensor) -> torch.Tensor:
    """ti_torch.py:152-176 -> int8mm_kernel.cu:8-34: exact int32 [m,k]x[k,n] (zero padding of
    k and n to multiples of 4 does not change the result)."""
    return (lhs.to(torch.int32) @ rhs.to(torch.int32)).contiguous()


# --------------------------------------------------------------------------------------
# max-pool
# --------------------------------------------------------------------------------------
def maxpool_fwd(x: torch.Tensor, kernel_size=2, stride=2, padding=0) -> torch.Tensor:
    """int8pool_kernel.cu:28-80: NHWC int8 max pooling (padding never wins a maximum)."""
    y = F.max_pool2d(_nhwc_to_nchw(x).contiguous(), kernel_size, stride, padding)
    return y.permute(0, 2, 3, 1).contiguous()


def maxpool_bwd(y, dy, x, kernel_size=2, stride=2, padding=0, ties="first"):
    """int8pool_kernel.cu:82-138: route dy to the input position holding the window maximum.
    ties="first": first maximum in (kh,kw) row-major scan order gets dy (torch CPU rule);
    ties="all": every position equal to the maximum gets dy.  Overlapping windows add."""
    xn = x.numpy().astype(np.int32)
    yn = y.numpy().astype(np.int32)
    dyn = dy.numpy().astype(np.int32)
    N, H, W, C = xn.shape
    _, P, Q, _ = yn.shape
    dx = np.zeros((N, H, W, C), dtype=np.int32)
    for p in range(P):
        for q in range(Q):
            taken = np.zeros((N, C), dtype=bool)
            for kh in range(kernel_size):
                h = p * stride - padding + kh
                if h < 0 or h >= H:
                    continue
                for kw in range(kernel_size):
                    w = q * stride - padding + kw
                    if w < 0 or w >= W:
                        continue
                    hit = xn[:, h, w, :] == yn[:, p, q, :]
                    if ties == "first":
                        hit = hit & ~taken
                        taken |= hit
                    dx[:, h, w, :] += np.where(hit, dyn[:, p, q, :], 0)
    return torch.from_numpy(dx).to(torch.int8)


# --------------------------------------------------------------------------------------
# integer cross-entropy gradient
# --------------------------------------------------------------------------------------
# 1/k! for k = 0..18 as the nearest doubles (hex literals: the same bits in niti_oracle.c and in the HIP kernel)
EXP2_COEF = [float.fromhex(h) for h in (
    "0x1.0000000000000p+0", "0x1.0000000000000p+0", "0x1.0000000000000p-1", "0x1.5555555555555p-3",
    "0x1.5555555555555p-5", "0x1.1111111111111p-7", "0x1.6c16c16c16c17p-10", "0x1.a01a01a01a01ap-13",
    "0x1.a01a01a01a01ap-16", "0x1.71de3a556c734p-19", "0x1.27e4fb7789f5cp-22", "0x1.ae64567f544e4p-26",
    "0x1.1eed8eff8d898p-29", "0x1.6124613a86d09p-33", "0x1.93974a8c07c9dp-37", "0x1.ae7f3e733b81fp-41",
    "0x1.ae7f3e733b81fp-45", "0x1.952c77030ad4ap-49", "0x1.6827863b97d97p-53")]
EXP2_LN2 = float.fromhex("0x1.62e42fefa39efp-1")


def exp2_contract(s: torch.Tensor) -> torch.Tensor:
    """``2 ** s`` of ti_loss.py:24 for a float32 tensor, as a fixed sequence of IEEE double operations, so
    that host and device agree bit for bit (a library pow differs by an ulp between platforms, which can
    flip the truncations that follow):  n = floor(s), x = (s - n) * ln2, p = sum x^k / k! by Horner's rule
    with a separately rounded product and sum per step (no fused multiply-add), result = float32(p * 2^n).
    The truncation error is below 2^-60, so the result is the correctly rounded float32 power except when
    the true value lies within about 2^-52 (relative) of a rounding boundary."""
    d = s.to(torch.float64)
    n = torch.floor(d)
    x = (d - n) * EXP2_LN2
    p = torch.full_like(x, EXP2_COEF[-1])
    for c in reversed(EXP2_COEF[:-1]):
        p = p * x
        p = p + c
    return torch.ldexp(p, n.to(torch.int32)).to(torch.float32)


def ti_loss_pre_round(out_val: torch.Tensor, out_exp: int, target: torch.Tensor, pow2=exp2_contract) -> torch.Tensor:
    """ti_loss.py:6-34: everything before the final StoShift; returns the int32 tensor that
    StoShift(.., 4) consumes.  fp32 arithmetic exactly as the reference's op sequence; ``2 ** s`` of
    line 24 through ``pow2`` (default: the deterministic statement above; ``lambda s: 2 ** s`` gives the
    platform's own float pow)."""
    s = out_val.to(torch.int64)
    out_exp = int(out_exp)
    if out_exp > -7:
        s = s * 47274 / (2 ** 15)                    # true division -> fp32
        if out_exp >= 0:
            s = s * 2 ** out_exp
        else:
            s = s / (2 ** -out_exp)
        out_max, _ = torch.max(s, dim=1)
        offset = out_max - 10
        s = s - offset.view(-1, 1)
        s = torch.max(s, torch.tensor(0, dtype=torch.int8).to(torch.int64))
        out_grad = pow2(s) - 1
    else:
        e = torch.tensor(out_exp, dtype=torch.int64)
        out_grad = 2 ** (1 - 2 * e) + s * 2 ** (1 - e) + s * s
    out_sum = out_grad.sum(1, dtype=torch.int64)
    out_grad = out_grad * (2 ** 11) / out_sum.view(-1, 1)
    out_grad[torch.arange(out_val.size(0)), target] -= out_grad.sum(1, dtype=torch.int64)
    return out_grad.to(torch.int32)


def ti_loss(out_val, out_exp, target, rand, div_mode=FLOOR):
    """ti_loss.py:35-36: int8 error = StoShift(pre_round, 4), exponent 0."""
    return StoShift(ti_loss_pre_round(out_val, out_exp, target), 4, rand, div_mode), 0


# --------------------------------------------------------------------------------------
# float -> int8 quantisers
# --------------------------------------------------------------------------------------
def ceil_log2_f32(r: float) -> int:
    """ceil(log2(r)) of a positive float32 as exact arithmetic on its exponent and mantissa (what
    ``torch.ceil(torch.log2(r))`` of ti_torch.py:336,348 means mathematically): r = m * 2^e with
    0.5 <= m < 1 gives e - 1 for m == 0.5 (a power of two) and e otherwise."""
    m, e = math.frexp(float(np.float32(r)))
    return e - 1 if m == 0.5 else e


def float_to_int8(x: torch.Tensor, bits: int = BITWIDTH, log2_mode: str = "exact") -> Tuple[torch.Tensor, int]:
    """TiFloatToInt8, ti_torch.py:341-356: r = max|x|, bw = ceil(log2 r), exponent bw - bits,
    values clamp(round_half_even(x * 2^(bits - bw)), -128, 127) as int8 (same shape as x).
    log2_mode "exact": ceil_log2_f32 (the contract of the HIP path); "f32": the reference's literal
    float32 ``ceil(log2(r))`` on this host.  The two differ only for r in the first few float32 values
    above a power of two >= 16, where float32(k + log2(1 + d)) rounds back to k.
    An all-zero tensor gives zeros and exponent 0 (the reference's sequence yields NaN there)."""
    x = x.to(torch.float32)
    r = torch.max(torch.abs(x))
    if float(r) == 0.0:
        return torch.zeros(x.shape, dtype=torch.int8), 0
    if log2_mode == "exact":
        bw = ceil_log2_f32(float(r))
    elif log2_mode == "f32":
        bw = int(torch.ceil(torch.log2(r)))
    else:
        raise ValueError(log2_mode)
    norm = x * torch.tensor(2.0 ** (bits - bw), dtype=torch.float32)
    q = torch.clamp(torch.round(norm), -128, 127).to(torch.int8)
    return q, bw - bits


def quantize_input_nhwc(x_nchw: torch.Tensor, bits: int = BITWIDTH) -> Tuple[torch.Tensor, int]:
    """TiNet.forward, ti_net.py:18-19: TiFloatToInt8 of the float NCHW batch, then permute(0,2,3,1).contiguous()."""
    q, e = float_to_int8(x_nchw, bits)
    return q.permute(0, 2, 3, 1).contiguous(), e


def weight_quant(w: torch.Tensor, log2_mode: str = "exact") -> Tuple[torch.Tensor, int]:
    """weight_quant, ti_torch.py:334-339: int8 = round_half_even(w / max|w| * 127) (float32 quotient, then
    float32 product), exponent ceil(log2(max|w|)) - 7."""
    w = w.to(torch.float32)
    r = torch.max(torch.abs(w))
    bw = ceil_log2_f32(float(r)) if log2_mode == "exact" else int(torch.ceil(torch.log2(r)))
    q = torch.round(w / r * (2 ** 7 - 1)).to(torch.int8)
    return q, bw - 7
