"""Integer cross-entropy gradient with the reference's ``ti_loss.TiLoss`` interface."""
import torch
from torch.nn.modules import Module

from . import ops, ti_torch


class TiLoss(Module):
    """ti_loss.py:5-36: base-2 soft-max approximation of the cross-entropy gradient, rounded to int8
    with StoShift(.., 4).  One launch of the library's kernel, which keeps the reference's float32
    operation sequence per sample (``2 ** s`` by a fixed sequence of double operations, see exp2_f32); the ``out_exp > -7`` case split happens on the device, so there is no
    host synchronisation.  ``rand`` (int32 in [0,16), one per logit) replaces the random integers the kernel
    otherwise draws itself (Philox4x32-10 on a small state in device memory, ops.rng_state)."""

    rng = None      # RngBox of the network; without one the device's shared generator state is used

    def forward(self, out_val, out_exp, target, rand=None):
        dev = out_val.device
        e = ti_torch._exp_tensor(out_exp, dev)
        if rand is None:    # the kernel draws the random integers itself
            state = self.rng.state(dev) if self.rng is not None else ops.rng_state(dev)
            self.out_grad = ops.loss_grad_rng(out_val.contiguous(), e, target.to(torch.int64).contiguous(), state, ti_torch.DIV_MODE)
        else:
            self.out_grad = ops.loss_grad(out_val.contiguous(), e, target.to(torch.int64).contiguous(),
                                          rand.to(torch.int32).contiguous(), ti_torch.DIV_MODE)
        return self.out_grad, 0


# 1 / k!, k = 0 .. 18, and ln 2 as the nearest doubles (the constants of the kernel's exp2_contract)
_EXP2_COEF = [float.fromhex(h) for h in (
    "0x1.0000000000000p+0", "0x1.0000000000000p+0", "0x1.0000000000000p-1", "0x1.5555555555555p-3",
    "0x1.5555555555555p-5", "0x1.1111111111111p-7", "0x1.6c16c16c16c17p-10", "0x1.a01a01a01a01ap-13",
    "0x1.a01a01a01a01ap-16", "0x1.71de3a556c734p-19", "0x1.27e4fb7789f5cp-22", "0x1.ae64567f544e4p-26",
    "0x1.1eed8eff8d898p-29", "0x1.6124613a86d09p-33", "0x1.93974a8c07c9dp-37", "0x1.ae7f3e733b81fp-41",
    "0x1.ae7f3e733b81fp-45", "0x1.952c77030ad4ap-49", "0x1.6827863b97d97p-53")]
_LN2 = float.fromhex("0x1.62e42fefa39efp-1")


def exp2_f32(s):
    """``2 ** s`` (ti_loss.py:24) for a non-negative float32 tensor by the kernel's fixed sequence of double operations:
    n = floor(s), x = (s - n) ln2, Horner's rule over 1/k! with separately rounded products and sums, float32(p 2^n).
    Every step is an IEEE operation, so the result does not depend on the device's math library."""
    d = s.to(torch.float64)
    n = torch.floor(d)
    x = (d - n) * _LN2
    p = torch.full_like(x, _EXP2_COEF[-1])
    for c in reversed(_EXP2_COEF[:-1]):
        p = p * x
        p = p + c
    return torch.ldexp(p, n.to(torch.int32)).to(torch.float32)


def loss_grad_tensor_ops(out_val, out_exp, target, rand):
    """The same gradient written as the reference's sequence of float32 tensor operations (ti_loss.py:5-36),
    both cases of the exponent split evaluated and selected on the device.  Kept as an independent statement
    of what the kernel computes; tests compare the two."""
    dev = out_val.device
    e = ti_torch._exp_tensor(out_exp, dev).to(torch.int64).reshape(())
    s0 = out_val.type(torch.int64)
    big = e > -7
    # case out_exp > -7
    ef = torch.clamp(e, min=-7).to(torch.float32)
    s = s0 * 47274 / (2 ** 15)
    s = torch.where(ef >= 0, s * 2 ** ef, s / (2 ** -ef))
    out_max, _ = torch.max(s, dim=1)
    s = s - (out_max - 10).view(-1, 1)
    s = torch.max(s, torch.zeros((), dtype=torch.int64, device=dev))
    grad_big = exp2_f32(s) - 1
    # case out_exp <= -7: 1 + e^x ~ 1 + x + x^2/2, in integers
    es = torch.clamp(e, max=-7)
    grad_small = 2 ** (1 - 2 * es) + s0 * 2 ** (1 - es) + s0 * s0
    out_sum = torch.where(big, grad_big.sum(1, dtype=torch.int64), grad_small.sum(1, dtype=torch.int64))
    out_grad = torch.where(big, grad_big, grad_small.to(torch.float32))
    out_grad = out_grad * (2 ** 11) / out_sum.view(-1, 1)
    rows = torch.arange(out_val.size(0), device=dev)
    out_grad[rows, target] -= out_grad.sum(1, dtype=torch.int64)
    return ti_torch.StoShift(out_grad.type(torch.int32), 4, rand)
