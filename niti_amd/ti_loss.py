"""Integer cross-entropy gradient with the reference's ``ti_loss.TiLoss`` interface."""
import torch
from torch.nn.modules import Module

from . import ops, ti_torch


class TiLoss(Module):
    """ti_loss.py:5-36: base-2 soft-max approximation of the cross-entropy gradient, rounded to int8
    with StoShift(.., 4).  One launch of the library's kernel, which keeps the reference's float32
    operation sequence per sample; the ``out_exp > -7`` case split happens on the device, so there is no
    host synchronisation.  ``rand`` (int32 in [0,16), one per logit) replaces the device random draw
    when given."""

    def forward(self, out_val, out_exp, target, rand=None):
        dev = out_val.device
        e = ti_torch._exp_tensor(out_exp, dev)
        if rand is None:
            rand = torch.randint(0, 16, out_val.shape, dtype=torch.int32, device=dev)
        self.out_grad = ops.loss_grad(out_val.contiguous(), e, target.to(torch.int64).contiguous(),
                                      rand.to(torch.int32).contiguous(), ti_torch.DIV_MODE)
        return self.out_grad, 0


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
    grad_big = 2 ** s - 1
    # case out_exp <= -7: 1 + e^x ~ 1 + x + x^2/2, in integers
    es = torch.clamp(e, max=-7)
    grad_small = 2 ** (1 - 2 * es) + s0 * 2 ** (1 - es) + s0 * s0
    out_sum = torch.where(big, grad_big.sum(1, dtype=torch.int64), grad_small.sum(1, dtype=torch.int64))
    out_grad = torch.where(big, grad_big, grad_small.to(torch.float32))
    out_grad = out_grad * (2 ** 11) / out_sum.view(-1, 1)
    rows = torch.arange(out_val.size(0), device=dev)
    out_grad[rows, target] -= out_grad.sum(1, dtype=torch.int64)
    return ti_torch.StoShift(out_grad.type(torch.int32), 4, rand)
