"""CPU oracle of the reference's layer stack and training step -- TEST INFRASTRUCTURE, NOT PRODUCT.

Restates ti_torch.py:11-21,235-455 (layers), ti_net.py:17-32 (forward / reverse-order backward) and
ti_vgg.py:10-42 (VGG configurations) on CPU tensors with Python-int exponents, built only from the
functions of oracle/niti_oracle.py.  Random inputs of the reference (StoShift draws, dropout mask)
are explicit arguments so both sides of a parity test can be fed the same values."""
from __future__ import annotations

import torch

from . import niti_oracle as po


class Cfg:
    """The module-level switches of ti_torch.py:457-464 plus main.py's injected globals."""

    def __init__(self, act="round", err="round", grad="psto", grad_bitwidth=5, div_mode="floor", bw_mode="int",
                 f32_epilogue=True, pool_ties="first", training=True):
        self.act, self.err, self.grad = act, err, grad
        self.grad_bitwidth = grad_bitwidth
        self.div_mode, self.bw_mode = div_mode, bw_mode
        self.f32_epilogue = f32_epilogue
        self.pool_ties = pool_ties
        self.training = training


class _Update:
    def weight_update(self, cfg, rand=None):
        """ti_torch.py:16-21."""
        self.grad, grad_shift = po.grad_calc(self.grad_int32acc.to(torch.int32), cfg.grad_bitwidth, cfg.grad,
                                             cfg.div_mode, rand, cfg.bw_mode)
        self.grad_shift = grad_shift
        self.grad_exp = self.err_exp + grad_shift + self.act_in_exp
        self.weight = po.weight_update(self.weight, self.grad)


class OConv2d(_Update):
    """ti_torch.py:379-437."""

    def __init__(self, weight, weight_exp, stride=1, padding=1, first_layer=False):
        self.weight, self.weight_exp = weight.clone(), int(weight_exp)
        self.stride, self.padding, self.first_layer = stride, padding, first_layer

    def forward(self, inp, cfg, rand=None):
        self.act, self.act_in_exp = inp
        self.acc = po.conv2d_int8(self.act, self.weight, self.stride, self.padding, cfg.f32_epilogue)
        return po.act_calc(self.acc, self.act_in_exp + self.weight_exp, cfg.act, cfg.div_mode, rand, cfg.bw_mode)

    def backward(self, inp, cfg, rand=None, grad_rand=None):
        err_in, self.err_exp = inp
        if not self.first_layer:
            acc = po.conv2d_dgrad_i32(err_in, self.weight, self.stride, self.padding, cfg.f32_epilogue)
            err_out, shift = po.err_calc(acc, cfg.err, cfg.div_mode, rand, cfg.bw_mode)
            self.err_exp = self.err_exp + shift + self.weight_exp
        if self.first_layer:
            self.grad_int32acc = po.conv2d_weight_int8(self.act, self.weight.shape, err_in, self.stride, self.padding)
        else:
            self.grad_int32acc = po.conv2d_wgrad_i32(self.act, err_in, self.stride, self.padding, cfg.f32_epilogue)
        self.weight_update(cfg, grad_rand)
        if not self.first_layer:
            return err_out, self.err_exp
        return None


class OLinear(_Update):
    """ti_torch.py:235-266."""

    def __init__(self, weight, weight_exp):
        self.weight, self.weight_exp = weight.clone(), int(weight_exp)

    def forward(self, inp, cfg, rand=None):
        self.act_in = inp
        act_in, exp_in = inp
        acc = po.int8mm(act_in, self.weight.transpose(0, 1).contiguous())
        return po.act_calc(acc, exp_in + self.weight_exp, cfg.act, cfg.div_mode, rand, cfg.bw_mode)

    def backward(self, inp, cfg, rand=None, grad_rand=None):
        err_in, self.err_exp = inp
        act, self.act_in_exp = self.act_in
        err_out, shift = po.err_calc(po.int8mm(err_in, self.weight), cfg.err, cfg.div_mode, rand, cfg.bw_mode)
        self.err_exp = self.err_exp + shift + self.weight_exp
        self.grad_int32acc = po.int8mm(err_in.transpose(0, 1).contiguous(), act)
        self.weight_update(cfg, grad_rand)
        return err_out, self.err_exp


class OReLU:
    """ti_torch.py:268-290."""

    def forward(self, inp, cfg):
        self.act_in = inp
        a, e = inp
        return torch.clamp(a, min=0), e

    def backward(self, inp, cfg):
        err, e = inp
        return torch.where(self.act_in[0] > 0, err, torch.zeros_like(err)), e


class OMaxpool2d:
    """ti_torch.py:292-316."""

    def __init__(self, kernel_size=2, stride=2, padding=0):
        self.k, self.s, self.p = kernel_size, stride, padding

    def forward(self, inp, cfg):
        self.act_in, e = inp
        self.act_out = po.maxpool_fwd(self.act_in, self.k, self.s, self.p)
        return self.act_out, e

    def backward(self, inp, cfg):
        err, e = inp
        return po.maxpool_bwd(self.act_out, err, self.act_in, self.k, self.s, self.p, cfg.pool_ties), e


class OFlat:
    """ti_torch.py:318-332."""

    def forward(self, inp, cfg):
        self.shape = inp[0].shape
        return inp[0].reshape(inp[0].shape[0], -1), inp[1]

    def backward(self, inp, cfg):
        return inp[0].reshape(self.shape), inp[1]


class ODropout:
    """ti_torch.py:439-455 with the per-feature mask supplied by the caller."""

    def __init__(self, mask):
        self.mask = mask

    def forward(self, inp, cfg):
        if not cfg.training:
            return inp
        return inp[0] * self.mask, inp[1] + 1

    def backward(self, inp, cfg):
        return inp[0] * self.mask, inp[1]


class ONet:
    """ti_net.py:8-32 over a flat list of the layers above."""

    def __init__(self, layers, cfg: Cfg):
        self.layers, self.cfg = layers, cfg

    def forward_int8(self, x, x_exp=0):
        cur = (x, x_exp)
        self.trace = []
        for l in self.layers:
            cur = l.forward(cur, self.cfg)
            self.trace.append(cur)
        self.out, self.out_exp = cur
        return cur

    def backward_from(self, err, err_exp=0):
        cur = (err, err_exp)
        self.btrace = []
        for l in reversed(self.layers):
            cur = l.backward(cur, self.cfg)
            self.btrace.append(cur)
        return cur

    def backward(self, target, loss_rand):
        err, e = po.ti_loss(self.out, self.out_exp, target, loss_rand, self.cfg.div_mode)
        self.loss_err = err
        return self.backward_from(err, e)


def build_vgg(cfg_list, weights, weight_exps, cfg: Cfg, dropout_mask=None):
    """ti_vgg.py:25-42 from explicit int8 weights (one per conv, then the FC weight)."""
    layers = []
    wi = 0
    for idx, x in enumerate(cfg_list):
        if x == 'M':
            layers.append(OMaxpool2d(2, 2))
        else:
            layers.append(OConv2d(weights[wi], weight_exps[wi], first_layer=(idx == 0)))
            layers.append(OReLU())
            wi += 1
    layers.append(OFlat())
    if dropout_mask is not None:
        layers.append(ODropout(dropout_mask))
    layers.append(OLinear(weights[wi], weight_exps[wi]))
    return ONet(layers, cfg)
