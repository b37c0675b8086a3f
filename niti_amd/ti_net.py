"""Network container with the reference's ``ti_net.TiNet`` interface (ti_net.py:8-48)."""
import collections

import torch
from torch.nn.modules import Module

from . import ops, ti_torch
from .ti_loss import TiLoss


class TiNet(Module):
    def __init__(self):
        super().__init__()
        self.loss = TiLoss()
        self.rng = ti_torch.RngBox()      # random draws made inside the kernels (dropout mask, loss gradient rounding)
        self.loss.rng = self.rng
        # the classifier TiLinear whose forward launch can evaluate the loss gradient (kept out of the module tree: it
        # already is a member of forward_layers)
        self.__dict__["_head"] = None

    def fuse(self):
        """Fold each TiReLU that directly follows a TiConv2d into that layer's requantisation."""
        layers = list(self.forward_layers)
        for a, b in zip(layers, layers[1:]):
            if isinstance(a, ti_torch.TiConv2d) and isinstance(b, ti_torch.TiReLU):
                a.fuse_relu = True
                b.fused = True
        # TiConv2d -> fused ReLU -> 2x2 / stride-2 max-pool: the convolution's launch writes the pooled tensor as well
        for a, b, c in zip(layers, layers[1:], layers[2:]):
            if (isinstance(a, ti_torch.TiConv2d) and isinstance(b, ti_torch.TiReLU) and b.fused and isinstance(c, ti_torch.TiMaxpool2d)
                    and (c.kernel_size, c.stride, c.padding) == (2, 2, 0)):
                a.pool_after = c
        # ReLU [-> max-pool] -> TiConv2d: the convolution zeroes its data gradient where its own input (the ReLU's
        # possibly pooled output) is not positive, which is that ReLU's backward pass (a max-pool routes gradients
        # only to elements equal to the pooled maximum, so masking before or after its backward is the same)
        for i, l in enumerate(layers):
            if not isinstance(l, ti_torch.TiReLU):
                continue
            j = i + 1
            if j < len(layers) and isinstance(layers[j], ti_torch.TiMaxpool2d):
                j += 1
            if j < len(layers) and isinstance(layers[j], ti_torch.TiConv2d) and not layers[j].first_layer:
                layers[j].relu_below = True
                l.bwd_folded = True
                if j == i + 2 and (layers[i + 1].kernel_size, layers[i + 1].stride, layers[i + 1].padding) == (2, 2, 0):
                    # ... and the data gradient writes its result through that max-pool's backward pass as well
                    layers[j].pool_below = layers[i + 1]
            elif j == i + 2:
                # ReLU -> max-pool -> anything else: the pooling's backward pass applies the mask to its own output
                layers[i + 1].relu_below = True
                l.bwd_folded = True
        # [TiDropout ->] TiLinear with few outputs at the end: the classifier's launches apply the dropout mask (and
        # draw it), and its forward launch evaluates the loss gradient when forward() is given the targets
        if layers and isinstance(layers[-1], ti_torch.TiLinear) and layers[-1].weight.shape[0] <= 16:
            self.__dict__["_head"] = layers[-1]
            self._head.rng = self.rng
            if len(layers) > 1 and isinstance(layers[-2], ti_torch.TiDropout):
                # plain attributes, not sub-modules: the two layers refer to each other
                layers[-1].__dict__["drop_below"] = layers[-2]
                layers[-2].__dict__["head"] = layers[-1]
            # 2x2 / stride-2 max-pool -> TiFlat -> [TiDropout ->] classifier: the classifier's backward launch routes its
            # data gradient through that pool's backward pass as well
            j = len(layers) - 2
            if j >= 0 and isinstance(layers[j], ti_torch.TiDropout):
                j -= 1
            if (j >= 1 and isinstance(layers[j], ti_torch.TiFlat) and isinstance(layers[j - 1], ti_torch.TiMaxpool2d)
                    and (layers[j - 1].kernel_size, layers[j - 1].stride, layers[j - 1].padding) == (2, 2, 0)):
                layers[-1].__dict__["pool_below"] = layers[j - 1]
        return self

    def forward(self, x, target=None):
        """ti_net.py:17-23: float NCHW batch -> (int8 logits, exponent).  ``target`` (not in the reference): the
        class indices that backward() will be called with; the classifier's forward launch then computes the loss
        gradient as well and backward(target) with the same tensor starts from it."""
        x_data, x_exp = self.quantize_input(x)
        return self.forward_int8(x_data, x_exp, target)

    @staticmethod
    def quantize_input(x):
        """TiFloatToInt8 + NCHW -> NHWC (ti_net.py:18-19): (int8 NHWC batch, exponent).  A contiguous float32 batch on
        the GPU takes the library's two launches (channels come zero-padded to 16, which the first convolution
        would do next anyway); anything else - and BW_MODE "f32", whose range exponent is the reference's float32
        ``ceil(log2(r))`` rather than the exact one - the reference's tensor operations."""
        x = x.to(ti_torch.GPU)
        if x.dtype == torch.float32 and x.dim() == 4 and x.is_contiguous() and x.is_cuda and ti_torch.BW_MODE == "int":
            return ops.quantize_input(x, ti_torch.BITWIDTH)
        x_data, x_exp = ti_torch.TiFloatToInt8(x)
        return x_data.permute(0, 2, 3, 1).contiguous(), x_exp

    def forward_int8(self, x_data, x_exp=0, target=None, loss_rand=None):
        """Same as forward() for a batch that already is int8 NHWC with exponent ``x_exp``."""
        ops.sync_arena.reset(x_data.device)     # one fill for the range-exchange words of the whole step
        if self._head is not None:
            self._head.next_target = None
            if target is not None and ti_torch.TRAINING and target.dtype == torch.int64 and target.is_contiguous() and target.is_cuda:
                self._head.next_target = (target, loss_rand)
        self.out, self.out_exp = self.forward_layers((x_data, x_exp))
        return self.out, self.out_exp

    @property
    def out_bits(self):
        """ti_net.py:22 (computed on demand: it needs a device->host copy)."""
        return ti_torch.RangeEstimate(self.out)

    def backward(self, target, loss_rand=None):
        """ti_net.py:25-32."""
        done = self._head.loss_grad if self._head is not None else None
        if done is not None and done[0] is target and loss_rand is None:
            self._head.loss_grad = None
            self.loss.out_grad = done[1]        # the classifier's forward launch has evaluated TiLoss already
            x = (done[1], 0)
        else:
            x = self.loss(self.out, self.out_exp, target, loss_rand)
        return self.backward_from(x)

    def backward_from(self, x):
        """Back-propagate a given (int8 error, exponent) pair through the layers in reverse."""
        for layer in reversed(self.forward_layers):
            if isinstance(layer, torch.nn.Sequential):
                for block in reversed(layer):
                    x = block.backward(x)
            else:
                x = layer.backward(x)
        return x

    def state_dict(self):
        """ti_net.py:34-41: ``layers.<idx>.weight`` (int8) and ``layers.<idx>.weight_exp`` (0-d float)."""
        state_dict = collections.OrderedDict()
        for idx, l in enumerate(self.forward_layers):
            if hasattr(l, "weight"):
                prefix = "layers." + str(idx) + "."
                state_dict[prefix + "weight"] = l.weight
                state_dict[prefix + "weight_exp"] = l.weight_exp
        return state_dict

    def load_state_dict(self, state_dict):
        """ti_net.py:43-48."""
        self.__dict__.pop("_step_graphs", None)     # captured steps (train.StepGraph) point at the tensors replaced here
        for idx, l in enumerate(self.forward_layers):
            if hasattr(l, "weight"):
                prefix = "layers." + str(idx) + "."
                l.weight = state_dict[prefix + "weight"].to(ti_torch.GPU).contiguous()
                l.weight_exp = state_dict[prefix + "weight_exp"]
