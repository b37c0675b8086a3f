"""Stand-in for the reference's ``int8conv_cuda`` extension (pytorch/int8conv-extension/int8conv.cpp:66-70)."""
import torch

from .. import ops


def group_conv(input, weight, stride, padding, dilation, groups):
    """int8conv.cpp:35-44 -> int8conv_kernel.cu:248-334: grouped NHWC int8 convolution with float32
    NPQK output (the reference uses it for the first layer's weight gradient only)."""
    from . import check_input
    check_input(input, "input")
    check_input(weight, "weight")
    if input.dtype != torch.int8 or weight.dtype != torch.int8:
        raise RuntimeError("expected scalar type Char")
    return ops.group_conv_f32(input, weight, int(stride), int(padding), int(dilation), int(groups))


def int8_conv(*args, **kwargs):
    raise NotImplementedError("int8conv_cuda.int8_conv is never called by the reference's Python")


def find_algo(*args, **kwargs):
    raise NotImplementedError("int8conv_cuda.find_algo is a cuDNN algorithm benchmark printer; nothing to replace")
