"""Stand-in for the reference's ``cutlassconv_cuda`` extension
(pytorch/cutlass-extension/cutlassconv.cpp:105-113)."""
import torch

from .. import ops


def _check(t, name):
    from . import check_input
    check_input(t, name)
    if t.dtype != torch.int8:
        raise RuntimeError("expected scalar type Char but found %s" % t.dtype)  # what .data<int8_t>() raises


def sp_conv(input, weight, stride_h, padding_h):
    """cutlassconv.cpp:57-64 -> cutlassconv_kernel.cu:180-319: NHWC int8 x KRSC int8 -> new NPQK
    int32 tensor, cross-correlation, same stride/padding in both dimensions, results passed through
    fp32 as the CUTLASS epilogue does."""
    _check(input, "input")
    _check(weight, "weight")
    return ops.conv2d_fprop(input, weight, int(stride_h), int(padding_h), f32_epilogue=True)


def sp_conv_optimized(input, weight, stride_h, padding_h):
    """cutlassconv.cpp:66-73 -> cutlassconv_kernel.cu:38-177 (same arithmetic as sp_conv; the
    reference's R,S <= 32 limit of this variant does not exist here)."""
    return sp_conv(input, weight, stride_h, padding_h)


def int8_conv(input, weight):
    """cutlassconv.cpp:49-54: fixed stride 1, padding 1."""
    return sp_conv(input, weight, 1, 1)


def int8_conv_optimized(input, weight):
    """cutlassconv.cpp:76-81."""
    return sp_conv(input, weight, 1, 1)


def _dead(name):
    def f(*args, **kwargs):
        raise NotImplementedError(
            "cutlassconv_cuda.%s is never called by the reference's Python and is not part of the int8 hot path" % name)
    f.__name__ = name
    return f


int4_conv = _dead("int4_conv")
int4_conv_optimized = _dead("int4_conv_optimized")
weight_grad = _dead("weight_grad")  # the reference's body is a stub returning uninitialised memory
