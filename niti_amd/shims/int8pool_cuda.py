"""Stand-in for the reference's ``int8pool_cuda`` extension (pytorch/int8pool-extension/int8pool.cpp:81-86)."""
import torch

from .. import ops

TIES = "first"  # which of several equal maxima receives the gradient ("first" or "all")


def int8_pool(input, kernel_size, stride, padding):
    """int8pool.cpp:37-44 -> int8pool_kernel.cu:28-80: NHWC int8 max pooling."""
    from . import check_input
    check_input(input, "input")
    return ops.maxpool_fwd(input, int(kernel_size), int(stride), int(padding))


def int8_pool_backward(y, dy, x, kernel_size, stride, padding):
    """int8pool.cpp:46-57 -> int8pool_kernel.cu:82-138.  The reference passes half tensors because cuDNN
    has no int8 pooling backward (ti_torch.py:309-314) and gets a half tensor back; int8 tensors are
    accepted too and then an int8 tensor is returned."""
    from . import check_input
    for t, n in ((y, "y"), (dy, "dy"), (x, "x")):
        check_input(t, n)
    as_half = dy.dtype == torch.float16
    conv = (lambda t: t.to(torch.int8)) if as_half else (lambda t: t)
    dx = ops.maxpool_bwd(conv(y), conv(dy), conv(x), int(kernel_size), int(stride), int(padding), TIES)
    return dx.half() if as_half else dx


def average_pool(*args, **kwargs):
    raise NotImplementedError("int8pool_cuda.average_pool is never called by the reference's Python")


def average_pool_backward(*args, **kwargs):
    raise NotImplementedError("int8pool_cuda.average_pool_backward is never called by the reference's Python")
