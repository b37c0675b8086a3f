"""Stand-in for the reference's ``int8mm_cuda`` extension (pytorch/int8mm-extension/int8mm.cpp:9-18)."""
import torch

from .. import ops


def int8_mm(lhs, rhs):
    """int8mm_kernel.cu:8-34: [m,k] x [k,n] -> exact int32 [m,n], returned like the reference as the
    transposed view of an [n,m] buffer (callers do ``.contiguous()``, ti_torch.py:176)."""
    from . import check_input
    check_input(lhs, "lhs")
    check_input(rhs, "rhs")
    if lhs.dtype != torch.int8 or rhs.dtype != torch.int8:
        raise RuntimeError("expected scalar type Char")
    # [n,m] = rhs^T lhs^T: rhs is stored [k,n] ("a" transposed), lhs is stored [m,k] ("b" transposed)
    out_t = ops.gemm(rhs, lhs, trans_a=True, trans_b=True)
    return out_t.transpose(0, 1)
