"""ctypes front end of oracle/libniti_oracle.so (plain-C oracle) -- TEST INFRASTRUCTURE.

Takes and returns torch CPU tensors so tests can compare it directly with
oracle/niti_oracle.py and with the HIP path.  Build with ``make -C oracle``."""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "libniti_oracle.so")
_lib = None


def build(force: bool = False) -> str:
    if force or not os.path.exists(_SO) or os.path.getmtime(_SO) < os.path.getmtime(os.path.join(_HERE, "niti_oracle.c")):
        subprocess.check_call(["make", "-C", _HERE, "-B", "libniti_oracle.so"], stdout=subprocess.DEVNULL)
    return _SO


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            build()
        _lib = C.CDLL(_SO)
        _lib.nito_round_shift1.restype = C.c_int8
        _lib.nito_sto_shift1.restype = C.c_int8
        _lib.nito_psto_shift1.restype = C.c_int8
        _lib.nito_absmax.restype = C.c_uint32
        _lib.nito_exp2_contract.restype = C.c_float
        _lib.nito_exp2_contract.argtypes = [C.c_float]
    return _lib


def _p(t: torch.Tensor):
    assert t.is_contiguous() and t.device.type == "cpu"
    return C.c_void_p(t.data_ptr())


def _out_dim(i, pad, k, st):
    return (i + 2 * pad - k) // st + 1


def num_threads() -> int:
    return int(lib().nito_num_threads())


def round_shift(x, s, trunc=False):
    x = x.contiguous()
    y = torch.empty(x.shape, dtype=torch.int8)
    lib().nito_round_shift(_p(x), _p(y), C.c_int64(x.numel()), int(s), int(trunc))
    return y


def sto_shift(x, s, u, trunc=False):
    x = x.contiguous()
    u = u.to(torch.int32).contiguous()
    y = torch.empty(x.shape, dtype=torch.int8)
    lib().nito_sto_shift(_p(x), _p(u), _p(y), C.c_int64(x.numel()), int(s), int(trunc))
    return y


def psto_shift(x, s, trunc=False):
    x = x.contiguous()
    y = torch.empty(x.shape, dtype=torch.int8)
    lib().nito_psto_shift(_p(x), _p(y), C.c_int64(x.numel()), int(s), int(trunc))
    return y


def bitwidth_int(r: int) -> int:
    return int(lib().nito_bitwidth_int(C.c_uint32(r)))


def bitwidth_f32_libm(r: int) -> int:
    return int(lib().nito_bitwidth_f32_libm(C.c_uint32(r)))


def absmax(x) -> int:
    x = x.contiguous()
    return int(lib().nito_absmax(_p(x), C.c_int64(x.numel())))


_METHOD = {"round": 0, "sto": 1, "psto": 2}


def requant(x, target_bits, method="round", trunc=False, u=None):
    """Returns (int8 tensor, shift)."""
    x = x.to(torch.int32).contiguous()
    y = torch.empty(x.shape, dtype=torch.int8)
    if u is None:
        u = torch.zeros(1, dtype=torch.int32)
        assert method != "sto"
    u = u.to(torch.int32).contiguous()
    s = lib().nito_requant(_p(x), _p(u), _p(y), C.c_int64(x.numel()), int(target_bits), _METHOD[method], int(trunc))
    return y, int(s)


def weight_update(w, g):
    w = w.clone().contiguous()
    lib().nito_weight_update(_p(w), _p(g.contiguous()), C.c_int64(w.numel()))
    return w


def f32_roundtrip(x):
    x = x.contiguous()
    y = torch.empty_like(x)
    lib().nito_f32_roundtrip(_p(x), _p(y), C.c_int64(x.numel()))
    return y


def conv_fprop(x, w, stride=1, pad=1):
    x, w = x.contiguous(), w.contiguous()
    N, H, W, Cc = x.shape
    K, R, S, _ = w.shape
    y = torch.empty((N, _out_dim(H, pad, R, stride), _out_dim(W, pad, S, stride), K), dtype=torch.int32)
    lib().nito_conv_fprop(_p(x), _p(w), _p(y), N, H, W, Cc, K, R, S, stride, pad)
    return y


def conv_dgrad(err, w, H, W, stride=1, pad=1):
    err, w = err.contiguous(), w.contiguous()
    N = err.shape[0]
    K, R, S, Cc = w.shape
    dx = torch.empty((N, H, W, Cc), dtype=torch.int32)
    lib().nito_conv_dgrad(_p(err), _p(w), _p(dx), N, H, W, Cc, K, R, S, stride, pad)
    return dx


def conv_wgrad(act, err, R, S, stride=1, pad=1):
    act, err = act.contiguous(), err.contiguous()
    N, H, W, Cc = act.shape
    K = err.shape[3]
    dw = torch.empty((K, R, S, Cc), dtype=torch.int32)
    lib().nito_conv_wgrad(_p(act), _p(err), _p(dw), N, H, W, Cc, K, R, S, stride, pad)
    return dw


def gemm(a, b):
    a, b = a.contiguous(), b.contiguous()
    m, k = a.shape
    n = b.shape[1]
    c = torch.empty((m, n), dtype=torch.int32)
    lib().nito_gemm(_p(a), _p(b), _p(c), m, n, k)
    return c


def maxpool_fwd(x, ks=2, stride=2, pad=0):
    x = x.contiguous()
    N, H, W, Cc = x.shape
    y = torch.empty((N, _out_dim(H, pad, ks, stride), _out_dim(W, pad, ks, stride), Cc), dtype=torch.int8)
    lib().nito_maxpool_fwd(_p(x), _p(y), N, H, W, Cc, ks, stride, pad)
    return y


def maxpool_bwd(y, dy, x, ks=2, stride=2, pad=0, ties="first"):
    y, dy, x = y.contiguous(), dy.contiguous(), x.contiguous()
    N, H, W, Cc = x.shape
    dx = torch.empty_like(x)
    lib().nito_maxpool_bwd(_p(y), _p(dy), _p(x), _p(dx), N, H, W, Cc, ks, stride, pad, int(ties == "all"))
    return dx


def exp2_contract(s: float) -> float:
    return float(lib().nito_exp2_contract(float(s)))


def ti_loss_pre_round(out_val, out_exp, target):
    out_val = out_val.contiguous()
    target = target.to(torch.int64).contiguous()
    n, classes = out_val.shape
    pre = torch.empty((n, classes), dtype=torch.int32)
    lib().nito_ti_loss_pre_round(_p(out_val), n, classes, int(out_exp), _p(target), _p(pre))
    return pre


def float_to_int8(x, bits=7):
    x = x.to(torch.float32).contiguous()
    y = torch.empty(x.shape, dtype=torch.int8)
    e = lib().nito_float_to_int8(_p(x), _p(y), C.c_int64(x.numel()), int(bits))
    return y, int(e)


def weight_quant(w):
    w = w.to(torch.float32).contiguous()
    y = torch.empty(w.shape, dtype=torch.int8)
    e = lib().nito_weight_quant(_p(w), _p(y), C.c_int64(w.numel()))
    return y, int(e)
