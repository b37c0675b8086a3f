"""ctypes binding of libniti_gfx950.so (the C ABI declared in include/niti_gfx950.h).

The library is the only implementation of the hot path: if it cannot be loaded every op of
this package raises, there is no fallback."""
from __future__ import annotations

import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
SO_PATH = os.path.join(_HERE, "libniti_gfx950.so")

OK = 0
EPI_F32_ROUNDTRIP = 1
CONV_FILTER_PREPARED = 2
CONV_FILTER_FORWARD_COPY = 4
CONV_SHIFT_HINT = 8
RQ_RELU = 1
RQ_SHIFT_HINT = 2
ROUND = {"round": 0, "sto": 1, "psto": 2}
DIV = {"floor": 0, "trunc": 1}
BW = {"int": 0, "f32": 1}
TIES = {"first": 0, "all": 1}
POOL_BWD_RELU = 2

_vp, _i, _u, _i64, _sz = C.c_void_p, C.c_int, C.c_uint, C.c_int64, C.c_size_t

# name -> (restype, argtypes); must list every symbol of include/niti_gfx950.h
SIGNATURES = {
    "niti_version": (_i, []),
    "niti_status_string": (C.c_char_p, [_i]),
    "niti_last_error": (C.c_char_p, []),
    "niti_bitwidth": (_i, [C.c_uint32, _i]),
    "niti_sync_timeouts": (_i, [_vp, _i, _vp]),
    "niti_fill_u32": (_i, [_vp, _i64, C.c_uint32, _vp]),
    "niti_conv2d_i8_filter_workspace": (_sz, [_i] * 10),
    "niti_conv2d_i8_filter_prepare": (_i, [_vp, _vp, _sz] + [_i] * 10 + [_vp]),
    "niti_conv2d_i8_fprop": (_i, [_vp, _vp, _vp] + [_i] * 9 + [_u, _vp, _vp, _sz, _vp]),
    "niti_conv2d_i8_dgrad": (_i, [_vp, _vp, _vp] + [_i] * 9 + [_u, _vp, _vp, _sz, _vp]),
    "niti_conv2d_i8_requant_sync_words": (_sz, [_i] * 10),
    "niti_conv2d_i8_fprop_requant": (_i, [_vp, _vp, _vp] + [_i] * 9 + [_u, _i, _i, _i, _i, _u, _vp, _sz, _vp, _vp, _vp, _vp, _vp, _sz, _vp]),
    "niti_conv2d_i8_fprop_requant_pool": (_i, [_vp, _vp, _vp, _vp] + [_i] * 9 + [_u, _i, _i, _i, _i, _u, _vp, _sz, _vp, _vp, _vp, _vp, _vp, _sz, _vp]),
    "niti_static_scratch_bytes": (_sz, []),
    "niti_conv2d_i8_fprop_requant_sto": (_i, [_vp, _vp, _vp, _vp, _vp] + [_i] * 9 + [_u, _i, _i, _i, _u, _vp, _sz, _vp, _vp, _vp, _vp, _vp, _sz, _vp]),
    "niti_conv2d_i8_dgrad_requant_sto": (_i, [_vp, _vp, _vp, _vp] + [_i] * 9 + [_u, _i, _i, _i, _u, _vp, _vp, _sz, _vp, _vp, _vp, _vp, _vp, _sz, _vp]),
    "niti_conv2d_i8_fprop_requant_static": (_i, [_vp, _vp, _vp] + [_i] * 9 + [_u, _i, _i, _i, _i, _u, _vp, _vp, _vp, _vp, _vp, _vp]),
    "niti_conv2d_i8_dgrad_requant": (_i, [_vp, _vp, _vp] + [_i] * 9 + [_u, _i, _i, _i, _i, _u, _vp, _vp, _sz, _vp, _vp, _vp, _vp, _vp, _sz, _vp]),
    "niti_conv2d_i8_dgrad_requant_unpool": (_i, [_vp, _vp, _vp, _vp, _vp, _i] + [_i] * 9 + [_u, _i, _i, _i, _i, _u, _vp, _sz, _vp, _vp, _vp, _vp,
                                                 _vp, _sz, _vp]),
    "niti_conv2d_i8_wgrad_workspace": (_sz, [_i] * 8),
    "niti_conv2d_i8_wgrad": (_i, [_vp, _vp, _vp] + [_i] * 9 + [_u, _vp, _vp, _sz, _vp]),
    "niti_conv2d_i8_wgrad_update_sync_words": (_sz, [_i] * 9),
    "niti_conv2d_i8_wgrad_update": (_i, [_vp, _vp, _vp] + [_i] * 10 + [_u, _i, _i, _i, _i, _vp, _sz, _vp, _vp, _vp, _vp, _vp, _vp,
                                         _vp, _vp, _sz, _vp]),
    "niti_gemm_i8_workspace": (_sz, [_i] * 5),
    "niti_gemm_i8": (_i, [_i, _i, _vp, _vp, _vp, _i, _i, _i, _u, _vp, _vp, _sz, _vp]),
    "niti_absmax_i32": (_i, [_vp, _i64, _vp, _vp]),
    "niti_requant_i32_i8": (_i, [_vp, _vp, _i64, _vp, _i, _i, _i, _i, _vp, _u, _vp, _vp, _vp, _vp, _vp]),
    "niti_grad_update_i8": (_i, [_vp, _vp, _i64, _vp, _i, _i, _i, _i, _vp, _vp, _vp, _vp, _vp, _vp, _vp]),
    "niti_pad_rows_i8": (_i, [_vp, _vp, _i64, _i, _i, _vp]),
    "niti_weight_update_i8": (_i, [_vp, _vp, _i64, _vp]),
    "niti_relu_i8_fwd": (_i, [_vp, _vp, _i64, _vp]),
    "niti_relu_i8_bwd": (_i, [_vp, _vp, _vp, _i64, _vp]),
    "niti_mask_features_i8": (_i, [_vp, _vp, _vp, _i64, _i, _vp, _vp, _i, _vp]),
    "niti_quantize_f32_i8": (_i, [_vp, _vp, _i, _i, _i, _i, _i, _i, _vp, _vp, _vp]),
    "niti_maxpool_i8_fwd": (_i, [_vp, _vp] + [_i] * 7 + [_vp]),
    "niti_maxpool_i8_bwd": (_i, [_vp, _vp, _vp, _vp] + [_i] * 8 + [_vp]),
    "niti_fc_i8_sync_words": (_sz, [_i] * 4),
    "niti_fc_i8_fwd_requant": (_i, [_vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _i, _u, _vp, _sz, _vp, _vp, _vp, _vp, _vp]),
    "niti_fc_i8_dgrad_requant": (_i, [_vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _i, _vp, _sz, _vp, _vp, _vp, _vp, _vp]),
    "niti_fc_i8_wgrad_update": (_i, [_vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _i, _vp, _sz, _vp, _vp, _vp, _vp, _vp, _vp]),
    "niti_linear_i8_sync_words": (_sz, [_i] * 4),
    "niti_linear_i8_fwd_requant": (_i, [_vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _i, _u, _vp, _vp, _sz, _vp, _vp, _vp, _vp, _vp]),
    "niti_linear_i8_dgrad_requant": (_i, [_vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _i, _vp, _vp, _sz, _vp, _vp, _vp, _vp, _vp]),
    "niti_linear_i8_wgrad_update": (_i, [_vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _i, _vp, _vp, _sz, _vp, _vp, _vp, _vp, _vp, _vp]),
    "niti_loss_grad_i8": (_i, [_vp, _vp, _vp, _vp, _vp, _i, _i, _i, _vp]),
    "niti_loss_grad_i8_rng": (_i, [_vp, _vp, _vp, _vp, _vp, _i, _i, _i, _vp]),
    "niti_rng_words_u32": (_i, [_vp, _u, _vp, _sz, _vp]),
    "niti_head_i8_sync_words": (_sz, [_i] * 4),
    "niti_head_i8_forward": (_i, [_vp, _vp, _vp, _i, _i, _i, _i, _vp, _vp, _i, _vp, _vp, _vp, _i, _i, _i, _i, _u, _vp, _sz,
                                  _vp, _vp, _vp, _vp, _vp]),
    "niti_head_i8_backward": (_i, [_vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _i, _i, _i, _vp, _sz, _vp, _vp, _vp,
                                   _vp, _vp, _vp, _i, _vp, _vp, _vp]),
    "niti_head_i8_backward_unpool": (_i, [_vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _i, _i, _i, _vp, _sz, _vp, _vp, _vp,
                                   _vp, _vp, _vp, _i, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _vp]),
    "niti_mfma_probe_i8": (_i, [_vp, _sz, _i, _i, _vp, _vp, _vp]),
    "niti_group_conv_i8_f32": (_i, [_vp, _vp, _vp] + [_i] * 12 + [_vp]),
}

_lib = None


class NitiError(RuntimeError):
    """A C-ABI call returned a non-zero status (the reference's extensions call exit() here)."""


def lib() -> C.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(SO_PATH):
            raise ImportError(
                "niti_amd: %s is missing; build it with `python -m niti_amd.build` "
                "(there is no fallback implementation)" % SO_PATH)
        handle = C.CDLL(SO_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(handle, name)
            fn.restype = res
            fn.argtypes = args
        _lib = handle
    return _lib


def check(status: int, what: str) -> None:
    if status != OK:
        l = lib()
        raise NitiError("%s: %s (%s)" % (what, l.niti_status_string(status).decode(), l.niti_last_error().decode()))
