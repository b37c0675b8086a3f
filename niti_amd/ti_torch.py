"""Integer layer library with the reference's ``ti_torch`` API (class and function names, tuple
conventions ``(int8 tensor, exponent)``, module-level switches) on top of libniti_gfx950.so.

Differences in mechanism, not in results:
  * every requantisation is one device kernel that reads the tensor range the producing
    conv/GEMM kernel left in device memory; shifts and exponents stay on the device as 1-element
    int32 tensors, so a training step contains no host synchronisation (the reference
    synchronises twice per requantisation, ti_torch.py:369-377);
  * dgrad and wgrad are C-ABI entry points instead of flip/transpose/contiguous copies around the
    forward convolution (ti_torch.py:404-405, 430-432);
  * the weight gradient is rounded and applied to the weights in one pass (ti_torch.py:16-21).

Switches (module globals, like the reference's ti_torch.py:457-464 plus the two that main.py
injects): BITWIDTH, ACT_ROUND_METHOD, ERROR_ROUND_METHOD, GRAD_ROUND_METHOD, WEIGHT_INIT_METHOD,
GPU, GRAD_BITWIDTH, TRAINING.  Added here: DIV_MODE ("floor" = meaning of ``//`` on torch >= 1.13,
"trunc" = torch <= 1.12), BW_MODE ("int" exact ceil(log2) / "f32" the reference's float
evaluation), F32_EPILOGUE (reproduce the CUTLASS int32->fp32->int32 epilogue), POOL_TIES.
"""
from __future__ import annotations

import math

import torch
import torch.nn.functional as F
from torch.nn.modules import Module

from . import ops

GPU = "cuda"
BITWIDTH = 7
GRAD_BITWIDTH = 5      # main.py:72-77 sets 5 -> 4 -> 3 over the epochs
TRAINING = True        # main.py:146-149
DIV_MODE = "floor"
BW_MODE = "int"
F32_EPILOGUE = True
POOL_TIES = "first"


# ------------------------------------------------------------------------------------------
# small helpers
# ------------------------------------------------------------------------------------------
_EXP_CONSTANTS = {}


def _exp_tensor(e, device) -> torch.Tensor:
    """Exponent as a 1-element int32 device tensor (accepts int, float, 0-d or 1-element tensors).
    Host values are uploaded once and cached, so steady-state steps issue no host-to-device copies
    (which also keeps a step capturable into a HIP graph)."""
    if isinstance(e, torch.Tensor):
        if e.is_cuda:
            return e.reshape(1) if e.dtype == torch.int32 else e.reshape(1).to(torch.int32)
        e = int(e)
    key = (int(e), str(device))
    t = _EXP_CONSTANTS.get(key)
    if t is None:
        t = torch.tensor([int(e)], dtype=torch.int32, device=device)
        _EXP_CONSTANTS[key] = t
    return t


def _planted_absmax(shift: int, target_bits: int, device) -> torch.Tensor:
    """A range whose bit-width is exactly target_bits + shift (so a kernel applies that shift)."""
    bits = target_bits + int(shift)
    if not 1 <= int(shift) or bits > 31:
        raise ValueError("shift %d out of range" % shift)
    key = ("absmax", bits, str(device))
    t = _EXP_CONSTANTS.get(key)
    if t is None:
        t = torch.tensor([2 ** (bits - 1) + 1], dtype=torch.int64, device=device).to(torch.int32)
        _EXP_CONSTANTS[key] = t
    return t


def _standalone(x: torch.Tensor, shift: int, method: str, rand=None) -> torch.Tensor:
    x32 = x.to(torch.int32).contiguous()
    am = _planted_absmax(shift, BITWIDTH, x32.device)
    y, _ = ops.requant(x32, am, BITWIDTH, method, DIV_MODE, "int", rand)
    return y


def RoundShift(input, shift):
    """ti_torch.py:23-31."""
    return _standalone(input, shift, "round")


def StoShift(input, shift, rand=None):
    """ti_torch.py:33-46; ``rand`` (int32, one per element, in [0, 2**shift)) replaces the device
    ``torch.randint`` when given."""
    if rand is None:
        rand = torch.randint(0, 2 ** shift, input.shape, dtype=torch.int32, device=input.device)
    return _standalone(input, shift, "sto", rand.to(torch.int32).contiguous())


def PstoShift(input, shift):
    """ti_torch.py:48-69."""
    return _standalone(input, shift, "psto")


ACT_ROUND_METHOD = RoundShift
ERROR_ROUND_METHOD = RoundShift
GRAD_ROUND_METHOD = PstoShift


def _method_name(fn) -> str:
    if fn is RoundShift:
        return "round"
    if fn is StoShift:
        return "sto"
    if fn is PstoShift:
        return "psto"
    raise ValueError("rounding method must be RoundShift, StoShift or PstoShift")


def _rand_bits_like(x: torch.Tensor) -> torch.Tensor:
    """31 uniform random bits per element; the kernel keeps the low `shift` ones."""
    return torch.randint(0, 2 ** 31 - 1, x.shape, dtype=torch.int32, device=x.device)


def int8_clip(input, clip_val=127):
    """ti_torch.py:71-72."""
    return torch.clamp(input, -clip_val, clip_val).type(torch.int8)


def Int8Tensor(val):
    return torch.tensor(val, dtype=torch.int8).to(GPU)


def Int8zeros(size):
    return torch.zeros(size=size, dtype=torch.int8, device=GPU)


def roundoff4(size):
    return (size + 3) // 4 * 4


# ------------------------------------------------------------------------------------------
# range estimate and requantisation (ti_torch.py:103-147, 366-377)
# ------------------------------------------------------------------------------------------
def TensorBitwidth(val):
    """ti_torch.py:366-367 (host value; synchronises)."""
    from . import _lib
    return int(_lib.lib().niti_bitwidth(int(val), _lib.BW[BW_MODE]))


def RangeEstimate(input):
    """ti_torch.py:369-377.  Returns a Python int like the reference, which costs a device->host
    copy; the layers below never call it."""
    am = ops.absmax_i32(input.to(torch.int32).contiguous())
    return TensorBitwidth(int(am.item()) & 0xFFFFFFFF)


def _requant(acc, target_bits, fn, absmax=None, rand=None, relu=False, exp_a=None, exp_b=None, want_exp=False):
    acc = acc.contiguous()
    if acc.dtype != torch.int32:
        acc = acc.to(torch.int32)        # first-layer gradients arrive as integer-valued float32
    if absmax is None:
        absmax = ops.absmax_i32(acc)
    method = _method_name(fn)
    if method == "sto" and rand is None:
        rand = _rand_bits_like(acc)
    exp_out = torch.empty(1, dtype=torch.int32, device=acc.device) if want_exp else None
    y, shift = ops.requant(acc, absmax, target_bits, method, DIV_MODE, BW_MODE, rand, relu,
                           exp_a=exp_a, exp_b=exp_b, exp_out=exp_out)
    return y, shift, exp_out


def act_calc(int32_acc, exp_in, absmax=None, rand=None):
    """ti_torch.py:103-117.  Returns (int8 tensor, exp_out) with exp_out a 1-element int32 device
    tensor equal to exp_in + shift."""
    e = _exp_tensor(exp_in, int32_acc.device)
    y, _, exp_out = _requant(int32_acc, BITWIDTH, ACT_ROUND_METHOD, absmax, rand, exp_a=e, want_exp=True)
    return y, exp_out


def err_calc(int32_acc, absmax=None, rand=None):
    """ti_torch.py:119-133.  Returns (int8 tensor, shift) with shift a 1-element int32 device tensor."""
    y, shift, _ = _requant(int32_acc, BITWIDTH, ERROR_ROUND_METHOD, absmax, rand)
    return y, shift


def grad_calc(int32_acc, mu, absmax=None, rand=None):
    """ti_torch.py:135-147."""
    y, shift, _ = _requant(int32_acc, mu, GRAD_ROUND_METHOD, absmax, rand)
    return y, shift


FUSE_CONV_REQUANT = True     # run convolution + requantisation as one launch where the library covers the shape
KEEP_INT32_GRAD = False      # also store layer.grad_int32acc when the weight gradient is rounded and applied in one call
_fused_refused = set()       # (dgrad, input shape, filter shape, stride, padding) the device turned out too small for


def _conv_requant_fused(dgrad, x, w, stride, padding, fn, rand, relu, exp_a, exp_b, relu_mask=None, prepared_filter=None,
                        forward_filter=None, shift_state=None, pool_out=None, unpool=None):
    """conv (forward or data gradient) + act_calc / err_calc as one launch.  Returns (int8 tensor, shift,
    exp_out) or None when the call needs the two-pass path: a shape outside the single-launch kernel, more
    workgroups than the device holds at once, or StoShift (ti_torch.py:33-46) on a 2 x 2 map or together with the
    pooling's backward pass.  StoShift otherwise runs inside the launch on ``rand`` (int32, shaped like the output;
    drawn here when the caller gives none)."""
    method = _method_name(fn)
    if not FUSE_CONV_REQUANT or (method != "sto" and rand is not None):
        return None
    key = (dgrad, tuple(x.shape), tuple(w.shape), stride, padding, unpool is not None)
    if key in _fused_refused:
        return None
    N = x.shape[0]
    K, R, S, C = w.shape
    H, W = (x.shape[1] - 2 * padding + R - 1, x.shape[2] - 2 * padding + S - 1) if dgrad else (x.shape[1], x.shape[2])
    if ops.conv_requant_sync_words(N, H, W, C, K, R, S, stride, padding, dgrad) == 0:
        _fused_refused.add(key)
        return None
    if method == "sto":
        if unpool is not None or H == 2:
            return None
        out_shape = (N, H, W, C) if dgrad else (N, (H + 2 * padding - R) // stride + 1, (W + 2 * padding - S) // stride + 1, K)
        if rand is None:
            rand = torch.randint(0, 2 ** 31 - 1, out_shape, dtype=torch.int32, device=x.device)
        elif rand.dtype != torch.int32 or tuple(rand.shape) != out_shape:
            return None
        rand = rand.contiguous()
    from ._lib import NitiError
    exp_out = torch.empty(1, dtype=torch.int32, device=x.device)
    call = ops.conv2d_dgrad_requant if dgrad else ops.conv2d_fprop_requant
    kw = dict(relu=relu, prepared_filter=prepared_filter) if not dgrad else dict(relu_mask=relu_mask, forward_filter=forward_filter)
    if pool_out is not None:
        kw.update(pool_out=pool_out)
    if unpool is not None:
        kw.update(unpool=unpool)
    if shift_state is not None:     # the tensor's shift of the previous step: the kernel's prediction for this one
        kw.update(shift_out=shift_state, shift_hint=True)
    if method == "sto":
        kw.update(rand=rand)
    try:
        y, shift, _ = call(x, w, stride, padding, f32_epilogue=F32_EPILOGUE, target_bits=BITWIDTH, method=method,
                           div_mode=DIV_MODE, bw_mode=BW_MODE, exp_a=exp_a, exp_b=exp_b, exp_out=exp_out, **kw)
    except NitiError as e:
        if "do not fit" not in str(e):
            raise
        _fused_refused.add(key)
        return None
    return y, shift, exp_out


# ------------------------------------------------------------------------------------------
# op wrappers (ti_torch.py:152-233)
# ------------------------------------------------------------------------------------------
def int8mm(lhs, rhs):
    """ti_torch.py:152-176: [m,k] x [k,n] -> contiguous int32 [m,n] (any m, n, k)."""
    return ops.gemm(lhs.contiguous(), rhs.contiguous())


def _pad_channels16(t):
    if t.size(3) % 16 == 0:
        return t
    if t.is_cuda and t.dtype == torch.int8:
        return ops.pad_last_dim(t.contiguous(), 16)
    return F.pad(t, (0, 16 - t.size(3) % 16), "constant", 0)


def conv2d_int8(input, weight, stride=1, padding=1, absmax=None):
    """ti_torch.py:178-192: NHWC int8 x KRSC int8 -> NPQK int32."""
    return ops.conv2d_fprop(_pad_channels16(input).contiguous(), _pad_channels16(weight).contiguous(), stride, padding,
                            f32_epilogue=F32_EPILOGUE, absmax=absmax)


def conv2d_weight_int8(input, weight_size, grad_output, stride=1, padding=0, dilation=1):
    """ti_torch.py:194-233: first-layer weight gradient, returned like the reference as an
    integer-valued float32 KRSC tensor."""
    if stride != 1 or dilation != 1:
        raise RuntimeError("conv2d_weight_int8: only stride 1, dilation 1 (as guarded in the reference, ti_torch.py:413)")
    dw = ops.conv2d_wgrad(input.contiguous(), grad_output.contiguous(), weight_size[1], weight_size[2], stride, padding)
    return dw.float()


# ------------------------------------------------------------------------------------------
# quantisers / initialisers (ti_torch.py:77-99, 334-364)
# ------------------------------------------------------------------------------------------
def _ceil_log2(r):
    """``torch.ceil(torch.log2(r))`` of ti_torch.py:336,348.  BW_MODE "int" (default): exact arithmetic on the float's
    exponent and mantissa (r = m * 2^e, 0.5 <= m < 1: e - 1 for a power of two, e otherwise), so that every device
    gives the same integer.  BW_MODE "f32": the reference's own float32 expression, whose log2 rounds
    k + log2(1 + d) back to k for the first float32 values above 2^k, k >= 4 (nextafter(16) gives 4 where the exact
    value is 5: the exponent is then one lower and the largest value saturates at 127).  0-d float tensor."""
    if BW_MODE == "f32":
        return torch.ceil(torch.log2(r.float()))
    m, e = torch.frexp(r.float())
    return torch.where(m == 0.5, e - 1, e).to(torch.float32)


def weight_quant(input):
    """ti_torch.py:334-339.  Returns (int8 weights on the GPU, exponent as a 0-d float tensor)."""
    input_range = torch.max(torch.abs(input))
    input_bitwidth = _ceil_log2(input_range)
    act_exp = input_bitwidth - 7
    round_val = torch.round(input / input_range * (2 ** 7 - 1)).type(torch.int8).to(GPU)
    return round_val, act_exp


def UniformWeights(size):
    """ti_torch.py:77-85 (Xavier-uniform drawn in KCRS, stored KRSC)."""
    if len(size) == 4:
        temp = torch.zeros(size).permute(0, 3, 1, 2).contiguous()
        torch.nn.init.xavier_uniform_(temp)
        return weight_quant(temp.permute(0, 2, 3, 1).contiguous())
    temp = torch.zeros(size)
    torch.nn.init.xavier_uniform_(temp)
    return weight_quant(temp)


def NormalWeight(size):
    """ti_torch.py:87-95."""
    if len(size) == 4:
        temp = torch.zeros(size).permute(0, 3, 1, 2).contiguous()
        torch.nn.init.xavier_normal_(temp)
        return weight_quant(temp.permute(0, 2, 3, 1).contiguous())
    temp = torch.zeros(size)
    torch.nn.init.xavier_normal_(temp)
    return weight_quant(temp)


WEIGHT_INIT_METHOD = UniformWeights


def TiFloatToInt8(input):
    """ti_torch.py:341-356: float tensor -> (int8 tensor on the GPU, exponent).  The exponent is
    returned as a 0-d float tensor like the reference; no host synchronisation.  The range is a tensor-library
    reduction, whose multi-block form clears its scratch words with a memset node: keep this call outside a captured
    HIP graph (train.StepGraph quantises eagerly and captures forward_int8 + backward)."""
    input = input.to(GPU)
    input_range = torch.max(torch.abs(input))
    input_bitwidth = _ceil_log2(input_range)
    act_exp = input_bitwidth - BITWIDTH
    norm_val = input * (2 ** (BITWIDTH - input_bitwidth))
    round_val = torch.round(norm_val)
    clamp_val = torch.clamp(round_val, -128, 127).type(torch.int8)
    return clamp_val, act_exp


def TiInt8ToFloat(input):
    """ti_torch.py:358-364."""
    act_in, exp_in = input
    if not isinstance(exp_in, torch.Tensor):
        exp_in = torch.tensor(float(exp_in), device=act_in.device)
    return act_in.float() * (2 ** (exp_in.float().reshape(())))


# ------------------------------------------------------------------------------------------
# layers
# ------------------------------------------------------------------------------------------
class UpdateWeight(Module):
    """ti_torch.py:11-21: vanilla integer SGD shared by TiConv2d and TiLinear.  grad_calc and the
    saturating subtraction run as one kernel; ``self.grad`` (the rounded int8 gradient) is kept only
    when ``keep_grad`` is set."""
    keep_grad = False

    def _init_weight(self, size):
        w, e = WEIGHT_INIT_METHOD(size)
        self.weight = w.to(GPU).contiguous()
        self.weight_exp = e if isinstance(e, torch.Tensor) else torch.tensor(float(e))

    def _wexp(self):
        """weight_exp (a host-side 0-d float tensor, as in the reference) as a cached device int32."""
        cached = getattr(self, "_wexp_cache", None)
        if cached is None or cached[0] is not self.weight_exp:
            cached = (self.weight_exp, _exp_tensor(self.weight_exp, self.weight.device))
            self._wexp_cache = cached
        return cached[1]

    def weight_update(self, absmax=None, rand=None):
        g = self.grad_int32acc
        if g.dtype != torch.int32:
            g = g.to(torch.int32)
        g = g.contiguous()
        if absmax is None:
            absmax = ops.absmax_i32(g)
        method = _method_name(GRAD_ROUND_METHOD)
        if method == "sto" and rand is None:
            rand = _rand_bits_like(g)
        self.grad_exp = torch.empty(1, dtype=torch.int32, device=g.device)
        if not self.weight.is_contiguous():
            self.weight = self.weight.contiguous()
        self.grad, self.grad_shift = ops.grad_update(
            g, self.weight, absmax, GRAD_BITWIDTH, method, DIV_MODE, BW_MODE, rand, want_grad=self.keep_grad,
            exp_a=_exp_tensor(self.err_exp, g.device), exp_b=_exp_tensor(self.act_in_exp, g.device), exp_out=self.grad_exp)
        self._wprep_key = None      # any kernel-ready copy of the old weights is stale now


class TiConv2d(UpdateWeight):
    """ti_torch.py:379-437: int8 convolution layer, NHWC activations, KRSC weights.
    ``fuse_relu`` folds the following TiReLU's forward into the activation requantisation."""

    def __init__(self, in_channels, out_channels, kernel_size=3, stride=1, padding=1, first_layer=False):
        super().__init__()
        self._init_weight(torch.Size([out_channels, kernel_size, kernel_size, in_channels]))
        self.first_layer = first_layer
        self.stride = stride
        self.padding = padding
        self.fuse_relu = False
        self.relu_below = False
        self.pool_after = None      # the 2x2 / stride-2 TiMaxpool2d behind this layer's (fused) ReLU, if its forward is folded in
        self.pool_below = None      # the 2x2 / stride-2 TiMaxpool2d in front of this layer, if its backward pass is folded in

    def forward(self, input, rand=None):
        self.act, self.act_in_exp = input
        dev = self.act.device
        self.act16 = _pad_channels16(self.act).contiguous()      # channel-padded copy, reused by the weight gradient
        # With an up-to-date kernel-ready filter copy the padded weights are passed for their shape only: the first
        # layer then reuses the padded tensor the copy was made from instead of padding the weights again every step.
        key = (self.weight.data_ptr(), self.weight._version, tuple(self.act16.shape))
        shape_only = (self.weight.shape[3] % 16 != 0 and getattr(self, "_wprep_key", None) == key
                      and getattr(self, "_wprep", None) is not None and getattr(self, "_w16_kept", None) is not None)
        w16 = self._w16_kept if shape_only else _pad_channels16(self.weight).contiguous()
        self._w16_kept = w16 if self.weight.shape[3] % 16 != 0 else None
        exp_a, exp_b = _exp_tensor(self.act_in_exp, dev), self._wexp()
        pooled = None
        N, H, W, _ = self.act16.shape
        if self.pool_after is not None and self.fuse_relu and self.stride == 1 and self.padding == 1 and H == W and H >= 2 and H % 2 == 0:
            pooled = torch.empty((N, H // 2, W // 2, self.weight.shape[0]), dtype=torch.int8, device=dev)
        fused = _conv_requant_fused(False, self.act16, w16, self.stride, self.padding, ACT_ROUND_METHOD, rand,
                                    self.fuse_relu, exp_a, exp_b, prepared_filter=self._forward_filter(w16),
                                    shift_state=self._shift_state("act", dev), pool_out=pooled)
        if fused is not None:
            if pooled is not None:      # the pooling layer finds its result ready when it sees this tensor
                self.pool_after.preset = (fused[0], pooled)
            return fused[0], fused[2]
        if shape_only:
            w16 = self._w16_kept = _pad_channels16(self.weight).contiguous()
        am = ops.new_scalar_u32(dev)
        acc = ops.conv2d_fprop(self.act16, w16, self.stride, self.padding, f32_epilogue=F32_EPILOGUE, absmax=am)
        act_out, _, exp_out = _requant(acc, BITWIDTH, ACT_ROUND_METHOD, am, rand, relu=self.fuse_relu,
                                       exp_a=exp_a, exp_b=exp_b, want_exp=True)
        return act_out, exp_out

    def backward(self, input, rand=None, grad_rand=None):
        err_in, err_exp = input
        err_in = err_in.contiguous()
        dev = err_in.device
        self.err_exp_in = _exp_tensor(err_exp, dev)
        self.err_exp = self.err_exp_in
        if not self.first_layer:
            # data gradient with the weights as they were in the forward pass
            # relu_below: the ReLU in front of this layer (possibly with a max-pool in between) leaves its backward
            # pass to this layer, whose input is that ReLU's (pooled) output
            from ._lib import NitiError
            mask = self.act.contiguous() if self.relu_below else None
            try:
                err_out, new_exp = self._data_gradient(err_in, rand, mask, self._dgrad_filter())
            except NitiError as e:
                if "forward filter copy" not in str(e):
                    raise
                self._dgrad_own_copy = True     # this shape's data gradient runs a kernel that needs its own copy
                err_out, new_exp = self._data_gradient(err_in, rand, mask, None)
            self.err_exp = new_exp
        K, R, S, C = self.weight.shape
        if self._wgrad_update_fused(err_in, grad_rand):
            if not self.first_layer:
                return err_out, self.err_exp
            return None
        amg = ops.new_scalar_u32(dev)
        dw = ops.conv2d_wgrad(self.act16, err_in, R, S, self.stride, self.padding,
                              f32_epilogue=F32_EPILOGUE and not self.first_layer, absmax=amg,
                              workspace=self._wgrad_workspace(err_in))
        # zero-padded input channels give zero gradient columns: drop them (they cannot raise the range)
        self.grad_int32acc = dw if dw.shape[3] == C else dw[..., :C].contiguous()
        self.weight_update(amg, grad_rand)
        if not self.first_layer:
            return err_out, self.err_exp

    def _shift_state(self, which, device):
        """1-element int32 device tensor that keeps the requantisation shift of this layer's activations ("act") or
        errors ("err") from one step to the next; the single-launch kernels take it as their prediction."""
        states = self.__dict__.setdefault("_shift_states", {})
        key = (which, str(device))
        if key not in states:
            states[key] = torch.zeros(1, dtype=torch.int32, device=device)
        return states[key]

    def _dgrad_filter(self):
        """The forward pass's kernel-ready filter copy, which the data gradient can read in place of a copy of its
        own while it matches the weights, or None."""
        if getattr(self, "_dgrad_own_copy", False) or self.act16.shape[3] != self.weight.shape[3]:
            return None
        return self._synced_filter()

    def _data_gradient(self, err_in, rand, mask, forward_filter):
        """err_calc(conv_dgrad(err_in, weight)) (ti_torch.py:422-427), the ReLU mask applied; -> (int8 error, exponent)."""
        pool = self.pool_below
        if (pool is not None and mask is not None and err_in.shape[1] >= 2 and getattr(pool, "act_out", None) is not None
                and pool.act_out.data_ptr() == mask.data_ptr() and pool.act_in.is_contiguous()):
            # the max-pool in front of this layer: its backward pass is written by this launch's epilogue
            fused = _conv_requant_fused(True, err_in, self.weight, self.stride, self.padding, ERROR_ROUND_METHOD, rand,
                                        False, self.err_exp_in, self._wexp(), relu_mask=mask, forward_filter=forward_filter,
                                        shift_state=self._shift_state("err", err_in.device), unpool=(pool.act_in, POOL_TIES))
            if fused is not None:
                pool.bwd_done = fused[0]
                return fused[0], fused[2]
        fused = _conv_requant_fused(True, err_in, self.weight, self.stride, self.padding, ERROR_ROUND_METHOD, rand,
                                    False, self.err_exp_in, self._wexp(), relu_mask=mask, forward_filter=forward_filter,
                                    shift_state=self._shift_state("err", err_in.device))
        if fused is not None:
            err_out, _, new_exp = fused
            return err_out, new_exp
        am = ops.new_scalar_u32(err_in.device)
        dx = ops.conv2d_dgrad(err_in, self.weight, self.stride, self.padding, f32_epilogue=F32_EPILOGUE, absmax=am,
                              forward_filter=forward_filter)
        err_out, _, new_exp = _requant(dx, BITWIDTH, ERROR_ROUND_METHOD, am, rand,
                                       exp_a=self.err_exp_in, exp_b=self._wexp(), want_exp=True)
        if mask is not None:
            err_out = ops.relu_bwd(mask, err_out)
        return err_out, new_exp

    def _forward_filter(self, w16):
        """Kernel-ready copy of the (channel-padded) filter for the forward pass.  Made when the weight tensor was
        replaced or modified through torch; the fused weight update keeps it in step with its own changes."""
        key = (self.weight.data_ptr(), self.weight._version, tuple(self.act16.shape))
        if getattr(self, "_wprep_key", None) != key:
            N, H, W, _ = self.act16.shape
            self._wprep = ops.conv_filter_prepare(w16, N, H, W, self.stride, self.padding)
            self._wprep_key = key
        return self._wprep

    def _wgrad_workspace(self, err_in):
        from . import _lib
        N, H, W, C16 = self.act16.shape
        K, R, S, _ = self.weight.shape
        return ops.scratch(_lib.lib().niti_conv2d_i8_wgrad_workspace(N, H, W, C16, K, R, S, self.padding), err_in.device)

    def _synced_filter(self):
        """The forward filter copy if it matches the weights as they are now (then the update maintains it)."""
        key = getattr(self, "_wprep_key", None)
        if key is None or self._wprep is None or key[:2] != (self.weight.data_ptr(), self.weight._version):
            self._wprep_key = None
            return None
        return self._wprep

    def _wgrad_update_fused(self, err_in, grad_rand):
        """Weight gradient, grad_calc and the weight update as one call into the library (no int32 gradient in
        memory unless KEEP_INT32_GRAD).  False when the call needs the separate steps."""
        method = _method_name(GRAD_ROUND_METHOD)
        if not FUSE_CONV_REQUANT or method == "sto" or grad_rand is not None or not self.weight.is_contiguous():
            return False
        N, H, W, C16 = self.act16.shape
        K, R, S, C = self.weight.shape
        if ops.wgrad_update_sync_words(N, H, W, C16, K, R, S, self.stride, self.padding) == 0:
            return False
        dev = err_in.device
        key = ("wgrad_update", tuple(self.act16.shape), tuple(self.weight.shape))
        if key in _fused_refused:
            return False
        from ._lib import NitiError
        self.grad_exp = torch.empty(1, dtype=torch.int32, device=dev)
        try:
            return self._wgrad_update_call(err_in, method, dev, C)
        except NitiError as e:
            if "do not fit" not in str(e):
                raise
            _fused_refused.add(key)     # a device too small for the finishing kernel's grid: separate steps from now on
            return False

    def _wgrad_update_call(self, err_in, method, dev, C):
        self.grad, dw, self.grad_shift, _ = ops.conv2d_wgrad_update(
            self.act16, err_in, self.weight, self.stride, self.padding, f32_epilogue=F32_EPILOGUE and not self.first_layer,
            mu=GRAD_BITWIDTH, method=method, div_mode=DIV_MODE, bw_mode=BW_MODE, want_grad=self.keep_grad,
            want_dw=KEEP_INT32_GRAD, exp_a=_exp_tensor(self.err_exp, dev), exp_b=_exp_tensor(self.act_in_exp, dev),
            exp_out=self.grad_exp, workspace=self._wgrad_workspace(err_in), prepared_filter=self._synced_filter(),
            shift_out=self._shift_state("grad", dev), shift_hint=True)
        self.grad_int32acc = None if dw is None else (dw if dw.shape[3] == C else dw[..., :C].contiguous())
        return True


class TiLinear(UpdateWeight):
    """ti_torch.py:235-266: int8 fully connected layer, weight [out_features, in_features]."""

    def __init__(self, in_features, out_features, last_layer=False):
        super().__init__()
        self._init_weight(torch.Size([out_features, in_features]))
        self.last_layer = last_layer
        self.__dict__["drop_below"] = None   # the TiDropout in front of this layer whose masking this layer's kernels take over
        self.rng = None             # RngBox of the network (dropout mask / loss rounding drawn inside the kernels)
        self.next_target = None     # (targets, random integers or None): evaluate the loss gradient in the next forward
        self.loss_grad = None       # (targets, loss gradient) left by that forward
        self._dropped = None        # dropout mask the last forward applied itself

    def _head(self, which, M, methods, rands):
        """The pass runs as one of the classifier-head kernels (dropout, loss gradient, both backward products and the
        update folded in) when the shape is inside them and no rounding needs random input."""
        O, F = self.weight.shape
        return (FUSE_CONV_REQUANT and all(r is None for r in rands) and all(_method_name(m) != "sto" for m in methods)
                and self.weight.is_contiguous() and ("head", which, M, O, F) not in _fused_refused
                and ops.head_sync_words(which, M, O, F) > 0)

    def _rng_state(self, dev):
        return self.rng.state(dev) if self.rng is not None else ops.rng_state(dev)

    def _one_launch(self, which, M, fn, rand):
        """The pass runs as one of the library's kernels for few output features (operands read as stored,
        requantisation folded in) when the shape is inside them and the rounding needs no random input."""
        O, F = self.weight.shape
        return (FUSE_CONV_REQUANT and rand is None and _method_name(fn) != "sto" and self.weight.is_contiguous()
                and (which, M, O, F) not in _fused_refused and ops.fc_sync_words(which, M, O, F) > 0)

    def _wide(self, which, M):
        """The pass runs as one of the library's any-width kernels (operands as stored, requantisation folded in, random
        rounding included) when the shape is inside them and the layer has more than a few output features."""
        O, F = self.weight.shape
        return (FUSE_CONV_REQUANT and O > 16 and self.weight.is_contiguous() and ("wide", which, M, O, F) not in _fused_refused
                and ops.linear_sync_words(which, M, O, F) > 0)

    @staticmethod
    def _sto_rand(fn, rand, shape, dev):
        """Random integers for a stochastic rounding of a tensor of ``shape`` (the caller's, or drawn here)."""
        if _method_name(fn) != "sto":
            return None
        return rand if rand is not None else torch.randint(0, 2 ** 31 - 1, shape, dtype=torch.int32, device=dev)

    def _try(self, which, M, call):
        """``call()``, or None when the device turned out too small to hold the kernel's grid at once."""
        from ._lib import NitiError
        try:
            return call()
        except NitiError as e:
            if "do not fit" not in str(e):
                raise
            _fused_refused.add((which, M) + tuple(self.weight.shape))
            return None

    def forward(self, input, rand=None):
        self.act_in = input
        act_in, exp_in = input
        act_in = act_in.contiguous()
        dev = act_in.device
        drop, self._dropped, self.loss_grad = self.drop_below, None, None
        pending = drop is not None and drop.pending is not None and drop.pending[0] is input[0]
        want_loss, self.next_target = self.next_target, None
        if (pending or want_loss is not None) and self._head("forward", act_in.shape[0], (ACT_ROUND_METHOD,), (rand,)):
            M = act_in.shape[0]
            exp_out = torch.empty(1, dtype=torch.int32, device=dev)
            given = drop.pending[1] if pending else None
            draws = (pending and given is None) or (want_loss is not None and want_loss[1] is None)
            done = self._try("head-forward", M, lambda: ops.head_forward(
                act_in, self.weight, BITWIDTH, _method_name(ACT_ROUND_METHOD), DIV_MODE, BW_MODE,
                dropout=None if not pending else ("draw" if given is None else "given"), drop_mask=given,
                rng=self._rng_state(dev) if draws else None, exp_bias=1 if pending else 0,
                target=want_loss[0] if want_loss is not None else None, loss_rand=want_loss[1] if want_loss is not None else None,
                exp_a=_exp_tensor(exp_in, dev), exp_b=self._wexp(), exp_out=exp_out))
            if done is not None:
                if pending:
                    drop.drop_mask = self._dropped = done[1]
                    drop.pending = None
                if want_loss is not None:
                    self.loss_grad = (want_loss[0], done[2])
                return done[0], exp_out
        if pending:   # the dropout left its work to this layer, which cannot take it: do it now
            act_in, exp_in = drop.apply_now(act_in, exp_in)
            self.act_in = (act_in, exp_in)
        if self._one_launch("forward", act_in.shape[0], ACT_ROUND_METHOD, rand):
            exp_out = torch.empty(1, dtype=torch.int32, device=dev)
            act_out, _, _ = ops.fc_fwd_requant(act_in, self.weight, BITWIDTH, _method_name(ACT_ROUND_METHOD), DIV_MODE, BW_MODE,
                                               exp_a=_exp_tensor(exp_in, dev), exp_b=self._wexp(), exp_out=exp_out)
            return act_out, exp_out
        if self._wide("forward", act_in.shape[0]):
            exp_out = torch.empty(1, dtype=torch.int32, device=dev)
            M, O = act_in.shape[0], self.weight.shape[0]
            done = self._try("wide-forward", M, lambda: ops.linear_fwd_requant(
                act_in, self.weight, BITWIDTH, _method_name(ACT_ROUND_METHOD), DIV_MODE, BW_MODE,
                rand=self._sto_rand(ACT_ROUND_METHOD, rand, (M, O), dev), exp_a=_exp_tensor(exp_in, dev), exp_b=self._wexp(),
                exp_out=exp_out))
            if done is not None:
                return done[0], exp_out
        am = ops.new_scalar_u32(dev)
        acc = ops.gemm(act_in, self.weight, trans_b=True, absmax=am)            # act @ W^T, W read as stored
        act_out, _, exp_out = _requant(acc, BITWIDTH, ACT_ROUND_METHOD, am, rand,
                                       exp_a=_exp_tensor(exp_in, dev), exp_b=self._wexp(), want_exp=True)
        return act_out, exp_out

    def backward(self, input, rand=None, grad_rand=None):
        err_in, err_exp = input
        err_in = err_in.contiguous()
        dev = err_in.device
        act, self.act_in_exp = self.act_in
        act = act.contiguous()
        M = err_in.shape[0]
        self.err_exp_in = _exp_tensor(err_exp, dev)
        mask = self._dropped     # the forward pass read ``act`` through this mask: act_in is the tensor in front of the dropout
        if not KEEP_INT32_GRAD and self._head("backward", M, (ERROR_ROUND_METHOD, GRAD_ROUND_METHOD), (rand, grad_rand)):
            exps = torch.empty(2, dtype=torch.int32, device=dev)
            # the 2x2 max-pool whose flattened output this layer read (TiNet.fuse): its backward pass in the same launch
            pool = self.__dict__.get("pool_below")
            unpool = None
            if (pool is not None and getattr(pool, "act_out", None) is not None and pool.act_out.data_ptr() == act.data_ptr()
                    and pool.act_out.numel() == act.numel() and pool.act_in.dim() == 4 and pool.act_in.is_contiguous()
                    and pool.act_in.dtype == torch.int8 and pool.act_in.shape[3] % 64 == 0):
                unpool = (pool.act_in, POOL_TIES, pool.relu_below)
            done = self._try("head-backward", M, lambda: ops.head_backward(
                err_in, act, self.weight, BITWIDTH, _method_name(ERROR_ROUND_METHOD), GRAD_BITWIDTH, _method_name(GRAD_ROUND_METHOD),
                DIV_MODE, BW_MODE, drop_mask=mask, want_grad=self.keep_grad, exp_err=self.err_exp_in, exp_w=self._wexp(),
                exp_act=_exp_tensor(self.act_in_exp, dev), exp_act_bias=1 if mask is not None else 0,
                err_exp_out=exps[0:1], grad_exp_out=exps[1:2], unpool=unpool))
            if done is not None:
                self.err_exp, self.grad_exp = exps[0:1], exps[1:2]
                self.grad, self.grad_shift, self.grad_int32acc = done[1], done[3], None
                if mask is not None:
                    self.drop_below.bwd_done = done[0]     # masked already
                if unpool is not None:
                    pool.bwd_routed = (done[0], done[5])
                return done[0], self.err_exp
        if mask is not None:     # the separate passes want the masked activations and their exponent
            act, self.act_in_exp = ops.mask_features(act, mask, _exp_tensor(self.act_in_exp, dev), 1)
        done = None
        if self._one_launch("dgrad", M, ERROR_ROUND_METHOD, rand):
            new_exp = torch.empty(1, dtype=torch.int32, device=dev)
            done = self._try("dgrad", M, lambda: ops.fc_dgrad_requant(
                err_in, self.weight, BITWIDTH, _method_name(ERROR_ROUND_METHOD), DIV_MODE, BW_MODE,
                exp_a=self.err_exp_in, exp_b=self._wexp(), exp_out=new_exp))
        if done is None and self._wide("dgrad", M):
            new_exp = torch.empty(1, dtype=torch.int32, device=dev)
            done = self._try("wide-dgrad", M, lambda: ops.linear_dgrad_requant(
                err_in, self.weight, BITWIDTH, _method_name(ERROR_ROUND_METHOD), DIV_MODE, BW_MODE,
                rand=self._sto_rand(ERROR_ROUND_METHOD, rand, (M, self.weight.shape[1]), dev), exp_a=self.err_exp_in,
                exp_b=self._wexp(), exp_out=new_exp))
        if done is not None:
            err_out, self.err_exp = done[0], new_exp
        else:
            am = ops.new_scalar_u32(dev)
            dx = ops.gemm(err_in, self.weight, absmax=am)                             # err @ W
            err_out, _, self.err_exp = _requant(dx, BITWIDTH, ERROR_ROUND_METHOD, am, rand,
                                                exp_a=self.err_exp_in, exp_b=self._wexp(), want_exp=True)
        done = None
        if not KEEP_INT32_GRAD and self._one_launch("wgrad", M, GRAD_ROUND_METHOD, grad_rand):
            self.grad_exp = torch.empty(1, dtype=torch.int32, device=dev)
            done = self._try("wgrad", M, lambda: ops.fc_wgrad_update(
                err_in, act, self.weight, GRAD_BITWIDTH, _method_name(GRAD_ROUND_METHOD), DIV_MODE, BW_MODE,
                want_grad=self.keep_grad, exp_a=_exp_tensor(self.err_exp, dev), exp_b=_exp_tensor(self.act_in_exp, dev),
                exp_out=self.grad_exp))
        if done is None and not KEEP_INT32_GRAD and self._wide("wgrad", M):
            self.grad_exp = torch.empty(1, dtype=torch.int32, device=dev)
            done = self._try("wide-wgrad", M, lambda: ops.linear_wgrad_update(
                err_in, act, self.weight, GRAD_BITWIDTH, _method_name(GRAD_ROUND_METHOD), DIV_MODE, BW_MODE,
                rand=self._sto_rand(GRAD_ROUND_METHOD, grad_rand, tuple(self.weight.shape), dev), want_grad=self.keep_grad,
                exp_a=_exp_tensor(self.err_exp, dev), exp_b=_exp_tensor(self.act_in_exp, dev), exp_out=self.grad_exp))
        if done is not None:
            self.grad, self.grad_shift, self.grad_int32acc = done[0], done[1], None
        else:
            amg = ops.new_scalar_u32(dev)
            self.grad_int32acc = ops.gemm(err_in, act, trans_a=True, absmax=amg)     # err^T @ act
            self.weight_update(amg, grad_rand)
        return err_out, self.err_exp


class TiReLU(Module):
    """ti_torch.py:268-290.  With ``fused`` set the preceding TiConv2d already clamped at zero and
    forward only records its input (the clamped tensor: ``act > 0`` is the same test on it)."""

    def __init__(self):
        super().__init__()
        self.fused = False
        self.bwd_folded = False

    def forward(self, input):
        self.act_in = input
        act_in, exp_in = input
        if self.fused:
            return input
        return ops.relu_fwd(act_in.contiguous()), exp_in

    def backward(self, input):
        if self.bwd_folded:      # the convolution or pooling above this layer masked its data gradient already
            return input
        err_in, err_exp = input
        act, _ = self.act_in
        return ops.relu_bwd(act.contiguous(), err_in.contiguous()), err_exp


class TiMaxpool2d(Module):
    """ti_torch.py:292-316."""

    def __init__(self, kernel_size, stride, padding=0):
        super().__init__()
        self.kernel_size = kernel_size
        self.stride = stride
        self.padding = padding
        self.relu_below = False     # the ReLU in front of this layer leaves its backward pass to this layer
        self.preset = None          # (input tensor, pooled tensor) left by the convolution that computed both
        self.bwd_done = None        # the error tensor a convolution behind this layer has already routed through it
        self.bwd_routed = None      # (error tensor, routed result) left by the classifier behind this layer

    def forward(self, input):
        self.act_in, exp_in = input
        preset, self.preset = self.preset, None
        if preset is not None and preset[0] is self.act_in:
            self.act_out = preset[1]
            return self.act_out, exp_in
        self.act_in = self.act_in.contiguous()
        self.act_out = ops.maxpool_fwd(self.act_in, self.kernel_size, self.stride, self.padding)
        return self.act_out, exp_in

    def backward(self, input):
        err_in, err_exp = input
        done, self.bwd_done = self.bwd_done, None
        if done is not None and done is err_in:
            return input        # the data gradient behind this layer wrote its result through this pooling already
        routed, self.bwd_routed = self.bwd_routed, None
        if routed is not None and routed[0].data_ptr() == err_in.data_ptr() and routed[0].numel() == err_in.numel():
            return routed[1], err_exp     # the classifier's backward launch has run this pass
        err_out = ops.maxpool_bwd(self.act_out, err_in.contiguous(), self.act_in, self.kernel_size, self.stride,
                                  self.padding, POOL_TIES, relu=self.relu_below)
        return err_out, err_exp


class TiFlat(Module):
    """ti_torch.py:318-332."""

    def forward(self, input):
        self.act_in = input
        act_in, exp_in = input
        return act_in.view(-1, act_in.nelement() // act_in.size(0)), exp_in

    def backward(self, input):
        err_in, err_exp = input
        act, _ = self.act_in
        return err_in.view_as(act), err_exp


class TiDropout(Module):
    """ti_torch.py:439-455: one keep/drop decision per feature (not per sample), exponent + 1.
    ``mask`` (int8 0/1 per feature) can be supplied for reproducible runs.  With ``head`` set (TiNet.fuse: the
    TiLinear that follows) the masking is left to that layer's kernels, which also draw the mask."""

    def __init__(self):
        super().__init__()
        self.__dict__["head"] = None   # the TiLinear behind this layer that applies the mask in its own launches
        self.pending = None      # (activation tensor, given mask or None) handed to that layer
        self.bwd_done = None     # the error tensor that layer has already masked

    def forward(self, input, mask=None):
        if TRAINING:
            act_in, exp_in = input
            if mask is not None:
                mask = mask.to(act_in.device)
            if (self.head is not None and FUSE_CONV_REQUANT and act_in.is_cuda and act_in.dtype == torch.int8 and act_in.dim() == 2
                    and act_in.is_contiguous() and (mask is None or (mask.dtype == torch.int8 and mask.is_contiguous()))):
                self.pending = (act_in, mask)
                return input
            return self.apply_now(act_in, exp_in, mask)
        self.pending = None
        return input

    def apply_now(self, act_in, exp_in, mask=None):
        if mask is None and self.pending is not None:
            mask = self.pending[1]
        self.pending = None
        if mask is None:
            mask = torch.randint(low=0, high=2, size=(act_in.size(1),), dtype=torch.int8, device=act_in.device)
        self.drop_mask = mask.to(act_in.device)
        if self._one_launch(act_in):
            return ops.mask_features(act_in, self.drop_mask, _exp_tensor(exp_in, act_in.device), 1)
        return act_in * self.drop_mask, _exp_tensor(exp_in, act_in.device) + 1

    def _one_launch(self, t):
        m = self.drop_mask
        return (t.is_cuda and t.dtype == torch.int8 and m.dtype == torch.int8 and t.dim() == 2 and t.is_contiguous()
                and m.is_contiguous() and t.shape[1] % 16 == 0 and t.data_ptr() % 16 == 0 and m.data_ptr() % 16 == 0)

    def backward(self, input):
        err_in, err_exp = input
        done, self.bwd_done = self.bwd_done, None
        if done is not None and done is err_in:
            return input        # the layer behind this one masked its data gradient already
        if self._one_launch(err_in):
            return ops.mask_features(err_in, self.drop_mask), err_exp
        return err_in * self.drop_mask, err_exp


class RngBox:
    """The generator state (ops.rng_state) of one network, created on first use with a key drawn from torch's default
    CPU generator: two networks built after the same ``torch.manual_seed`` draw the same sequence."""

    def __init__(self):
        self._state = {}

    def state(self, device):
        key = str(device)
        if key not in self._state:
            if torch.cuda.is_current_stream_capturing():
                raise RuntimeError("RngBox: first use under graph capture; run one step eagerly first")
            self._state[key] = ops.rng_state(device, int(torch.empty((), dtype=torch.int64).random_().item()))
        return self._state[key]
