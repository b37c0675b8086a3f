"""Tensor-level front end of the C ABI: takes torch device tensors, allocates outputs and
workspaces with the torch allocator, launches on torch's current stream.  Nothing here
computes: every function is one (or a few) calls into libniti_gfx950.so."""
from __future__ import annotations

from typing import Optional, Tuple

import torch

from . import _lib as L


def _stream(t: torch.Tensor):
    return torch.cuda.current_stream(t.device).cuda_stream


def _chk_dev(*ts: torch.Tensor) -> None:
    for t in ts:
        if t is None:
            continue
        if not t.is_cuda:
            raise RuntimeError("niti_amd: tensor must live on the GPU")
        if not t.is_contiguous():
            raise RuntimeError("niti_amd: tensor must be contiguous")


def _ptr(t: Optional[torch.Tensor]):
    return None if t is None else t.data_ptr()


def new_scalar_u32(device) -> torch.Tensor:
    """Zeroed device scalar the kernels fold max|x| into (stored as int32 bits of a uint32)."""
    return torch.zeros(1, dtype=torch.int32, device=device)


def _flags(f32_epilogue: bool) -> int:
    return L.EPI_F32_ROUNDTRIP if f32_epilogue else 0


def conv_filter_prepare(w, N, H, W, stride=1, padding=1, dgrad=False):
    """Kernel-ready copy of the [K,R,S,C] filter for a convolution over an [N,H,W,*] input (forward) or
    the data gradient of one (dgrad=True).  Returns None when the kernels read the filter as stored."""
    _chk_dev(w)
    K, R, S, C = w.shape
    nbytes = L.lib().niti_conv2d_i8_filter_workspace(N, H, W, C, K, R, S, stride, padding, int(dgrad))
    if nbytes == 0:
        return None
    dst = torch.empty(nbytes, dtype=torch.int8, device=w.device)
    st = L.lib().niti_conv2d_i8_filter_prepare(_ptr(w), _ptr(dst), nbytes, N, H, W, C, K, R, S, stride, padding,
                                               int(dgrad), _stream(w))
    L.check(st, "niti_conv2d_i8_filter_prepare")
    return dst


def conv2d_fprop(x, w, stride=1, padding=1, f32_epilogue=False, absmax: Optional[torch.Tensor] = None,
                 prepared_filter=None):
    """x [N,H,W,C] int8, w [K,R,S,C] int8 -> [N,P,Q,K] int32.  ``prepared_filter``: the output of
    conv_filter_prepare(w, N, H, W, stride, padding), to keep the filter copy out of the call."""
    _chk_dev(x, w, absmax, prepared_filter)
    if x.dtype != torch.int8 or w.dtype != torch.int8:
        raise RuntimeError("conv2d_fprop: int8 tensors expected")
    N, H, W, C = x.shape
    K, R, S, C2 = w.shape
    if C2 != C:
        raise RuntimeError("conv2d_fprop: channel mismatch %d vs %d" % (C, C2))
    P = (H + 2 * padding - R) // stride + 1
    Q = (W + 2 * padding - S) // stride + 1
    y = torch.empty((N, max(P, 0), max(Q, 0), K), dtype=torch.int32, device=x.device)
    flags = _flags(f32_epilogue)
    if prepared_filter is not None:
        st = L.lib().niti_conv2d_i8_fprop(_ptr(x), _ptr(prepared_filter), _ptr(y), N, H, W, C, K, R, S, stride, padding,
                                          flags | L.CONV_FILTER_PREPARED, _ptr(absmax), None, 0, _stream(x))
    else:
        nbytes = L.lib().niti_conv2d_i8_filter_workspace(N, H, W, C, K, R, S, stride, padding, 0)
        ws = torch.empty(nbytes, dtype=torch.int8, device=x.device) if nbytes else None
        st = L.lib().niti_conv2d_i8_fprop(_ptr(x), _ptr(w), _ptr(y), N, H, W, C, K, R, S, stride, padding, flags,
                                          _ptr(absmax), _ptr(ws), nbytes, _stream(x))
    L.check(st, "niti_conv2d_i8_fprop")
    return y


def conv2d_dgrad(err, w, stride=1, padding=1, f32_epilogue=False, absmax=None, prepared_filter=None, forward_filter=None):
    """err [N,P,Q,K] int8, w [K,R,S,C] int8 -> dx [N,H,W,C] int32 (stride 1).  ``prepared_filter``:
    the output of conv_filter_prepare(w, N, H, W, stride, padding, dgrad=True).  ``forward_filter``: the copy the
    FORWARD pass reads (conv_filter_prepare(.., dgrad=False)), for shapes where both passes run the 3x3 kernel."""
    _chk_dev(err, w, absmax, prepared_filter, forward_filter)
    N, P, Q, K = err.shape
    K2, R, S, C = w.shape
    if K2 != K:
        raise RuntimeError("conv2d_dgrad: channel mismatch")
    H = P - 2 * padding + R - 1
    W = Q - 2 * padding + S - 1
    dx = torch.empty((N, H, W, C), dtype=torch.int32, device=err.device)
    flags = _flags(f32_epilogue)
    if forward_filter is not None:
        prepared_filter, flags = forward_filter, flags | L.CONV_FILTER_FORWARD_COPY
    if prepared_filter is not None:
        st = L.lib().niti_conv2d_i8_dgrad(_ptr(err), _ptr(prepared_filter), _ptr(dx), N, H, W, C, K, R, S, stride, padding,
                                          flags | L.CONV_FILTER_PREPARED, _ptr(absmax), None, 0, _stream(err))
    else:
        nbytes = L.lib().niti_conv2d_i8_filter_workspace(N, H, W, C, K, R, S, stride, padding, 1)
        ws = torch.empty(max(nbytes, 16), dtype=torch.int8, device=err.device)
        st = L.lib().niti_conv2d_i8_dgrad(_ptr(err), _ptr(w), _ptr(dx), N, H, W, C, K, R, S, stride, padding,
                                          flags, _ptr(absmax), _ptr(ws), nbytes, _stream(err))
    L.check(st, "niti_conv2d_i8_dgrad")
    return dx


def conv_requant_sync_words(N, H, W, C, K, R=3, S=3, stride=1, padding=1, dgrad=False) -> int:
    """uint32 words of the sync buffer conv2d_fprop_requant / conv2d_dgrad_requant need for a convolution with
    INPUT [N,H,W,C] and filter [K,R,S,C]; 0 when only the two-pass path (conv2d_* then requant) covers the shape."""
    return int(L.lib().niti_conv2d_i8_requant_sync_words(N, H, W, C, K, R, S, stride, padding, int(dgrad)))


def _conv_requant(entry, dgrad, x, w, out_shape, dims, stride, padding, f32_epilogue, target_bits, method, div_mode,
                  bw_mode, relu, sync, shift_out, exp_a, exp_b, exp_out, prepared_filter, relu_mask=None, forward_filter=None,
                  shift_hint=False, pool_out=None, unpool=None, rand=None):
    _chk_dev(x, w, sync, shift_out, exp_a, exp_b, exp_out, prepared_filter, relu_mask, forward_filter, rand)
    if method == "sto":
        # StoShift folded in: one random integer per output element (its low `shift` bits are used)
        if rand is None or rand.dtype != torch.int32 or tuple(rand.shape) != tuple(out_shape) or not rand.is_contiguous():
            raise RuntimeError("%s: stochastic rounding needs `rand`, a contiguous int32 tensor shaped like the output" % entry)
        if unpool is not None:
            raise L.NitiError("%s: stochastic rounding is not folded in together with the pooling's backward pass" % entry)
    elif rand is not None:
        raise RuntimeError("%s: `rand` is only used by method='sto'" % entry)
    if relu_mask is not None and (relu_mask.dtype != torch.int8 or tuple(relu_mask.shape) != tuple(out_shape)):
        raise RuntimeError("%s: relu_mask must be int8 and shaped like the output" % entry)
    if unpool is not None:      # (pooling input [N,2H,2W,C], tie rule): the result is written at that size
        pool_in, ties = unpool
        _chk_dev(x, pool_in)
        n_, h_, w_, c_ = out_shape
        if relu_mask is None or pool_in.dtype != torch.int8 or tuple(pool_in.shape) != (n_, 2 * h_, 2 * w_, c_) or not pool_in.is_contiguous():
            raise RuntimeError("%s: unpool needs relu_mask (the pooled map) and a contiguous int8 [N,2H,2W,C] pooling input" % entry)
        entry = "niti_conv2d_i8_dgrad_requant_unpool"
        out_shape = tuple(pool_in.shape)
    if x.dtype != torch.int8 or w.dtype != torch.int8:
        raise RuntimeError("%s: int8 tensors expected" % entry)
    N, H, W, C, K, R, S = dims
    words = conv_requant_sync_words(N, H, W, C, K, R, S, stride, padding, dgrad)
    if words == 0:
        raise L.NitiError("%s: shape not covered by the single-launch path" % entry)
    if sync is None:
        sync = sync_arena.take(words, x.device)
    elif sync.dtype != torch.int32 or sync.numel() < words:
        raise RuntimeError("%s: sync must be a zeroed int32 tensor of at least %d words" % (entry, words))
    y = torch.empty(out_shape, dtype=torch.int8, device=x.device)
    if shift_out is None:
        if shift_hint:
            raise RuntimeError("%s: shift_hint needs shift_out, holding the predicted shift" % entry)
        shift_out = torch.empty(1, dtype=torch.int32, device=x.device)
    flags = _flags(f32_epilogue)
    if forward_filter is not None:
        prepared_filter, flags = forward_filter, flags | L.CONV_FILTER_FORWARD_COPY
    if prepared_filter is not None:
        wptr, ws, nbytes, flags = _ptr(prepared_filter), None, 0, flags | L.CONV_FILTER_PREPARED
    else:
        nbytes = L.lib().niti_conv2d_i8_filter_workspace(N, H, W, C, K, R, S, stride, padding, int(dgrad))
        ws = torch.empty(max(nbytes, 16), dtype=torch.int8, device=x.device)
        wptr = _ptr(w)
    head = (_ptr(x), wptr, _ptr(y), N, H, W, C, K, R, S, stride, padding, flags, target_bits, L.ROUND[method],
            L.DIV[div_mode], L.BW[bw_mode], (L.RQ_RELU if relu else 0) | (L.RQ_SHIFT_HINT if shift_hint else 0))
    tail = (_ptr(sync), sync.numel(), _ptr(shift_out), _ptr(exp_a), _ptr(exp_b), _ptr(exp_out), _ptr(ws), nbytes, _stream(x))
    if method == "sto":         # entries of their own: (pooled output,) random integers behind the output, no method argument
        entry = "niti_conv2d_i8_dgrad_requant_sto" if dgrad else "niti_conv2d_i8_fprop_requant_sto"
        head = head[:3] + ((_ptr(rand),) if dgrad else (_ptr(pool_out), _ptr(rand))) + head[3:14] + head[15:]
    elif pool_out is not None:    # the entry with the pooled output takes it right after the output
        head = head[:3] + (_ptr(pool_out),) + head[3:]
    if unpool is not None:
        head = head[:3] + (_ptr(relu_mask), _ptr(unpool[0]), L.TIES[unpool[1]]) + head[3:]
        st = getattr(L.lib(), entry)(*(head + tail))
    else:
        st = getattr(L.lib(), entry)(*(head + ((_ptr(relu_mask),) if dgrad else ()) + tail))
    L.check(st, entry)
    return y, shift_out, sync


def conv2d_fprop_requant(x, w, stride=1, padding=1, f32_epilogue=False, target_bits=7, method="round", div_mode="floor",
                         bw_mode="int", relu=False, sync=None, shift_out=None, exp_a=None, exp_b=None, exp_out=None,
                         prepared_filter=None, shift_hint=False, pool_out=None, rand=None):
    """conv2d_fprop + requant as one launch: x [N,H,W,C] int8, w [K,R,S,C] int8 -> ([N,P,Q,K] int8, device shift,
    sync).  method "sto" takes ``rand`` (int32, shaped like the output).  ``pool_out`` ([N,P/2,Q/2,K] int8): also receives the 2x2 / stride-2 maximum of the output.  sync[0] holds max|sum| afterwards, sync[1] != 0 flags a timed-out wait (invalid output).  ``sync``, if
    given, must hold conv_requant_sync_words(...) zeroed int32 words.  ``shift_hint``: ``shift_out`` holds a
    predicted shift on entry (e.g. this tensor's shift of the previous training step); a good prediction saves the
    kernel a second store pass, the results do not depend on it."""
    N, H, W, C = x.shape
    K, R, S, C2 = w.shape
    if C2 != C:
        raise RuntimeError("conv2d_fprop_requant: channel mismatch %d vs %d" % (C, C2))
    P = (H + 2 * padding - R) // stride + 1
    Q = (W + 2 * padding - S) // stride + 1
    if pool_out is not None:
        _chk_dev(x, pool_out)
        if pool_out.dtype != torch.int8 or tuple(pool_out.shape) != (N, P // 2, Q // 2, K) or not pool_out.is_contiguous():
            raise RuntimeError("conv2d_fprop_requant: pool_out must be a contiguous int8 [N,P/2,Q/2,K] tensor")
    entry = "niti_conv2d_i8_fprop_requant_pool" if pool_out is not None else "niti_conv2d_i8_fprop_requant"
    return _conv_requant(entry, False, x, w, (N, P, Q, K), (N, H, W, C, K, R, S), stride, padding,
                         f32_epilogue, target_bits, method, div_mode, bw_mode, relu, sync, shift_out, exp_a, exp_b, exp_out,
                         prepared_filter, shift_hint=shift_hint, pool_out=pool_out, rand=rand)


def conv2d_fprop_requant_static(x, w, stride=1, padding=1, f32_epilogue=False, target_bits=7, method="round", div_mode="floor",
                                bw_mode="int", relu=False, y=None, shift_out=None, exp_a=None, exp_b=None, exp_out=None,
                                prepared_filter=None, range_out=None):
    """conv2d_fprop_requant through the entry point that takes no scratch memory from the caller (the library keeps its
    sync words and filter copy in a device array of its own): only the tensors given here are touched, and when ``y``,
    ``shift_out`` are passed in nothing is allocated at all.  ``range_out``: int32[2], receives max|sum| and the
    timed-out flag.  Calls on one GPU must not overlap.  Returns (y, shift_out)."""
    _chk_dev(x, w, y, shift_out, exp_a, exp_b, exp_out, prepared_filter, range_out)
    if x.dtype != torch.int8 or w.dtype != torch.int8:
        raise RuntimeError("conv2d_fprop_requant_static: int8 tensors expected")
    N, H, W, C = x.shape
    K, R, S, C2 = w.shape
    if C2 != C:
        raise RuntimeError("conv2d_fprop_requant_static: channel mismatch %d vs %d" % (C, C2))
    P = (H + 2 * padding - R) // stride + 1
    Q = (W + 2 * padding - S) // stride + 1
    if y is None:
        y = torch.empty((N, P, Q, K), dtype=torch.int8, device=x.device)
    elif y.dtype != torch.int8 or tuple(y.shape) != (N, P, Q, K) or not y.is_contiguous():
        raise RuntimeError("conv2d_fprop_requant_static: y must be a contiguous int8 [N,P,Q,K] tensor")
    if shift_out is None:
        shift_out = torch.empty(1, dtype=torch.int32, device=x.device)
    if range_out is not None and (range_out.dtype != torch.int32 or range_out.numel() < 2):
        raise RuntimeError("conv2d_fprop_requant_static: range_out must hold two int32 words")
    flags = _flags(f32_epilogue) | (L.CONV_FILTER_PREPARED if prepared_filter is not None else 0)
    st = L.lib().niti_conv2d_i8_fprop_requant_static(
        _ptr(x), _ptr(prepared_filter if prepared_filter is not None else w), _ptr(y), N, H, W, C, K, R, S, stride, padding, flags,
        target_bits, L.ROUND[method], L.DIV[div_mode], L.BW[bw_mode], L.RQ_RELU if relu else 0, _ptr(shift_out), _ptr(exp_a),
        _ptr(exp_b), _ptr(exp_out), _ptr(range_out), _stream(x))
    L.check(st, "niti_conv2d_i8_fprop_requant_static")
    return y, shift_out


def conv2d_dgrad_requant(err, w, stride=1, padding=1, f32_epilogue=False, target_bits=7, method="round", div_mode="floor",
                         bw_mode="int", sync=None, shift_out=None, exp_a=None, exp_b=None, exp_out=None,
                         prepared_filter=None, relu_mask=None, forward_filter=None, shift_hint=False, unpool=None, rand=None):
    """conv2d_dgrad + requant as one launch: err [N,P,Q,K] int8, w [K,R,S,C] int8 -> ([N,H,W,C] int8, shift, sync).
    method "sto" takes ``rand`` (int32, shaped like the output; not together with ``unpool``).
    ``unpool`` = (pool_in [N,2H,2W,C] int8, "first" | "all") with ``relu_mask`` = the pooled map: the backward pass of
    the 2x2 / stride-2 max-pool in front of the layer is folded in and the result has pool_in's shape.
    ``relu_mask`` (int8 [N,H,W,C]): results whose mask element is not positive are stored as zero, after range
    and rounding were taken from the unmasked sums (the backward pass of a ReLU in front of the layer).
    ``forward_filter``: the copy the forward pass reads, in place of ``prepared_filter`` (see conv2d_dgrad)."""
    N, P, Q, K = err.shape
    K2, R, S, C = w.shape
    if K2 != K:
        raise RuntimeError("conv2d_dgrad_requant: channel mismatch")
    H = P - 2 * padding + R - 1
    W = Q - 2 * padding + S - 1
    return _conv_requant("niti_conv2d_i8_dgrad_requant", True, err, w, (N, H, W, C), (N, H, W, C, K, R, S), stride, padding,
                         f32_epilogue, target_bits, method, div_mode, bw_mode, False, sync, shift_out, exp_a, exp_b, exp_out,
                         prepared_filter, relu_mask, forward_filter, shift_hint, unpool=unpool, rand=rand)


_scratch = {}


def scratch(nbytes: int, device) -> torch.Tensor:
    """One grow-only int8 buffer per device for kernel workspaces that live only inside a call.  Calls on one
    stream run in order, so they can all use the same memory - which also keeps the partial sums of
    consecutive weight-gradient launches in the same cache-resident region instead of walking through fresh
    allocations.  Not for use from several streams at once."""
    key = str(device)
    buf = _scratch.get(key)
    if buf is None or buf.numel() < nbytes:
        buf = torch.empty(max(nbytes, 1 << 20), dtype=torch.int8, device=device)
        _scratch[key] = buf
    return buf


class _SyncArena:
    """Zeroed int32 words for the single-launch kernels of one training step: one fill per step instead of one
    per kernel.  ``reset`` zeroes the arena and starts handing out slices from its beginning; ``take`` returns the
    next zeroed slice.  Slices are handed out once per reset, so a kernel never sees words another kernel of the
    same step wrote.  An arena that runs out (or was never reset) grows by another zeroed chunk, which later
    resets zero as well, so ``timed_out`` covers every slice handed out since the last reset."""

    WORDS = 1 << 16
    MAX_CHUNKS = 8

    def __init__(self):
        self.chunks = {}    # device -> list of int32 tensors
        self.pos = {}       # device -> (chunk index, offset)
        self.taken = {}     # device -> list of (chunk index, offset)

    def reset(self, device):
        key = str(device)
        if key not in self.chunks:
            self.chunks[key] = [torch.zeros(self.WORDS, dtype=torch.int32, device=device)]
        else:
            for c in self.chunks[key]:
                c.zero_()
        self.pos[key] = (0, 0)
        self.taken[key] = []

    def take(self, words, device):
        key = str(device)
        if key not in self.chunks:
            self.reset(device)
        ci, off = self.pos[key]
        chunks = self.chunks[key]
        while off + words > chunks[ci].numel():
            ci, off = ci + 1, 0
            if ci == len(chunks):
                if torch.cuda.is_current_stream_capturing():
                    raise RuntimeError("sync arena: out of words while a graph is being captured; run one step eagerly first")
                if len(chunks) >= self.MAX_CHUNKS and words <= self.WORDS:
                    # a caller that never resets: start over (the fill is ordered behind the launches that used the
                    # words; their flags are gone from here but stay in the device-wide word, see sync_timeouts)
                    self.reset(device)
                    ci, off, chunks = 0, 0, self.chunks[key]
                    break
                chunks.append(torch.zeros(max(self.WORDS, words), dtype=torch.int32, device=device))
        self.pos[key] = (ci, off + (words + 31) // 32 * 32)
        self.taken[key].append((ci, off))
        return chunks[ci][off:off + words]

    def timed_out(self, device) -> bool:
        """True if a single-launch kernel that used a slice since the last reset flagged that its grid-wide wait ran
        into the time limit (its output is then invalid).  Copies the flags to the host: for the end of a step or an
        epoch, not for the inner loop."""
        key = str(device)
        flags = [self.chunks[key][ci][off + 1] for ci, off in self.taken.get(key, [])]
        if not flags:
            return False
        return bool(torch.stack(flags).ne(0).any().item())


def sync_timeouts(device=None, clear=True) -> bool:
    """True if any grid-wide wait of the library's kernels on ``device`` gave up since the flag was last cleared
    (niti_sync_timeouts): some int8 output or weight update since then was made with a wrong shift.  Unlike
    ``sync_arena.timed_out`` this survives the arena's resets.  Waits for the device's current stream."""
    import ctypes
    dev = torch.device("cuda", torch.cuda.current_device()) if device is None else torch.device(device)
    flag = ctypes.c_uint32(0)
    with torch.cuda.device(dev):
        st = L.lib().niti_sync_timeouts(ctypes.byref(flag), int(clear), torch.cuda.current_stream(dev).cuda_stream)
    L.check(st, "niti_sync_timeouts")
    return flag.value != 0


sync_arena = _SyncArena()


def conv2d_wgrad(act, err, R, S, stride=1, padding=1, f32_epilogue=False, absmax=None, workspace=None):
    """act [N,H,W,C] int8, err [N,P,Q,K] int8 -> dw [K,R,S,C] int32 (stride 1).  ``workspace``: int8 tensor of
    at least niti_conv2d_i8_wgrad_workspace bytes (default: a fresh allocation)."""
    _chk_dev(act, err, absmax, workspace)
    N, H, W, C = act.shape
    K = err.shape[3]
    dw = torch.empty((K, R, S, C), dtype=torch.int32, device=act.device)
    nbytes = L.lib().niti_conv2d_i8_wgrad_workspace(N, H, W, C, K, R, S, padding)
    ws = workspace if workspace is not None else torch.empty(max(nbytes, 16), dtype=torch.int8, device=act.device)
    if ws.numel() < nbytes:
        raise RuntimeError("conv2d_wgrad: workspace of %d bytes needed, got %d" % (nbytes, ws.numel()))
    st = L.lib().niti_conv2d_i8_wgrad(_ptr(act), _ptr(err), _ptr(dw), N, H, W, C, K, R, S, stride, padding,
                                      _flags(f32_epilogue), _ptr(absmax), _ptr(ws), nbytes, _stream(act))
    L.check(st, "niti_conv2d_i8_wgrad")
    return dw


def wgrad_update_sync_words(N, H, W, C, K, R=3, S=3, stride=1, padding=1) -> int:
    """uint32 words of the sync buffer conv2d_wgrad_update needs; 0 when only the two-pass path covers the shape."""
    return int(L.lib().niti_conv2d_i8_wgrad_update_sync_words(N, H, W, C, K, R, S, stride, padding))


def conv2d_wgrad_update(act, err, w, stride=1, padding=1, f32_epilogue=False, mu=5, method="psto", div_mode="floor",
                        bw_mode="int", sync=None, want_grad=False, want_dw=False, shift_out=None, exp_a=None, exp_b=None,
                        exp_out=None, workspace=None, prepared_filter=None, shift_hint=False):
    """Weight gradient + grad_calc + weight update: act [N,H,W,C] int8 (C may carry zero channel padding), err
    [N,H,W,K] int8, w [K,3,3,Cw] int8 updated in place.  Returns (g8 or None, dw int32 or None, device shift, sync).
    ``prepared_filter``: conv_filter_prepare(w padded to C channels, N, H, W) made earlier; it receives the updated
    weights too and stays valid for the next forward pass.  ``shift_hint``: ``shift_out`` holds a predicted shift
    on entry (the previous step's): the update's stores then overlap the wait for the tensor's range."""
    if shift_hint and shift_out is None:
        raise RuntimeError("conv2d_wgrad_update: shift_hint needs shift_out, holding the predicted shift")
    _chk_dev(act, err, w, sync, shift_out, exp_a, exp_b, exp_out, workspace, prepared_filter)
    if act.dtype != torch.int8 or err.dtype != torch.int8 or w.dtype != torch.int8:
        raise RuntimeError("conv2d_wgrad_update: int8 tensors expected")
    N, H, W, C = act.shape
    K, R, S, Cw = w.shape
    if err.shape[3] != K:
        raise RuntimeError("conv2d_wgrad_update: channel mismatch")
    words = wgrad_update_sync_words(N, H, W, C, K, R, S, stride, padding)
    if words == 0:
        raise L.NitiError("conv2d_wgrad_update: shape not covered by the single-pass path")
    if sync is None:
        sync = sync_arena.take(words, act.device)
    elif sync.dtype != torch.int32 or sync.numel() < words:
        raise RuntimeError("conv2d_wgrad_update: sync must be a zeroed int32 tensor of at least %d words" % words)
    nbytes = L.lib().niti_conv2d_i8_wgrad_workspace(N, H, W, C, K, R, S, padding)
    ws = workspace if workspace is not None else torch.empty(max(nbytes, 16), dtype=torch.int8, device=act.device)
    if ws.numel() < nbytes:
        raise RuntimeError("conv2d_wgrad_update: workspace of %d bytes needed, got %d" % (nbytes, ws.numel()))
    g8 = torch.empty(w.shape, dtype=torch.int8, device=w.device) if want_grad else None
    dw = torch.empty((K, R, S, C), dtype=torch.int32, device=w.device) if want_dw else None
    if shift_out is None:
        shift_out = torch.empty(1, dtype=torch.int32, device=w.device)
    st = L.lib().niti_conv2d_i8_wgrad_update(_ptr(act), _ptr(err), _ptr(w), Cw, N, H, W, C, K, R, S, stride, padding,
                                             _flags(f32_epilogue) | (L.CONV_SHIFT_HINT if shift_hint else 0), mu, L.ROUND[method],
                                             L.DIV[div_mode], L.BW[bw_mode],
                                             _ptr(sync), sync.numel(), _ptr(g8), _ptr(dw), _ptr(prepared_filter), _ptr(shift_out), _ptr(exp_a),
                                             _ptr(exp_b), _ptr(exp_out), _ptr(ws), nbytes, _stream(act))
    L.check(st, "niti_conv2d_i8_wgrad_update")
    return g8, dw, shift_out, sync


def gemm(a, b, trans_a=False, trans_b=False, absmax=None, out=None, f32_epilogue=False):
    """c[m,n] = op(a) @ op(b), int8 x int8 -> int32.  trans_a: a stored [k,m]; trans_b: b stored [n,k].
    f32_epilogue: every sum takes the int32 -> float32 -> int32 round trip of the reference's convolution epilogue."""
    _chk_dev(a, b, absmax, out)
    if a.dtype != torch.int8 or b.dtype != torch.int8:
        raise RuntimeError("gemm: int8 tensors expected")
    m, k = (a.shape[1], a.shape[0]) if trans_a else (a.shape[0], a.shape[1])
    n, k2 = (b.shape[0], b.shape[1]) if trans_b else (b.shape[1], b.shape[0])
    if k != k2:
        raise RuntimeError("gemm: inner extents differ (%d vs %d)" % (k, k2))
    c = out if out is not None else torch.empty((m, n), dtype=torch.int32, device=a.device)
    nbytes = L.lib().niti_gemm_i8_workspace(int(trans_a), int(trans_b), m, n, k)
    ws = torch.empty(nbytes, dtype=torch.int8, device=a.device) if nbytes else None
    st = L.lib().niti_gemm_i8(int(trans_a), int(trans_b), _ptr(a), _ptr(b), _ptr(c), m, n, k,
                              L.EPI_F32_ROUNDTRIP if f32_epilogue else 0, _ptr(absmax),
                              _ptr(ws), nbytes, _stream(a))
    L.check(st, "niti_gemm_i8")
    return c


def absmax_i32(x, absmax=None):
    _chk_dev(x, absmax)
    if absmax is None:
        absmax = new_scalar_u32(x.device)
    st = L.lib().niti_absmax_i32(_ptr(x), x.numel(), _ptr(absmax), _stream(x))
    L.check(st, "niti_absmax_i32")
    return absmax


def requant(x, absmax, target_bits=7, method="round", div_mode="floor", bw_mode="int", rand=None, relu=False,
            shift_out=None, exp_a=None, exp_b=None, exp_out=None):
    """int32 -> int8 (act_calc / err_calc / grad_calc).  Returns (int8 tensor, device int32 shift).
    exp_out (device int32), when given, receives shift + exp_a + exp_b."""
    _chk_dev(x, absmax, rand, shift_out, exp_a, exp_b, exp_out)
    if x.dtype != torch.int32:
        raise RuntimeError("requant: int32 input expected")
    if rand is not None and (rand.dtype != torch.int32 or rand.numel() != x.numel()):
        raise RuntimeError("requant: rand must be int32 with one entry per element")
    y = torch.empty(x.shape, dtype=torch.int8, device=x.device)
    if shift_out is None:
        shift_out = torch.empty(1, dtype=torch.int32, device=x.device)
    st = L.lib().niti_requant_i32_i8(_ptr(x), _ptr(y), x.numel(), _ptr(absmax), target_bits, L.ROUND[method],
                                     L.DIV[div_mode], L.BW[bw_mode], _ptr(rand), L.RQ_RELU if relu else 0,
                                     _ptr(shift_out), _ptr(exp_a), _ptr(exp_b), _ptr(exp_out), _stream(x))
    L.check(st, "niti_requant_i32_i8")
    return y, shift_out


def grad_update(g, w, absmax, mu, method="psto", div_mode="floor", bw_mode="int", rand=None, want_grad=False,
                shift_out=None, exp_a=None, exp_b=None, exp_out=None):
    """Fused grad_calc + weight update, in place on w.  Returns (int8 grad or None, device shift)."""
    _chk_dev(g, w, absmax, rand, shift_out, exp_a, exp_b, exp_out)
    if g.dtype != torch.int32 or w.dtype != torch.int8 or g.numel() != w.numel():
        raise RuntimeError("grad_update: int32 grad and int8 weight of equal size expected")
    g8 = torch.empty(w.shape, dtype=torch.int8, device=w.device) if want_grad else None
    if shift_out is None:
        shift_out = torch.empty(1, dtype=torch.int32, device=w.device)
    st = L.lib().niti_grad_update_i8(_ptr(g), _ptr(w), g.numel(), _ptr(absmax), mu, L.ROUND[method], L.DIV[div_mode],
                                     L.BW[bw_mode], _ptr(rand), _ptr(g8), _ptr(shift_out), _ptr(exp_a), _ptr(exp_b),
                                     _ptr(exp_out), _stream(g))
    L.check(st, "niti_grad_update_i8")
    return g8, shift_out


def weight_update(w, g):
    _chk_dev(w, g)
    st = L.lib().niti_weight_update_i8(_ptr(w), _ptr(g), w.numel(), _stream(w))
    L.check(st, "niti_weight_update_i8")
    return w


def relu_fwd(x):
    _chk_dev(x)
    y = torch.empty_like(x)
    L.check(L.lib().niti_relu_i8_fwd(_ptr(x), _ptr(y), x.numel(), _stream(x)), "niti_relu_i8_fwd")
    return y


def quantize_input(x, bits=7, cpad=16):
    """Float NCHW batch -> (int8 NHWC batch with the channels zero-padded to ``cpad``, exponent as a 1-element int32
    tensor): the reference's input quantiser and the layout change behind it in two launches."""
    _chk_dev(x)
    if x.dtype != torch.float32 or x.dim() != 4 or not x.is_contiguous():
        raise RuntimeError("quantize_input: contiguous float32 [N,C,H,W] tensor expected")
    N, C, H, W = x.shape
    cpad = max(cpad, (C + 3) // 4 * 4)
    y = torch.empty((N, H, W, cpad), dtype=torch.int8, device=x.device)
    am = torch.zeros(1, dtype=torch.int32, device=x.device)
    exp_out = torch.empty(1, dtype=torch.int32, device=x.device)
    L.check(L.lib().niti_quantize_f32_i8(_ptr(x), _ptr(y), N, C, H, W, cpad, bits, _ptr(am), _ptr(exp_out), _stream(x)),
            "niti_quantize_f32_i8")
    return y, exp_out


def mask_features(x, mask, exp_in=None, exp_add=None):
    """x [rows, F] int8 times a keep / drop byte per feature (mask [F] int8 0/1) in one launch.  With ``exp_add`` also
    returns a 1-element int32 tensor holding exp_in + exp_add."""
    _chk_dev(x, mask, exp_in)
    if x.dtype != torch.int8 or mask.dtype != torch.int8 or x.dim() != 2 or mask.numel() != x.shape[1]:
        raise RuntimeError("mask_features: int8 [rows, F] tensor and int8 [F] mask expected")
    y = torch.empty_like(x)
    exp_out = torch.empty(1, dtype=torch.int32, device=x.device) if exp_add is not None else None
    L.check(L.lib().niti_mask_features_i8(_ptr(x), _ptr(mask), _ptr(y), x.shape[0], x.shape[1], _ptr(exp_in), _ptr(exp_out),
                                         int(exp_add or 0), _stream(x)), "niti_mask_features_i8")
    return (y, exp_out) if exp_add is not None else y


def relu_bwd(act, dy):
    _chk_dev(act, dy)
    dx = torch.empty_like(dy)
    L.check(L.lib().niti_relu_i8_bwd(_ptr(act), _ptr(dy), _ptr(dx), dy.numel(), _stream(dy)), "niti_relu_i8_bwd")
    return dx


FC_PASS = {"forward": 0, "dgrad": 1, "wgrad": 2}


def fc_sync_words(which, M, O, F) -> int:
    """uint32 sync words the one-launch TiLinear kernels need for act [M,F], weight [O,F]; 0 when the shape is
    outside them (more than 16 output features, ...) and the GEMM entry point has to be used."""
    return int(L.lib().niti_fc_i8_sync_words(FC_PASS[which], M, O, F))


def _fc_sync(which, M, O, F, sync, device, who):
    words = fc_sync_words(which, M, O, F)
    if words == 0:
        raise L.NitiError("%s: shape not covered by the few-output-features kernels" % who)
    if sync is None:
        sync = sync_arena.take(words, device)
    elif sync.dtype != torch.int32 or sync.numel() < words:
        raise RuntimeError("%s: sync must be a zeroed int32 tensor of at least %d words" % (who, words))
    return sync


def fc_fwd_requant(act, w, target_bits=7, method="round", div_mode="floor", bw_mode="int", relu=False, sync=None,
                   shift_out=None, exp_a=None, exp_b=None, exp_out=None):
    """act_calc(act @ w^T) as one launch: act [M,F] int8, w [O,F] int8 (O <= 16) -> ([M,O] int8, shift, sync)."""
    _chk_dev(act, w, sync, shift_out, exp_a, exp_b, exp_out)
    if act.dtype != torch.int8 or w.dtype != torch.int8 or act.dim() != 2 or w.dim() != 2 or act.shape[1] != w.shape[1]:
        raise RuntimeError("fc_fwd_requant: int8 act [M,F] and w [O,F] expected")
    M, F = act.shape
    O = w.shape[0]
    sync = _fc_sync("forward", M, O, F, sync, act.device, "fc_fwd_requant")
    out = torch.empty((M, O), dtype=torch.int8, device=act.device)
    if shift_out is None:
        shift_out = torch.empty(1, dtype=torch.int32, device=act.device)
    st = L.lib().niti_fc_i8_fwd_requant(_ptr(act), _ptr(w), _ptr(out), M, O, F, target_bits, L.ROUND[method], L.DIV[div_mode],
                                        L.BW[bw_mode], L.RQ_RELU if relu else 0, _ptr(sync), sync.numel(), _ptr(shift_out),
                                        _ptr(exp_a), _ptr(exp_b), _ptr(exp_out), _stream(act))
    L.check(st, "niti_fc_i8_fwd_requant")
    return out, shift_out, sync


def fc_dgrad_requant(err, w, target_bits=7, method="round", div_mode="floor", bw_mode="int", sync=None, shift_out=None,
                     exp_a=None, exp_b=None, exp_out=None):
    """err_calc(err @ w) as one launch: err [M,O] int8, w [O,F] int8 (O <= 16) -> ([M,F] int8, shift, sync)."""
    _chk_dev(err, w, sync, shift_out, exp_a, exp_b, exp_out)
    if err.dtype != torch.int8 or w.dtype != torch.int8 or err.dim() != 2 or w.dim() != 2 or err.shape[1] != w.shape[0]:
        raise RuntimeError("fc_dgrad_requant: int8 err [M,O] and w [O,F] expected")
    M, O = err.shape
    F = w.shape[1]
    sync = _fc_sync("dgrad", M, O, F, sync, err.device, "fc_dgrad_requant")
    dx = torch.empty((M, F), dtype=torch.int8, device=err.device)
    if shift_out is None:
        shift_out = torch.empty(1, dtype=torch.int32, device=err.device)
    st = L.lib().niti_fc_i8_dgrad_requant(_ptr(err), _ptr(w), _ptr(dx), M, O, F, target_bits, L.ROUND[method], L.DIV[div_mode],
                                          L.BW[bw_mode], _ptr(sync), sync.numel(), _ptr(shift_out), _ptr(exp_a), _ptr(exp_b),
                                          _ptr(exp_out), _stream(err))
    L.check(st, "niti_fc_i8_dgrad_requant")
    return dx, shift_out, sync


def fc_wgrad_update(err, act, w, mu=5, method="psto", div_mode="floor", bw_mode="int", sync=None, want_grad=False,
                    shift_out=None, exp_a=None, exp_b=None, exp_out=None):
    """g = grad_calc(err^T @ act, mu); w = clip(w - g) in place, as one launch: err [M,O], act [M,F], w [O,F] int8
    (O <= 16, M <= 512) -> (g as int8 [O,F] if want_grad else None, shift, sync)."""
    _chk_dev(err, act, w, sync, shift_out, exp_a, exp_b, exp_out)
    if err.dtype != torch.int8 or act.dtype != torch.int8 or w.dtype != torch.int8 or err.dim() != 2 or act.dim() != 2 \
            or tuple(w.shape) != (err.shape[1], act.shape[1]) or err.shape[0] != act.shape[0]:
        raise RuntimeError("fc_wgrad_update: int8 err [M,O], act [M,F] and w [O,F] expected")
    M, O = err.shape
    F = act.shape[1]
    sync = _fc_sync("wgrad", M, O, F, sync, err.device, "fc_wgrad_update")
    g8 = torch.empty_like(w) if want_grad else None
    if shift_out is None:
        shift_out = torch.empty(1, dtype=torch.int32, device=err.device)
    st = L.lib().niti_fc_i8_wgrad_update(_ptr(err), _ptr(act), _ptr(w), M, O, F, mu, L.ROUND[method], L.DIV[div_mode],
                                         L.BW[bw_mode], _ptr(sync), sync.numel(), _ptr(g8), _ptr(shift_out), _ptr(exp_a),
                                         _ptr(exp_b), _ptr(exp_out), _stream(err))
    L.check(st, "niti_fc_i8_wgrad_update")
    return g8, shift_out, sync


def linear_sync_words(which, M, O, F) -> int:
    """uint32 words of the sync buffer the any-width TiLinear kernels need for a pass ("forward", "dgrad", "wgrad") on
    the current device; 0 when the shape is outside them (then: gemm + requant / grad_update)."""
    return int(L.lib().niti_linear_i8_sync_words({"forward": 0, "dgrad": 1, "wgrad": 2}[which], M, O, F))


def _linear_sync(which, M, O, F, sync, device, who):
    words = linear_sync_words(which, M, O, F)
    if words == 0:
        raise L.NitiError("%s: shape not covered by the any-width linear kernels" % who)
    if sync is None:
        sync = sync_arena.take(words, device)
    elif sync.dtype != torch.int32 or sync.numel() < words:
        raise RuntimeError("%s: sync must be a zeroed int32 tensor of at least %d words" % (who, words))
    return sync


def _chk_rand(rand, shape, who):
    if rand is not None and (rand.dtype != torch.int32 or tuple(rand.shape) != tuple(shape) or not rand.is_contiguous()):
        raise RuntimeError("%s: rand must be a contiguous int32 tensor shaped like the output" % who)


def linear_fwd_requant(act, w, target_bits=7, method="round", div_mode="floor", bw_mode="int", relu=False, rand=None, sync=None,
                       shift_out=None, exp_a=None, exp_b=None, exp_out=None):
    """act_calc(act @ w^T) in one launch for a layer of any width: act [M,F] int8, w [O,F] int8 -> ([M,O] int8, shift,
    sync).  ``rand`` (int32 [M,O]) for method "sto"."""
    _chk_dev(act, w, rand, sync, shift_out, exp_a, exp_b, exp_out)
    M, F = act.shape
    O = w.shape[0]
    _chk_rand(rand, (M, O), "linear_fwd_requant")
    sync = _linear_sync("forward", M, O, F, sync, act.device, "linear_fwd_requant")
    y = torch.empty((M, O), dtype=torch.int8, device=act.device)
    if shift_out is None:
        shift_out = torch.empty(1, dtype=torch.int32, device=act.device)
    L.check(L.lib().niti_linear_i8_fwd_requant(_ptr(act), _ptr(w), _ptr(y), M, O, F, target_bits, L.ROUND[method], L.DIV[div_mode],
                                               L.BW[bw_mode], L.RQ_RELU if relu else 0, _ptr(rand), _ptr(sync), sync.numel(),
                                               _ptr(shift_out), _ptr(exp_a), _ptr(exp_b), _ptr(exp_out), _stream(act)),
            "niti_linear_i8_fwd_requant")
    return y, shift_out, sync


def linear_dgrad_requant(err, w, target_bits=7, method="round", div_mode="floor", bw_mode="int", rand=None, sync=None,
                         shift_out=None, exp_a=None, exp_b=None, exp_out=None):
    """err_calc(err @ w) in one launch: err [M,O] int8, w [O,F] int8 -> ([M,F] int8, shift, sync)."""
    _chk_dev(err, w, rand, sync, shift_out, exp_a, exp_b, exp_out)
    M, O = err.shape
    F = w.shape[1]
    _chk_rand(rand, (M, F), "linear_dgrad_requant")
    sync = _linear_sync("dgrad", M, O, F, sync, err.device, "linear_dgrad_requant")
    y = torch.empty((M, F), dtype=torch.int8, device=err.device)
    if shift_out is None:
        shift_out = torch.empty(1, dtype=torch.int32, device=err.device)
    L.check(L.lib().niti_linear_i8_dgrad_requant(_ptr(err), _ptr(w), _ptr(y), M, O, F, target_bits, L.ROUND[method], L.DIV[div_mode],
                                                 L.BW[bw_mode], _ptr(rand), _ptr(sync), sync.numel(), _ptr(shift_out), _ptr(exp_a),
                                                 _ptr(exp_b), _ptr(exp_out), _stream(err)), "niti_linear_i8_dgrad_requant")
    return y, shift_out, sync


def linear_wgrad_update(err, act, w, mu=5, method="psto", div_mode="floor", bw_mode="int", rand=None, sync=None, want_grad=False,
                        shift_out=None, exp_a=None, exp_b=None, exp_out=None):
    """grad_calc(err^T @ act) and the weight update in one launch: err [M,O], act [M,F], w [O,F] int8 updated in place.
    Returns (int8 gradient or None, shift, sync)."""
    _chk_dev(err, act, w, rand, sync, shift_out, exp_a, exp_b, exp_out)
    M, O = err.shape
    F = act.shape[1]
    _chk_rand(rand, (O, F), "linear_wgrad_update")
    sync = _linear_sync("wgrad", M, O, F, sync, err.device, "linear_wgrad_update")
    g8 = torch.empty((O, F), dtype=torch.int8, device=w.device) if want_grad else None
    if shift_out is None:
        shift_out = torch.empty(1, dtype=torch.int32, device=w.device)
    L.check(L.lib().niti_linear_i8_wgrad_update(_ptr(err), _ptr(act), _ptr(w), M, O, F, mu, L.ROUND[method], L.DIV[div_mode],
                                                L.BW[bw_mode], _ptr(rand), _ptr(sync), sync.numel(), _ptr(g8), _ptr(shift_out),
                                                _ptr(exp_a), _ptr(exp_b), _ptr(exp_out), _stream(err)), "niti_linear_i8_wgrad_update")
    return g8, shift_out, sync


def pad_last_dim(t, multiple=16):
    """``t`` with zeros appended along its last dimension up to a multiple of ``multiple`` (``t`` itself when it
    already is one): the channel padding of conv2d_int8 (ti_torch.py:182-187) as one launch."""
    c = t.shape[-1]
    if c % multiple == 0:
        return t
    _chk_dev(t)
    if t.dtype != torch.int8:
        raise RuntimeError("pad_last_dim: int8 tensor expected")
    cp = (c + multiple - 1) // multiple * multiple
    out = torch.empty(tuple(t.shape[:-1]) + (cp,), dtype=torch.int8, device=t.device)
    L.check(L.lib().niti_pad_rows_i8(_ptr(t), _ptr(out), t.numel() // c, c, cp, _stream(t)), "niti_pad_rows_i8")
    return out


def loss_grad(out_val, out_exp, target, rand, div_mode="floor"):
    """TiLoss.forward (ti_loss.py:5-36) as one launch: int8 logits [n, classes] with exponent ``out_exp`` (1-element
    int32 device tensor), int64 targets [n], int32 random integers [n, classes] -> int8 gradient (exponent 0)."""
    _chk_dev(out_val, out_exp, target, rand)
    if out_val.dtype != torch.int8 or out_val.dim() != 2 or not out_val.is_contiguous():
        raise RuntimeError("loss_grad: contiguous int8 [n, classes] logits expected")
    if out_exp.dtype != torch.int32 or target.dtype != torch.int64 or rand.dtype != torch.int32:
        raise RuntimeError("loss_grad: int32 exponent, int64 targets and int32 random integers expected")
    n, classes = out_val.shape
    if target.numel() != n or tuple(rand.shape) != (n, classes) or not rand.is_contiguous() or not target.is_contiguous():
        raise RuntimeError("loss_grad: shape mismatch")
    grad = torch.empty_like(out_val)
    st = L.lib().niti_loss_grad_i8(_ptr(out_val), _ptr(out_exp), _ptr(target), _ptr(rand), _ptr(grad), n, classes,
                                   L.DIV[div_mode], _stream(out_val))
    L.check(st, "niti_loss_grad_i8")
    return grad


def loss_grad_rng(out_val, out_exp, target, rng, div_mode="floor"):
    """``loss_grad`` with the random integers drawn in the kernel from the generator state ``rng`` (see rng_state)."""
    _chk_dev(out_val, out_exp, target, rng)
    if out_val.dtype != torch.int8 or out_val.dim() != 2 or not out_val.is_contiguous():
        raise RuntimeError("loss_grad_rng: contiguous int8 [n, classes] logits expected")
    if out_exp.dtype != torch.int32 or target.dtype != torch.int64 or target.numel() != out_val.shape[0] or not target.is_contiguous():
        raise RuntimeError("loss_grad_rng: int32 exponent and int64 targets [n] expected")
    _check_rng(rng, "loss_grad_rng")
    n, classes = out_val.shape
    grad = torch.empty_like(out_val)
    L.check(L.lib().niti_loss_grad_i8_rng(_ptr(out_val), _ptr(out_exp), _ptr(target), _ptr(rng), _ptr(grad), n, classes,
                                          L.DIV[div_mode], _stream(out_val)), "niti_loss_grad_i8_rng")
    return grad


RNG_STREAM = {"dropout": 1, "loss": 2}
_rng_states = {}


def _check_rng(rng, who):
    if rng.dtype != torch.int32 or rng.numel() != 4 or not rng.is_contiguous() or not rng.is_cuda:
        raise RuntimeError("%s: the generator state is a contiguous int32 tensor of 4 words on the GPU" % who)


def rng_state(device=None, key=None):
    """Generator state for the kernels that draw their own random integers (dropout mask, loss gradient rounding):
    int32[4] = {key0, key1, step, 0}.  Without ``key`` returns the device's shared state, created on first use with
    a key taken from torch's default CPU generator (so ``torch.manual_seed`` fixes the sequence); with ``key`` (an
    int, 64 bits used) a fresh state at step 0.  Creating a state copies to the device: not under graph capture."""
    dev = torch.device("cuda", torch.cuda.current_device()) if device is None else torch.device(device)
    if dev.index is None:
        dev = torch.device("cuda", torch.cuda.current_device())
    if key is None:
        if str(dev) not in _rng_states:
            if torch.cuda.is_current_stream_capturing():
                raise RuntimeError("rng_state: first use under graph capture; run one step eagerly first")
            k = int(torch.empty((), dtype=torch.int64).random_().item())
            _rng_states[str(dev)] = rng_state(dev, k)
        return _rng_states[str(dev)]
    words = [key & 0xFFFFFFFF, (key >> 32) & 0xFFFFFFFF, 0, 0]
    return torch.tensor([w - (1 << 32) if w >= (1 << 31) else w for w in words], dtype=torch.int32).to(dev)


def rng_words(rng, stream, n):
    """The first ``n`` words (int32 tensor, to be read as unsigned) of stream "dropout" / "loss" that a kernel launched
    now would draw from ``rng``; the state is not advanced."""
    _check_rng(rng, "rng_words")
    out = torch.empty(n, dtype=torch.int32, device=rng.device)
    L.check(L.lib().niti_rng_words_u32(_ptr(rng), RNG_STREAM[stream] if isinstance(stream, str) else int(stream), _ptr(out), n,
                                       _stream(rng)), "niti_rng_words_u32")
    return out


def head_sync_words(which, M, O, F) -> int:
    """uint32 sync words of the classifier-head kernels ("forward" / "backward"); 0 = shape not covered."""
    return int(L.lib().niti_head_i8_sync_words(1 if which == "backward" else 0, M, O, F))


def head_forward(act, w, target_bits=7, method="round", div_mode="floor", bw_mode="int", relu=False, dropout=None,
                 drop_mask=None, rng=None, exp_bias=0, target=None, loss_rand=None, sync=None, shift_out=None, exp_a=None,
                 exp_b=None, exp_out=None):
    """Classifier forward in one launch (niti_head_i8_forward): act_calc((act * mask) @ w^T) for act [M,F], w [O,F],
    O <= 16.  ``dropout``: None, "given" (``drop_mask`` int8 [F] of 0 / 1 is read) or "draw" (the mask is drawn from
    ``rng`` and written to ``drop_mask``, allocated here when None).  With ``target`` (int64 [M]) the loss gradient
    of the logits is computed as well, rounded with ``loss_rand`` (int32 [M,O]) or with draws from ``rng``.
    Returns (out8 [M,O], drop_mask or None, loss gradient [M,O] or None, shift, sync)."""
    _chk_dev(act, w, sync, shift_out, exp_a, exp_b, exp_out, drop_mask, rng, target, loss_rand)
    if act.dtype != torch.int8 or w.dtype != torch.int8 or act.dim() != 2 or w.dim() != 2 or act.shape[1] != w.shape[1]:
        raise RuntimeError("head_forward: int8 act [M,F] and w [O,F] expected")
    if not act.is_contiguous() or not w.is_contiguous():
        raise RuntimeError("head_forward: contiguous operands expected")
    M, F = act.shape
    O = w.shape[0]
    mode = {None: 0, "given": 1, "draw": 2}[dropout]
    if mode == 2 and drop_mask is None:
        drop_mask = torch.empty(F, dtype=torch.int8, device=act.device)
    if mode != 0 and (drop_mask is None or drop_mask.dtype != torch.int8 or drop_mask.numel() != F or not drop_mask.is_contiguous()):
        raise RuntimeError("head_forward: drop_mask must be a contiguous int8 tensor of F elements")
    if rng is not None:
        _check_rng(rng, "head_forward")
    loss_grad_out = None
    if target is not None:
        if target.dtype != torch.int64 or target.numel() != M or not target.is_contiguous():
            raise RuntimeError("head_forward: int64 targets [M] expected")
        if loss_rand is not None and (loss_rand.dtype != torch.int32 or tuple(loss_rand.shape) != (M, O) or not loss_rand.is_contiguous()):
            raise RuntimeError("head_forward: loss_rand must be a contiguous int32 [M,O] tensor")
        loss_grad_out = torch.empty((M, O), dtype=torch.int8, device=act.device)
    words = head_sync_words("forward", M, O, F)
    if words == 0:
        raise L.NitiError("head_forward: shape not covered by the few-output-features kernels")
    if sync is None:
        sync = sync_arena.take(words, act.device)
    elif sync.dtype != torch.int32 or sync.numel() < words:
        raise RuntimeError("head_forward: sync must be a zeroed int32 tensor of at least %d words" % words)
    out = torch.empty((M, O), dtype=torch.int8, device=act.device)
    if shift_out is None:
        shift_out = torch.empty(1, dtype=torch.int32, device=act.device)
    st = L.lib().niti_head_i8_forward(_ptr(act), _ptr(w), _ptr(out), M, O, F, mode, _ptr(drop_mask) if mode else None, _ptr(rng),
                                      int(exp_bias), _ptr(target), _ptr(loss_rand), _ptr(loss_grad_out), target_bits,
                                      L.ROUND[method], L.DIV[div_mode], L.BW[bw_mode], L.RQ_RELU if relu else 0, _ptr(sync),
                                      sync.numel(), _ptr(shift_out), _ptr(exp_a), _ptr(exp_b), _ptr(exp_out), _stream(act))
    L.check(st, "niti_head_i8_forward")
    return out, (drop_mask if mode else None), loss_grad_out, shift_out, sync


def head_backward(err, act, w, err_bits=7, err_method="psto", grad_bits=5, grad_method="psto", div_mode="floor", bw_mode="int",
                  drop_mask=None, want_grad=False, sync=None, exp_err=None, exp_w=None, exp_act=None, exp_act_bias=0,
                  err_exp_out=None, grad_exp_out=None, unpool=None):
    """Classifier backward in one launch (niti_head_i8_backward): err [M,O], act [M,F] (in front of the dropout),
    w [O,F] (updated in place), ``drop_mask`` int8 [F] of 0 / 1 or None.  Returns (dx8 [M,F] with the mask applied,
    rounded gradient [O,F] or None, err shift, grad shift, sync).
    ``unpool`` = (pool_in [M,2P,2Q,C], ties, relu): act is the flattened output of a 2 x 2 max-pool over pool_in; the launch
    also routes dx8 through that pool's backward pass (niti_head_i8_backward_unpool) and a sixth element is returned:
    the gradient [M,2P,2Q,C]."""
    _chk_dev(err, act, w, drop_mask, sync, exp_err, exp_w, exp_act, err_exp_out, grad_exp_out)
    if (err.dtype != torch.int8 or act.dtype != torch.int8 or w.dtype != torch.int8 or err.dim() != 2 or act.dim() != 2
            or w.dim() != 2 or err.shape[0] != act.shape[0] or tuple(w.shape) != (err.shape[1], act.shape[1])):
        raise RuntimeError("head_backward: int8 err [M,O], act [M,F], w [O,F] expected")
    if not (err.is_contiguous() and act.is_contiguous() and w.is_contiguous()):
        raise RuntimeError("head_backward: contiguous operands expected")
    M, O = err.shape
    F = act.shape[1]
    if drop_mask is not None and (drop_mask.dtype != torch.int8 or drop_mask.numel() != F or not drop_mask.is_contiguous()):
        raise RuntimeError("head_backward: drop_mask must be a contiguous int8 tensor of F elements")
    words = head_sync_words("backward", M, O, F)
    if words == 0:
        raise L.NitiError("head_backward: shape not covered (M <= 256, O <= 16, F a multiple of 64)")
    if sync is None:
        sync = sync_arena.take(words, err.device)
    elif sync.dtype != torch.int32 or sync.numel() < words:
        raise RuntimeError("head_backward: sync must be a zeroed int32 tensor of at least %d words" % words)
    dx = torch.empty((M, F), dtype=torch.int8, device=err.device)
    g8 = torch.empty_like(w) if want_grad else None
    shifts = torch.empty(2, dtype=torch.int32, device=err.device)
    if unpool is not None:
        pool_in, ties, relu = unpool
        _chk_dev(pool_in)
        if pool_in.dtype != torch.int8 or pool_in.dim() != 4 or not pool_in.is_contiguous() or pool_in.shape[0] != M:
            raise RuntimeError("head_backward: unpool wants the pool's contiguous int8 input [M,2P,2Q,C]")
        H2, W2, C = pool_in.shape[1:]
        if H2 % 2 or W2 % 2 or (H2 // 2) * (W2 // 2) * C != F:
            raise RuntimeError("head_backward: the pool's input %s does not pool to %d features" % (tuple(pool_in.shape), F))
        out = torch.empty_like(pool_in)
        st = L.lib().niti_head_i8_backward_unpool(
            _ptr(err), _ptr(act), _ptr(drop_mask), _ptr(w), _ptr(dx), M, O, F, err_bits, L.ROUND[err_method], grad_bits,
            L.ROUND[grad_method], L.DIV[div_mode], L.BW[bw_mode], _ptr(sync), sync.numel(), _ptr(g8), _ptr(shifts[0:1]),
            _ptr(shifts[1:2]), _ptr(exp_err), _ptr(exp_w), _ptr(exp_act), int(exp_act_bias), _ptr(err_exp_out), _ptr(grad_exp_out),
            _ptr(pool_in), _ptr(out), H2 // 2, W2 // 2, C, L.TIES[ties] | (L.POOL_BWD_RELU if relu else 0), _stream(err))
        L.check(st, "niti_head_i8_backward_unpool")
        return dx, g8, shifts[0:1], shifts[1:2], sync, out
    st = L.lib().niti_head_i8_backward(_ptr(err), _ptr(act), _ptr(drop_mask), _ptr(w), _ptr(dx), M, O, F, err_bits,
                                       L.ROUND[err_method], grad_bits, L.ROUND[grad_method], L.DIV[div_mode], L.BW[bw_mode],
                                       _ptr(sync), sync.numel(), _ptr(g8), _ptr(shifts[0:1]), _ptr(shifts[1:2]), _ptr(exp_err),
                                       _ptr(exp_w), _ptr(exp_act), int(exp_act_bias), _ptr(err_exp_out), _ptr(grad_exp_out),
                                       _stream(err))
    L.check(st, "niti_head_i8_backward")
    return dx, g8, shifts[0:1], shifts[1:2], sync


def mfma_probe(operands, workgroups=512, iters=1200):
    """Times the library's register-resident int8 MFMA loop over the given operand bytes (int8 tensor, >= 128 bytes).
    Returns (tera-operations per second, shader clock in GHz during the loop): the matrix-unit ceiling for operands
    with these values."""
    _chk_dev(operands)
    if operands.dtype != torch.int8 or not operands.is_contiguous():
        raise RuntimeError("mfma_probe: contiguous int8 tensor expected")
    out = torch.empty(workgroups * 512, dtype=torch.int32, device=operands.device)
    clocks = torch.zeros(2, dtype=torch.int64, device=operands.device)
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)

    def launch():
        L.check(L.lib().niti_mfma_probe_i8(_ptr(operands), operands.numel(), workgroups, iters, _ptr(out), _ptr(clocks),
                                           _stream(operands)), "niti_mfma_probe_i8")
    for _ in range(3):
        launch()
    e0.record()
    launch()
    e1.record()
    torch.cuda.synchronize()
    ms = e0.elapsed_time(e1)
    c = clocks.tolist()
    tops = workgroups * 8 * iters * 12 * 65536.0 / (ms * 1e-3) / 1e12
    return tops, (c[0] / (c[1] * 10.0) if c[1] else 0.0)


def maxpool_fwd(x, kernel_size=2, stride=2, padding=0):
    _chk_dev(x)
    if x.dtype != torch.int8:
        raise RuntimeError("maxpool_fwd: int8 tensor expected")
    N, H, W, C = x.shape
    P = (H + 2 * padding - kernel_size) // stride + 1
    Q = (W + 2 * padding - kernel_size) // stride + 1
    y = torch.empty((N, max(P, 0), max(Q, 0), C), dtype=torch.int8, device=x.device)
    st = L.lib().niti_maxpool_i8_fwd(_ptr(x), _ptr(y), N, H, W, C, kernel_size, stride, padding, _stream(x))
    L.check(st, "niti_maxpool_i8_fwd")
    return y


def maxpool_bwd(y, dy, x, kernel_size=2, stride=2, padding=0, ties="first", relu=False):
    """``relu``: also zero the gradient where x <= 0 (the backward pass of a ReLU whose output x is)."""
    _chk_dev(y, dy, x)
    N, H, W, C = x.shape
    dx = torch.empty_like(x)
    st = L.lib().niti_maxpool_i8_bwd(_ptr(y), _ptr(dy), _ptr(x), _ptr(dx), N, H, W, C, kernel_size, stride, padding,
                                     L.TIES[ties] | (L.POOL_BWD_RELU if relu else 0), _stream(x))
    L.check(st, "niti_maxpool_i8_bwd")
    return dx


def group_conv_f32(x, w, stride, padding, dilation, groups):
    _chk_dev(x, w)
    N, H, W, C = x.shape
    K, R, S, Cg = w.shape
    P = (H + 2 * padding - dilation * (R - 1) - 1) // stride + 1
    Q = (W + 2 * padding - dilation * (S - 1) - 1) // stride + 1
    y = torch.empty((N, max(P, 0), max(Q, 0), K), dtype=torch.float32, device=x.device)
    st = L.lib().niti_group_conv_i8_f32(_ptr(x), _ptr(w), _ptr(y), N, H, W, C, K, R, S, Cg, stride, padding, dilation,
                                        groups, _stream(x))
    L.check(st, "niti_group_conv_i8_f32")
    return y
