"""Pins the oracle's convolution / GEMM / pooling statements: library routines, brute force,
the operand rewrites the reference itself relies on (ti_torch.py:404-405, 430-432), adjoint
identities and hand-checkable special cases."""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import c_oracle as co
from oracle import niti_oracle as po


def ri8(g, *shape, lo=-127, hi=127):
    return torch.randint(lo, hi + 1, shape, generator=g, dtype=torch.int8)


CASES = [  # N,H,W,C,K,R,S,stride,pad
    (2, 5, 5, 4, 3, 3, 3, 1, 1),
    (1, 6, 7, 16, 8, 3, 3, 1, 1),
    (2, 8, 8, 3, 5, 3, 3, 1, 1),
    (2, 7, 9, 8, 4, 3, 3, 2, 1),
    (1, 8, 8, 4, 6, 5, 5, 1, 2),
    (3, 4, 4, 2, 2, 1, 1, 1, 0),
    (2, 6, 6, 4, 3, 3, 3, 1, 0),
]


@pytest.mark.parametrize("case", CASES)
def test_fprop_three_ways(case):
    N, H, W, C, K, R, S, st, pad = case
    g = torch.Generator().manual_seed(11)
    x, w = ri8(g, N, H, W, C), ri8(g, K, R, S, C)
    brute = po.conv2d_fprop_loops(x, w, st, pad)
    lib = po.conv2d_fprop_i32(x, w, st, pad)
    f64 = F.conv2d(x.permute(0, 3, 1, 2).double(), w.permute(0, 3, 1, 2).double(), stride=st, padding=pad)
    cc = co.conv_fprop(x, w, st, pad)
    assert torch.equal(lib.to(torch.int64), brute)
    assert torch.equal(cc.to(torch.int64), brute)
    assert torch.equal(f64.permute(0, 2, 3, 1).to(torch.int64), brute)


def test_fprop_special_cases():
    g = torch.Generator().manual_seed(12)
    x = ri8(g, 2, 6, 6, 4)
    # centre-tap delta filter copies channel c to output k=c
    w = torch.zeros(4, 3, 3, 4, dtype=torch.int8)
    for c in range(4):
        w[c, 1, 1, c] = 1
    assert torch.equal(po.conv2d_fprop_i32(x, w), x.to(torch.int32))
    assert torch.equal(co.conv_fprop(x, w), x.to(torch.int32))
    # off-centre delta (r=0,s=2) shifts: y[p,q] = x[p-1,q+1]
    w = torch.zeros(1, 3, 3, 4, dtype=torch.int8)
    w[0, 0, 2, 1] = 1
    y = co.conv_fprop(x, w)
    ref = torch.zeros(2, 6, 6, 1, dtype=torch.int32)
    ref[:, 1:, :5, 0] = x[:, :5, 1:, 1].to(torch.int32)
    assert torch.equal(y, ref) and torch.equal(po.conv2d_fprop_i32(x, w), ref)
    # all-ones: window population * C  (corner 4C, edge 6C, interior 9C)
    ones = torch.ones(1, 5, 5, 6, dtype=torch.int8)
    y = co.conv_fprop(ones, torch.ones(2, 3, 3, 6, dtype=torch.int8))
    assert y[0, 0, 0, 0] == 24 and y[0, 0, 2, 1] == 36 and y[0, 2, 2, 0] == 54
    # channel zero-padding (ti_torch.py:180-183) is a no-op; linearity in x
    w = ri8(g, 3, 3, 3, 4)
    assert torch.equal(po.conv2d_int8(x, w), po.conv2d_fprop_i32(x, w))
    xa, xb = ri8(g, 2, 6, 6, 4, lo=-60, hi=60), ri8(g, 2, 6, 6, 4, lo=-60, hi=60)
    assert torch.equal(po.conv2d_fprop_i32(xa + xb, w), po.conv2d_fprop_i32(xa, w) + po.conv2d_fprop_i32(xb, w))


@pytest.mark.parametrize("case", [c for c in CASES])
def test_dgrad_wgrad_definitions(case):
    N, H, W, C, K, R, S, st, pad = case
    g = torch.Generator().manual_seed(13)
    x, w = ri8(g, N, H, W, C), ri8(g, K, R, S, C)
    P, Q = (H + 2 * pad - R) // st + 1, (W + 2 * pad - S) // st + 1
    e = ri8(g, N, P, Q, K)
    dx_def = po.conv2d_dgrad_def(e, w, H, W, st, pad)
    dw_def = po.conv2d_wgrad_def(x, e, R, S, st, pad)
    assert torch.equal(co.conv_dgrad(e, w, H, W, st, pad).to(torch.int64), dx_def)
    assert torch.equal(co.conv_wgrad(x, e, R, S, st, pad).to(torch.int64), dw_def)
    # adjoint identities, exact in int64: <fprop(x,w),e> == <x,dgrad(e,w)> == <w,wgrad(x,e)>
    y = po.conv2d_fprop_i32(x, w, st, pad).to(torch.int64)
    lhs = int((y * e.to(torch.int64)).sum())
    assert lhs == int((x.to(torch.int64) * dx_def).sum())
    assert lhs == int((w.to(torch.int64) * dw_def).sum())
    if st == 1 and 2 * pad == R - 1:
        # the reference's operand rewrites give the same tensors
        assert torch.equal(po.conv2d_dgrad_i32(e, w, st, pad).to(torch.int64), dx_def)
        assert torch.equal(po.conv2d_wgrad_i32(x, e, st, pad).to(torch.int64), dw_def)
        assert torch.equal(po.conv2d_weight_int8(x, w.shape, e, st, pad).to(torch.int64), dw_def)


def test_gemm():
    g = torch.Generator().manual_seed(14)
    for m, k, n in [(5, 7, 3), (16, 64, 32), (33, 100, 10), (128, 256, 12)]:
        a, b = ri8(g, m, k), ri8(g, k, n)
        ref = torch.from_numpy(a.numpy().astype(np.int64) @ b.numpy().astype(np.int64))
        assert torch.equal(po.int8mm(a, b).to(torch.int64), ref)
        assert torch.equal(co.gemm(a, b).to(torch.int64), ref)
    a, b = ri8(g, 32, 64), ri8(g, 64, 16)
    assert torch.equal(torch._int_mm(a, b), po.int8mm(a, b))


POOL = [(2, 8, 8, 16, 2, 2, 0), (1, 6, 6, 5, 2, 2, 0), (2, 7, 7, 4, 3, 2, 1), (1, 5, 5, 3, 2, 1, 0), (1, 9, 9, 2, 3, 3, 0)]


@pytest.mark.parametrize("case", POOL)
def test_maxpool(case):
    N, H, W, C, ks, st, pad = case
    g = torch.Generator().manual_seed(15)
    for lo, hi in ((-127, 127), (-3, 3), (0, 1)):          # the narrow ranges force ties
        x = ri8(g, N, H, W, C, lo=lo, hi=hi)
        y = po.maxpool_fwd(x, ks, st, pad)
        assert torch.equal(y, co.maxpool_fwd(x, ks, st, pad))
        dy = ri8(g, *y.shape, lo=-20, hi=20)
        # torch CPU autograd routes to the first maximum in scan order
        xf = x.permute(0, 3, 1, 2).double().requires_grad_(True)
        F.max_pool2d(xf, ks, st, pad).backward(dy.permute(0, 3, 1, 2).double())
        ref = xf.grad.permute(0, 2, 3, 1).to(torch.int32)
        assert torch.equal(po.maxpool_bwd(y, dy, x, ks, st, pad, "first").to(torch.int32), ref.to(torch.int8).to(torch.int32))
        assert torch.equal(co.maxpool_bwd(y, dy, x, ks, st, pad, "first"), po.maxpool_bwd(y, dy, x, ks, st, pad, "first"))
        assert torch.equal(co.maxpool_bwd(y, dy, x, ks, st, pad, "all"), po.maxpool_bwd(y, dy, x, ks, st, pad, "all"))
    # no ties inside any (n, c) plane: both rules coincide; without window overlap dx sums to dy
    planes = torch.stack([torch.randperm(H * W, generator=g) for _ in range(N * C)]).reshape(N, C, H, W)
    x = (planes - 60).permute(0, 2, 3, 1).contiguous().to(torch.int8)
    y = po.maxpool_fwd(x, ks, st, pad)
    dy = ri8(g, *y.shape, lo=-20, hi=20)
    a, b = po.maxpool_bwd(y, dy, x, ks, st, pad, "first"), po.maxpool_bwd(y, dy, x, ks, st, pad, "all")
    assert torch.equal(a, b)
    if st >= ks:
        assert int(a.to(torch.int64).sum()) == int(dy.to(torch.int64).sum())
        assert int((a != 0).sum()) <= dy.numel()


def test_ti_loss_shapes_and_sign():
    g = torch.Generator().manual_seed(16)
    out = ri8(g, 16, 10)
    tgt = torch.randint(0, 10, (16,), generator=g)
    for e in (-9, -7, -3, 0, 1):
        pre = po.ti_loss_pre_round(out, e, tgt)
        assert pre.shape == (16, 10) and pre.dtype == torch.int32
        # softmax-minus-onehot: the target column is <= 0, every other column >= 0
        rows = torch.arange(16)
        assert bool((pre[rows, tgt] <= 0).all())
        mask = torch.ones_like(pre, dtype=torch.bool)
        mask[rows, tgt] = False
        assert bool((pre[mask] >= 0).all())
        u = torch.randint(0, 16, pre.shape, generator=g, dtype=torch.int32)
        err, ee = po.ti_loss(out, e, tgt, u)
        assert err.dtype == torch.int8 and ee == 0
