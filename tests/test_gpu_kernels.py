"""GPU parity of every C-ABI entry point against the CPU oracle on seeded inputs (bit-exact)."""
import sys

import pytest
import torch

pytestmark = pytest.mark.gpu


def _say(*a):
    print("[case]", *a, flush=True)
    sys.stdout.flush()


@pytest.fixture(scope="module")
def dev():
    assert torch.cuda.is_available(), "GPU tests need a GPU"
    return torch.device("cuda:0")


def ri8(g, *shape, lo=-127, hi=127):
    return torch.randint(lo, hi + 1, shape, generator=g, dtype=torch.int8)


CONV_CASES = [  # N,H,W,C,K,R,S,stride,pad
    (1, 4, 4, 16, 16, 3, 3, 1, 1),
    (2, 8, 8, 16, 32, 3, 3, 1, 1),
    (3, 7, 9, 32, 40, 3, 3, 1, 1),       # ragged M and K
    (2, 8, 8, 64, 128, 3, 3, 1, 1),
    (2, 9, 9, 48, 130, 3, 3, 2, 1),      # stride 2, K not a multiple of 4... of 128
    (2, 8, 8, 16, 10, 5, 5, 1, 2),       # K = 10: scalar store tail
    (4, 16, 16, 128, 128, 3, 3, 1, 1),
    (1, 6, 6, 80, 24, 1, 1, 1, 0),
    (2, 6, 6, 16, 8, 3, 3, 1, 0),        # no padding
    (8, 32, 32, 128, 128, 3, 3, 1, 1),
    (2, 40, 40, 16, 16, 36, 36, 1, 1),   # filter wider than 32 (the reference's sp_conv case)
    (8, 8, 8, 64, 128, 3, 3, 1, 1),      # 3x3 kernel with LDS-resident halo: whole small images per workgroup
    (4, 8, 8, 80, 24, 3, 3, 1, 1),       # ... ragged channel slice and channel tile
    (1, 16, 16, 16, 40, 3, 3, 1, 1),
    (2, 32, 32, 16, 64, 3, 3, 1, 1),
    (3, 16, 16, 192, 260, 3, 3, 1, 1),   # three channel slices, three channel tiles
    (12, 8, 8, 512, 128, 3, 3, 1, 1),
]


@pytest.mark.parametrize("case", CONV_CASES)
def test_conv_fprop(dev, case):
    from niti_amd import ops
    from oracle import niti_oracle as po
    N, H, W, C, K, R, S, st, pad = case
    _say("conv_fprop", case)
    g = torch.Generator().manual_seed(100 + N + C + K)
    x, w = ri8(g, N, H, W, C), ri8(g, K, R, S, C)
    ref = po.conv2d_fprop_i32(x, w, st, pad)
    am = ops.new_scalar_u32(dev)
    y = ops.conv2d_fprop(x.to(dev), w.to(dev), st, pad, absmax=am)
    torch.cuda.synchronize()
    assert torch.equal(y.cpu(), ref)
    assert int(am.cpu()) == po.absmax(ref)
    y2 = ops.conv2d_fprop(x.to(dev), w.to(dev), st, pad, f32_epilogue=True)
    assert torch.equal(y2.cpu(), po.f32_roundtrip(ref))


def test_conv_fprop_f32_epilogue_rounds_large_sums(dev):
    from niti_amd import ops
    from oracle import niti_oracle as po
    _say("conv_fprop f32 epilogue, |acc| > 2^24")
    # all +-127 operands and a long reduction: |acc| reaches 127*127*9*256 = 37.2M > 2^24
    x = torch.full((1, 6, 6, 256), 127, dtype=torch.int8)
    x[0, 2, 2, 0] = 126                      # odd sums so the round trip is visible
    w = torch.full((16, 3, 3, 256), 127, dtype=torch.int8)
    w[1] = -127
    w[2, 0, 0, 5] = 1
    ref = po.conv2d_fprop_i32(x, w)
    assert int(ref.abs().max()) > 2 ** 24
    rt = po.f32_roundtrip(ref)
    assert not torch.equal(rt, ref)
    y = ops.conv2d_fprop(x.to(dev), w.to(dev), 1, 1, f32_epilogue=True)
    assert torch.equal(y.cpu(), rt)
    y = ops.conv2d_fprop(x.to(dev), w.to(dev), 1, 1, f32_epilogue=False)
    assert torch.equal(y.cpu(), ref)


DGRAD_CASES = [(4, 8, 8, 96, 48, 3, 1), (1, 32, 32, 32, 16, 3, 1), (2, 16, 16, 256, 128, 3, 1), (2, 8, 8, 16, 16, 3, 1), (2, 8, 8, 32, 48, 3, 1), (3, 7, 9, 40, 32, 3, 1), (2, 16, 16, 128, 128, 3, 1),
               (2, 8, 8, 16, 32, 5, 2), (2, 8, 8, 24, 16, 3, 0), (2, 6, 6, 3, 16, 3, 1)]


@pytest.mark.parametrize("case", DGRAD_CASES)
def test_conv_dgrad(dev, case):
    from niti_amd import ops
    from oracle import c_oracle as co
    from oracle import niti_oracle as po
    N, H, W, C, K, R, pad = case
    _say("conv_dgrad", case)
    g = torch.Generator().manual_seed(200 + C + K)
    P, Q = H + 2 * pad - R + 1, W + 2 * pad - R + 1
    e, w = ri8(g, N, P, Q, K), ri8(g, K, R, R, C)
    ref = co.conv_dgrad(e, w, H, W, 1, pad)
    if 2 * pad == R - 1:
        assert torch.equal(ref, po.conv2d_dgrad_i32(e, w, 1, pad, f32_epilogue=False))
    am = ops.new_scalar_u32(dev)
    dx = ops.conv2d_dgrad(e.to(dev), w.to(dev), 1, pad, absmax=am)
    assert torch.equal(dx.cpu(), ref)
    assert int(am.cpu()) == po.absmax(ref)


# convolution + requantisation in one launch: N,Q,C,K (3x3, stride 1, pad 1), small sums / large sums / ragged tiles
FUSED_CASES = [(4, 8, 16, 16), (4, 8, 64, 128), (8, 8, 80, 144), (1, 16, 16, 48), (3, 16, 192, 272), (2, 32, 16, 64),
               (8, 32, 128, 128), (12, 8, 512, 128), (16, 4, 64, 128), (48, 4, 256, 80), (64, 2, 512, 512), (128, 2, 32, 48),
               (5, 2, 48, 16), (33, 2, 16, 80), (256, 2, 160, 96), (1, 2, 96, 32),
               # more than 512 tiles of 256 pixels x 64 channels: workgroups of 512 pixels
               (256, 32, 16, 64), (1024, 16, 32, 48), (144, 32, 48, 64),
               # more workgroups than the device holds at once: two launches, the second one settling the shift
               (264, 16, 16, 272), (600, 32, 16, 48)]


@pytest.fixture(params=["auto", "32", "64", "128"])
def halo_tile(request):
    """Channel tile of the 3x3 halo kernel: the library's own choice, or pinned to either width."""
    import os
    old = os.environ.get("NITI_HALO_KT")
    if request.param != "auto":
        os.environ["NITI_HALO_KT"] = request.param
    yield request.param
    if old is None:
        os.environ.pop("NITI_HALO_KT", None)
    else:
        os.environ["NITI_HALO_KT"] = old


@pytest.mark.parametrize("case", [(8, 8, 64, 128), (4, 8, 80, 24), (3, 16, 192, 260), (2, 32, 16, 64), (8, 32, 128, 256), (12, 8, 512, 128),
                                  (32, 4, 128, 256), (16, 4, 48, 16), (64, 2, 256, 128), (192, 2, 64, 32),
                                  (7, 2, 48, 20), (40, 2, 16, 132), (1, 2, 32, 4)])
def test_conv_halo_tiles(dev, case, halo_tile):
    """Forward, data gradient and the requantising variant with both channel tiles of the halo kernel."""
    from niti_amd import ops
    from oracle import c_oracle as co
    from oracle import niti_oracle as po
    N, Q, C, K = case
    _say("conv_halo_tiles", case, halo_tile)
    g = torch.Generator().manual_seed(990 + C + K)
    x, w = ri8(g, N, Q, Q, C), ri8(g, K, 3, 3, C)
    ref = po.conv2d_fprop_i32(x, w, 1, 1)
    am = ops.new_scalar_u32(dev)
    y = ops.conv2d_fprop(x.to(dev), w.to(dev), 1, 1, absmax=am)
    assert torch.equal(y.cpu(), ref) and int(am.cpu()) == po.absmax(ref)
    if K % 16 == 0:
        r8, sh_ref = po.act_calc(ref, 0)
        y8, sh, sync = ops.conv2d_fprop_requant(x.to(dev), w.to(dev))
        assert int(sync.cpu()[1]) == 0 and int(sync.cpu()[0]) == po.absmax(ref)
        assert torch.equal(y8.cpu(), r8) and int(sh.cpu()) == sh_ref
        e = ri8(g, N, Q, Q, K)
        dref = co.conv_dgrad(e, w, Q, Q, 1, 1)
        d8, dsh = po.err_calc(dref)
        dx = ops.conv2d_dgrad(e.to(dev), w.to(dev), 1, 1)
        assert torch.equal(dx.cpu(), dref)
        dx8, sh, sync = ops.conv2d_dgrad_requant(e.to(dev), w.to(dev))
        assert int(sync.cpu()[1]) == 0 and torch.equal(dx8.cpu(), d8) and int(sh.cpu()) == dsh
        # the data gradient reading the copy of the filter that the forward pass uses
        wf = ops.conv_filter_prepare(w.to(dev), N, Q, Q)
        dx = ops.conv2d_dgrad(e.to(dev), w.to(dev), 1, 1, forward_filter=wf)
        assert torch.equal(dx.cpu(), dref)
        dx8, sh, sync = ops.conv2d_dgrad_requant(e.to(dev), w.to(dev), forward_filter=wf)
        assert int(sync.cpu()[1]) == 0 and torch.equal(dx8.cpu(), d8) and int(sh.cpu()) == dsh
        # ... and zeroing the gradient where the layer's input was not positive
        mask = ri8(g, N, Q, Q, C)
        dx8, sh, sync = ops.conv2d_dgrad_requant(e.to(dev), w.to(dev), forward_filter=wf, relu_mask=mask.to(dev))
        assert int(sync.cpu()[1]) == 0 and int(sh.cpu()) == dsh
        assert torch.equal(dx8.cpu(), torch.where(mask > 0, d8, torch.zeros_like(d8)))


@pytest.mark.parametrize("div_mode", ["floor", "trunc"])
@pytest.mark.parametrize("method", ["round", "psto"])
@pytest.mark.parametrize("case", FUSED_CASES)
def test_conv_fprop_requant(dev, case, method, div_mode):
    from niti_amd import ops
    from oracle import niti_oracle as po
    N, Q, C, K = case
    _say("conv_fprop_requant", case, method, div_mode)
    g = torch.Generator().manual_seed(900 + N + C + K)
    x, w = ri8(g, N, Q, Q, C), ri8(g, K, 3, 3, C)
    acc = po.conv2d_fprop_i32(x, w, 1, 1)
    words = ops.conv_requant_sync_words(N, Q, Q, C, K)
    assert words >= 16 + (N * Q * Q // 256) * ((K + 127) // 128)
    for tgt, relu in ((7, False), (7, True), (4, False)):
        ref, sh_ref = po.act_calc(acc, 0, method, div_mode) if tgt == 7 else po.grad_calc(acc, tgt, method, div_mode)
        ea = torch.tensor([3], dtype=torch.int32, device=dev)
        eb = torch.tensor([-11], dtype=torch.int32, device=dev)
        eo = torch.zeros(1, dtype=torch.int32, device=dev)
        y, sh, sync = ops.conv2d_fprop_requant(x.to(dev), w.to(dev), 1, 1, target_bits=tgt, method=method, div_mode=div_mode,
                                               relu=relu, exp_a=ea, exp_b=eb, exp_out=eo)
        torch.cuda.synchronize()
        sync = sync.cpu()
        assert int(sync[1]) == 0, "grid-wide wait timed out"
        assert int(sync[0]) == po.absmax(acc)
        assert int(sh.cpu()) == sh_ref and int(eo.cpu()) == sh_ref + 3 - 11
        assert torch.equal(y.cpu(), ref.clamp(min=0) if relu else ref)
        if Q >= 2:
            # the same launch also writing the 2x2 / stride-2 maximum of its output
            pooled = torch.full((N, Q // 2, Q // 2, K), 77, dtype=torch.int8, device=dev)
            y2, sh2, sync2 = ops.conv2d_fprop_requant(x.to(dev), w.to(dev), 1, 1, target_bits=tgt, method=method, div_mode=div_mode,
                                                      relu=relu, pool_out=pooled)
            assert int(sync2.cpu()[1]) == 0 and torch.equal(y2, y) and int(sh2.cpu()) == sh_ref
            assert torch.equal(pooled.cpu(), po.maxpool_fwd(y.cpu()))


STO_CASES = [(4, 8, 16, 16), (8, 8, 80, 144), (3, 16, 192, 272), (2, 32, 16, 64), (8, 32, 128, 128), (16, 4, 64, 128),
             (256, 32, 16, 64),      # workgroups of 512 pixels
             (264, 16, 16, 272)]     # two launches, the second one settling the shift


@pytest.mark.parametrize("div_mode", ["floor", "trunc"])
@pytest.mark.parametrize("case", STO_CASES)
def test_conv_requant_sto(dev, case, div_mode):
    """StoShift (ti_torch.py:33-46) inside the single-launch convolutions: same random integers, same bytes as the
    oracle's act_calc / err_calc / grad_calc with method 'sto'; wide random integers count by their low `shift` bits;
    a wrong prediction (second store pass with another shift) changes nothing."""
    from niti_amd import ops
    from oracle import niti_oracle as po
    N, Q, C, K = case
    _say("conv_requant_sto", case, div_mode)
    g = torch.Generator().manual_seed(990 + N + C + K)
    x, w = ri8(g, N, Q, Q, C), ri8(g, K, 3, 3, C)
    acc = po.conv2d_fprop_i32(x, w, 1, 1)
    for tgt, relu in ((7, False), (7, True), (4, False)):
        s = max(po.RangeEstimate(acc) - tgt, 1)
        u = torch.randint(0, 2 ** s, acc.shape, generator=g, dtype=torch.int32)
        ref, sh_ref = po.act_calc(acc, 0, "sto", div_mode, u) if tgt == 7 else po.grad_calc(acc, tgt, "sto", div_mode, u)
        wide = u + (torch.randint(0, 2 ** (30 - s), acc.shape, generator=g, dtype=torch.int32) << s)
        for rand, hint in ((u, None), (wide, 0), (wide, sh_ref + 2), (u, max(sh_ref - 1, 0))):
            kw = {}
            if hint is not None:
                kw = dict(shift_out=torch.tensor([hint], dtype=torch.int32, device=dev), shift_hint=True)
            y, sh, sync = ops.conv2d_fprop_requant(x.to(dev), w.to(dev), 1, 1, target_bits=tgt, method="sto", div_mode=div_mode,
                                                   relu=relu, rand=rand.to(dev), **kw)
            sync = sync.cpu()
            assert int(sync[1]) == 0 and int(sync[0]) == po.absmax(acc) and int(sh.cpu()) == sh_ref
            assert torch.equal(y.cpu(), ref.clamp(min=0) if relu else ref), (tgt, relu, hint)
    # with the pooled output next to it
    pooled = torch.empty((N, Q // 2, Q // 2, K), dtype=torch.int8, device=dev)
    y2, _, _ = ops.conv2d_fprop_requant(x.to(dev), w.to(dev), 1, 1, target_bits=4, method="sto", div_mode=div_mode, rand=u.to(dev),
                                        pool_out=pooled)
    assert torch.equal(y2.cpu(), ref) and torch.equal(pooled.cpu(), po.maxpool_fwd(ref))
    # data gradient (the error map has K channels, the result C), with the ReLU mask of the layer below
    e = ri8(g, N, Q, Q, K)
    dacc = po.conv2d_dgrad_i32(e, w, 1, 1, f32_epilogue=False)
    s = max(po.RangeEstimate(dacc) - 7, 1)
    u = torch.randint(0, 2 ** s, dacc.shape, generator=g, dtype=torch.int32)
    dref, dsh = po.err_calc(dacc, "sto", div_mode, u)
    mask = ri8(g, N, Q, Q, C)
    fwd_copy = ops.conv_filter_prepare(w.to(dev), N, Q, Q)
    for kw in (dict(), dict(forward_filter=fwd_copy), dict(relu_mask=mask.to(dev))):
        d8, sh, sync = ops.conv2d_dgrad_requant(e.to(dev), w.to(dev), 1, 1, method="sto", div_mode=div_mode, rand=u.to(dev), **kw)
        assert int(sync.cpu()[1]) == 0 and int(sh.cpu()) == dsh
        assert torch.equal(d8.cpu(), torch.where(mask > 0, dref, torch.zeros_like(dref)) if "relu_mask" in kw else dref)


def test_conv_requant_sto_refusals(dev):
    from niti_amd import ops
    from niti_amd._lib import NitiError
    g = torch.Generator().manual_seed(991)
    x, w = ri8(g, 32, 2, 2, 32).to(dev), ri8(g, 32, 3, 3, 32).to(dev)
    u = torch.zeros((32, 2, 2, 32), dtype=torch.int32, device=dev)
    with pytest.raises(NitiError):       # 2 x 2 maps keep the two-pass path for StoShift
        ops.conv2d_fprop_requant(x, w, method="sto", rand=u)
    with pytest.raises(RuntimeError):    # no random integers
        ops.conv2d_fprop_requant(x, w, method="sto")
    with pytest.raises(RuntimeError):    # random integers of the wrong shape
        ops.conv2d_fprop_requant(x, w, method="sto", rand=u[:1])


def test_conv_fprop_requant_wraps_when_no_shift(dev):
    """Sums that already fit 7 bits (+ the 128 -> -128 wrap of the reference's int32 -> int8 cast)."""
    from niti_amd import ops
    from oracle import niti_oracle as po
    _say("conv_fprop_requant no shift")
    x = torch.zeros((4, 8, 8, 16), dtype=torch.int8)
    w = torch.zeros((16, 3, 3, 16), dtype=torch.int8)
    x[0, 3, 3, 0] = 64
    w[2, 1, 1, 0] = 2          # one sum of exactly 128: bit width 7, shift 0, low byte wraps to -128
    x[1, 2, 2, 1] = -5
    w[3, 1, 1, 1] = 7
    acc = po.conv2d_fprop_i32(x, w, 1, 1)
    ref, sh_ref = po.act_calc(acc, 0)
    assert sh_ref == 0 and int(ref.min()) == -128
    y, sh, sync = ops.conv2d_fprop_requant(x.to(dev), w.to(dev))
    assert torch.equal(y.cpu(), ref) and int(sh.cpu()) == 0 and int(sync.cpu()[1]) == 0


def test_conv_fprop_requant_f32_epilogue(dev):
    from niti_amd import ops
    from oracle import niti_oracle as po
    _say("conv_fprop_requant f32 epilogue, |acc| > 2^24")
    x = torch.full((4, 8, 8, 256), 127, dtype=torch.int8)
    x[0, 2, 2, 0] = 126
    w = torch.full((16, 3, 3, 256), 127, dtype=torch.int8)
    w[1] = -127
    w[2, 0, 0, 5] = 1
    acc = po.conv2d_fprop_i32(x, w)
    assert int(acc.abs().max()) > 2 ** 24
    for f32 in (True, False):
        a = po.f32_roundtrip(acc) if f32 else acc
        ref, sh_ref = po.act_calc(a, 0)
        y, sh, sync = ops.conv2d_fprop_requant(x.to(dev), w.to(dev), f32_epilogue=f32)
        assert torch.equal(y.cpu(), ref) and int(sh.cpu()) == sh_ref and int(sync.cpu()[0]) == po.absmax(a)


VGG_LAYERS = [(3, 128, 32), (128, 128, 32), (128, 256, 16), (256, 256, 16), (256, 512, 8), (512, 512, 8)]


@pytest.mark.parametrize("layer", VGG_LAYERS)
def test_conv_triple_at_benchmark_size(dev, layer):
    """The six layer shapes of the benchmark at batch 128, where the CPU oracle would take minutes: checked through
    what does not depend on size - the oracle on a few images of the batch (convolutions are per sample), the
    adjoint identities <fprop(x,w),e> = <x,dgrad(e,w)> = <w,wgrad(x,e)> in 64-bit integers, additivity of the
    weight gradient over the batch, and the single-launch forms against convolution + requantisation as two
    launches (that chain is checked against the oracle at small sizes)."""
    import torch.nn.functional as F
    from niti_amd import ops
    from oracle import c_oracle as co
    from oracle import niti_oracle as po
    C, K, Q = layer
    N = 128
    _say("conv_triple_at_benchmark_size", layer)
    g = torch.Generator().manual_seed(7000 + C + K + Q)
    x, w = ri8(g, N, Q, Q, C), ri8(g, K, 3, 3, C)
    e = torch.clamp(torch.round(torch.distributions.Laplace(0.0, 16.0).sample((N, Q, Q, K))), -127, 127).to(torch.int8)
    x16 = (F.pad(x, (0, 16 - C % 16)) if C % 16 else x).contiguous()
    w16 = (F.pad(w, (0, 16 - C % 16)) if C % 16 else w).contiguous()
    xd, wd, ed, x16d, w16d = x.to(dev), w.to(dev), e.to(dev), x16.to(dev), w16.to(dev)
    sub = [0, 77, 127]
    # forward
    am = ops.new_scalar_u32(dev)
    y = ops.conv2d_fprop(x16d, w16d, 1, 1, absmax=am)
    assert torch.equal(y[sub].cpu(), co.conv_fprop(x[sub].contiguous(), w, 1, 1))
    assert int(am.cpu()) == int(y.abs().max())
    y8, sh, sync = ops.conv2d_fprop_requant(x16d, w16d)
    r8, rsh = ops.requant(y, am, 7, "round")
    assert int(sync.cpu()[1]) == 0 and int(sync.cpu()[0]) == int(am.cpu())
    assert torch.equal(y8, r8) and int(sh.cpu()) == int(rsh.cpu())
    lhs = int((y.to(torch.int64) * ed.to(torch.int64)).sum())
    # weight gradient
    amw = ops.new_scalar_u32(dev)
    dw = ops.conv2d_wgrad(x16d, ed, 3, 3, 1, 1, absmax=amw)[..., :C]
    assert int((dw.to(torch.int64) * wd.to(torch.int64)).sum()) == lhs
    half = ops.conv2d_wgrad(x16d[:64].contiguous(), ed[:64].contiguous(), 3, 3, 1, 1)[..., :C] + \
        ops.conv2d_wgrad(x16d[64:].contiguous(), ed[64:].contiguous(), 3, 3, 1, 1)[..., :C]
    assert torch.equal(dw, half)
    one = ops.conv2d_wgrad(x16d[5:7].contiguous(), ed[5:7].contiguous(), 3, 3, 1, 1)[..., :C]
    assert torch.equal(one.cpu(), co.conv_wgrad(x[5:7].contiguous(), e[5:7].contiguous(), 3, 3, 1, 1))
    if C % 16 == 0:
        wnew, wtwo = wd.clone(), wd.clone()
        g8, _, sh, sync = ops.conv2d_wgrad_update(x16d, ed, wnew, mu=5, method="psto", want_grad=True)
        g8two, shtwo = ops.grad_update(dw.contiguous(), wtwo, amw, 5, "psto", want_grad=True)
        assert int(sync.cpu()[1]) == 0 and int(sync.cpu()[0]) == int(amw.cpu())
        assert torch.equal(g8, g8two) and int(sh.cpu()) == int(shtwo.cpu()) and torch.equal(wnew, wtwo)
        assert torch.equal(wnew.cpu(), po.weight_update(w, g8.cpu()))
    # data gradient (the first layer has none)
    if C % 16 == 0:
        amd = ops.new_scalar_u32(dev)
        dx = ops.conv2d_dgrad(ed, wd, 1, 1, absmax=amd)
        assert torch.equal(dx[sub].cpu(), co.conv_dgrad(e[sub].contiguous(), w, Q, Q, 1, 1))
        assert int((dx.to(torch.int64) * xd.to(torch.int64)).sum()) == lhs
        wf = ops.conv_filter_prepare(wd, N, Q, Q)
        d8, sh, sync = ops.conv2d_dgrad_requant(ed, wd, forward_filter=wf)
        r8, rsh = ops.requant(dx, amd, 7, "round")
        assert int(sync.cpu()[1]) == 0 and torch.equal(d8, r8) and int(sh.cpu()) == int(rsh.cpu())


@pytest.mark.parametrize("case", [(8, 32, 64, 128), (16, 8, 256, 64), (4, 16, 32, 48),
                                  (264, 16, 16, 272), (136, 32, 16, 144)])   # the last two: more workgroups than fit at once
def test_conv_requant_predicted_shift(dev, case):
    """A predicted shift (right, too small, too large, absurd) changes how often the kernel stores, never what."""
    from niti_amd import ops
    from oracle import c_oracle as co
    from oracle import niti_oracle as po
    N, Q, C, K = case
    _say("conv_requant_predicted_shift", case)
    g = torch.Generator().manual_seed(8200 + C + K)
    x, w, e = ri8(g, N, Q, Q, C), ri8(g, K, 3, 3, C), ri8(g, N, Q, Q, K)
    acc = po.conv2d_fprop_i32(x, w, 1, 1)
    ref, sh_ref = po.act_calc(acc, 0)
    dacc = co.conv_dgrad(e, w, Q, Q, 1, 1)
    dref, dsh = po.err_calc(dacc)
    for guess in (sh_ref, sh_ref - 1, sh_ref + 1, 0, 31):
        so = torch.tensor([max(guess, 0)], dtype=torch.int32, device=dev)
        y, sh, sync = ops.conv2d_fprop_requant(x.to(dev), w.to(dev), shift_out=so, shift_hint=True)
        assert sh is so and int(sync.cpu()[1]) == 0
        assert torch.equal(y.cpu(), ref) and int(so.cpu()) == sh_ref
        so = torch.tensor([max(guess, 0)], dtype=torch.int32, device=dev)
        d8, sh, sync = ops.conv2d_dgrad_requant(e.to(dev), w.to(dev), shift_out=so, shift_hint=True)
        assert torch.equal(d8.cpu(), dref) and int(so.cpu()) == dsh
    # all-zero input: no shift at all, whatever was predicted
    so = torch.tensor([5], dtype=torch.int32, device=dev)
    y, sh, sync = ops.conv2d_fprop_requant(torch.zeros_like(x).to(dev), w.to(dev), shift_out=so, shift_hint=True)
    assert int(y.abs().max()) == 0 and int(so.cpu()) == 0


def test_conv_requant_oversubscribed_range_set_by_one_tile(dev):
    """Two-launch form (more workgroups than fit at once): one image with large values among images of tiny ones makes
    nearly every workgroup of the second launch compute and store its tile again; with the mask of a ReLU below and
    with the pooled output."""
    from niti_amd import ops
    from oracle import c_oracle as co
    from oracle import niti_oracle as po
    N, Q, C, K = 136, 32, 144, 144
    _say("conv_requant_oversubscribed_range_set_by_one_tile")
    g = torch.Generator().manual_seed(6160)
    x = ri8(g, N, Q, Q, C, lo=-1, hi=1)
    x[77] = ri8(g, Q, Q, C)
    w = ri8(g, K, 3, 3, C)
    acc = po.conv2d_fprop_i32(x, w, 1, 1)
    ref, sh_ref = po.act_calc(acc, 0)
    pooled = torch.empty((N, Q // 2, Q // 2, K), dtype=torch.int8, device=dev)
    y, sh, sync = ops.conv2d_fprop_requant(x.to(dev), w.to(dev), relu=True, pool_out=pooled)
    assert int(sync.cpu()[1]) == 0 and int(sync.cpu()[0]) == po.absmax(acc) and int(sh.cpu()) == sh_ref
    assert torch.equal(y.cpu(), ref.clamp(min=0)) and torch.equal(pooled.cpu(), po.maxpool_fwd(ref.clamp(min=0)))
    e = ri8(g, N, Q, Q, K, lo=-1, hi=1)
    e[5] = ri8(g, Q, Q, K)
    dacc = co.conv_dgrad(e, w, Q, Q, 1, 1)
    dref, dsh = po.err_calc(dacc)
    mask = ri8(g, N, Q, Q, C)
    wf = ops.conv_filter_prepare(w.to(dev), N, Q, Q)
    for kw in (dict(), dict(forward_filter=wf)):
        d8, sh, sync = ops.conv2d_dgrad_requant(e.to(dev), w.to(dev), relu_mask=mask.to(dev), **kw)
        assert int(sync.cpu()[1]) == 0 and int(sh.cpu()) == dsh
        assert torch.equal(d8.cpu(), torch.where(mask > 0, dref, torch.zeros_like(dref)))


@pytest.mark.parametrize("hot", [0, 3, 7])
def test_conv_requant_range_set_by_one_tile(dev, hot):
    """The single-launch kernels store results with the range seen so far and store again when a later workgroup
    raises it: one image with large values among images of tiny ones makes most workgroups take that second pass."""
    from niti_amd import ops
    from oracle import c_oracle as co
    from oracle import niti_oracle as po
    N, Q, C, K = 8, 32, 64, 128
    _say("conv_requant_range_set_by_one_tile", hot)
    g = torch.Generator().manual_seed(5150 + hot)
    x = ri8(g, N, Q, Q, C, lo=-1, hi=1)
    x[hot] = ri8(g, Q, Q, C)
    w = ri8(g, K, 3, 3, C)
    acc = po.conv2d_fprop_i32(x, w, 1, 1)
    for method in ("round", "psto"):
        ref, sh_ref = po.act_calc(acc, 0, method)
        for rep in range(3):     # the order in which workgroups finish differs from launch to launch
            y, sh, sync = ops.conv2d_fprop_requant(x.to(dev), w.to(dev), method=method)
            assert int(sync.cpu()[1]) == 0 and int(sync.cpu()[0]) == po.absmax(acc)
            assert torch.equal(y.cpu(), ref) and int(sh.cpu()) == sh_ref
    e = ri8(g, N, Q, Q, K, lo=-1, hi=1)
    e[hot] = ri8(g, Q, Q, K)
    dacc = co.conv_dgrad(e, w, Q, Q, 1, 1)
    dref, dsh = po.err_calc(dacc)
    mask = ri8(g, N, Q, Q, C)
    for rep in range(3):
        d8, sh, sync = ops.conv2d_dgrad_requant(e.to(dev), w.to(dev), relu_mask=mask.to(dev))
        assert int(sync.cpu()[1]) == 0 and int(sh.cpu()) == dsh
        assert torch.equal(d8.cpu(), torch.where(mask > 0, dref, torch.zeros_like(dref)))


@pytest.mark.parametrize("case", [(4, 8, 96, 48), (1, 16, 32, 16), (2, 16, 256, 128), (8, 32, 128, 128), (4, 8, 16, 32),
                                  (256, 32, 64, 64), (1024, 16, 48, 32)])   # the last two: workgroups of 512 pixels
def test_conv_dgrad_requant(dev, case):
    from niti_amd import ops
    from oracle import c_oracle as co
    from oracle import niti_oracle as po
    N, Q, C, K = case
    _say("conv_dgrad_requant", case)
    g = torch.Generator().manual_seed(950 + C + K)
    e, w = ri8(g, N, Q, Q, K), ri8(g, K, 3, 3, C)
    acc = co.conv_dgrad(e, w, Q, Q, 1, 1)
    for method in ("round", "psto"):
        ref, sh_ref = po.err_calc(acc, method)
        wt = ops.conv_filter_prepare(w.to(dev), N, Q, Q, dgrad=True)
        for prepared in (None, wt):
            y, sh, sync = ops.conv2d_dgrad_requant(e.to(dev), w.to(dev), 1, 1, method=method, prepared_filter=prepared)
            assert int(sync.cpu()[1]) == 0
            assert torch.equal(y.cpu(), ref) and int(sh.cpu()) == sh_ref and int(sync.cpu()[0]) == po.absmax(acc)
        y, sh, sync = ops.conv2d_dgrad_requant(e.to(dev), w.to(dev), 1, 1, method=method,
                                               forward_filter=ops.conv_filter_prepare(w.to(dev), N, Q, Q))
        assert int(sync.cpu()[1]) == 0
        assert torch.equal(y.cpu(), ref) and int(sh.cpu()) == sh_ref and int(sync.cpu()[0]) == po.absmax(acc)
        # ReLU backward of the layer below folded in: zero where the mask is not positive, range from the unmasked sums
        mask = ri8(g, N, Q, Q, C)
        mask[0, 0, 0, :4] = torch.tensor([0, -128, 1, 127], dtype=torch.int8)
        y, sh, sync = ops.conv2d_dgrad_requant(e.to(dev), w.to(dev), 1, 1, method=method, relu_mask=mask.to(dev))
        assert torch.equal(y.cpu(), torch.where(mask > 0, ref, torch.zeros_like(ref)))
        assert int(sh.cpu()) == sh_ref and int(sync.cpu()[0]) == po.absmax(acc)


@pytest.fixture(params=["0", "1"])
def wgrad_arrangement(request):
    """Pin the native 3x3 weight-gradient kernel to its 128 x 64 tiles (0) or its 128 x 32 tiles with two pixel halves (1)."""
    import os
    old = os.environ.get("NITI_WGRAD_NARROW")
    os.environ["NITI_WGRAD_NARROW"] = request.param
    yield request.param
    if old is None:
        os.environ.pop("NITI_WGRAD_NARROW", None)
    else:
        os.environ["NITI_WGRAD_NARROW"] = old


@pytest.mark.parametrize("case", [(4, 8, 16, 16), (8, 8, 80, 144), (1, 16, 64, 64), (5, 16, 48, 272), (1, 32, 32, 16), (3, 32, 16, 80),
                                  (20, 8, 96, 32), (4, 16, 256, 64), (64, 8, 64, 256)])
def test_conv_wgrad_arrangements(dev, case, wgrad_arrangement):
    from niti_amd import ops
    from oracle import c_oracle as co
    from oracle import niti_oracle as po
    N, Q, C, K = case
    _say("conv_wgrad_arrangements", case, wgrad_arrangement)
    g = torch.Generator().manual_seed(980 + C + K)
    act, err = ri8(g, N, Q, Q, C), ri8(g, N, Q, Q, K)
    ref = co.conv_wgrad(act, err, 3, 3, 1, 1)
    am = ops.new_scalar_u32(dev)
    dw = ops.conv2d_wgrad(act.to(dev), err.to(dev), 3, 3, 1, 1, absmax=am)
    assert torch.equal(dw.cpu(), ref)
    assert int(am.cpu()) == po.absmax(ref)


@pytest.mark.parametrize("case", [(4, 32, 16, 32), (8, 16, 128, 64), (6, 8, 80, 144), (64, 8, 64, 256), (16, 16, 256, 128),
                                  (2, 8, 16, 16), (4, 8, 3, 16), (8, 32, 3, 128), (32, 8, 512, 512), (16, 4, 64, 128), (64, 4, 512, 256), (64, 2, 128, 64), (256, 2, 512, 512),
                                  (3, 32, 3, 64), (2, 32, 3, 32), (2, 32, 3, 256), (5, 32, 2, 64), (1, 32, 1, 128),
                                  (8, 4, 64, 128), (3, 2, 32, 32), (37, 4, 96, 160), (300, 2, 64, 32)])   # any batch size on 4 x 4 / 2 x 2 maps
@pytest.mark.parametrize("div_mode", ["floor", "trunc"])
@pytest.mark.parametrize("launches", ["one", "pair"])
def test_conv_wgrad_update(dev, case, div_mode, launches, monkeypatch):
    """wgrad + grad_calc + weight update in one call against the oracle's three steps.  `pair` pins the main + finishing
    launches for the shapes that otherwise run both parts as one launch."""
    import torch.nn.functional as F
    from niti_amd import ops
    from oracle import c_oracle as co
    from oracle import niti_oracle as po
    N, Q, C, K = case
    if launches == "pair":
        if Q < 8 or C < 16 or (N * Q * Q) % 256 != 0:
            pytest.skip("this shape has no one-launch form of the general kernel to pin away from")
        monkeypatch.setenv("NITI_WGRAD_ONE_LAUNCH", "0")
    _say("conv_wgrad_update", case, div_mode, launches)
    g = torch.Generator().manual_seed(970 + C + K)
    act, err, w = ri8(g, N, Q, Q, C), ri8(g, N, Q, Q, K, lo=-40, hi=40), ri8(g, K, 3, 3, C)
    dw_ref = co.conv_wgrad(act, err, 3, 3, 1, 1)
    act16 = F.pad(act, (0, 16 - C % 16)) if C % 16 else act
    for method, mu in (("psto", 5), ("round", 3)):
        g8_ref, sh_ref = po.grad_calc(dw_ref, mu, method, div_mode)
        w_ref = po.weight_update(w, g8_ref)
        wd = w.to(dev).clone()
        ea = torch.tensor([-4], dtype=torch.int32, device=dev)
        eo = torch.zeros(1, dtype=torch.int32, device=dev)
        g8, dw, sh, sync = ops.conv2d_wgrad_update(act16.to(dev).contiguous(), err.to(dev), wd, mu=mu, method=method,
                                                   div_mode=div_mode, want_grad=True, want_dw=True, exp_a=ea, exp_out=eo)
        torch.cuda.synchronize()
        sync = sync.cpu()
        assert int(sync[1]) == 0, "grid-wide wait timed out"
        assert int(sync[0]) == po.absmax(dw_ref)
        assert torch.equal(dw.cpu()[..., :C], dw_ref)
        assert int(sh.cpu()) == sh_ref and int(eo.cpu()) == sh_ref - 4
        assert torch.equal(g8.cpu(), g8_ref)
        assert torch.equal(wd.cpu(), w_ref)
        # a predicted shift (right, too small, too large) changes when the update is stored, never its result
        for guess in (sh_ref, max(sh_ref - 1, 0), sh_ref + 2):
            wd3 = w.to(dev).clone()
            so = torch.tensor([guess], dtype=torch.int32, device=dev)
            g8p, _, shp, syncp = ops.conv2d_wgrad_update(act16.to(dev).contiguous(), err.to(dev), wd3, mu=mu, method=method,
                                                         div_mode=div_mode, want_grad=True, shift_out=so, shift_hint=True)
            assert int(syncp.cpu()[1]) == 0 and int(so.cpu()) == sh_ref
            assert torch.equal(g8p.cpu(), g8_ref) and torch.equal(wd3.cpu(), w_ref)
        # without the optional outputs, and with a kernel-ready forward filter copy that has to follow the update
        wd2 = w.to(dev).clone()
        w16 = (F.pad(w, (0, 16 - C % 16)) if C % 16 else w).to(dev).contiguous()
        wp = ops.conv_filter_prepare(w16, N, Q, Q)
        ops.conv2d_wgrad_update(act16.to(dev).contiguous(), err.to(dev), wd2, mu=mu, method=method, div_mode=div_mode,
                                prepared_filter=wp)
        assert torch.equal(wd2.cpu(), w_ref)
        if wp is not None:
            w16_ref = (F.pad(w_ref, (0, 16 - C % 16)) if C % 16 else w_ref).to(dev).contiguous()
            assert torch.equal(wp.cpu(), ops.conv_filter_prepare(w16_ref, N, Q, Q).cpu())


@pytest.mark.parametrize("case", [(128, 10, 8192), (5, 3, 64), (33, 16, 272), (512, 10, 1024), (1, 1, 16), (100, 7, 4000), (37, 10, 384),
                                  (48, 16, 128)])
@pytest.mark.parametrize("div_mode", ["floor", "trunc"])
def test_fc_few_outputs(dev, case, div_mode):
    """TiLinear's three passes as one launch each (few output features) against GEMM + requantisation of the oracle."""
    from niti_amd import ops
    from oracle import niti_oracle as po
    M, O, F = case
    _say("fc_few_outputs", case, div_mode)
    g = torch.Generator().manual_seed(4100 + M + O + F)
    act, w, err = ri8(g, M, F), ri8(g, O, F), ri8(g, M, O, lo=-40, hi=40)
    ea = torch.tensor([-3], dtype=torch.int32, device=dev)
    eb = torch.tensor([-5], dtype=torch.int32, device=dev)
    # forward: act_calc(act @ w^T)
    acc = po.int8mm(act, w.t().contiguous())
    for method in ("round", "psto"):
        ref, sh_ref = po.act_calc(acc, 0, method, div_mode)
        eo = torch.zeros(1, dtype=torch.int32, device=dev)
        y, sh, sync = ops.fc_fwd_requant(act.to(dev), w.to(dev), 7, method, div_mode, exp_a=ea, exp_b=eb, exp_out=eo)
        sync = sync.cpu()
        assert int(sync[0]) == po.absmax(acc) and int(sync[1]) == 0
        assert torch.equal(y.cpu(), ref) and int(sh.cpu()) == sh_ref and int(eo.cpu()) == sh_ref - 8
        # data gradient: err_calc(err @ w)
        dacc = po.int8mm(err, w)
        dref, dsh = po.err_calc(dacc, method, div_mode)
        dx, sh, sync = ops.fc_dgrad_requant(err.to(dev), w.to(dev), 7, method, div_mode, exp_a=ea, exp_out=eo)
        sync = sync.cpu()
        assert int(sync[0]) == po.absmax(dacc) and int(sync[1]) == 0
        assert torch.equal(dx.cpu(), dref) and int(sh.cpu()) == dsh and int(eo.cpu()) == dsh - 3
        # weight gradient, grad_calc, update
        if M <= 512:
            gacc = po.int8mm(err.t().contiguous(), act)
            for mu in (5, 3):
                g8_ref, gsh = po.grad_calc(gacc, mu, method, div_mode)
                w_ref = po.weight_update(w, g8_ref)
                wd = w.to(dev).clone()
                g8, sh, sync = ops.fc_wgrad_update(err.to(dev), act.to(dev), wd, mu, method, div_mode, want_grad=True,
                                                   exp_a=ea, exp_b=eb, exp_out=eo)
                sync = sync.cpu()
                assert int(sync[0]) == po.absmax(gacc) and int(sync[1]) == 0
                assert torch.equal(g8.cpu(), g8_ref) and int(sh.cpu()) == gsh and int(eo.cpu()) == gsh - 8
                assert torch.equal(wd.cpu(), w_ref)
                wd2 = w.to(dev).clone()
                ops.fc_wgrad_update(err.to(dev), act.to(dev), wd2, mu, method, div_mode)
                assert torch.equal(wd2.cpu(), w_ref)
    # shapes outside the kernels are reported, not run
    assert ops.fc_sync_words("forward", 128, 17, 8192) == 0 and ops.fc_sync_words("wgrad", 513, 10, 64) == 0
    assert ops.fc_sync_words("dgrad", 8, 10, 24) == 0


def test_conv_requant_rejects_what_it_does_not_cover(dev):
    from niti_amd import ops
    from niti_amd._lib import NitiError
    _say("conv_requant unsupported shapes")
    assert ops.conv_requant_sync_words(3, 7, 9, 32, 40) == 0        # not square / not 8, 16, 32
    assert ops.conv_requant_sync_words(2, 8, 8, 16, 10) == 0        # 128 pixels: not whole workgroups
    assert ops.conv_requant_sync_words(4096, 32, 32, 16, 128) == 0  # far more workgroups than any device holds
    x = torch.zeros((2, 8, 8, 16), dtype=torch.int8, device=dev)
    w = torch.zeros((16, 3, 3, 16), dtype=torch.int8, device=dev)
    with pytest.raises(NitiError):
        ops.conv2d_fprop_requant(x, w)
    # the forward filter copy stands in for the data gradient's own only where both passes run the 3x3 kernel
    e = torch.zeros((3, 7, 9, 32), dtype=torch.int8, device=dev)
    with pytest.raises(NitiError):
        ops.conv2d_dgrad(e, torch.zeros((32, 3, 3, 16), dtype=torch.int8, device=dev), forward_filter=torch.zeros(64, dtype=torch.int8, device=dev))
    # a launch that would not be resident at once runs as two launches that do not wait for each other
    from oracle import niti_oracle as po
    N = 2048                                                          # 2048 tiles of 256 pixels
    assert ops.conv_requant_sync_words(N, 16, 16, 16, 16) > 0
    g = torch.Generator().manual_seed(31)
    x, w = ri8(g, N, 16, 16, 16), ri8(g, 16, 3, 3, 16)
    ref, sh_ref = po.act_calc(po.conv2d_fprop_i32(x, w, 1, 1), 0)
    y, sh, sync = ops.conv2d_fprop_requant(x.to(dev), w.to(dev))
    assert int(sync.cpu()[1]) == 0 and int(sh.cpu()) == sh_ref and torch.equal(y.cpu(), ref)
    # internal flag bits are not part of the interface
    from niti_amd import _lib as L
    xs = torch.zeros((4, 8, 8, 16), dtype=torch.int8, device=dev)
    y8 = torch.empty((4, 8, 8, 16), dtype=torch.int8, device=dev)
    words = ops.conv_requant_sync_words(4, 8, 8, 16, 16)
    sync = torch.zeros(words, dtype=torch.int32, device=dev)
    ws = torch.empty(1 << 20, dtype=torch.int8, device=dev)
    st = L.lib().niti_conv2d_i8_fprop_requant(xs.data_ptr(), w.to(dev).data_ptr(), y8.data_ptr(), 4, 8, 8, 16, 16, 3, 3, 1, 1, 0, 7, 0, 0, 0,
                                              1 << 30, sync.data_ptr(), words, None, None, None, None, ws.data_ptr(), ws.numel(), None)
    assert st != 0


WGRAD_CASES = [(4, 32, 32, 16, 32, 3, 1), (8, 16, 16, 128, 64, 3, 1), (6, 8, 8, 80, 144, 3, 1), (2, 32, 32, 64, 128, 3, 1),
               (64, 8, 8, 64, 256, 3, 1), (16, 16, 16, 256, 128, 3, 1), (2, 8, 8, 16, 16, 3, 1), (16, 8, 8, 32, 48, 3, 1), (5, 7, 9, 40, 24, 3, 1), (32, 16, 16, 64, 128, 3, 1),
               (4, 8, 8, 3, 16, 3, 1), (6, 8, 8, 16, 10, 5, 2), (3, 6, 6, 8, 8, 3, 0), (128, 8, 8, 16, 16, 3, 1),
               (16, 4, 4, 64, 128, 3, 1), (48, 4, 4, 272, 80, 3, 1), (256, 4, 4, 32, 16, 3, 1), (8, 4, 4, 16, 16, 3, 1),
               (64, 2, 2, 64, 128, 3, 1), (192, 2, 2, 272, 48, 3, 1), (256, 2, 2, 512, 512, 3, 1), (32, 2, 2, 16, 16, 3, 1)]


@pytest.mark.parametrize("case", WGRAD_CASES)
def test_conv_wgrad(dev, case):
    from niti_amd import ops
    from oracle import c_oracle as co
    from oracle import niti_oracle as po
    N, H, W, C, K, R, pad = case
    _say("conv_wgrad", case)
    g = torch.Generator().manual_seed(300 + C + K)
    P, Q = H + 2 * pad - R + 1, W + 2 * pad - R + 1
    a, e = ri8(g, N, H, W, C), ri8(g, N, P, Q, K)
    ref = co.conv_wgrad(a, e, R, R, 1, pad)
    if 2 * pad == R - 1:
        assert torch.equal(ref, po.conv2d_wgrad_i32(a, e, 1, pad, f32_epilogue=False))
    am = ops.new_scalar_u32(dev)
    dw = ops.conv2d_wgrad(a.to(dev), e.to(dev), R, R, 1, pad, absmax=am)
    assert torch.equal(dw.cpu(), ref)
    assert int(am.cpu()) == po.absmax(ref)


# the last six take the kernel that reads operands with a slow reduction index as stored (n and k multiples of 32):
# several staged chunks, a chunk tail, row counts that are not multiples of the 128-row tile, the three products of a
# fully connected layer 8192 -> 1024 on a batch of 128; then shapes for the kernel that stages whole lines (n and k
# multiples of 128, in the doubly transposed form m and k): a row tail, a reduction split unevenly over workgroups
# (5 chunks in 2 parts), a single chunk, several tiles, a row tail in the transposed store
GEMM_CASES = [(128, 10, 8192), (16, 16, 16), (128, 128, 64), (100, 10, 512), (7, 5, 3), (130, 70, 100), (128, 1024, 1024), (33, 12, 8192),
              (48, 32, 32), (200, 64, 96), (160, 96, 2080), (64, 7, 1056), (128, 1024, 8192), (128, 8192, 1024), (1024, 8192, 128),
              (100, 128, 256), (40, 256, 640), (128, 128, 128), (96, 384, 1152), (256, 40, 640)]


@pytest.mark.parametrize("mnk", GEMM_CASES)
@pytest.mark.parametrize("ta,tb", [(False, True), (False, False), (True, False), (True, True)])
def test_gemm(dev, mnk, ta, tb):
    from niti_amd import ops
    from oracle import niti_oracle as po
    m, n, k = mnk
    _say("gemm", mnk, ta, tb)
    g = torch.Generator().manual_seed(400 + m + n + k)
    A, B = ri8(g, m, k), ri8(g, k, n)
    ref = po.int8mm(A, B)
    a = (A.t().contiguous() if ta else A).to(dev)
    b = (B.t().contiguous() if tb else B).to(dev)
    am = ops.new_scalar_u32(dev)
    c = ops.gemm(a, b, ta, tb, absmax=am)
    assert torch.equal(c.cpu(), ref)
    assert int(am.cpu()) == po.absmax(ref)


@pytest.mark.parametrize("mnk", [(160, 64, 2080), (160, 128, 2176), (384, 2048, 2176)])
@pytest.mark.parametrize("ta,tb", [(False, False), (True, False), (True, True)])
def test_gemm_f32_epilogue_above_2_24(dev, ta, tb, mnk):
    """Sums beyond 2**24 through the kernel that reads both operands as stored: with the flag every sum takes the
    reference epilogue's int32 -> float32 -> int32 round trip (linear_combination_clamp.h:371-389), without it none.
    The second shape takes the whole-line kernel with the reduction split over workgroups (the round trip then happens
    where the parts are added), the third the same kernel without a split."""
    from niti_amd import ops
    from oracle import niti_oracle as po
    _say("gemm f32 epilogue", ta, tb, mnk)
    g = torch.Generator().manual_seed(411)
    m, n, k = mnk
    A, B = ri8(g, m, k), ri8(g, k, n)
    A[:40] = 127
    B[:, :20] = 127
    B[:, 20:30] = -127
    B[5, :30] = 126          # odd sums: not representable in float32 above 2**24
    ref = po.int8mm(A, B)
    assert int(ref.abs().max()) > 2 ** 24 + 2 ** 20
    rt = ref.to(torch.float32).to(torch.int64).clamp(max=2 ** 31 - 1).to(torch.int32)
    assert not torch.equal(rt, ref)
    a = (A.t().contiguous() if ta else A).to(dev)
    b = (B.t().contiguous() if tb else B).to(dev)
    for f32 in (False, True):
        am = ops.new_scalar_u32(dev)
        c = ops.gemm(a, b, ta, tb, absmax=am, f32_epilogue=f32)
        want = rt if f32 else ref
        assert torch.equal(c.cpu(), want)
        assert int(am.cpu()) == po.absmax(want)


@pytest.mark.parametrize("div_mode", ["floor", "trunc"])
@pytest.mark.parametrize("method", ["round", "psto", "sto"])
def test_requant(dev, method, div_mode):
    from niti_amd import ops
    from oracle import niti_oracle as po
    g = torch.Generator().manual_seed(500)
    for n, hi in [(1, 5), (15, 128), (16, 129), (4099, 300), (70001, 40000), (1 << 18, 3000000), (1000, 2 ** 31 - 1)]:
        for tgt in (7, 5, 3):
            _say("requant", method, div_mode, n, hi, tgt)
            x = torch.randint(-hi, hi + 1, (n,), generator=g, dtype=torch.int64).to(torch.int32)
            x[0] = hi
            s = max(po.RangeEstimate(x) - tgt, 0)
            u = torch.randint(0, 2 ** max(s, 1), (n,), generator=g, dtype=torch.int32)
            if tgt == 7:
                ref, e = po.act_calc(x, 0, method, div_mode, u)
            else:
                ref, e = po.grad_calc(x, tgt, method, div_mode, u)
            xd = x.to(dev)
            am = ops.absmax_i32(xd)
            assert int(am.cpu()) == po.absmax(x)
            y, sh = ops.requant(xd, am, tgt, method, div_mode, rand=u.to(dev) if method == "sto" else None)
            assert torch.equal(y.cpu(), ref)
            assert int(sh.cpu()) == e == s
            yr, _ = ops.requant(xd, am, tgt, method, div_mode, rand=u.to(dev) if method == "sto" else None, relu=True)
            assert torch.equal(yr.cpu(), ref.clamp(min=0))


def test_requant_special_cases(dev, kat):
    from niti_amd import ops
    from oracle import niti_oracle as po
    _say("requant special cases")
    for vals, want_shift in (([0, 0, 0, 0, 0], 0), ([128, -128, 127, 5, -3], 0), ([129, -129, 1, -1, 0], 1)):
        x = torch.tensor(vals, dtype=torch.int32)
        ref, e = po.act_calc(x, 0)
        am = ops.absmax_i32(x.to(dev))
        y, sh = ops.requant(x.to(dev), am, 7)
        assert y.cpu().tolist() == ref.tolist() and int(sh.cpu()) == want_shift
    # known-answer table through the kernel: fix the shift by planting the range in absmax
    X = torch.tensor(kat["X"], dtype=torch.int32)
    for mode in ("floor", "trunc"):
        am = torch.tensor([2 ** 14], dtype=torch.int32, device=dev)   # bitwidth 14 -> shift 7
        y, sh = ops.requant(X.to(dev), am, 7, "round", mode)
        assert y.cpu().tolist() == kat[f"round_s7_{mode}"] and int(sh.cpu()) == 7
        y, _ = ops.requant(X.to(dev), am, 7, "psto", mode)
        assert y.cpu().tolist() == kat[f"psto_s7_{mode}"]
    # bit-width evaluated the reference's float way inside the thin band above 2^22
    x = torch.tensor([2 ** 22 + 2, -5, 77], dtype=torch.int32)
    am = ops.absmax_i32(x.to(dev))
    _, s_int = ops.requant(x.to(dev), am, 7, bw_mode="int")
    _, s_f32 = ops.requant(x.to(dev), am, 7, bw_mode="f32")
    assert int(s_int.cpu()) == 23 - 7 and int(s_f32.cpu()) == 22 - 7 == po.bitwidth_f32(2 ** 22 + 2) - 7


def _band_operands(g, N, Q, C, K):
    """Activations and a filter whose largest convolution sum is exactly 2**22 + 2 (at one output pixel, channel 0):
    260 products 127 * 127, one 127 * 6 and one 4 * 1 under the 3 x 3 x 32 window of pixel (0, 3, 3); everything else
    is non-negative and smaller.  In (2**22, 2**22 (1 + 7e-7)] the reference's float evaluation of the bit width
    (ti_torch.py:366-377) gives 22 where the exact integer form gives 23."""
    x = torch.zeros((N, Q, Q, C), dtype=torch.int8)
    w = torch.randint(0, 3, (K, 3, 3, C), generator=g, dtype=torch.int8)
    xv = [127] * 260 + [127, 4] + [0] * (9 * 32 - 262)
    wv = [127] * 260 + [6, 1] + [0] * (9 * 32 - 262)
    x[0, 2:5, 2:5, :32] = torch.tensor(xv, dtype=torch.int8).view(3, 3, 32)
    w[0, :, :, :] = 0
    w[0, :, :, :32] = torch.tensor(wv, dtype=torch.int8).view(3, 3, 32)
    x[1:] = torch.randint(0, 4, (N - 1, Q, Q, C), generator=g, dtype=torch.int8)
    return x, w


def test_fused_epilogues_in_both_bitwidth_modes(dev):
    """The tensor-wide range lands in the thin band above 2**22 where the two bit-width rules differ: forward
    convolution + act_calc, data gradient + err_calc and weight gradient + grad_calc + update, each as its one-launch
    form, in the exact integer mode and in the reference's float mode."""
    from niti_amd import ops
    from oracle import c_oracle as co
    from oracle import niti_oracle as po
    g = torch.Generator().manual_seed(977)
    N, Q, C, K = 8, 8, 64, 64
    T = 2 ** 22 + 2
    assert po.bitwidth_int(T) == 23 and po.bitwidth_f32(T) == 22
    x, w = _band_operands(g, N, Q, C, K)
    acc = co.conv_fprop(x, w, 1, 1)
    assert int(acc.abs().max()) == T
    for mode, want in (("int", 16), ("f32", 15)):
        _say("band fprop", mode)
        ref, e = po.act_calc(acc, 0, "round", "floor", None, mode)
        y, sh, _ = ops.conv2d_fprop_requant(x.to(dev), w.to(dev), bw_mode=mode)
        assert int(sh.cpu()) == want == e
        assert torch.equal(y.cpu(), ref)
    # data gradient: the error map plays the activations' part; flipping the filter's taps and swapping its channel
    # roles turns the forward sums above into data-gradient sums (ti_torch.py:403-405)
    wd = torch.flip(w, [1, 2]).permute(3, 1, 2, 0).contiguous()
    accd = co.conv_dgrad(x, wd, Q, Q, 1, 1)
    assert torch.equal(accd, acc)
    for mode, want in (("int", 16), ("f32", 15)):
        _say("band dgrad", mode)
        ref, e = po.err_calc(accd, "round", "floor", None, mode)
        dx, sh, _ = ops.conv2d_dgrad_requant(x.to(dev), wd.to(dev), bw_mode=mode)
        assert int(sh.cpu()) == want == e
        assert torch.equal(dx.cpu(), ref)
    # weight gradient: 260 pixels with 127 in activation channel 0 and error channel 0, two isolated pixels carrying
    # 127 * 6 and 4 * 1; the centre tap sums them all, every other tap loses at least one pair
    Nw = 8
    act = torch.zeros((Nw, Q, Q, C), dtype=torch.int8)
    err = torch.zeros((Nw, Q, Q, K), dtype=torch.int8)
    flat_a, flat_e = act.view(-1, C), err.view(-1, K)
    flat_a[:260, 0] = 127
    flat_e[:260, 0] = 127
    flat_a[5 * 64 + 18, 0], flat_e[5 * 64 + 18, 0] = 127, 6
    flat_a[6 * 64 + 45, 0], flat_e[6 * 64 + 45, 0] = 4, 1
    act[7] = torch.randint(0, 3, (Q, Q, C), generator=g, dtype=torch.int8)
    err[7] = torch.randint(0, 3, (Q, Q, K), generator=g, dtype=torch.int8)
    act[7, :, :, 0] = 0     # nothing more for the element that carries the range
    accw = co.conv_wgrad(act, err, 3, 3, 1, 1)
    assert int(accw.abs().max()) == T == int(accw[0, 1, 1, 0])
    w0 = torch.randint(-127, 128, (K, 3, 3, C), generator=g, dtype=torch.int8)
    for mode, want in (("int", 18), ("f32", 17)):
        _say("band wgrad", mode)
        g8, e = po.grad_calc(accw, 5, "psto", "floor", None, mode)
        wdev = w0.clone().to(dev)
        got_g8, _, sh, _ = ops.conv2d_wgrad_update(act.to(dev), err.to(dev), wdev, mu=5, method="psto", bw_mode=mode, want_grad=True)
        assert int(sh.cpu()) == want == e
        assert torch.equal(got_g8.cpu(), g8)
        assert torch.equal(wdev.cpu(), po.weight_update(w0, g8))


@pytest.mark.parametrize("div_mode", ["floor", "trunc"])
def test_grad_update_and_weight_update(dev, div_mode):
    from niti_amd import ops
    from oracle import niti_oracle as po
    g = torch.Generator().manual_seed(600)
    for n in (7, 1152, 128 * 9 * 128 + 3):
        for mu in (5, 4, 3):
            for method in ("psto", "round"):
                _say("grad_update", div_mode, n, mu, method)
                gi = torch.randint(-900000, 900001, (n,), generator=g, dtype=torch.int32)
                w = ri8(g, n)
                g8, s = po.grad_calc(gi, mu, method, div_mode)
                wref = po.weight_update(w, g8)
                wd = w.to(dev)
                am = ops.absmax_i32(gi.to(dev))
                g8d, sh = ops.grad_update(gi.to(dev), wd, am, mu, method, div_mode, want_grad=True)
                assert torch.equal(g8d.cpu(), g8) and torch.equal(wd.cpu(), wref) and int(sh.cpu()) == s
                w2 = w.to(dev)
                ops.weight_update(w2, g8.to(dev))
                assert torch.equal(w2.cpu(), wref)


def test_relu(dev):
    from niti_amd import ops
    g = torch.Generator().manual_seed(700)
    for n in (5, 64, 100003):
        _say("relu", n)
        x, dy = ri8(g, n, lo=-128), ri8(g, n)
        assert torch.equal(ops.relu_fwd(x.to(dev)).cpu(), x.clamp(min=0))
        assert torch.equal(ops.relu_bwd(x.to(dev), dy.to(dev)).cpu(), torch.where(x > 0, dy, torch.zeros_like(dy)))


POOL_CASES = [(2, 8, 8, 16, 2, 2, 0), (1, 6, 6, 5, 2, 2, 0), (2, 7, 7, 32, 3, 2, 1), (1, 5, 5, 3, 2, 1, 0),
              (1, 9, 9, 16, 3, 3, 0), (8, 32, 32, 128, 2, 2, 0), (3, 7, 7, 16, 2, 2, 0), (5, 4, 6, 48, 2, 2, 0), (2, 2, 2, 16, 2, 2, 0)]


@pytest.mark.parametrize("case", POOL_CASES)
def test_maxpool(dev, case):
    from niti_amd import ops
    from oracle import c_oracle as co
    N, H, W, C, ks, st, pad = case
    g = torch.Generator().manual_seed(800 + C)
    for lo, hi in ((-128, 127), (-2, 2), (0, 1)):
        _say("maxpool", case, lo, hi)
        x = ri8(g, N, H, W, C, lo=lo, hi=hi)
        yref = co.maxpool_fwd(x, ks, st, pad)
        y = ops.maxpool_fwd(x.to(dev), ks, st, pad)
        assert torch.equal(y.cpu(), yref)
        dy = ri8(g, *yref.shape, lo=-30, hi=30)
        for ties in ("first", "all"):
            ref = co.maxpool_bwd(yref, dy, x, ks, st, pad, ties)
            dx = ops.maxpool_bwd(y, dy.to(dev), x.to(dev), ks, st, pad, ties)
            assert torch.equal(dx.cpu(), ref), ties
            # with the backward pass of a ReLU in front of the pooling folded in
            dxr = ops.maxpool_bwd(y, dy.to(dev), x.to(dev), ks, st, pad, ties, relu=True)
            assert torch.equal(dxr.cpu(), torch.where(x > 0, ref, torch.zeros_like(ref))), ties


def test_quantize_input(dev):
    """The input quantiser (two launches: range, then quantise + NHWC + channel padding) against the CPU oracle's
    TiFloatToInt8 + permute, including ranges at and next to a power of two (where ceil(log2 r) jumps), the hand-derived
    known answers, round-half-even ties and both clamps; the tensor-operation form of the package gives the same."""
    import json
    import os
    from niti_amd import ops, ti_torch
    from oracle import niti_oracle as po
    _say("quantize_input")
    g = torch.Generator().manual_seed(77)
    for shape, top in (((128, 3, 32, 32), None), ((5, 3, 7, 9), 4.0), ((2, 3, 8, 8), 4.000001), ((2, 3, 8, 8), 3.9999998),
                       ((3, 17, 4, 4), 0.3), ((1, 1, 1, 1), 100.0), ((2, 3, 8, 8), 16.000002), ((2, 3, 4, 4), 1e-3),
                       ((2, 3, 4, 4), 3e4)):
        x = torch.randn(shape, generator=g)
        if top is not None:
            x = x / x.abs().max() * 0.9 * top
            x.view(-1)[min(3, x.numel() - 1)] = -top
        ref, ref_exp = po.quantize_input_nhwc(x)
        xd = x.to(dev)
        y, e = ops.quantize_input(xd)
        C = shape[1]
        assert y.shape[3] == max(16, (C + 3) // 4 * 4) and int(e.cpu()) == ref_exp, (shape, top)
        assert torch.equal(y[..., :C].cpu(), ref) and int(y[..., C:].abs().max()) == 0, (shape, top)
        t, te = ti_torch.TiFloatToInt8(xd)
        assert int(te.cpu()) == ref_exp and torch.equal(t.permute(0, 2, 3, 1).cpu(), ref), (shape, top)
    with open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "quantize_kat.json")) as f:
        kat = json.load(f)
    for c in kat["float_to_int8"]:
        x = torch.tensor(c["x"], dtype=torch.float32).reshape(1, -1, 1, 1)     # the values as channels of one pixel
        y, e = ops.quantize_input(x.to(dev))
        assert y[0, 0, 0, :x.shape[1]].cpu().tolist() == c["q"] and int(e.cpu()) == c["exp"], c["name"]
    for c in kat["weight_quant"]:
        q, e = ti_torch.weight_quant(torch.tensor(c["w"], dtype=torch.float32))
        assert q.cpu().tolist() == c["q"] and int(e.cpu()) == c["exp"], c["name"]
    w = torch.randn((64, 3, 3, 32), generator=g) * 0.07
    q, e = ti_torch.weight_quant(w.to(dev))
    qr, er = po.weight_quant(w)
    assert torch.equal(q.cpu(), qr) and int(e.cpu()) == er
    y, e = ops.quantize_input(torch.zeros((2, 3, 4, 4), device=dev))
    assert int(y.abs().max()) == 0 and int(e.cpu()) == 0


def test_mask_features(dev):
    """Dropout as one launch: a keep / drop byte per feature times every row, exponent + 1."""
    from niti_amd import ops
    _say("mask_features")
    g = torch.Generator().manual_seed(4242)
    for rows, feats in ((128, 8192), (7, 48), (1, 16), (256, 512)):
        x = ri8(g, rows, feats, lo=-128)
        mask = torch.randint(0, 2, (feats,), generator=g, dtype=torch.int8)
        e = torch.tensor([-9], dtype=torch.int32, device=dev)
        y, eo = ops.mask_features(x.to(dev), mask.to(dev), e, 1)
        assert torch.equal(y.cpu(), x * mask) and int(eo.cpu()) == -8
        assert torch.equal(ops.mask_features(x.to(dev), mask.to(dev)).cpu(), x * mask)
    with pytest.raises(Exception):
        ops.mask_features(torch.zeros((4, 24), dtype=torch.int8, device=dev), torch.ones(24, dtype=torch.int8, device=dev))


def test_pad_last_dim(dev):
    import torch.nn.functional as F
    from niti_amd import ops
    g = torch.Generator().manual_seed(77)
    for shape in ((128, 32, 32, 3), (7, 3, 3, 3), (5, 40), (2, 2, 2, 16), (3, 1, 1, 17)):
        _say("pad_last_dim", shape)
        x = ri8(g, *shape)
        y = ops.pad_last_dim(x.to(dev), 16)
        c = shape[-1]
        ref = F.pad(x, (0, (16 - c % 16) % 16))
        assert y.dtype == torch.int8 and torch.equal(y.cpu(), ref)


def test_group_conv_first_layer_wgrad(dev):
    """The reference's first-layer weight gradient (ti_torch.py:194-233) routed through the
    group_conv stand-in gives the true weight gradient as float32."""
    from niti_amd import ops
    from oracle import niti_oracle as po
    _say("group_conv")
    g = torch.Generator().manual_seed(900)
    N, H, W, C, K = 4, 8, 8, 3, 16
    act, err = ri8(g, N, H, W, C), ri8(g, N, H, W, K)
    # operand preparation exactly as conv2d_weight_int8 does it
    go = err.permute(0, 3, 1, 2).contiguous().repeat(1, C, 1, 1)
    go = go.contiguous().reshape(N * C * K, 1, H, W).permute(0, 2, 3, 1).contiguous()
    inp = act.permute(0, 3, 1, 2).contiguous().reshape(1, N * C, H, W).permute(0, 2, 3, 1).contiguous()
    out = ops.group_conv_f32(inp.to(dev), go.to(dev), 1, 1, 1, C * N).cpu()
    gw = out.permute(0, 3, 1, 2)
    gw = gw.view(N, gw.shape[1] // N, gw.shape[2], gw.shape[3]).sum(dim=0)
    gw = gw.view(C, K, gw.shape[1], gw.shape[2]).transpose(0, 1).narrow(2, 0, 3).narrow(3, 0, 3)
    gw = gw.permute(0, 2, 3, 1).contiguous()
    assert gw.dtype == torch.float32
    assert torch.equal(gw, po.conv2d_weight_int8(act, (K, 3, 3, C), err, 1, 1))


@pytest.mark.parametrize("case", [(128, 8192, 1024), (40, 256, 64), (300, 512, 96), (16, 64, 32), (64, 320, 32), (128, 1024, 2048),
                                  (7, 4096, 128), (40, 384, 384), (33, 128, 256)])   # M, F, O; the last two: a ring of three
                                                                                     # stages that wraps, ragged sample tiles
@pytest.mark.parametrize("div_mode", ["floor", "trunc"])
def test_linear_any_width(dev, case, div_mode):
    """TiLinear's three passes as single launches on operands as stored, all rounding methods (stochastic rounding on
    supplied random integers), against int8mm + act_calc / err_calc / grad_calc / weight_update of the oracle."""
    from niti_amd import ops
    from oracle import c_oracle as co
    from oracle import niti_oracle as po
    M, F, O = case
    _say("linear_any_width", case, div_mode)
    g = torch.Generator().manual_seed(5000 + M + O)
    act, w, err = ri8(g, M, F), ri8(g, O, F), ri8(g, M, O, lo=-60, hi=60)
    acc_f = co.gemm(act, w.t().contiguous())            # [M,O]
    acc_d = co.gemm(err, w)                             # [M,F]
    acc_w = co.gemm(err.t().contiguous(), act)          # [O,F]
    assert torch.equal(acc_f, po.int8mm(act, w.t().contiguous()))
    ad, wd, ed = act.to(dev), w.to(dev), err.to(dev)
    for method in ("round", "psto", "sto"):
        uf = torch.randint(0, 1 << 24, (M, O), generator=g, dtype=torch.int32)
        ud = torch.randint(0, 1 << 24, (M, F), generator=g, dtype=torch.int32)
        uw = torch.randint(0, 1 << 24, (O, F), generator=g, dtype=torch.int32)
        sto = method == "sto"

        def low(u, acc, bits):    # the low `shift` bits, as the reference's randint(0, 2^shift) would give
            s = max(po.bitwidth_int(po.absmax(acc)) - bits, 0)
            return u & ((1 << s) - 1) if s > 0 else torch.zeros_like(u)
        if ops.linear_sync_words("forward", M, O, F):
            ref, e_ref = po.act_calc(acc_f, -5, method, div_mode, rand=low(uf, acc_f, 7) if sto else None)
            ea = torch.tensor([-5], dtype=torch.int32, device=dev)
            eo = torch.zeros(1, dtype=torch.int32, device=dev)
            y, sh, sync = ops.linear_fwd_requant(ad, wd, 7, method, div_mode, rand=uf.to(dev) if sto else None, exp_a=ea, exp_out=eo)
            sync = sync.cpu()
            assert int(sync[1]) == 0 and int(sync[0]) == po.absmax(acc_f), method
            assert torch.equal(y.cpu(), ref) and int(eo.cpu()) == e_ref, method
            yr, _, _ = ops.linear_fwd_requant(ad, wd, 7, method, div_mode, relu=True, rand=uf.to(dev) if sto else None)
            assert torch.equal(yr.cpu(), torch.clamp(ref, min=0)), method
        else:
            assert O % 4 or F % 16
        if ops.linear_sync_words("dgrad", M, O, F):
            ref, sh_ref = po.err_calc(acc_d, method, div_mode, rand=low(ud, acc_d, 7) if sto else None)
            y, sh, sync = ops.linear_dgrad_requant(ed, wd, 7, method, div_mode, rand=ud.to(dev) if sto else None)
            sync = sync.cpu()
            assert int(sync[1]) == 0 and int(sync[0]) == po.absmax(acc_d), method
            assert int(sh.cpu()) == sh_ref and torch.equal(y.cpu(), ref), method
        else:
            assert O % 32 or F % 32
        if ops.linear_sync_words("wgrad", M, O, F):
            g8_ref, sh_ref = po.grad_calc(acc_w, 5, method, div_mode, rand=low(uw, acc_w, 5) if sto else None)
            w_ref = po.weight_update(w, g8_ref)
            wu = wd.clone()
            g8, sh, sync = ops.linear_wgrad_update(ed, ad, wu, 5, method, div_mode, rand=uw.to(dev) if sto else None, want_grad=True)
            sync = sync.cpu()
            assert int(sync[1]) == 0 and int(sync[0]) == po.absmax(acc_w), method
            assert int(sh.cpu()) == sh_ref and torch.equal(g8.cpu(), g8_ref) and torch.equal(wu.cpu(), w_ref), method
        else:
            assert O % 16 or F % 16
    assert ops.linear_sync_words("forward", 128, 1024, 8192) > 0 and ops.linear_sync_words("dgrad", 128, 1024, 8192) > 0
    assert ops.linear_sync_words("wgrad", 128, 1024, 8192) > 0


@pytest.mark.parametrize("case", [(4, 8, 16, 32), (8, 16, 128, 64), (2, 16, 48, 80), (16, 4, 64, 128), (8, 32, 32, 16), (1024, 16, 48, 32),
                                  (264, 16, 16, 272), (64, 2, 64, 128), (40, 2, 48, 80)])   # N, Q (pooled map), C, K; 512-pixel tiles, two-launch form, 2 x 2 maps
def test_conv_dgrad_requant_unpool(dev, case):
    """Data gradient + err_calc + ReLU mask + the backward pass of the 2x2 max-pool in front of the layer in one launch,
    against the oracle's three steps; windows with several equal maxima under both tie rules."""
    from niti_amd import ops
    from oracle import c_oracle as co
    from oracle import niti_oracle as po
    N, Q, C, K = case
    _say("conv_dgrad_requant_unpool", case)
    g = torch.Generator().manual_seed(990 + C + K)
    e, w = ri8(g, N, Q, Q, K), ri8(g, K, 3, 3, C)
    pool_in = ri8(g, N, 2 * Q, 2 * Q, C, lo=-3, hi=5)            # few distinct values: many ties, many non-positive maxima
    pooled = po.maxpool_fwd(pool_in)
    acc = co.conv_dgrad(e, w, Q, Q, 1, 1)
    ed, wd, pd, xd = e.to(dev), w.to(dev), pooled.to(dev), pool_in.to(dev)
    for method in ("round", "psto"):
        dx, sh_ref = po.err_calc(acc, method)
        dx = torch.where(pooled > 0, dx, torch.zeros_like(dx))
        for ties in ("first", "all"):
            ref = co.maxpool_bwd(pooled, dx, pool_in, 2, 2, 0, ties)
            y, sh, sync = ops.conv2d_dgrad_requant(ed, wd, 1, 1, method=method, relu_mask=pd, unpool=(xd, ties))
            assert tuple(y.shape) == tuple(pool_in.shape) and int(sync.cpu()[1]) == 0
            assert int(sh.cpu()) == sh_ref and int(sync.cpu()[0]) == po.absmax(acc)
            assert torch.equal(y.cpu(), ref), (method, ties)
        # the forward filter copy as the filter operand, and a wrong shift prediction (stores twice)
        so = torch.tensor([max(sh_ref - 2, 0)], dtype=torch.int32, device=dev)
        y, sh, _ = ops.conv2d_dgrad_requant(ed, wd, 1, 1, method=method, relu_mask=pd, unpool=(xd, "first"),
                                            forward_filter=ops.conv_filter_prepare(wd, N, Q, Q), shift_out=so, shift_hint=True)
        assert int(so.cpu()) == sh_ref and torch.equal(y.cpu(), co.maxpool_bwd(pooled, dx, pool_in, 2, 2, 0, "first")), method


@pytest.mark.parametrize("seed", [11, 12, 13])
def test_whole_line_kernels_on_drawn_shapes(dev, seed):
    """The kernels that stage whole 128-byte lines (int32 GEMM with a slow reduction index in both storage forms, TiLinear
    forward and data gradient) on shapes drawn per seed: row counts that leave ragged tiles, one to a dozen chunks of the
    reduction (so the split over workgroups comes out even, uneven and absent), against the oracle's int8mm and
    act_calc / err_calc."""
    import random
    from niti_amd import ops
    from oracle import niti_oracle as po
    rnd = random.Random(seed)
    g = torch.Generator().manual_seed(7000 + seed)
    for _ in range(4):
        m = rnd.choice([1, 7, 31, 33, 64, 100, 128, 200, 257])
        n, k = 128 * rnd.randint(1, 6), 128 * rnd.randint(1, 12)
        _say("whole_line gemm", seed, m, n, k)
        A, B = ri8(g, m, k), ri8(g, k, n)
        ref = po.int8mm(A, B)
        am = ops.new_scalar_u32(dev)
        assert torch.equal(ops.gemm(A.to(dev), B.to(dev), False, False, absmax=am).cpu(), ref)
        assert int(am.cpu()) == po.absmax(ref)
        am = ops.new_scalar_u32(dev)
        assert torch.equal(ops.gemm(B.to(dev), A.to(dev), True, True, absmax=am).cpu(), ref.t().contiguous())   # [n,m] = B^T A^T
        assert int(am.cpu()) == po.absmax(ref)
    for _ in range(3):
        M = rnd.choice([1, 5, 16, 31, 33, 64, 100, 160])
        Fi, O = 128 * rnd.randint(1, 8), 128 * rnd.randint(1, 6)
        _say("whole_line linear", seed, M, Fi, O)
        act, w, err = ri8(g, M, Fi), ri8(g, O, Fi), ri8(g, M, O, lo=-60, hi=60)
        for method in ("round", "sto"):
            ud = torch.randint(0, 1 << 24, (M, Fi), generator=g, dtype=torch.int32)
            uf = torch.randint(0, 1 << 24, (M, O), generator=g, dtype=torch.int32)

            def low(u, acc):
                s = max(po.bitwidth_int(po.absmax(acc)) - 7, 0)
                return u & ((1 << s) - 1) if s > 0 else torch.zeros_like(u)
            sto = method == "sto"
            assert ops.linear_sync_words("dgrad", M, O, Fi) and ops.linear_sync_words("forward", M, O, Fi)
            acc = po.int8mm(err, w)
            ref, sh = po.err_calc(acc, method, "floor", rand=low(ud, acc) if sto else None)
            y, s2, sync = ops.linear_dgrad_requant(err.to(dev), w.to(dev), 7, method, "floor", rand=ud.to(dev) if sto else None)
            assert torch.equal(y.cpu(), ref) and int(s2.cpu()) == sh and int(sync.cpu()[1]) == 0, (M, Fi, O, method)
            acc = po.int8mm(act, w.t().contiguous())
            ref, _ = po.act_calc(acc, 0, method, "floor", rand=low(uf, acc) if sto else None)
            y, _, sync = ops.linear_fwd_requant(act.to(dev), w.to(dev), 7, method, "floor", rand=uf.to(dev) if sto else None)
            assert torch.equal(y.cpu(), ref) and int(sync.cpu()[1]) == 0, (M, Fi, O, method)
