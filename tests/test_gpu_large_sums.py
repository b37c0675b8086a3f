"""GPU parity on the corners the other files leave out: sums beyond 2^24 through the float32 round trip of the backward
kernels, the float32 bit-width rule inside fused kernels with a planted range, and whole training steps at the batch
sizes of the benchmark configurations (fused launches against the two-pass launches, bit for bit)."""
import sys

import pytest
import torch
import torch.nn.functional as F

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


def _extreme(g, *shape):
    """+-127 everywhere in large same-sign blocks, with a sprinkling of 126 / -125 so that sums are odd."""
    t = torch.full(shape, 127, dtype=torch.int8)
    flat = t.view(-1)
    idx = torch.randperm(flat.numel(), generator=g)[: max(flat.numel() // 50, 3)]
    flat[idx] = 126
    return t


@pytest.mark.parametrize("case", [(4, 8, 16, 256), (1, 16, 32, 256), (64, 2, 32, 1024), (16, 4, 16, 512)])   # N, Q, C, K
def test_dgrad_sums_beyond_2_24(dev, case):
    """linear_combination_clamp.h:371-389 applies to the data gradient too (ti_torch.py:405): with |sum| > 2^24 the
    float32 round trip changes values, with and without the requantisation folded in."""
    from niti_amd import ops
    from oracle import c_oracle as co
    from oracle import niti_oracle as po
    N, Q, C, K = case
    _say("dgrad > 2^24", case)
    g = torch.Generator().manual_seed(4100 + Q)
    e = _extreme(g, N, Q, Q, K)
    e[N // 2:] = -e[N // 2:] if N > 1 else e[N // 2:]
    w = _extreme(g, K, 3, 3, C)
    w[:, :, :, 1::2] = -w[:, :, :, 1::2]          # odd input channels negative
    w[0, 1, 1, 0] = 1
    acc = co.conv_dgrad(e, w, Q, Q, 1, 1)
    assert int(acc.abs().max()) > 2 ** 24 and int(acc.to(torch.int64).abs().max()) < 2 ** 31
    rt = po.f32_roundtrip(acc)
    assert not torch.equal(rt, acc)
    ed, wd = e.to(dev), w.to(dev)
    assert torch.equal(ops.conv2d_dgrad(ed, wd, 1, 1, f32_epilogue=True).cpu(), rt)
    assert torch.equal(ops.conv2d_dgrad(ed, wd, 1, 1, f32_epilogue=False).cpu(), acc)
    if ops.conv_requant_sync_words(N, Q, Q, C, K, dgrad=True):
        for f32, src in ((True, rt), (False, acc)):
            for method in ("round", "psto"):
                ref, sh_ref = po.err_calc(src, method)
                y, sh, sync = ops.conv2d_dgrad_requant(ed, wd, 1, 1, f32_epilogue=f32, method=method)
                sync = sync.cpu()
                assert int(sync[1]) == 0 and int(sync[0]) == po.absmax(src), (f32, method)
                assert int(sh.cpu()) == sh_ref and torch.equal(y.cpu(), ref), (f32, method)
                fwd_copy = ops.conv_filter_prepare(wd, N, Q, Q)
                y, sh, _ = ops.conv2d_dgrad_requant(ed, wd, 1, 1, f32_epilogue=f32, method=method, forward_filter=fwd_copy)
                assert int(sh.cpu()) == sh_ref and torch.equal(y.cpu(), ref), (f32, method, "forward copy")


def test_fprop_requant_on_2x2_maps_beyond_2_24(dev):
    from niti_amd import ops
    from oracle import niti_oracle as po
    N, Q, C, K = 64, 2, 1024, 48
    _say("fprop 2x2 > 2^24")
    g = torch.Generator().manual_seed(4200)
    x, w = _extreme(g, N, Q, Q, C), _extreme(g, K, 3, 3, C)
    w[K // 2:] = -w[K // 2:]
    w[1, 1, 1, 3] = 2
    acc = po.conv2d_fprop_i32(x, w)
    assert int(acc.abs().max()) > 2 ** 24
    for f32 in (True, False):
        src = po.f32_roundtrip(acc) if f32 else acc
        ref, _ = po.act_calc(src, 0, "round")
        y, sh, sync = ops.conv2d_fprop_requant(x.to(dev), w.to(dev), f32_epilogue=f32)
        assert int(sync.cpu()[1]) == 0 and int(sync.cpu()[0]) == po.absmax(src)
        assert torch.equal(y.cpu(), ref), f32


@pytest.mark.parametrize("case", [(8, 16, 16, 16), (2, 32, 16, 32), (32, 8, 32, 16), (128, 4, 16, 16), (512, 2, 16, 32)])   # N, Q, C, K
def test_wgrad_sums_beyond_2_24(dev, case):
    """The weight gradient is where sums approach 2^24 in real training (ti_torch.py:430-432 runs it through the same
    CUTLASS epilogue): constant +-127 operands over more than 1041 pixels, round trip on and off, two-pass and
    single-pass forms."""
    from niti_amd import ops
    from oracle import c_oracle as co
    from oracle import niti_oracle as po
    N, Q, C, K = case
    _say("wgrad > 2^24", case)
    g = torch.Generator().manual_seed(4300 + Q)
    act, err = _extreme(g, N, Q, Q, C), _extreme(g, N, Q, Q, K)
    err[..., 1::2] = -err[..., 1::2]
    act[0, 0, 0, 0] = 3
    w = ri8(g, K, 3, 3, C)
    dw = co.conv_wgrad(act, err, 3, 3, 1, 1)
    assert int(dw.abs().max()) > 2 ** 24
    rt = po.f32_roundtrip(dw)
    assert not torch.equal(rt, dw)
    ad, ed = act.to(dev), err.to(dev)
    assert torch.equal(ops.conv2d_wgrad(ad, ed, 3, 3, 1, 1, f32_epilogue=True).cpu(), rt)
    assert torch.equal(ops.conv2d_wgrad(ad, ed, 3, 3, 1, 1, f32_epilogue=False).cpu(), dw)
    for f32, src in ((True, rt), (False, dw)):
        for method, mu in (("psto", 5), ("round", 4)):
            g8_ref, sh_ref = po.grad_calc(src, mu, method)
            w_ref = po.weight_update(w, g8_ref)
            wd = w.to(dev).clone()
            g8, dwo, sh, sync = ops.conv2d_wgrad_update(ad, ed, wd, f32_epilogue=f32, mu=mu, method=method, want_grad=True, want_dw=True)
            sync = sync.cpu()
            assert int(sync[1]) == 0 and int(sync[0]) == po.absmax(src), (f32, method)
            assert torch.equal(dwo.cpu(), src) and int(sh.cpu()) == sh_ref, (f32, method)
            assert torch.equal(g8.cpu(), g8_ref) and torch.equal(wd.cpu(), w_ref), (f32, method)


@pytest.mark.parametrize("case", [(12, 16, 128, 128), (48, 8, 64, 256)])   # N, Q, C, K
def test_wgrad_one_launch_partial_sums_beyond_2_23(dev, case, monkeypatch):
    """The one-launch weight gradient hands its partial sums over as 24-bit values unless a workgroup's own sums need
    more: few, long workgroups (NITI_WGRAD_BLOCKS) and constant +-127 operands in the first input-channel tile of the
    first pixel range make exactly one kind of workgroup write 32-bit sums, next to others of the same slice and of the
    same tile that do not."""
    from niti_amd import ops
    from oracle import c_oracle as co
    from oracle import niti_oracle as po
    N, Q, C, K = case
    _say("wgrad one launch, partial sums > 2^23", case)
    monkeypatch.setenv("NITI_WGRAD_BLOCKS", "16")
    g = torch.Generator().manual_seed(4400 + Q)
    act, err, w = ri8(g, N, Q, Q, C, lo=-20, hi=20), ri8(g, N, Q, Q, K, lo=-20, hi=20), ri8(g, K, 3, 3, C)
    n_hot = N // 4                      # the first of at least four pixel ranges
    act[:n_hot, :, :, :32] = 127
    err[:n_hot] = 127
    err[:n_hot, :, :, 1::2] = -127
    dw = co.conv_wgrad(act, err, 3, 3, 1, 1)
    assert int(dw.abs().max()) > 2 ** 23 and int(dw[:, :, :, 32:].abs().max()) < 2 ** 22
    for method, mu in (("psto", 5), ("round", 4)):
        g8_ref, sh_ref = po.grad_calc(dw, mu, method)
        w_ref = po.weight_update(w, g8_ref)
        wd = w.to(dev).clone()
        g8, dwo, sh, sync = ops.conv2d_wgrad_update(act.to(dev), err.to(dev), wd, mu=mu, method=method, want_grad=True, want_dw=True)
        sync = sync.cpu()
        assert int(sync[1]) == 0 and int(sync[0]) == po.absmax(dw), method
        assert torch.equal(dwo.cpu(), dw) and int(sh.cpu()) == sh_ref, method
        assert torch.equal(g8.cpu(), g8_ref) and torch.equal(wd.cpu(), w_ref), method


PLANT = 2 ** 22 + 2     # bit width 23 as an integer, 22 under the reference's float32 log2 (ti_torch.py:366-377)


def _planted_terms(n):
    """n (a, b) pairs with sum a*b == 2^22 + 2: 260 x 127*127 + 127*6 + 4*1, the rest zero."""
    a = [127] * 260 + [127, 4] + [0] * (n - 262)
    b = [127] * 260 + [6, 1] + [0] * (n - 262)
    assert sum(x * y for x, y in zip(a, b)) == PLANT
    return torch.tensor(a, dtype=torch.int8), torch.tensor(b, dtype=torch.int8)


def test_f32_bitwidth_rule_inside_the_fused_convolution(dev):
    """A tensor whose largest sum is exactly 2^22 + 2: shift 16 with the exact rule, 15 with the float32 rule."""
    from niti_amd import ops
    from oracle import niti_oracle as po
    _say("bw_mode f32, fused conv")
    g = torch.Generator().manual_seed(4400)
    N, Q, C, K = 4, 8, 32, 16
    a, b = _planted_terms(9 * C)
    x = torch.zeros((N, Q, Q, C), dtype=torch.int8)
    x[1, 2:5, 3:6, :] = a.view(3, 3, C)
    w = ri8(g, K, 3, 3, C, lo=-3, hi=3)
    w[5] = b.view(3, 3, C)
    acc = po.conv2d_fprop_i32(x, w)
    assert po.absmax(acc) == PLANT and int(acc[1, 3, 4, 5]) == PLANT
    assert po.bitwidth_int(PLANT) == 23 and po.bitwidth_f32(PLANT) == 22 and po.bitwidth_f32_model(PLANT) == 22
    for bw_mode, shift in (("int", 16), ("f32", 15)):
        for method in ("round", "psto"):
            ref, e_ref = po.act_calc(acc, 0, method, "floor", bw_mode=bw_mode)
            assert e_ref == shift
            y, sh, sync = ops.conv2d_fprop_requant(x.to(dev), w.to(dev), method=method, bw_mode=bw_mode)
            assert int(sh.cpu()) == shift and int(sync.cpu()[0]) == PLANT and torch.equal(y.cpu(), ref), (bw_mode, method)


def test_f32_bitwidth_rule_inside_the_fused_weight_gradient(dev):
    from niti_amd import ops
    from oracle import c_oracle as co
    from oracle import niti_oracle as po
    _say("bw_mode f32, fused wgrad")
    g = torch.Generator().manual_seed(4500)
    N, Q, C, K = 8, 8, 16, 16
    a, b = _planted_terms(N * Q * Q)
    act = torch.zeros((N, Q, Q, C), dtype=torch.int8)
    err = ri8(g, N, Q, Q, K, lo=-2, hi=2)
    act[..., 3] = a.view(N, Q, Q)
    err[..., 7] = b.view(N, Q, Q)
    w = ri8(g, K, 3, 3, C)
    dw = co.conv_wgrad(act, err, 3, 3, 1, 1)
    assert po.absmax(dw) == PLANT and int(dw[7, 1, 1, 3]) == PLANT
    for bw_mode, shift in (("int", 18), ("f32", 17)):
        for method in ("psto", "round"):
            g8_ref, sh_ref = po.grad_calc(dw, 5, method, "floor", bw_mode=bw_mode)
            assert sh_ref == shift
            wd = w.to(dev).clone()
            g8, _, sh, sync = ops.conv2d_wgrad_update(act.to(dev), err.to(dev), wd, mu=5, method=method, bw_mode=bw_mode, want_grad=True)
            assert int(sh.cpu()) == shift and int(sync.cpu()[0]) == PLANT, (bw_mode, method)
            assert torch.equal(g8.cpu(), g8_ref) and torch.equal(wd.cpu(), po.weight_update(w, g8_ref)), (bw_mode, method)


# (7, 256): the reference's default batch (options.py:3); its two 128-channel layers on 32 x 32 maps have more tiles than the
# device holds at once and run the two-launch form inside the step
@pytest.mark.parametrize("depth,N", [(7, 128), (7, 256), (13, 256)])
def test_full_batch_steps_fused_against_two_pass(dev, depth, N):
    """Two training steps at the batch size of the benchmark configurations: the network with every single-launch
    form switched on against the same network on the two-pass launches (int32 results + separate requantisation),
    every activation the layers keep, every error exponent and every weight bit for bit; the first convolution of
    three images against the plain-C statement of the reference."""
    from niti_amd import ops, ti_torch, ti_vgg
    from oracle import c_oracle as co
    from oracle import niti_oracle as po
    _say("full batch", depth, N)
    saved = (ti_torch.FUSE_CONV_REQUANT, ti_torch.TRAINING, ti_torch.GRAD_BITWIDTH)
    try:
        ti_torch.TRAINING, ti_torch.GRAD_BITWIDTH = True, 5
        g = torch.Generator().manual_seed(4600 + depth)
        proto = ti_vgg.TiVGG_cifar(depth)
        weights = [ri8(g, *l.weight.shape) for l in proto.forward_layers if hasattr(l, "weight")]
        x = ri8(g, N, 32, 32, 3)
        target = torch.randint(0, 10, (N,), generator=g)
        loss_rand = torch.randint(0, 16, (N, 10), generator=g, dtype=torch.int32)
        fc_in = weights[-1].shape[1]
        masks = [torch.randint(0, 2, (fc_in,), generator=g, dtype=torch.int8) for _ in range(2)]

        def run(fused):
            ti_torch.FUSE_CONV_REQUANT = fused
            net = ti_vgg.TiVGG_cifar(depth, fuse=fused)
            ws = iter(weights)
            for l in net.forward_layers:
                if hasattr(l, "weight"):
                    l.weight, l.weight_exp = next(ws).to(dev).clone(), torch.tensor(-8.0)
            drop = [l for l in net.forward_layers if isinstance(l, ti_torch.TiDropout)][0]
            orig = drop.forward
            trace = []
            for step in range(2):
                drop.forward = lambda inp, m=masks[step]: orig(inp, m.to(dev))
                y, e = net.forward_int8(x.to(dev), 0)
                trace.append(("logits", y.cpu().clone(), int(e.item()) if isinstance(e, torch.Tensor) else int(e)))
                net.backward(target.to(dev), loss_rand.to(dev))
                torch.cuda.synchronize()
                assert not ops.sync_arena.timed_out(dev) and not ops.sync_timeouts(dev)
                for i, l in enumerate(net.forward_layers):
                    if hasattr(l, "weight"):
                        ge = l.grad_exp
                        trace.append(("w%d" % i, l.weight.cpu().clone(), int(ge.item()) if isinstance(ge, torch.Tensor) else int(ge)))
                        ee = getattr(l, "err_exp", None)
                        if ee is not None:
                            trace.append(("err_exp%d" % i, None, int(ee.item()) if isinstance(ee, torch.Tensor) else int(ee)))
            return trace

        fused, plain = run(True), run(False)
        assert len(fused) == len(plain)
        for (na, ta, ea), (nb, tb, eb) in zip(fused, plain):
            assert na == nb and ea == eb, (na, ea, eb)
            if ta is not None and tb is not None:
                assert torch.equal(ta, tb), na
        # the first convolution + act_calc + ReLU of three images against the plain-C statement
        w1 = F.pad(weights[0], (0, 13))
        x3 = F.pad(x[:3], (0, 13))
        acc = po.f32_roundtrip(co.conv_fprop(x3, w1, 1, 1))
        full = ops.conv2d_fprop(F.pad(x, (0, 13)).to(dev), w1.to(dev), 1, 1, f32_epilogue=True)
        assert torch.equal(full[:3].cpu(), acc)
        y8, sh, _ = ops.conv2d_fprop_requant(F.pad(x, (0, 13)).to(dev), w1.to(dev), f32_epilogue=True, relu=True)
        shift = int(sh.cpu())
        want = torch.clamp(po.RoundShift(acc, shift), min=0) if shift > 0 else None
        assert want is not None and torch.equal(y8[:3].cpu(), want)
    finally:
        ti_torch.FUSE_CONV_REQUANT, ti_torch.TRAINING, ti_torch.GRAD_BITWIDTH = saved
