"""The classifier head (dropout + TiLinear + TiLoss in two launches) and the kernels' own random draws, against the
CPU oracle and a numpy statement of Philox4x32-10."""
import sys

import numpy as np
import pytest
import torch


def _say(*a):
    print("[case]", *a, flush=True)
    sys.stdout.flush()


def ri8(g, *shape, lo=-127, hi=127):
    return torch.randint(lo, hi + 1, shape, generator=g, dtype=torch.int8)


# ---- Philox4x32-10 (Salmon et al., SC'11) in numpy -------------------------------------------------------------
def philox4x32_10(ctr, key):
    """ctr: uint32 [n, 4], key: (k0, k1) -> uint32 [n, 4]."""
    c = [ctr[:, i].astype(np.uint64) for i in range(4)]
    k0, k1 = np.uint64(key[0]), np.uint64(key[1])
    m32 = np.uint64(0xFFFFFFFF)
    for _ in range(10):
        p0 = np.uint64(0xD2511F53) * c[0]
        p1 = np.uint64(0xCD9E8D57) * c[2]
        c = [(p1 >> np.uint64(32)) ^ c[1] ^ k0, p1 & m32, (p0 >> np.uint64(32)) ^ c[3] ^ k1, p0 & m32]
        k0 = (k0 + np.uint64(0x9E3779B9)) & m32
        k1 = (k1 + np.uint64(0xBB67AE85)) & m32
    return np.stack(c, axis=1).astype(np.uint32)


def stream_words(key, step, stream, n):
    """The first n words of a stream as the kernels define them: word i = output (i & 3) of counter {i >> 2, stream, step, 0}."""
    q = (n + 3) // 4
    ctr = np.zeros((q, 4), dtype=np.uint32)
    ctr[:, 0] = np.arange(q, dtype=np.uint32)
    ctr[:, 1] = stream
    ctr[:, 2] = step
    return philox4x32_10(ctr, key).reshape(-1)[:n]


def test_philox_known_answers():
    """The numpy statement against the known-answer vectors published with the generator (Random123 kat_vectors,
    philox4x32 with 10 rounds)."""
    kat = [
        ((0, 0, 0, 0), (0, 0), (0x6627e8d5, 0xe169c58d, 0xbc57ac4c, 0x9b00dbd8)),
        ((0xffffffff,) * 4, (0xffffffff, 0xffffffff), (0x408f276d, 0x41c83b0e, 0xa20bc7c6, 0x6d5451fd)),
        ((0x243f6a88, 0x85a308d3, 0x13198a2e, 0x03707344), (0xa4093822, 0x299f31d0), (0xd16cfe09, 0x94fdcceb, 0x5001e420, 0x24126ea1)),
    ]
    for ctr, key, want in kat:
        got = philox4x32_10(np.array([ctr], dtype=np.uint32), key)[0]
        assert tuple(int(v) for v in got) == want


@pytest.fixture(scope="module")
def dev():
    assert torch.cuda.is_available(), "GPU tests need a GPU"
    return torch.device("cuda:0")


def _u32(t):
    return t.cpu().numpy().view(np.uint32)


KEY = 0x9E3779B97F4A7C15


@pytest.mark.gpu
def test_rng_words_and_step(dev):
    from niti_amd import ops
    from oracle import niti_oracle as po
    _say("rng words")
    rng = ops.rng_state(dev, KEY)
    key = (KEY & 0xFFFFFFFF, KEY >> 32)
    assert [int(v) for v in _u32(rng)] == [key[0], key[1], 0, 0]
    for stream, sid in (("dropout", 1), ("loss", 2)):
        for n in (1, 4, 5, 1000, 8192):
            assert np.array_equal(_u32(ops.rng_words(rng, stream, n)), stream_words(key, 0, sid, n))
    assert [int(v) for v in _u32(rng)] == [key[0], key[1], 0, 0]          # looking does not advance
    # a launch that draws advances the step by one, whatever its grid
    g = torch.Generator().manual_seed(5)
    for step, (n, classes) in enumerate([(128, 10), (3, 10), (256, 16), (7, 5)]):
        out = ri8(g, n, classes)
        tgt = torch.randint(0, classes, (n,), generator=g)
        e = torch.tensor([-3], dtype=torch.int32)
        words = stream_words(key, step, 2, n * classes)
        assert np.array_equal(_u32(ops.rng_words(rng, "loss", n * classes)), words)
        got = ops.loss_grad_rng(out.to(dev), e.to(dev), tgt.to(dev), rng)
        ref = po.ti_loss(out, -3, tgt, torch.from_numpy((words & 15).astype(np.int32)).view(n, classes))[0]
        assert torch.equal(got.cpu(), ref)
        assert [int(v) for v in _u32(rng)] == [key[0], key[1], step + 1, 0]


# F a multiple of 128 takes the forward kernel that stages whole lines through LDS (unless the mask of 32768 features
# leaves no room for its stages): 384 = wavefronts with two, one and no line; 128 = a single line
HEAD_CASES = [(128, 10, 8192), (256, 10, 512), (20, 10, 512), (16, 7, 64), (33, 16, 1088), (1, 1, 64), (24, 10, 32768), (37, 10, 384),
              (48, 16, 128)]


@pytest.mark.gpu
@pytest.mark.parametrize("case", HEAD_CASES)
@pytest.mark.parametrize("div_mode", ["floor", "trunc"])
def test_head_forward(dev, case, div_mode):
    """niti_head_i8_forward against TiDropout.forward + TiLinear.forward + TiLoss.forward of the oracle."""
    from niti_amd import ops
    from oracle import niti_oracle as po
    M, O, F = case
    _say("head_forward", case, div_mode)
    g = torch.Generator().manual_seed(7000 + M + O + F)
    act, w = ri8(g, M, F), ri8(g, O, F, lo=-20, hi=20)
    tgt = torch.randint(0, O, (M,), generator=g)
    ea = torch.tensor([-6], dtype=torch.int32, device=dev)
    eb = torch.tensor([-9], dtype=torch.int32, device=dev)
    key = (KEY & 0xFFFFFFFF, KEY >> 32)
    for method in ("round", "psto"):
        for dropout in (None, "given", "draw"):
            rng = ops.rng_state(dev, KEY)
            if dropout == "given":
                mask = torch.randint(0, 2, (F,), generator=g, dtype=torch.int8)
                mask_d = mask.to(dev)
            elif dropout == "draw":
                mask = torch.from_numpy((stream_words(key, 0, 1, F) & 1).astype(np.int8))
                mask_d = None
            else:
                mask, mask_d = torch.ones(F, dtype=torch.int8), None
            bias = 0 if dropout is None else 1
            acc = po.int8mm(act * mask, w.t().contiguous())
            ref, sh_ref = po.act_calc(acc, 0, method, div_mode)
            e_ref = sh_ref - 15 + bias
            for with_loss in (None, "given", "draw"):
                eo = torch.zeros(1, dtype=torch.int32, device=dev)
                rng = ops.rng_state(dev, KEY)
                lr = torch.randint(0, 2 ** 31 - 1, (M, O), generator=g, dtype=torch.int32) if with_loss == "given" else None
                y, mk, lg, sh, sync = ops.head_forward(
                    act.to(dev), w.to(dev), 7, method, div_mode, dropout=dropout, drop_mask=mask_d, rng=rng, exp_bias=bias,
                    target=tgt.to(dev) if with_loss else None, loss_rand=lr.to(dev) if lr is not None else None,
                    exp_a=ea, exp_b=eb, exp_out=eo)
                sync = sync.cpu()
                assert int(sync[0]) == po.absmax(acc) and int(sync[1]) == 0
                assert torch.equal(y.cpu(), ref) and int(sh.cpu()) == sh_ref and int(eo.cpu()) == e_ref
                if dropout == "draw":
                    assert torch.equal(mk.cpu(), mask)
                if with_loss:
                    r = lr if lr is not None else torch.from_numpy((stream_words(key, 0, 2, M * O) & 15).astype(np.int32)).view(M, O)
                    assert torch.equal(lg.cpu(), po.ti_loss(ref, e_ref, tgt, r & 15, div_mode)[0])
                else:
                    assert lg is None
                drew = dropout == "draw" or with_loss == "draw"
                assert int(_u32(rng)[2]) == (1 if drew else 0) and int(_u32(rng)[3]) == 0


@pytest.mark.gpu
def test_head_forward_loss_branches(dev):
    """Both branches of the loss (out_exp > -7 and the quadratic form below) through the fused forward."""
    from niti_amd import ops
    from oracle import niti_oracle as po
    g = torch.Generator().manual_seed(99)
    M, O, F = 64, 10, 256
    act, w = ri8(g, M, F), ri8(g, O, F)
    tgt = torch.randint(0, O, (M,), generator=g)
    for e_in in (-30, -14, -10, -3, 0):
        _say("head loss branch", e_in)
        ea = torch.tensor([e_in], dtype=torch.int32, device=dev)
        eo = torch.zeros(1, dtype=torch.int32, device=dev)
        lr = torch.randint(0, 16, (M, O), generator=g, dtype=torch.int32)
        y, _, lg, sh, _ = ops.head_forward(act.to(dev), w.to(dev), target=tgt.to(dev), loss_rand=lr.to(dev), exp_a=ea, exp_out=eo)
        e = int(eo.cpu())
        assert e == int(sh.cpu()) + e_in
        assert torch.equal(lg.cpu(), po.ti_loss(y.cpu(), e, tgt, lr)[0])
        sep = ops.loss_grad(y, eo, tgt.to(dev), lr.to(dev))
        assert torch.equal(lg, sep)


@pytest.mark.gpu
@pytest.mark.parametrize("case", [(128, 10, 8192), (256, 10, 512), (20, 10, 512), (16, 7, 64), (33, 16, 1088), (1, 1, 64), (200, 3, 128), (24, 10, 32768)])
@pytest.mark.parametrize("div_mode", ["floor", "trunc"])
def test_head_backward(dev, case, div_mode):
    """niti_head_i8_backward against TiLinear.backward + TiDropout.backward of the oracle."""
    from niti_amd import ops
    from oracle import niti_oracle as po
    M, O, F = case
    _say("head_backward", case, div_mode)
    g = torch.Generator().manual_seed(7100 + M + O + F)
    act, w, err = ri8(g, M, F), ri8(g, O, F), ri8(g, M, O, lo=-40, hi=40)
    e_err = torch.tensor([0], dtype=torch.int32, device=dev)
    e_w = torch.tensor([-7], dtype=torch.int32, device=dev)
    e_act = torch.tensor([-4], dtype=torch.int32, device=dev)
    for use_mask in (False, True):
        mask = torch.randint(0, 2, (F,), generator=g, dtype=torch.int8) if use_mask else torch.ones(F, dtype=torch.int8)
        dacc = po.int8mm(err, w)
        gacc = po.int8mm(err.t().contiguous(), act * mask)
        for em, gm, mu in (("psto", "psto", 5), ("round", "psto", 3), ("psto", "round", 4)):
            dref, dsh = po.err_calc(dacc, em, div_mode)
            g8_ref, gsh = po.grad_calc(gacc, mu, gm, div_mode)
            w_ref = po.weight_update(w, g8_ref)
            wd = w.to(dev).clone()
            eo = torch.zeros(2, dtype=torch.int32, device=dev)
            dx, g8, s_d, s_w, sync = ops.head_backward(
                err.to(dev), act.to(dev), wd, 7, em, mu, gm, div_mode, drop_mask=mask.to(dev) if use_mask else None,
                want_grad=True, exp_err=e_err, exp_w=e_w, exp_act=e_act, exp_act_bias=1 if use_mask else 0,
                err_exp_out=eo[0:1], grad_exp_out=eo[1:2])
            sync = sync.cpu()
            assert int(sync[0]) == po.absmax(dacc) and int(sync[2]) == po.absmax(gacc) and int(sync[1]) == 0
            assert int(s_d.cpu()) == dsh and int(s_w.cpu()) == gsh
            assert torch.equal(dx.cpu(), dref * mask)
            assert torch.equal(g8.cpu(), g8_ref) and torch.equal(wd.cpu(), w_ref)
            assert int(eo.cpu()[0]) == dsh - 7 and int(eo.cpu()[1]) == gsh + dsh - 7 - 4 + (1 if use_mask else 0)
    assert ops.head_sync_words("backward", 257, 10, 512) == 0 and ops.head_sync_words("backward", 128, 17, 512) == 0
    assert ops.head_sync_words("backward", 128, 10, 96) == 0 and ops.head_sync_words("forward", 128, 17, 512) == 0


@pytest.mark.gpu
@pytest.mark.parametrize("case", [(128, 10, 4, 4, 512), (37, 7, 2, 3, 64), (256, 16, 1, 1, 128)])   # M, O, P, Q, C
@pytest.mark.parametrize("ties", ["first", "all"])
def test_head_backward_unpool(dev, case, ties):
    """niti_head_i8_backward_unpool: the classifier's backward launch followed through the 2 x 2 max-pool in front of it,
    against niti_head_i8_backward's data gradient routed by the oracle's max-pool backward (+ the ReLU mask).  The pool's
    input has few distinct values: many windows with several equal maxima, many non-positive maxima."""
    from niti_amd import ops
    from oracle import niti_oracle as po
    M, O, P, Q, C = case
    F = P * Q * C
    _say("head_backward_unpool", case, ties)
    g = torch.Generator().manual_seed(7300 + M + O + F)
    x = ri8(g, M, 2 * P, 2 * Q, C, lo=-3, hi=5)
    y = po.maxpool_fwd(x)
    act = y.reshape(M, F).contiguous()
    w, err = ri8(g, O, F), ri8(g, M, O, lo=-40, hi=40)
    mask = torch.randint(0, 2, (F,), generator=g, dtype=torch.int8)
    for relu in (False, True):
        for use_mask in (False, True):
            wd = w.to(dev).clone()
            dx, _, _, _, sync, routed = ops.head_backward(err.to(dev), act.to(dev), wd, 7, "round", 5, "psto", "floor",
                                                          drop_mask=mask.to(dev) if use_mask else None,
                                                          unpool=(x.to(dev), ties, relu))
            wd2 = w.to(dev).clone()
            dx_plain, _, _, _, _ = ops.head_backward(err.to(dev), act.to(dev), wd2, 7, "round", 5, "psto", "floor",
                                                     drop_mask=mask.to(dev) if use_mask else None)
            assert int(sync.cpu()[1]) == 0
            assert torch.equal(dx.cpu(), dx_plain.cpu()) and torch.equal(wd.cpu(), wd2.cpu())
            ref = po.maxpool_bwd(y, dx_plain.cpu().reshape(M, P, Q, C), x, ties=ties)
            if relu:
                ref = torch.where(x > 0, ref, torch.zeros_like(ref))
            assert torch.equal(routed.cpu(), ref.to(torch.int8)), (relu, use_mask)
