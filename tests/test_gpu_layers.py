"""Layer- and step-level GPU parity: niti_amd.ti_torch / ti_net / ti_vgg against the CPU oracle
model on the same seeded int8 weights, inputs, labels and injected random draws.  Every int8
tensor, every exponent and every updated weight must match exactly."""
import sys

import pytest
import torch

pytestmark = pytest.mark.gpu


def _say(*a):
    print("[case]", *a, flush=True)


def ri8(g, *shape, lo=-127, hi=127):
    return torch.randint(lo, hi + 1, shape, generator=g, dtype=torch.int8)


def laplace_i8(g, shape, b=16.0):
    u = torch.rand(shape, generator=g, dtype=torch.float64) - 0.5
    v = -b * torch.sign(u) * torch.log1p(-2 * u.abs())
    return torch.clamp(torch.round(v), -127, 127).to(torch.int8)


@pytest.fixture()
def tt():
    from niti_amd import ti_torch
    saved = {k: getattr(ti_torch, k) for k in ("ACT_ROUND_METHOD", "ERROR_ROUND_METHOD", "GRAD_ROUND_METHOD",
                                               "GRAD_BITWIDTH", "DIV_MODE", "BW_MODE", "F32_EPILOGUE", "POOL_TIES", "TRAINING")}
    yield ti_torch
    for k, v in saved.items():
        setattr(ti_torch, k, v)


def _ei(e):
    return int(e.item()) if isinstance(e, torch.Tensor) else int(e)


@pytest.mark.parametrize("div_mode", ["floor", "trunc"])
@pytest.mark.parametrize("first", [False, True])
def test_conv_layer_fwd_bwd(tt, div_mode, first):
    from oracle import niti_model_oracle as mo
    dev = torch.device("cuda:0")
    g = torch.Generator().manual_seed(1000 + first)
    N, H, C, K = 8, 16, (3 if first else 32), 64
    _say("conv layer", div_mode, first)
    tt.DIV_MODE = div_mode
    w, x = ri8(g, K, 3, 3, C), ri8(g, N, H, H, C)
    err = laplace_i8(g, (N, H, H, K))
    cfg = mo.Cfg(div_mode=div_mode)
    o = mo.OConv2d(w, -9, first_layer=first)
    yo, eo = o.forward((x, -3), cfg)
    ro = o.backward((err, -5), cfg)
    layer = tt.TiConv2d(C, K, first_layer=first)
    layer.weight = w.to(dev)
    layer.weight_exp = torch.tensor(-9.0)
    layer.keep_grad = True
    y, e = layer.forward((x.to(dev), -3))
    assert torch.equal(y.cpu(), yo) and _ei(e) == eo
    r = layer.backward((err.to(dev), -5))
    assert torch.equal(layer.grad.cpu(), o.grad) and _ei(layer.grad_shift) == o.grad_shift
    assert torch.equal(layer.weight.cpu(), o.weight)
    assert _ei(layer.grad_exp) == o.grad_exp
    if first:
        assert r is None and ro is None
    else:
        assert torch.equal(r[0].cpu(), ro[0]) and _ei(r[1]) == ro[1]


def test_conv_layer_sto_runs_in_the_single_launch_kernels(tt):
    """ACT / ERROR_ROUND_METHOD = StoShift (selectable in the reference, ti_torch.py:460-463): the layer hands the random
    integers to the convolution launches instead of falling back to int32 results + a requantisation pass."""
    from oracle import niti_model_oracle as mo
    from oracle import niti_oracle as po
    from niti_amd import ops
    dev = torch.device("cuda:0")
    g = torch.Generator().manual_seed(1050)
    N, H, C, K = 8, 16, 32, 64
    _say("conv layer, StoShift")
    tt.ACT_ROUND_METHOD = tt.ERROR_ROUND_METHOD = tt.StoShift
    w, x, err = ri8(g, K, 3, 3, C), ri8(g, N, H, H, C), laplace_i8(g, (N, H, H, K))
    rf = torch.randint(0, 2 ** 20, (N, H, H, K), generator=g, dtype=torch.int32)
    rb = torch.randint(0, 2 ** 20, (N, H, H, C), generator=g, dtype=torch.int32)
    cfg = mo.Cfg(act="sto", err="sto")
    o = mo.OConv2d(w, -9)
    # the oracle's StoShift compares with the integer as it is: hand it the low `shift` bits the kernels use
    sf = max(po.RangeEstimate(po.conv2d_int8(x, w)) - 7, 1)
    sb = max(po.RangeEstimate(po.conv2d_dgrad_i32(err, w)) - 7, 1)
    yo, eo = o.forward((x, -3), cfg, rf & (2 ** sf - 1))
    ro = o.backward((err, -5), cfg, rb & (2 ** sb - 1))
    layer = tt.TiConv2d(C, K)
    layer.weight, layer.weight_exp = w.to(dev), torch.tensor(-9.0)
    calls = []
    real = ops.requant
    ops.requant = lambda *a, **k: calls.append(1) or real(*a, **k)
    try:
        y, e = layer.forward((x.to(dev), -3), rf.to(dev))
        r = layer.backward((err.to(dev), -5), rb.to(dev))
    finally:
        ops.requant = real
    assert not calls
    assert torch.equal(y.cpu(), yo) and _ei(e) == eo
    assert torch.equal(r[0].cpu(), ro[0]) and _ei(r[1]) == ro[1]
    assert torch.equal(layer.weight.cpu(), o.weight) and _ei(layer.grad_exp) == o.grad_exp
    # random integers drawn by the layer itself: between the results of the two extreme draws
    y2, _ = layer.forward((x.to(dev), -3))
    acc2 = po.conv2d_int8(x, o.weight)
    s2 = max(po.RangeEstimate(acc2) - 7, 1)
    a, _ = po.act_calc(acc2, 0, "sto", "floor", torch.zeros_like(acc2))
    b, _ = po.act_calc(acc2, 0, "sto", "floor", torch.full_like(acc2, 2 ** s2 - 1))
    y2 = y2.cpu().to(torch.int16)
    assert bool(((y2 >= torch.minimum(a, b).to(torch.int16)) & (y2 <= torch.maximum(a, b).to(torch.int16))).all())


def test_conv_layer_on_a_grid_larger_than_the_device(tt):
    """A layer whose convolutions have more workgroups than the device holds at once (136 images of 32 x 32, 80 -> 144
    channels: 1088 and 544 tiles): forward and data gradient run as two launches that do not wait.  Two training
    steps in a row, the second one predicting its shifts from the first."""
    from oracle import niti_model_oracle as mo
    dev = torch.device("cuda:0")
    g = torch.Generator().manual_seed(1100)
    N, H, C, K = 136, 32, 80, 144
    _say("conv layer, oversubscribed grid")
    w, x = ri8(g, K, 3, 3, C), ri8(g, N, H, H, C, lo=-60, hi=60)   # 139264 pixels: keeps the weight gradient's bound below 2^31
    cfg = mo.Cfg()
    o = mo.OConv2d(w, -9)
    layer = tt.TiConv2d(C, K)
    layer.weight = w.to(dev)
    layer.weight_exp = torch.tensor(-9.0)
    layer.relu_below = True
    for step in range(2):
        err = laplace_i8(g, (N, H, H, K), b=4.0 * (step + 1))
        yo, eo = o.forward((x, -3), cfg)
        ro = o.backward((err, -5), cfg)
        y, e = layer.forward((x.to(dev), -3))
        assert torch.equal(y.cpu(), yo) and _ei(e) == eo
        r = layer.backward((err.to(dev), -5))
        assert torch.equal(layer.weight.cpu(), o.weight) and _ei(layer.grad_exp) == o.grad_exp
        assert torch.equal(r[0].cpu(), torch.where(x > 0, ro[0], torch.zeros_like(ro[0]))) and _ei(r[1]) == ro[1]
    from niti_amd import ops
    assert not ops.sync_arena.timed_out(dev)


# sizes: a ragged small one, the fully connected configuration of the benchmark list (activations 128 x 8192,
# weights 1024 x 8192, stochastic rounding from seeded random integers), and the classifier (few output features)
@pytest.mark.parametrize("shape", [(32, 512, 48), (128, 8192, 1024), (128, 8192, 10)])
@pytest.mark.parametrize("methods", [("round", "round", "psto"), ("sto", "sto", "sto"), ("psto", "psto", "round")])
def test_linear_layer_fwd_bwd(tt, methods, shape):
    from oracle import niti_model_oracle as mo
    from oracle import niti_oracle as po
    dev = torch.device("cuda:0")
    g = torch.Generator().manual_seed(1100)
    m, kin, nout = shape
    if shape[2] == 1024 and methods[0] != "sto":
        pytest.skip("the large configuration runs with the rounding it names")
    _say("linear layer", methods, shape)
    fn = {"round": tt.RoundShift, "sto": tt.StoShift, "psto": tt.PstoShift}
    tt.ACT_ROUND_METHOD, tt.ERROR_ROUND_METHOD, tt.GRAD_ROUND_METHOD = (fn[x] for x in methods)
    w, x, err = ri8(g, nout, kin), ri8(g, m, kin), ri8(g, m, nout)
    # random integers for the three stochastic roundings, drawn for the shifts the oracle will see
    acc_f, acc_b, acc_g = po.int8mm(x, w.t().contiguous()), po.int8mm(err, w), po.int8mm(err.t().contiguous(), x)
    def draw(acc, tgt):
        s = max(po.RangeEstimate(acc) - tgt, 1)
        return torch.randint(0, 2 ** s, acc.shape, generator=g, dtype=torch.int32)
    rf, rb, rg = draw(acc_f, 7), draw(acc_b, 7), draw(acc_g, 5)
    cfg = mo.Cfg(*methods)
    o = mo.OLinear(w, -8)
    yo, eo = o.forward((x, 1), cfg, rf)
    ro = o.backward((err, -2), cfg, rb, rg)
    layer = tt.TiLinear(kin, nout)
    layer.weight, layer.weight_exp, layer.keep_grad = w.to(dev), torch.tensor(-8.0), True
    from niti_amd import ops
    gemm_calls = []
    real_gemm = ops.gemm
    if nout == 1024:
        # the wide layer runs as three launches that read the operands as stored: no GEMM into int32, no re-layout
        ops.gemm = lambda *a, **k: gemm_calls.append(1) or real_gemm(*a, **k)
    try:
        _run_linear_layer(tt, layer, x, err, rf, rb, rg, yo, eo, ro, o, dev)
    finally:
        ops.gemm = real_gemm
    assert not gemm_calls


def _run_linear_layer(tt, layer, x, err, rf, rb, rg, yo, eo, ro, o, dev):
    y, e = layer.forward((x.to(dev), 1), rf.to(dev))
    assert torch.equal(y.cpu(), yo) and _ei(e) == eo
    r = layer.backward((err.to(dev), -2), rb.to(dev), rg.to(dev))
    assert torch.equal(r[0].cpu(), ro[0]) and _ei(r[1]) == ro[1]
    assert torch.equal(layer.grad.cpu(), o.grad)
    assert torch.equal(layer.weight.cpu(), o.weight) and _ei(layer.grad_exp) == o.grad_exp


def test_standalone_shift_functions(tt, kat):
    dev = torch.device("cuda:0")
    _say("standalone RoundShift/PstoShift/StoShift")
    X = torch.tensor(kat["X"], dtype=torch.int32, device=dev)
    for mode in ("floor", "trunc"):
        tt.DIV_MODE = mode
        assert tt.RoundShift(X, 7).cpu().tolist() == kat[f"round_s7_{mode}"]
        assert tt.PstoShift(X, 7).cpu().tolist() == kat[f"psto_s7_{mode}"]
        r20 = torch.arange(-20, 21, dtype=torch.int32, device=dev)
        assert tt.StoShift(r20, 4, torch.full_like(r20, 7)).cpu().tolist() == kat[f"sto_s4_u7_m20_20_{mode}"]
        assert tt.PstoShift(r20, 4).cpu().tolist() == kat[f"psto_s4_m20_20_{mode}"]
    y = tt.StoShift(X, 3)          # device random draw: only the range is checkable
    assert int(y.min()) >= -127 and int(y.max()) <= 127


def _build_pair(tt, cfg_list, widths_in, N, seed, dropout, image=32):
    """Same int8 weights in the GPU model and in the oracle model."""
    from niti_amd import ti_vgg
    from oracle import niti_model_oracle as mo
    g = torch.Generator().manual_seed(seed)
    dev = torch.device("cuda:0")
    ti_vgg.cifar_cfg["test"] = cfg_list
    net = ti_vgg.TiVGG_cifar("test", fuse=True, dropout=dropout)
    weights, exps = [], []
    for l in net.forward_layers:
        if hasattr(l, "weight"):
            w = ri8(g, *l.weight.shape)
            e = -int(torch.randint(6, 12, (1,), generator=g))
            l.weight, l.weight_exp = w.to(dev), torch.tensor(float(e))
            weights.append(w)
            exps.append(e)
    fc_in = weights[-1].shape[1]
    mask = torch.randint(0, 2, (fc_in,), generator=g, dtype=torch.int8) if dropout else None
    onet = mo.build_vgg(cfg_list, weights, exps, mo.Cfg(), mask)
    x = ri8(g, N, image, image, 3)
    target = torch.randint(0, 10, (N,), generator=g)
    loss_rand = torch.randint(0, 16, (N, 10), generator=g, dtype=torch.int32)
    return net, onet, x, target, loss_rand, mask


@pytest.mark.parametrize("name,cfg_list,N", [
    ("vgg7-narrow", [16, 16, 'M', 32, 32, 'M', 512, 512, 'M'], 8),
    ("vgg7-full", [128, 128, 'M', 256, 256, 'M', 512, 512, 'M'], 16),
    ("vgg13", [64, 64, 'M', 128, 128, 'M', 256, 256, 'M', 512, 512, 'M', 512, 512, 'M'], 8),
    # cifar_cfg[8] and cifar_cfg[9] of the reference (ti_vgg.py:12-13): stages of three convolutions, i.e. convolutions
    # whose ReLU is followed by another convolution instead of a pooling
    # batches that are not whole tiles of the single-launch kernels: the last batch of a pass over a data set (80 =
    # 50000 mod 256, the reference trains on it: data.py:42-46) and an odd one (ti_torch.py:419-428)
    ("vgg7-narrow-batch80", [16, 16, 'M', 32, 32, 'M', 512, 512, 'M'], 80),
    ("vgg7-narrow-batch37", [16, 16, 'M', 32, 32, 'M', 512, 512, 'M'], 37),
    ("vgg8", [128, 128, 128, 'M', 256, 256, 'M', 512, 512, 'M'], 8),
    ("vgg9", [128, 128, 128, 'M', 256, 256, 256, 'M', 512, 512, 'M'], 8),
])
def test_training_step(tt, name, cfg_list, N):
    """One complete integer training step (forward, loss gradient, backward, weight update)."""
    from niti_amd import ti_torch
    dev = torch.device("cuda:0")
    _say("training step", name, N)
    net, onet, x, target, loss_rand, mask = _build_pair(tt, cfg_list, None, N, 2000, dropout=True)
    # forward
    yo, eo = onet.forward_int8(x, 0)
    drop = [l for l in net.forward_layers if isinstance(l, ti_torch.TiDropout)][0]
    orig_fwd = drop.forward
    drop.forward = lambda inp: orig_fwd(inp, mask.to(dev))
    y, e = net.forward_int8(x.to(dev), 0)
    assert torch.equal(y.cpu(), yo) and _ei(e) == eo
    # backward from the oracle's loss gradient (the float loss itself is compared separately)
    onet.backward(target, loss_rand)
    net.backward_from((onet.loss_err.to(dev), 0))
    gl = [l for l in net.forward_layers if hasattr(l, "weight")]
    ol = [l for l in onet.layers if hasattr(l, "weight")]
    assert len(gl) == len(ol)
    for i, (a, b) in enumerate(zip(gl, ol)):
        assert torch.equal(a.weight.cpu(), b.weight), "updated weight of layer %d" % i
        assert _ei(a.grad_exp) == b.grad_exp, "grad exponent of layer %d" % i
        if i > 0:
            assert _ei(a.err_exp) == b.err_exp, "error exponent of layer %d" % i
    # a second step on the updated weights keeps matching
    yo, eo = onet.forward_int8(x, 0)
    y, e = net.forward_int8(x.to(dev), 0)
    assert torch.equal(y.cpu(), yo) and _ei(e) == eo
    # a complete step with the targets known at forward time: the classifier's forward launch evaluates the loss
    # gradient, backward(target) starts from it
    from niti_amd import ops
    onet.backward(target, loss_rand)
    tgt = target.to(dev)
    calls = []
    orig_loss = ops.loss_grad
    ops.loss_grad = lambda *a, **k: calls.append("loss") or orig_loss(*a, **k)
    try:
        y, e = net.forward_int8(x.to(dev), 0, tgt, loss_rand.to(dev))
        assert torch.equal(y.cpu(), yo) and _ei(e) == eo
        net.backward(tgt)
    finally:
        ops.loss_grad = orig_loss
    assert calls == []
    from oracle import niti_oracle as po
    if not bool((po.ti_loss_pre_round(yo, eo, target) == -2 ** 31).any()):
        # (for exponents far from zero the reference's own formula, ti_loss.py:14-31, divides 0 by 0 and converts the NaN
        # to an integer, which host and device do differently: nothing to compare there)
        assert torch.equal(net.loss.out_grad.cpu(), onet.loss_err)
        for i, (a, b) in enumerate(zip(gl, ol)):
            assert torch.equal(a.weight.cpu(), b.weight), "updated weight of layer %d (second step)" % i
            assert _ei(a.grad_exp) == b.grad_exp
    assert not ops.sync_arena.timed_out(dev), "a single-launch kernel gave up waiting for its workgroups"


def test_ti_loss_matches_oracle_exactly(tt):
    """TiLoss is one kernel that keeps the reference's float32 operation sequence, with 2 ** s evaluated by a fixed
    sequence of double operations that the oracle repeats: every int8 of the gradient equals the CPU oracle's, in
    both branches of the exponent split, and the known answers of tests/golden/ti_loss_kat.json come out of the kernel."""
    import json
    import os
    from niti_amd.ti_loss import TiLoss, loss_grad_tensor_ops
    from oracle import niti_oracle as po
    dev = torch.device("cuda:0")
    g = torch.Generator().manual_seed(3000)
    for div_mode in ("floor", "trunc"):
        tt.DIV_MODE = div_mode
        for e in (-12, -9, -7, -6, -3, -1, 0, 2, 5):
            _say("ti_loss", e, div_mode)
            n = 64 if e != -3 else 1025         # more than one workgroup, ragged
            spread = 127 if e < 0 else 40
            out = torch.randint(-spread, spread + 1, (n, 10), generator=g, dtype=torch.int8)
            tgt = torch.randint(0, 10, (n,), generator=g)
            u = torch.randint(0, 16, (n, 10), generator=g, dtype=torch.int32)
            ref, _ = po.ti_loss(out, e, tgt, u, div_mode)
            got, ge = TiLoss()(out.to(dev), e, tgt.to(dev), u.to(dev))
            assert ge == 0 and got.dtype == torch.int8 and tuple(got.shape) == (n, 10)
            assert torch.equal(got.cpu(), ref), (e, div_mode)
            # the same sequence as device tensor operations
            alt = loss_grad_tensor_ops(out.to(dev), e, tgt.to(dev), u.to(dev))
            assert torch.equal(alt.cpu(), ref), (e, div_mode)
    tt.DIV_MODE = "floor"
    # known answers: with rand = 15 nothing is added (StoShift adds one when the remainder exceeds rand), so the kernel's
    # int8 output is clip(pre_round >> 4, +-127) of the golden pre-round values
    with open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "ti_loss_kat.json")) as f:
        cases = json.load(f)["cases"]
    for c in cases:
        out = torch.tensor([c["row"]], dtype=torch.int8)
        tgt = torch.tensor([c["target"]])
        u = torch.full((1, len(c["row"])), 15, dtype=torch.int32)
        want = torch.clamp(torch.tensor([c["expected"]], dtype=torch.int32) >> 4, -127, 127).to(torch.int8)
        got, _ = TiLoss()(out.to(dev), c["out_exp"], tgt.to(dev), u.to(dev))
        assert torch.equal(got.cpu(), want), c["name"]
    # drawing the random integers on the device (no ``rand``): between the results for the two extreme draws
    out = ri8(g, 64, 10)
    tgt = torch.randint(0, 10, (64,), generator=g)
    lo, _ = po.ti_loss(out, -3, tgt, torch.full((64, 10), 15, dtype=torch.int32))
    hi, _ = po.ti_loss(out, -3, tgt, torch.zeros((64, 10), dtype=torch.int32))
    got, _ = TiLoss()(out.to(dev), -3, tgt.to(dev))
    gc = got.cpu().to(torch.int16)
    assert bool(((gc >= torch.minimum(lo, hi).to(torch.int16)) & (gc <= torch.maximum(lo, hi).to(torch.int16))).all())


def test_shims_match_reference_conventions():
    """The four stand-in extension modules: names, return dtypes / shapes / strides, error behaviour."""
    import niti_amd.shims as shims
    from oracle import niti_oracle as po
    dev = torch.device("cuda:0")
    _say("shims")
    shims.install()
    import cutlassconv_cuda, int8conv_cuda, int8mm_cuda, int8pool_cuda
    g = torch.Generator().manual_seed(4000)
    x, w = ri8(g, 2, 8, 8, 16), ri8(g, 24, 3, 3, 16)
    y = cutlassconv_cuda.sp_conv_optimized(x.to(dev), w.to(dev), 1, 1)
    assert y.dtype == torch.int32 and y.is_contiguous() and tuple(y.shape) == (2, 8, 8, 24)
    assert torch.equal(y.cpu(), po.conv2d_int8(x, w))
    assert torch.equal(cutlassconv_cuda.sp_conv(x.to(dev), w.to(dev), 2, 1).cpu(), po.conv2d_int8(x, w, 2, 1))
    with pytest.raises(RuntimeError):
        cutlassconv_cuda.sp_conv(x, w.to(dev), 1, 1)                       # CPU tensor
    with pytest.raises(RuntimeError):
        cutlassconv_cuda.sp_conv(x.to(dev).permute(0, 2, 1, 3), w.to(dev), 1, 1)   # not contiguous
    a, b = ri8(g, 12, 32), ri8(g, 32, 20)
    c = int8mm_cuda.int8_mm(a.to(dev), b.to(dev))
    assert c.dtype == torch.int32 and tuple(c.shape) == (12, 20) and not c.is_contiguous() and c.stride() == (1, 12)
    assert torch.equal(c.contiguous().cpu(), po.int8mm(a, b))
    p = int8pool_cuda.int8_pool(x.to(dev), 2, 2, 0)
    assert torch.equal(p.cpu(), po.maxpool_fwd(x))
    dy = ri8(g, 2, 4, 4, 16, lo=-20, hi=20)
    dx = int8pool_cuda.int8_pool_backward(p.half(), dy.to(dev).half(), x.to(dev).half(), 2, 2, 0)
    assert dx.dtype == torch.float16
    assert torch.equal(dx.type(torch.int8).cpu(), po.maxpool_bwd(po.maxpool_fwd(x), dy, x))
    assert hasattr(int8conv_cuda, "group_conv") and hasattr(cutlassconv_cuda, "weight_grad")


@pytest.mark.parametrize("use_graph", [False, True])
def test_epoch_driver_learns_and_checkpoints(tt, tmp_path, use_graph):
    """The epoch driver (regime, train pass, evaluation pass, checkpoint files) on a synthetic ten-class task: the
    integer step must actually learn (chance is 10 %), and a checkpoint loaded into a fresh model must reproduce
    the trained model's outputs bit for bit."""
    import os
    from niti_amd import train
    from niti_amd.ti_vgg import TiVGG_cifar
    _say("epoch_driver")
    torch.manual_seed(3)
    model = TiVGG_cifar(depth=7)
    model.regime = [{'epoch': 0, 'gb': 5}, {'epoch': 3, 'gb': 4}]
    tr, te = train.synthetic_loaders(128, train_batches=16, test_batches=4, noise=0.5, seed=1)
    hist = train.fit(model, tr, te, epochs=4, save_path=str(tmp_path), save_all=True, use_graph=use_graph)
    if use_graph:   # training and evaluation steps at both gradient bit widths of the regime were captured, none refused
        graphs = model.__dict__["_step_graphs"]
        assert len(graphs) == 4 and all(g.graph is not None and not g.failed for g in graphs.values())
        # every replay (52 training and 4 evaluation steps, with eager work and host reads in between) did what the
        # eager step does: the same run issued launch by launch ends with the same numbers and the same weights
        torch.manual_seed(3)
        twin = TiVGG_cifar(depth=7)
        twin.regime = model.regime
        tr2, te2 = train.synthetic_loaders(128, train_batches=16, test_batches=4, noise=0.5, seed=1)
        hist2 = train.fit(twin, tr2, te2, epochs=4, use_graph=False)
        assert hist2 == hist
        for a, b in zip(model.state_dict().values(), twin.state_dict().values()):
            assert torch.equal(a, b)
    assert [h['grad_bitwidth'] for h in hist] == [5, 5, 5, 4]
    assert hist[0]['val_prec1'] < 60.0 and max(h['val_prec1'] for h in hist) > 80.0, hist
    assert sorted(os.listdir(tmp_path)) == ['checkpoint_epoch_0.pth.tar', 'checkpoint_epoch_1.pth.tar', 'checkpoint_epoch_2.pth.tar',
                                            'checkpoint_epoch_3.pth.tar', 'ckpt.pth', 'model_best.pth.tar']
    fresh = TiVGG_cifar(depth=7)
    ckpt = train.load_checkpoint(fresh, os.path.join(tmp_path, 'ckpt.pth'))
    assert ckpt['epoch'] == 3 and ckpt['best_prec1'] == hist[-1]['best_prec1']
    tt.TRAINING = False
    x, _ = next(iter(te))
    out_a, exp_a = model(x.to("cuda:0"))
    out_b, exp_b = fresh(x.to("cuda:0"))
    assert torch.equal(out_a, out_b) and _ei(exp_a) == _ei(exp_b)


@pytest.mark.parametrize("use_graph", [False, True])
def test_epoch_driver_trains_on_the_trailing_batch(tt, use_graph):
    """A pass over 128 + 80 images: the smaller last batch is a training step like any other (the reference's loaders
    do not drop it, data.py:42-46).  The pass must see all 208 samples, and its weights must equal those of the same
    two batches stepped by hand."""
    from niti_amd import train
    from niti_amd.ti_vgg import TiVGG_cifar
    _say("epoch_driver trailing batch", use_graph)
    g = torch.Generator().manual_seed(77)
    x = torch.randn(208, 3, 32, 32, generator=g)
    y = torch.randint(0, 10, (208,), generator=g)
    torch.manual_seed(11)
    model = TiVGG_cifar(depth=7)
    start = {k: v.clone() for k, v in model.state_dict().items()}
    loader = train.TensorLoader(x, y, 128)
    assert len(loader) == 2
    seen = []
    orig = train._add_metrics
    train._add_metrics = lambda out, e, t, sums: seen.append(int(t.numel())) or orig(out, e, t, sums)
    try:
        torch.manual_seed(12)      # the dropout masks and the loss gradient's random integers come from torch's device generator
        torch.cuda.manual_seed(12)
        train.run_epoch(loader, model, True, use_graph=use_graph)
    finally:
        train._add_metrics = orig
    assert seen == [128, 80]
    twin = TiVGG_cifar(depth=7)
    twin.load_state_dict(start)
    tt.TRAINING = True
    torch.manual_seed(12)
    torch.cuda.manual_seed(12)
    dev = torch.device("cuda:0")
    before = {k: v.clone() for k, v in start.items()}    # load_state_dict adopts the tensors it is given
    for lo, hi in ((0, 128), (128, 208)):
        tgt = y[lo:hi].to(dev)
        twin(x[lo:hi].to(dev), tgt)
        twin.backward(tgt)
    changed = 0
    for (k, a), b in zip(model.state_dict().items(), twin.state_dict().values()):
        assert torch.equal(a, b), k
        changed += int(not torch.equal(a.cpu(), before[k].cpu()))
    assert changed > 0
    from niti_amd import ops
    assert not ops.sync_timeouts(dev)


def test_epoch_driver_command_line(tt, tmp_path, monkeypatch):
    """The command line keeps the reference's option names; without a data file it trains on the synthetic set and
    leaves its checkpoints under ./results/<--save>; --init continues from one."""
    import os
    from niti_amd import train
    _say("epoch_driver_command_line")
    monkeypatch.chdir(tmp_path)
    hist = train.main(["--depth", "7", "--epochs", "1", "--batch-size", "128", "--seed", "5", "--save", "run1", "--log-interval", "8"])
    assert len(hist) == 1 and os.path.exists(os.path.join("results", "run1", "ckpt.pth"))
    again = train.main(["--depth", "7", "--epochs", "1", "--batch-size", "128", "--seed", "5", "--init", os.path.join("results", "run1", "ckpt.pth")])
    assert again[0]["val_prec1"] >= 0.0 and not os.path.exists(os.path.join("results", "test"))


def test_grid_wide_wait_gives_up_and_says_so():
    """With a wait limit of zero (set from the host, in a process of its own because the library reads the limit
    once) every wait of the single-launch kernels gives up after its first look: every workgroup still runs to its
    end, the launch completes, and the sync words of EVERY launch report that the result is not to be used - for the
    one-launch weight gradient both of its waits (bit 1: arrival of the partial sums, bit 0: range)."""
    import os
    import subprocess
    import sys
    code = r"""
import torch
from niti_amd import ops
dev = torch.device("cuda:0")
g = torch.Generator().manual_seed(1)
x = torch.randint(-127, 128, (64, 32, 32, 64), generator=g, dtype=torch.int8).to(dev)
w = torch.randint(-127, 128, (128, 3, 3, 64), generator=g, dtype=torch.int8).to(dev)
ops.sync_arena.reset(dev)
flagged = 0
for i in range(4):
    y, sh, sync = ops.conv2d_fprop_requant(x, w)
    torch.cuda.synchronize()
    flagged += int(sync.cpu()[1] == 1)
print("FLAGGED", flagged, "ARENA", int(ops.sync_arena.timed_out(dev)))
# the one-launch weight gradient waits twice (arrival of the partial sums, range): same limit, same flag
act = torch.randint(-127, 128, (16, 16, 16, 64), generator=g, dtype=torch.int8).to(dev)
err = torch.randint(-127, 128, (16, 16, 16, 128), generator=g, dtype=torch.int8).to(dev)
wflag = 0
for i in range(4):
    wd = w.clone()
    _, _, _, sync = ops.conv2d_wgrad_update(act, err, wd, mu=5, method="psto")
    torch.cuda.synchronize()
    wflag += int(sync.cpu()[1] == 3)
print("WGRAD_FLAGGED", wflag)
# the device-wide word survives the arena's reset, is cleared by a read, and the epoch driver's check raises on it
ops.sync_arena.reset(dev)
print("STICKY", int(ops.sync_arena.timed_out(dev)), int(ops.sync_timeouts(dev, clear=False)), int(ops.sync_timeouts(dev)),
      int(ops.sync_timeouts(dev)))
from niti_amd import train
y, sh, sync = ops.conv2d_fprop_requant(x, w)
try:
    train.check_waits(dev)
    print("RAISED 0")
except train.GridWaitTimeout:
    print("RAISED 1")
"""
    env = dict(os.environ, NITI_SYNC_TIMEOUT_MS="0")
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    out = subprocess.run([sys.executable, "-c", code], cwd=root, env=env, capture_output=True, text=True, timeout=120)
    assert out.returncode == 0, out.stderr[-2000:]
    line = [l for l in out.stdout.splitlines() if l.startswith("FLAGGED")][0].split()
    assert int(line[1]) == 4 and int(line[3]) == 1
    assert int([l for l in out.stdout.splitlines() if l.startswith("WGRAD_FLAGGED")][0].split()[1]) == 4
    sticky = [l for l in out.stdout.splitlines() if l.startswith("STICKY")][0].split()
    assert sticky[1:] == ["0", "1", "1", "0"], sticky
    assert "RAISED 1" in out.stdout
