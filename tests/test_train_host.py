"""Host logic of the epoch driver (no GPU): accuracy meter, regime schedule, checkpoint files, loaders."""
import os

import torch

from niti_amd import ti_torch, train


def test_accuracy_known_answers():
    # meters.py:56-70: rows = samples, precision@k = share of samples whose label is among the k largest outputs
    out = torch.tensor([[9, 1, 5, 0], [2, 8, 7, 1], [1, 2, 3, 4], [5, 4, 3, 2]], dtype=torch.int8)
    target = torch.tensor([0, 2, 0, 1])
    p1, p2, p4 = train.accuracy(out, target, topk=(1, 2, 4))
    assert float(p1) == 25.0      # only sample 0
    assert float(p2) == 75.0      # + sample 1 (7 is second) + sample 3 (4 is second)
    assert float(p4) == 100.0


def test_regime_sets_gradient_bitwidth():
    regime = [{'epoch': 0, 'gb': 5}, {'epoch': 100, 'gb': 4}, {'epoch': 150, 'gb': 3}]   # ti_vgg.py:21-23
    old = ti_torch.GRAD_BITWIDTH
    try:
        seen = []
        for epoch in (0, 1, 99, 100, 149, 150, 199):
            train.apply_regime(regime, epoch)
            seen.append(ti_torch.GRAD_BITWIDTH)
        assert seen == [5, 5, 5, 4, 4, 3, 3]
    finally:
        ti_torch.GRAD_BITWIDTH = old


def test_checkpoint_files(tmp_path):
    # log.py:219-226: ckpt file always, model_best copy when best, per-epoch copy when save_all
    state = {'epoch': 3, 'state_dict': {'layers.0.weight': torch.arange(6, dtype=torch.int8), 'layers.0.weight_exp': torch.tensor(-8.0)},
             'best_prec1': 12.5}
    train.save_checkpoint(state, False, str(tmp_path), 'ckpt.pth', False)
    assert sorted(os.listdir(tmp_path)) == ['ckpt.pth']
    train.save_checkpoint(state, True, str(tmp_path), 'ckpt.pth', True)
    assert sorted(os.listdir(tmp_path)) == ['checkpoint_epoch_3.pth.tar', 'ckpt.pth', 'model_best.pth.tar']
    back = torch.load(os.path.join(tmp_path, 'model_best.pth.tar'), weights_only=True)
    assert back['epoch'] == 3 and back['best_prec1'] == 12.5
    assert torch.equal(back['state_dict']['layers.0.weight'], state['state_dict']['layers.0.weight'])


def test_synthetic_loaders_are_deterministic_and_whole_batches():
    a, at = train.synthetic_loaders(8, train_batches=3, test_batches=2, seed=5)
    b, _ = train.synthetic_loaders(8, train_batches=3, test_batches=2, seed=5)
    assert len(a) == 3 and len(at) == 2
    xa = [x for x, _ in a]
    xb = [x for x, _ in b]
    assert all(x.shape == (8, 3, 32, 32) and x.dtype == torch.float32 for x in xa)
    assert all(torch.equal(p, q) for p, q in zip(xa, xb))
    ys = torch.cat([y for _, y in at])
    assert ys.dtype == torch.int64 and int(ys.min()) >= 0 and int(ys.max()) <= 9
    # a second pass reshuffles the training set and repeats the test set
    assert not all(torch.equal(p, q) for p, q in zip(xa, [x for x, _ in a]))
    assert all(torch.equal(p, q) for (p, _), (q, _) in zip(at, at))


def test_npz_loader(tmp_path):
    import numpy as np
    rng = np.random.default_rng(0)
    path = os.path.join(tmp_path, 'd.npz')
    np.savez(path, x_train=rng.integers(0, 256, (10, 32, 32, 3), dtype=np.uint8), y_train=rng.integers(0, 10, 10),
             x_test=rng.integers(0, 256, (4, 32, 32, 3), dtype=np.uint8), y_test=rng.integers(0, 10, 4))
    tr, te = train.npz_loaders(path, 4)
    # data.py:42-46 builds its loaders without drop_last: the two images left over are the last batch
    assert len(tr) == 3 and len(te) == 1
    assert [x.shape[0] for x, _ in tr] == [4, 4, 2]
    assert sorted(int(v) for _, y in tr for v in y) == sorted(int(v) for v in np.load(path)['y_train'])
    whole = train.TensorLoader(tr.x, tr.y, 4, drop_last=True)
    assert len(whole) == 2 and [x.shape[0] for x, _ in whole] == [4, 4]
    x, y = next(iter(te))
    assert x.shape == (4, 3, 32, 32) and float(x.min()) >= -1.0 and float(x.max()) <= 1.0 and y.dtype == torch.int64


def test_quantisers_follow_bw_mode():
    """BW_MODE "f32" makes TiFloatToInt8 / weight_quant take the range exponent from the reference's own float32
    expression (ti_torch.py:336,348); "int" (default) from the float's exponent and mantissa.  They differ for the
    first float32 values above 2^k, k >= 4, when log2 rounds to k: with torch's CPU log2, nextafter(16) gives 4."""
    import numpy as np
    r = torch.tensor(float(np.nextafter(np.float32(16.0), np.float32(32.0))))
    old = ti_torch.BW_MODE
    try:
        ti_torch.BW_MODE = "int"
        assert float(ti_torch._ceil_log2(r)) == 5.0
        assert float(ti_torch._ceil_log2(torch.tensor(16.0))) == 4.0 and float(ti_torch._ceil_log2(torch.tensor(0.75))) == 0.0
        ti_torch.BW_MODE = "f32"
        assert float(ti_torch._ceil_log2(r)) == float(torch.ceil(torch.log2(r)))
        assert float(ti_torch._ceil_log2(torch.tensor(16.0))) == 4.0 and float(ti_torch._ceil_log2(torch.tensor(17.0))) == 5.0
    finally:
        ti_torch.BW_MODE = old
