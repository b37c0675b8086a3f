"""Epoch driver with the reference's ``main.py`` behaviour (main.py:72-131 epoch loop, 133-193 ``forward``),
its accuracy meter (meters.py:56-70) and its checkpoint files (log.py:219-226), for any iterable of
``(float32 NCHW images, int64 labels)`` batches.

The reference reads CIFAR-10 through torchvision (data.py); neither is available offline, so the command line
here trains on ``--data-npz`` (arrays ``x_train, y_train, x_test, y_test``; images uint8 NHWC or float NCHW) or,
without it, on a synthetic ten-class set of noisy class patterns (``synthetic_loaders``).

    python -m niti_amd.train --depth 7 --epochs 2 --batch-size 128
"""
from __future__ import annotations

import argparse
import logging
import os
import shutil

import numpy as np
import torch
import torch.nn.functional as F

from . import ti_torch
from .ti_vgg import TiVGG_cifar


def accuracy(output, target, topk=(1,)):
    """Precision@k in percent for each k (meters.py:56-70), as 0-d tensors on the output's device."""
    maxk = max(topk)
    batch_size = target.size(0)
    _, pred = output.topk(maxk, 1, True, True)
    correct = pred.t().eq(target.view(1, -1).expand(maxk, batch_size))
    return [correct[:k].reshape(-1).float().sum(0) * (100.0 / batch_size) for k in topk]


def apply_regime(regime, epoch):
    """main.py:73-77: the gradient bit width changes at the epochs the model's regime names."""
    for s in regime:
        if s['epoch'] == epoch:
            ti_torch.GRAD_BITWIDTH = s['gb']
            logging.info("Change Grad Bitwidth to : %s", ti_torch.GRAD_BITWIDTH)
            break


def run_epoch(data_loader, model, training, log_interval=0, epoch=0):
    """One pass over ``data_loader`` (main.py:133-193).  Returns (loss, top-1 %, top-5 %) averaged over the
    samples.  The float cross-entropy is for display only, as in the reference (main.py:156-157); the sums stay on
    the device until the end of the pass so that the integer step is not held up by host reads."""
    ti_torch.TRAINING = bool(training)
    dev = torch.device(ti_torch.GPU)
    sums = torch.zeros(3, dtype=torch.float64, device=dev)
    count = 0
    for i, (inputs, target) in enumerate(data_loader):
        inputs = inputs.to(dev, non_blocking=True)
        target = target.to(dev, non_blocking=True)
        output, output_exp = model(inputs)
        scale = torch.exp2(torch.as_tensor(output_exp, device=dev).float().reshape(()))
        loss = F.cross_entropy(output.float() * scale, target)
        prec1, prec5 = accuracy(output.detach(), target, topk=(1, 5))
        n = inputs.size(0)
        sums += torch.stack([loss.double(), prec1.double(), prec5.double()]) * n
        count += n
        if training:
            model.backward(target)
            if log_interval and i % log_interval == 0:
                s = (sums / count).tolist()
                logging.info('[%d][%3d] loss %.3f @1 %.3f', epoch, i, s[0], s[1])
    if count == 0:
        return 0.0, 0.0, 0.0
    loss_avg, top1, top5 = (sums / count).tolist()
    return loss_avg, top1, top5


def save_checkpoint(state, is_best, path='.', filename='checkpoint.pth.tar', save_all=False):
    """log.py:219-226."""
    filename = os.path.join(path, filename)
    torch.save(state, filename)
    if is_best:
        shutil.copyfile(filename, os.path.join(path, 'model_best.pth.tar'))
    if save_all:
        shutil.copyfile(filename, os.path.join(path, 'checkpoint_epoch_%s.pth.tar' % state['epoch']))


def load_checkpoint(model, path):
    """main.py:61-64.  Checkpoints hold tensors and numbers only, so the loader that executes nothing from the
    file is enough."""
    ckpt = torch.load(path, map_location='cpu', weights_only=True)
    model.load_state_dict(ckpt['state_dict'])
    return ckpt


def fit(model, train_loader, test_loader, epochs, save_path=None, save_all=False, log_interval=0):
    """main.py:66-131 without the TensorBoard writer: per epoch apply the regime, train, evaluate, write
    ``ckpt.pth`` (and ``model_best.pth.tar``) under ``save_path``.  Returns one dict per epoch."""
    history = []
    best_prec1 = 0.0
    for epoch in range(epochs):
        apply_regime(model.regime, epoch)
        train_loss, train_prec1, _ = run_epoch(train_loader, model, True, log_interval, epoch)
        val_loss, val_prec1, _ = run_epoch(test_loader, model, False, 0, epoch)
        is_best = val_prec1 > best_prec1
        best_prec1 = max(val_prec1, best_prec1)
        if save_path is not None:
            os.makedirs(save_path, exist_ok=True)
            save_checkpoint({'epoch': epoch, 'state_dict': model.state_dict(), 'best_prec1': best_prec1},
                            is_best, save_path, 'ckpt.pth', save_all)
        logging.info('Epoch: %d Train Prec@1 %.3f Train Loss %.3f Valid Prec@1 %.3f Valid Loss %.3f',
                     epoch, train_prec1, train_loss, val_prec1, val_loss)
        history.append({'epoch': epoch, 'train_loss': train_loss, 'train_prec1': train_prec1,
                        'val_loss': val_loss, 'val_prec1': val_prec1, 'best_prec1': best_prec1,
                        'grad_bitwidth': ti_torch.GRAD_BITWIDTH})
    return history


class TensorLoader:
    """Minimal stand-in for a ``DataLoader`` over in-memory tensors: fixed-size batches (the last ragged one is
    dropped: the convolution kernels own whole tiles of a batch), reshuffled every pass when ``shuffle``."""

    def __init__(self, x, y, batch_size, shuffle=False, seed=0):
        self.x, self.y, self.batch_size, self.shuffle = x, y, batch_size, shuffle
        self.gen = torch.Generator().manual_seed(seed)

    def __len__(self):
        return self.x.shape[0] // self.batch_size

    def __iter__(self):
        n = len(self) * self.batch_size
        order = torch.randperm(self.x.shape[0], generator=self.gen)[:n] if self.shuffle else torch.arange(n)
        for b in range(len(self)):
            idx = order[b * self.batch_size:(b + 1) * self.batch_size]
            yield self.x[idx], self.y[idx]


def synthetic_loaders(batch_size, train_batches=16, test_batches=4, noise=0.5, seed=0, classes=10):
    """Ten classes of 3x32x32 images: a fixed random low-resolution pattern per class plus Gaussian noise."""
    g = torch.Generator().manual_seed(seed)
    coarse = torch.randn(classes, 3, 8, 8, generator=g)
    patterns = F.interpolate(coarse, size=(32, 32), mode='nearest')

    def make(nb):
        y = torch.randint(0, classes, (nb * batch_size,), generator=g)
        x = patterns[y] + noise * torch.randn(nb * batch_size, 3, 32, 32, generator=g)
        return x, y

    xtr, ytr = make(train_batches)
    xte, yte = make(test_batches)
    return TensorLoader(xtr, ytr, batch_size, True, seed + 1), TensorLoader(xte, yte, batch_size)


def npz_loaders(path, batch_size, seed=0):
    """Arrays x_train / y_train / x_test / y_test; uint8 NHWC images are scaled to [-1, 1] and laid out NCHW."""
    d = np.load(path)

    def images(a):
        t = torch.from_numpy(a)
        if t.dtype == torch.uint8:
            t = t.permute(0, 3, 1, 2).float() / 127.5 - 1.0
        return t.float().contiguous()

    return (TensorLoader(images(d['x_train']), torch.from_numpy(d['y_train']).long(), batch_size, True, seed),
            TensorLoader(images(d['x_test']), torch.from_numpy(d['y_test']).long(), batch_size))


def main(argv=None):
    # option names of the reference's options.py
    p = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    p.add_argument('--batch-size', type=int, default=256)
    p.add_argument('--seed', type=int, default=-1)
    p.add_argument('--log-interval', type=int, default=100)
    p.add_argument('--save-all', action='store_true', default=False)
    p.add_argument('--data-npz', type=str, default='')
    p.add_argument('--save', default='')
    p.add_argument('--epochs', default=200, type=int)
    p.add_argument('--init', help='init ckpt')
    p.add_argument('--depth', default=7, type=int)
    args = p.parse_args(argv)
    logging.basicConfig(level=logging.INFO, format='%(asctime)s %(message)s')
    if args.seed > 0:
        torch.manual_seed(args.seed)
    model = TiVGG_cifar(depth=args.depth)
    if args.init:
        load_checkpoint(model, args.init)
        logging.info("Init weights from: %s", args.init)
    if args.data_npz:
        train_loader, test_loader = npz_loaders(args.data_npz, args.batch_size, max(args.seed, 0))
    else:
        logging.info("no dataset given: synthetic class patterns")
        train_loader, test_loader = synthetic_loaders(args.batch_size, seed=max(args.seed, 0))
    save_path = os.path.join('./results/', args.save) if args.save else None
    return fit(model, train_loader, test_loader, args.epochs, save_path, args.save_all, args.log_interval)


if __name__ == '__main__':
    main()
