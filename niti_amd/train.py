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
import gc
import logging
import os
import shutil

import numpy as np
import torch
import torch.nn.functional as F

from . import ops, ti_torch
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


def _add_metrics(output, output_exp, target, sums):
    """Adds batch size x (display loss, top-1, top-5) to ``sums`` (main.py:156-163)."""
    scale = torch.exp2(torch.as_tensor(output_exp, device=output.device).float().reshape(()))
    loss = F.cross_entropy(output.float() * scale, target)
    prec1, prec5 = accuracy(output.detach(), target, topk=(1, 5))
    sums += torch.stack([loss.double(), prec1.double(), prec5.double()]) * target.size(0)


def _one_step(model, training, inputs, target, sums):
    """Forward (+ backward when training) on one batch of float images."""
    output, output_exp = model(inputs, target if training else None)
    _add_metrics(output, output_exp, target, sums)
    if training:
        model.backward(target)


class StepGraph:
    """The integer part of a training (or evaluation) step replayed from a captured HIP graph: a step is some forty
    short launches, and issuing them one by one from Python takes about twice as long as the device needs for them.
    Only the library's own kernels, fills and random-number kernels are captured.  The input quantisation and the
    display metrics - tensor-library reductions, whose multi-block forms clear their scratch words with memset
    nodes that do not replay reliably here - run eagerly before and after each replay, on static buffers.  The
    first ``eager_steps`` batches run eagerly (ordinary steps: nothing is run twice), the next one is captured, from
    then on batches are replays.  Falls back to eager steps if the capture is refused."""

    def __init__(self, model, training, inputs, target, eager_steps=3):
        self.model, self.training = model, training
        x_data, _ = model.quantize_input(inputs)
        self.x8 = torch.empty_like(x_data)                                               # quantised batch, NHWC
        self.x_exp = torch.empty(1, dtype=torch.int32, device=inputs.device)
        self.target = torch.empty_like(target)
        self.graph, self.failed, self.eager_left = None, False, eager_steps
        self.out = None
        self.side = torch.cuda.Stream()

    def _step(self):
        self.model.forward_int8(self.x8, self.x_exp, self.target if self.training else None)
        if self.training:
            self.model.backward(self.target)

    def __call__(self, inputs, target, sums):
        x_data, x_exp = self.model.quantize_input(inputs)       # ti_net.py:17-19
        self.x8.copy_(x_data)
        self.x_exp.copy_(x_exp.reshape(1))
        self.target.copy_(target, non_blocking=True)
        if self.graph is not None:
            self.graph.replay()
        elif self.eager_left > 0 or self.failed:
            self.eager_left -= 1
            cur = torch.cuda.current_stream()
            self.side.wait_stream(cur)
            with torch.cuda.stream(self.side):
                self._step()
            cur.wait_stream(self.side)
        else:
            torch.cuda.synchronize()
            # No cyclic garbage collection while the stream is capturing: a collection that frees device tensors of
            # the eager steps (allocated on another stream) makes the allocator record events, which a capturing
            # process may not do - the runtime aborts.  torch.cuda.graph collects once on entry, but a collection can
            # still start at any allocation inside the captured step.
            gc_was_on = gc.isenabled()
            gc.collect()
            gc.disable()
            try:
                try:
                    g = torch.cuda.CUDAGraph()
                    with torch.cuda.graph(g):
                        self._step()
                finally:
                    if gc_was_on:
                        gc.enable()
                self.graph = g
                self.out = (self.model.out, self.model.out_exp)     # where every replay leaves its logits
                g.replay()
            except Exception as e:      # keep training
                logging.warning("step graph capture failed (%s); running eager steps", e)
                torch.cuda.synchronize()
                self.failed = True
                self._step()
        output, output_exp = self.out if self.graph is not None else (self.model.out, self.model.out_exp)
        _add_metrics(output, output_exp, self.target, sums)


def run_epoch(data_loader, model, training, log_interval=0, epoch=0, use_graph=False):
    """One pass over ``data_loader`` (main.py:133-193).  Returns (loss, top-1 %, top-5 %) averaged over the
    samples.  The float cross-entropy is for display only, as in the reference (main.py:156-157); the sums stay on
    the device until the end of the pass so that the integer step is not held up by host reads.  ``use_graph``:
    replay the step from a HIP graph (StepGraph; batches must all have one shape)."""
    ti_torch.TRAINING = bool(training)
    dev = torch.device(ti_torch.GPU)
    sums = torch.zeros(3, dtype=torch.float64, device=dev)
    count = 0
    for i, (inputs, target) in enumerate(data_loader):
        inputs = inputs.to(dev, non_blocking=True)
        target = target.to(dev, non_blocking=True)
        if use_graph:
            # graphs are per mode, batch shape and gradient bit width (a kernel argument fixed at capture)
            key = (bool(training), tuple(inputs.shape), inputs.dtype, ti_torch.GRAD_BITWIDTH)
            cache = model.__dict__.setdefault('_step_graphs', {})
            runner = cache.get(key)
            if runner is None:
                runner = cache[key] = StepGraph(model, bool(training), inputs, target)
            runner(inputs, target, sums)
        else:
            _one_step(model, bool(training), inputs, target, sums)
        count += inputs.size(0)
        if training and log_interval and i % log_interval == 0:
            s = (sums / count).tolist()
            logging.info('[%d][%3d] loss %.3f @1 %.3f', epoch, i, s[0], s[1])
        # A shared device makes every grid-wide wait run into its limit and every step round with wrong shifts: find out
        # after the first steps and whenever the host reads the device anyway, not at the end of a pass that looked hung
        if i in (0, 3) or (training and log_interval and i % log_interval == 0):
            check_waits(dev)
    if count == 0:
        return 0.0, 0.0, 0.0
    loss_avg, top1, top5 = (sums / count).tolist()
    check_waits(dev)
    return loss_avg, top1, top5


class GridWaitTimeout(RuntimeError):
    """A kernel that exchanges a tensor-wide range between its workgroups gave up waiting for some of them."""


def check_waits(dev=None):
    """Raises if any single-launch kernel since the last check flagged a grid-wide wait that ran into its time limit
    (other work kept part of the device busy): activations, errors or weight updates since then were rounded with a
    wrong shift, so the pass is invalid and its weights must not be saved.  One 4-byte read per call; run_epoch calls
    it at the end of every pass, i.e. before fit() writes a checkpoint."""
    if ops.sync_timeouts(dev if dev is not None else torch.device(ti_torch.GPU), clear=True):
        raise GridWaitTimeout("a grid-wide wait of the int8 kernels timed out during this pass: the device was shared with "
                              "other work; results of the pass are invalid and nothing was saved")


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


def fit(model, train_loader, test_loader, epochs, save_path=None, save_all=False, log_interval=0, use_graph=False):
    """main.py:66-131 without the TensorBoard writer: per epoch apply the regime, train, evaluate, write
    ``ckpt.pth`` (and ``model_best.pth.tar``) under ``save_path``.  Returns one dict per epoch."""
    history = []
    best_prec1 = 0.0
    for epoch in range(epochs):
        apply_regime(model.regime, epoch)
        train_loss, train_prec1, _ = run_epoch(train_loader, model, True, log_interval, epoch, use_graph)
        val_loss, val_prec1, _ = run_epoch(test_loader, model, False, 0, epoch, use_graph)
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
    """Minimal stand-in for a ``DataLoader`` over in-memory tensors, reshuffled every pass when ``shuffle``.  Like the
    reference's loaders (data.py:42-46: no ``drop_last``) it ends a pass with the smaller batch that is left over -
    CIFAR-10 at batch 256 ends with 80 images; the layers run such a batch through whichever kernels cover its
    shape (the single-launch ones need whole tiles of 256 pixels) and the reference's own odd-batch case
    (ti_torch.py:419-428) needs no special path here.  ``drop_last=True`` keeps only whole batches."""

    def __init__(self, x, y, batch_size, shuffle=False, seed=0, drop_last=False):
        self.x, self.y, self.batch_size, self.shuffle, self.drop_last = x, y, batch_size, shuffle, drop_last
        self.gen = torch.Generator().manual_seed(seed)

    def __len__(self):
        n = self.x.shape[0]
        return n // self.batch_size if self.drop_last else (n + self.batch_size - 1) // self.batch_size

    def __iter__(self):
        n = self.x.shape[0]
        order = torch.randperm(n, generator=self.gen) if self.shuffle else torch.arange(n)
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
    p.add_argument('--no-graph', action='store_true', help='issue every launch of a step from Python instead of replaying a HIP graph')
    p.add_argument('--div-mode', choices=('floor', 'trunc'), default=ti_torch.DIV_MODE,
                   help="meaning of // on negative numbers in the rounding helpers: floor (torch >= 1.13, default) or "
                        "trunc (torch <= 1.12, what the reference's published runs used)")
    p.add_argument('--bw-mode', choices=('int', 'f32'), default=ti_torch.BW_MODE,
                   help="bit width of a range: exact integer ceil(log2 r) (default) or the reference's float32 evaluation")
    args = p.parse_args(argv)
    logging.basicConfig(level=logging.INFO, format='%(asctime)s %(message)s')
    if args.seed > 0:
        torch.manual_seed(args.seed)
    ti_torch.DIV_MODE, ti_torch.BW_MODE = args.div_mode, args.bw_mode
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
    return fit(model, train_loader, test_loader, args.epochs, save_path, args.save_all, args.log_interval, not args.no_graph)


if __name__ == '__main__':
    main()
