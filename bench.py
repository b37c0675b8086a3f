#!/usr/bin/env python3
"""Benchmark of the int8 hot path on one MI355X.

One "step" = one pass of the int8 conv layer triple over the six VGG-small conv layer shapes at
batch 128 (BASELINE.json configs[2]): for every layer the forward convolution + activation
requantisation, the data gradient + error requantisation (not for the first layer) and the weight
gradient + fused gradient rounding / weight update, all through the C ABI of libniti_gfx950.so.
Inputs are resident in HBM before the timed region.  The reported value is int8 TOPS =
algorithmic ops (2*N*P*Q*K*R*S*C per conv, real C) / time.

Also reported on the same JSON line: the roofline of the dominant kernel (the MFMA implicit-GEMM
convolution, timed per launch with HIP events on the launch stream inside the timed region), the
CPU baseline (plain-C oracle with OpenMP on the host cores, bounded sample) and the images/s of
a complete VGG-small integer training step (configs[3]).

Usage: python bench.py [--gpus 1] [--steps K] [--warmup W]
"""
from __future__ import annotations

import argparse
import gc
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

INT8_MFMA_PEAK_TOPS = 5000.0   # MI355X dense int8 matrix peak, 5.0 POP/s
HBM_PEAK_GBS = 8000.0

# (C_in, C_out, H=W) of the VGG-small conv stack
LAYERS = [(3, 128, 32), (128, 128, 32), (128, 256, 16), (256, 256, 16), (256, 512, 8), (512, 512, 8)]
BATCH = 128


def conv_ops(n, hw, c, k):
    return 2.0 * n * hw * hw * k * 9 * c


def laplace_i8(g, shape, b=16.0):
    import torch
    u = torch.rand(shape, generator=g, dtype=torch.float32) - 0.5
    v = -b * torch.sign(u) * torch.log1p(-2 * u.abs())
    return torch.clamp(torch.round(v), -127, 127).to(torch.int8)


class ConvTriple:
    """Device state and one step of the conv-triple workload."""

    def __init__(self, dev, seed=1236, restore_weights=True):
        import torch
        import torch.nn.functional as F
        from niti_amd import ops
        self.torch, self.ops, self.dev = torch, ops, dev
        self.restore_weights = restore_weights
        g = torch.Generator().manual_seed(seed)
        self.layers = []
        for (c, k, hw) in LAYERS:
            x = torch.randint(-127, 128, (BATCH, hw, hw, c), generator=g, dtype=torch.int8)
            w = torch.randint(-127, 128, (k, 3, 3, c), generator=g, dtype=torch.int8)
            e = laplace_i8(g, (BATCH, hw, hw, k))
            L = dict(c=c, k=k, hw=hw, x=x.to(dev), w=w.to(dev), err=e.to(dev))
            L["x16"] = F.pad(L["x"], (0, 16 - c % 16)).contiguous() if c % 16 else L["x"]
            # requantisation shifts of the layer's forward and data-gradient results, kept from step to step
            L["shift_f"] = torch.zeros(1, dtype=torch.int32, device=dev)
            L["shift_d"] = torch.zeros(1, dtype=torch.int32, device=dev)
            L["shift_w"] = torch.zeros(1, dtype=torch.int32, device=dev)
            self.layers.append(L)
        # zeroed words the single-launch conv + requantisation kernels exchange their tile ranges through
        off = 0
        for L in self.layers:
            for key, dgrad in (("sync_f", False), ("sync_d", True)):
                n = ops.conv_requant_sync_words(BATCH, L["hw"], L["hw"], L["x16"].shape[3] if not dgrad else L["c"], L["k"],
                                                dgrad=dgrad)
                L[key] = (off, n)
                off += n
            n = ops.wgrad_update_sync_words(BATCH, L["hw"], L["hw"], L["x16"].shape[3], L["k"])
            L["sync_w"] = (off, n)
            off += n
        sync_words = (max(off, 1) + 63) // 64 * 64
        self.ws = ops.scratch(256 << 20, dev)    # shared by all weight-gradient launches
        # Every step updates the weights (and their kernel-ready copies) in place.  So that each timed step multiplies
        # the operands the configuration names - weights uniform in [-127, 127] from the seed, not the saturated values
        # thousands of identical updates would leave - all weights and filter copies live in ONE buffer that the step
        # restores from a pristine copy with a single device copy before anything else.
        segs = []
        for L in self.layers:
            c, hw = L["c"], L["hw"]
            L["w16"] = F.pad(L["w"], (0, 16 - c % 16)).contiguous() if c % 16 else L["w"]
            L["wp"] = ops.conv_filter_prepare(L["w16"], BATCH, hw, hw)
            segs += [(L, "w"), (L, "wp")] if L["wp"] is not None else [(L, "w")]
        # ... and in front of them the words that every step must find zeroed (the sync words of all launches, then the
        # ranges of the two-pass paths): zeros in the pristine copy, so the one copy is also the step's only fill
        zero_bytes = ((sync_words + 3 * len(LAYERS)) * 4 + 255) // 256 * 256
        total = zero_bytes + sum((L[key].numel() + 255) // 256 * 256 for L, key in segs)
        self.wflat = torch.zeros(total, dtype=torch.int8, device=dev)
        self.zeroed = self.wflat[:zero_bytes].view(torch.int32)
        self.sync = self.zeroed[:sync_words]
        self.absmax = self.zeroed[sync_words:sync_words + 3 * len(LAYERS)]
        o = zero_bytes
        for L, key in segs:
            t = L[key]
            view = self.wflat[o:o + t.numel()].view(t.shape)
            view.copy_(t)
            if key == "w" and L["w16"] is t:
                L["w16"] = view
            L[key] = view
            o += (t.numel() + 255) // 256 * 256
        self.wpristine = self.wflat.clone()
        self.restore_bytes = total
        self.exp0 = torch.zeros(1, dtype=torch.int32, device=dev)
        self.ops_per_step = sum(conv_ops(BATCH, hw, c, k) * (2 if i == 0 else 3) for i, (c, k, hw) in enumerate(LAYERS))
        self.main_kernel_ops = []     # algorithmic ops of every launch bracketed by events, in launch order
        self.events = []           # forward and data-gradient launches (the dominant kernel)
        self.wgrad_events = []     # weight gradient + rounding + update (two kernels per bracket)

    def step(self, record=False):
        torch, ops = self.torch, self.ops
        import torch.nn.functional as F
        if self.restore_weights:
            self.wflat.copy_(self.wpristine)      # weights, filter copies and the zeroed words in one device copy
        else:
            self.zeroed.zero_()
        for i, L in enumerate(self.layers):
            c, k, hw = L["c"], L["k"], L["hw"]
            am = self.absmax[3 * i: 3 * i + 3]
            if L.get("wp") is None and c % 16:
                L["w16"] = F.pad(L["w"], (0, 16 - c % 16)).contiguous()
            w16 = L["w16"]        # with a maintained filter copy only its shape is used
            # forward + activation requantisation; the kernel-ready forward filter copy is made once and from then
            # on maintained by the weight update below
            wp = L.get("wp")
            if wp is None:
                wp = L["wp"] = ops.conv_filter_prepare(w16, BATCH, hw, hw)
            if record:
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                e0.record()
            so, sn = L["sync_f"]
            if sn:
                # the shift of the previous step is handed in as the prediction for this one
                ops.conv2d_fprop_requant(L["x16"], w16, 1, 1, f32_epilogue=True, sync=self.sync[so:so + sn], exp_a=self.exp0,
                                         exp_b=self.exp0, exp_out=torch.empty_like(self.exp0), prepared_filter=wp,
                                         shift_out=L["shift_f"], shift_hint=True)
            else:
                acc = ops.conv2d_fprop(L["x16"], w16, 1, 1, f32_epilogue=True, absmax=am[0:1], prepared_filter=wp)
            if record:
                e1.record()
                self.events.append((e0, e1, conv_ops(BATCH, hw, c, k), i, "fprop"))
            if not sn:
                ops.requant(acc, am[0:1], 7, "round", exp_a=self.exp0, exp_b=self.exp0, exp_out=torch.empty_like(self.exp0))
            # data gradient + error requantisation
            if i > 0:
                # the single-launch kernel reads the forward pass's filter copy; the two-pass path makes its own
                so, sn = L["sync_d"]
                wt = None if sn else ops.conv_filter_prepare(L["w"], BATCH, hw, hw, dgrad=True)
                if record:
                    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                    e0.record()
                if sn:
                    ops.conv2d_dgrad_requant(L["err"], L["w"], 1, 1, f32_epilogue=True, sync=self.sync[so:so + sn],
                                             forward_filter=wp, shift_out=L["shift_d"], shift_hint=True)
                else:
                    dx = ops.conv2d_dgrad(L["err"], L["w"], 1, 1, f32_epilogue=True, absmax=am[1:2], prepared_filter=wt)
                if record:
                    e1.record()
                    self.events.append((e0, e1, conv_ops(BATCH, hw, c, k), i, "dgrad"))
                if not sn:
                    ops.requant(dx, am[1:2], 7, "round")
            # weight gradient + gradient rounding + weight update
            so, sn = L["sync_w"]
            if record:
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                e0.record()
            if sn:
                ops.conv2d_wgrad_update(L["x16"], L["err"], L["w"], 1, 1, f32_epilogue=(i > 0), mu=5, method="psto",
                                        sync=self.sync[so:so + sn], workspace=self.ws, prepared_filter=L["wp"],
                                        shift_out=L["shift_w"], shift_hint=True)
            else:
                L["wp"] = None
                dw = ops.conv2d_wgrad(L["x16"], L["err"], 3, 3, 1, 1, f32_epilogue=(i > 0), absmax=am[2:3], workspace=self.ws)
                if c % 16:
                    dw = dw[..., :c].contiguous()     # zero-padded input channels give zero gradient columns
                ops.grad_update(dw, L["w"], am[2:3], 5, "psto")
            if record:
                e1.record()
                self.wgrad_events.append((e0, e1, conv_ops(BATCH, hw, c, k), i, "wgrad"))


class Runner:
    """Runs exactly n steps per call of run(n).  Warm up eagerly, then capture the step into HIP graphs (launch-bound
    chains of small kernels replay without per-launch host cost): one graph of a single step and, with unroll > 1, one
    of `unroll` consecutive steps - two consecutive graph launches leave the device idle for some microseconds, a
    longer graph has fewer such seams.  n steps = n // unroll replays of the long graph + n % unroll of the short one."""

    def __init__(self, step_fn, warmup, use_graph=True, unroll=1):
        import torch
        self.step_fn, self.mode, self.unroll, self.graphs = step_fn, "eager", 1, None
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for _ in range(max(warmup, 3)):
                step_fn()
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        if not use_graph:
            return
        try:
            graphs = []
            for u in ([1, unroll] if unroll > 1 else [1]):
                g = torch.cuda.CUDAGraph()
                # no cyclic garbage collection while capturing (freeing tensors of the eager warm-up, allocated on
                # another stream, makes the allocator record events, which a capturing process may not do)
                gc.collect()
                gc.disable()
                try:
                    with torch.cuda.graph(g):
                        for _ in range(u):
                            step_fn()
                finally:
                    gc.enable()
                g.replay()
                torch.cuda.synchronize()
                graphs.append(g)
            self.graphs, self.mode, self.unroll = graphs, "graph", max(unroll, 1)
        except Exception as e:  # capture refused: keep measuring, say so
            print("bench.py: graph capture failed (%s); timing eager launches" % e, file=sys.stderr)
            torch.cuda.synchronize()

    def run(self, n=1):
        if self.graphs is None:
            for _ in range(n):
                self.step_fn()
            return
        if self.unroll > 1:
            for _ in range(n // self.unroll):
                self.graphs[1].replay()
            n %= self.unroll
        for _ in range(n):
            self.graphs[0].replay()


def cpu_baseline(min_seconds=5.0):
    """The plain-C oracle (OpenMP) over the same six layer triples, on synthetic inputs of the same
    shapes, repeated until at least `min_seconds` of CPU work."""
    import torch
    from oracle import c_oracle as co
    co.build()
    g = torch.Generator().manual_seed(77)
    data = []
    for (c, k, hw) in LAYERS:
        data.append((torch.randint(-127, 128, (BATCH, hw, hw, c), generator=g, dtype=torch.int8),
                     torch.randint(-127, 128, (k, 3, 3, c), generator=g, dtype=torch.int8),
                     laplace_i8(g, (BATCH, hw, hw, k)), c, k, hw))
    ops_total, t_total, passes = 0.0, 0.0, 0
    while t_total < min_seconds and passes < 8:
        t0 = time.perf_counter()
        for i, (x, w, e, c, k, hw) in enumerate(data):
            acc = co.conv_fprop(x, w, 1, 1)
            co.requant(acc, 7, "round")
            if i > 0:
                co.requant(co.conv_dgrad(e, w, hw, hw, 1, 1), 7, "round")
            g8, _ = co.requant(co.conv_wgrad(x, e, 3, 3, 1, 1), 5, "psto")
            co.weight_update(w, g8)
            ops_total += conv_ops(BATCH, hw, c, k) * (2 if i == 0 else 3)
        t_total += time.perf_counter() - t0
        passes += 1
    return {"value": ops_total / t_total / 1e12, "unit": "TOPS", "cores": co.num_threads(), "kind": "port",
            "sample": "%d pass(es) of the full six-layer conv triple at batch %d (plain-C oracle, OpenMP), %.1f s" % (passes, BATCH, t_total)}


def cpu_baseline_train_step(batch=BATCH):
    """One complete integer training step of VGG-small (configs[3]) on the host cores: the reference's layer stack
    and reverse-order backward (ti_net.py:17-32, ti_torch.py:235-455) restated on torch CPU int32 tensors - integer
    convolutions through F.conv2d on int32 operands with the reference's own operand rewrites for the two gradients,
    int32 matrix products, the literal requantisation sequences.  One warm-up pass on a batch of 8, one timed pass."""
    import torch
    from oracle import niti_model_oracle as mo
    from niti_amd import ti_vgg
    cfg_list = ti_vgg.cifar_cfg[7]
    g = torch.Generator().manual_seed(1237 + 7)
    weights, c = [], 3
    for v in cfg_list:
        if v != 'M':
            weights.append(torch.randint(-127, 128, (v, 3, 3, c), generator=g, dtype=torch.int8))
            c = v
    weights.append(torch.randint(-127, 128, (10, 512 * 4 * 4), generator=g, dtype=torch.int8))
    mask = torch.randint(0, 2, (512 * 4 * 4,), generator=g, dtype=torch.int8)

    def one(n):
        net = mo.build_vgg(cfg_list, weights, [-8] * len(weights), mo.Cfg(), mask)
        x = torch.randint(-127, 128, (n, 32, 32, 3), generator=g, dtype=torch.int8)
        target = torch.randint(0, 10, (n,), generator=g)
        rand = torch.randint(0, 16, (n, 10), generator=g, dtype=torch.int32)
        t0 = time.perf_counter()
        net.forward_int8(x, 0)
        net.backward(target, rand)
        return time.perf_counter() - t0

    one(8)
    dt = one(batch)
    model = ""
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.startswith("model name"):
                    model = line.split(":", 1)[1].strip()
                    break
    except OSError:
        pass
    return {"value": batch / dt, "unit": "images/s", "seconds_per_step": round(dt, 3), "cores": torch.get_num_threads(),
            "os_cpu_count": os.cpu_count(), "cpu_model": model, "kind": "port",
            "sample": "1 warm-up pass at batch 8 + 1 timed pass of the full VGG-small (6 conv + FC) integer training step at "
                      "batch %d: forward, TiLoss gradient, backward, weight updates (torch CPU int32 restatement of the "
                      "reference's layers)" % batch}


def train_step_rate(dev, steps, warmup, depth=7, batch=BATCH, graph=True, unroll=1):
    """images/s of a complete integer training step: VGG-small (six conv + FC), batch 128 (configs[3]), or the
    ten-convolution VGG-13 widths, batch 256 (configs[4])."""
    import torch
    from niti_amd import ti_torch, ti_vgg
    g = torch.Generator().manual_seed(1237 + depth)
    net = ti_vgg.TiVGG_cifar(depth)
    for l in net.forward_layers:
        if hasattr(l, "weight"):
            l.weight = torch.randint(-127, 128, tuple(l.weight.shape), generator=g, dtype=torch.int8).to(dev)
            l.weight_exp = torch.tensor(-8.0)
    # the batch as the input quantiser delivers it (ops.quantize_input): int8 NHWC with the 3 channels zero-padded to 16
    x = torch.nn.functional.pad(torch.randint(-127, 128, (batch, 32, 32, 3), generator=g, dtype=torch.int8), (0, 13)).to(dev)
    target = torch.randint(0, 10, (batch,), generator=g).to(dev)
    ti_torch.TRAINING = True
    ti_torch.GRAD_BITWIDTH = 5

    def one():
        net.forward_int8(x, 0, target)      # the targets are known: the classifier's forward launch evaluates the loss gradient
        net.backward(target)

    runner = Runner(one, warmup, graph, unroll)
    runner.run(max(steps, 2 * runner.unroll))      # the clocks settle, both graphs have run
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    runner.run(steps)
    torch.cuda.synchronize()
    dt = (time.perf_counter() - t0) / steps
    return batch / dt, dt * 1e3, runner.mode


def _avg_us(fn, reps=20, warm=3):
    """Average duration of fn() in microseconds over `reps` back-to-back calls, by one HIP event pair on the launch
    stream around the whole run; a device sleep queued first lets the host run ahead, so the device never idles
    between the launches."""
    import torch
    for _ in range(warm):
        fn()
    torch.cuda.synchronize()
    torch.cuda._sleep(int(2e7))
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(reps):
        fn()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) * 1e3 / reps


def mfma_probe(dev):
    """What the matrix units sustain in a register-resident MFMA loop (no LDS, no memory traffic) for constant and for
    uniform random int8 operands: the shader clock follows the multipliers' power draw, so the second figure - not the
    datasheet peak - is the ceiling of kernels that multiply random data."""
    import torch
    from niti_amd import ops
    g = torch.Generator().manual_seed(4321)
    const = torch.ones(1 << 20, dtype=torch.int8, device=dev)
    rnd = torch.randint(-127, 128, (1 << 20,), generator=g, dtype=torch.int8).to(dev)
    zero = torch.zeros(1 << 20, dtype=torch.int8, device=dev)
    ops.mfma_probe(const)                              # clocks up
    # one workgroup (8 wavefronts) per compute unit: two wavefronts per SIMD, each issuing its run of products back to
    # back.  With two workgroups per compute unit the same loop reaches two thirds of this (four wavefronts of equal
    # priority take turns on a SIMD's matrix unit, and the changes of wavefront cost it idle clocks).
    one = dict(workgroups=256, iters=2400)
    zt, zg = ops.mfma_probe(zero, **one)
    ct, cg = ops.mfma_probe(const, **one)
    rt, rg = ops.mfma_probe(rnd, **one)
    rt2, rg2 = ops.mfma_probe(rnd)
    return {"zero_operands_tops": round(zt, 1), "zero_operands_clock_ghz": round(zg, 2),
            "constant_operands_tops": round(ct, 1), "constant_operands_clock_ghz": round(cg, 2),
            "random_operands_tops": round(rt, 1), "random_operands_clock_ghz": round(rg, 2),
            "random_operands_two_workgroups_per_cu_tops": round(rt2, 1), "random_operands_two_workgroups_per_cu_clock_ghz": round(rg2, 2),
            "note": "256 workgroups (one per compute unit) x 8 wavefronts x 2400 x 12 v_mfma_i32_32x32x32_i8 on register operands; "
                    "clock = shader cycle counter against the 100 MHz wall clock inside the loop; the last pair is the same loop "
                    "with 512 workgroups x 1200"}


def side_workloads(dev):
    """The other configurations and bandwidth kernels, each on its own roofline:
    config0  BASELINE configs[0]: one 128 -> 128 convolution on 128 x 32 x 32 + RoundShift requantisation
             (ti_torch.py:391-397), as one launch (MFMA roofline) and as the drop-in int32 convolution + separate
             requantisation (cutlassconv.cpp:57-73: HBM roofline, |x| + |w| + 4|y| bytes);
    config1  BASELINE configs[1]: fully connected layer 128 x 8192 x 1024, forward / data gradient / weight gradient
             with StoShift on supplied random integers (ti_torch.py:241-266, int8mm_kernel.cu:8-34), against the HBM
             roofline with m k + k n + m n bytes per pass;
    maxpool  2x2 / stride-2 int8 max-pool forward (1.25 |x| bytes) and backward (2.5 |x| bytes)."""
    import torch
    from niti_amd import ops
    g = torch.Generator().manual_seed(1234)
    out = {}
    # ---- config 0
    N, hw, c, k = 128, 32, 128, 128
    x = torch.randint(-127, 128, (N, hw, hw, c), generator=g, dtype=torch.int8).to(dev)
    w = torch.randint(-127, 128, (k, 3, 3, c), generator=g, dtype=torch.int8).to(dev)
    wp = ops.conv_filter_prepare(w, N, hw, hw)
    words = ops.conv_requant_sync_words(N, hw, hw, c, k)
    sync = torch.zeros(words, dtype=torch.int32, device=dev)
    shift = torch.zeros(1, dtype=torch.int32, device=dev)
    gop = conv_ops(N, hw, c, k) / 1e9

    def fused():
        sync.zero_()
        ops.conv2d_fprop_requant(x, w, f32_epilogue=True, sync=sync, prepared_filter=wp, shift_out=shift, shift_hint=True)

    def fill_only():
        sync.zero_()

    am = torch.zeros(1, dtype=torch.int32, device=dev)
    y32 = {}

    def dropin_conv():
        y32["y"] = ops.conv2d_fprop(x, w, 1, 1, f32_epilogue=True, prepared_filter=wp)

    def two_pass():
        am.zero_()
        acc = ops.conv2d_fprop(x, w, 1, 1, f32_epilogue=True, absmax=am, prepared_filter=wp)
        ops.requant(acc, am, 7, "round")

    t_fill = _avg_us(fill_only)
    t_fused = max(_avg_us(fused) - t_fill, 1e-3)
    t_conv = _avg_us(dropin_conv)
    t_two = max(_avg_us(two_pass) - t_fill, 1e-3)
    y_elems = N * hw * hw * k
    bytes_dropin = x.numel() + w.numel() + 4 * y_elems
    out["config0"] = {
        "workload": "BASELINE configs[0]: conv3x3 128->128 on 128x32x32 + RoundShift requantisation, %.2f GOP" % gop,
        "fused_us": round(t_fused, 2), "fused_tops": round(gop / t_fused * 1e3, 1),
        "fused_frac_mfma": round(gop / t_fused * 1e3 / INT8_MFMA_PEAK_TOPS, 4),
        "dropin_int32_conv_us": round(t_conv, 2), "dropin_gbs": round(bytes_dropin / t_conv * 1e-3, 1),
        "dropin_frac_hbm": round(bytes_dropin / t_conv * 1e-3 / HBM_PEAK_GBS, 4), "dropin_bytes": bytes_dropin,
        "two_pass_us": round(t_two, 2), "two_pass_tops": round(gop / t_two * 1e3, 1)}
    del y32, x, w
    # ---- config 1
    M, Fin, O = 128, 8192, 1024
    A = torch.randint(-127, 128, (M, Fin), generator=g, dtype=torch.int8).to(dev)
    W = torch.randint(-127, 128, (O, Fin), generator=g, dtype=torch.int8).to(dev)
    G = torch.randint(-127, 128, (M, O), generator=g, dtype=torch.int8).to(dev)
    u_f = torch.randint(0, 1 << 20, (M, O), generator=g, dtype=torch.int32).to(dev)
    u_d = torch.randint(0, 1 << 20, (M, Fin), generator=g, dtype=torch.int32).to(dev)
    u_w = torch.randint(0, 1 << 20, (O, Fin), generator=g, dtype=torch.int32).to(dev)
    Wu = W.clone()

    fsync = torch.zeros(max(ops.linear_sync_words(p, M, O, Fin) for p in ("forward", "dgrad", "wgrad")), dtype=torch.int32, device=dev)

    def fc_fwd():
        fsync.zero_()
        ops.linear_fwd_requant(A, W, 7, "sto", rand=u_f, sync=fsync)

    def fc_dgrad():
        fsync.zero_()
        ops.linear_dgrad_requant(G, W, 7, "sto", rand=u_d, sync=fsync)

    def fc_wgrad():
        fsync.zero_()
        ops.linear_wgrad_update(G, A, Wu, 5, "sto", rand=u_w, sync=fsync)

    fc = {"workload": "BASELINE configs[1]: fully connected 128x8192x1024, each pass one launch (int8 operands as stored, int32 "
                      "sums in registers, StoShift on supplied random integers); bytes = m k + k n + m n per pass "
                      "(the 4-byte random integer per output element is not counted)", "gop_per_pass": round(2.0 * M * Fin * O / 1e9, 3)}
    for name, fn, nbytes in (("fwd", fc_fwd, M * Fin + Fin * O + M * O), ("dgrad", fc_dgrad, M * O + O * Fin + M * Fin),
                             ("wgrad", fc_wgrad, O * M + M * Fin + O * Fin)):
        t = max(_avg_us(fn) - t_fill, 1e-3)
        fc[name + "_us"] = round(t, 2)
        fc[name + "_gbs"] = round(nbytes / t * 1e-3, 1)
        fc[name + "_frac_hbm"] = round(nbytes / t * 1e-3 / HBM_PEAK_GBS, 4)
        fc[name + "_tops"] = round(2.0 * M * Fin * O / t * 1e-6, 1)
    # what the weight-gradient launch moves: both operands, the weights in and out, one random integer per weight
    moved = O * M + M * Fin + 2 * O * Fin + 4 * O * Fin
    fc["wgrad_moved_bytes"] = moved
    fc["wgrad_moved_gbs"] = round(moved / fc["wgrad_us"] * 1e-3, 1)
    fc["wgrad_moved_frac_hbm"] = round(moved / fc["wgrad_us"] * 1e-3 / HBM_PEAK_GBS, 4)
    # the same three launches with the reference's default rounding (ti_torch.py:459-462: RoundShift for
    # activations and errors, PstoShift for gradients - no random integers to read)
    for name, fn in (("fwd_round", lambda: (fsync.zero_(), ops.linear_fwd_requant(A, W, 7, "round", sync=fsync))),
                     ("dgrad_round", lambda: (fsync.zero_(), ops.linear_dgrad_requant(G, W, 7, "round", sync=fsync))),
                     ("wgrad_psto", lambda: (fsync.zero_(), ops.linear_wgrad_update(G, A, Wu, 5, "psto", sync=fsync)))):
        fc[name + "_us"] = round(max(_avg_us(fn) - t_fill, 1e-3), 2)
    # the drop-in int32 products of the extension boundary, operands as the reference hands them over
    # (ti_torch.py:246,259,263: [m,k] and [k,n] row-major, the result the transposed view of an [n,m] buffer)
    from niti_amd.shims import int8mm_cuda
    Wt, Gt = W.t().contiguous(), G.t().contiguous()
    for name, lhs, rhs in (("fwd", A, Wt), ("dgrad", G, W), ("wgrad", Gt, A)):
        m_, k_, n_ = lhs.shape[0], lhs.shape[1], rhs.shape[1]
        t = _avg_us(lambda: int8mm_cuda.int8_mm(lhs, rhs))
        fc["dropin_int8_mm_" + name + "_us"] = round(t, 2)
        fc["dropin_int8_mm_" + name + "_gbs"] = round((m_ * k_ + k_ * n_ + 4 * m_ * n_) / t * 1e-3, 1)
    fc["dropin_note"] = "int8mm_cuda.int8_mm(lhs, rhs) -> int32, operands read as stored (one launch; the forward product splits its reduction over workgroups and adds the parts in a second launch); bytes = m k + k n + 4 m n"
    out["config1"] = fc
    del A, W, G, u_f, u_d, u_w, Wu, Wt, Gt
    # ---- max-pool
    xp = torch.randint(-127, 128, (128, 32, 32, 128), generator=g, dtype=torch.int8).to(dev)
    yp = ops.maxpool_fwd(xp)
    dy = torch.randint(-127, 128, tuple(yp.shape), generator=g, dtype=torch.int8).to(dev)
    t_f = _avg_us(lambda: ops.maxpool_fwd(xp))
    t_b = _avg_us(lambda: ops.maxpool_bwd(yp, dy, xp))
    nb = xp.numel()
    out["maxpool"] = {"workload": "2x2/stride-2 int8 max-pool on 128x32x32x128",
                      "fwd_us": round(t_f, 2), "fwd_gbs": round(1.25 * nb / t_f * 1e-3, 1), "fwd_frac_hbm": round(1.25 * nb / t_f * 1e-3 / HBM_PEAK_GBS, 4),
                      "bwd_us": round(t_b, 2), "bwd_gbs": round(2.5 * nb / t_b * 1e-3, 1), "bwd_frac_hbm": round(2.5 * nb / t_b * 1e-3 / HBM_PEAK_GBS, 4)}
    return out


TRAIN_STEPS = (("train_step", 7, BATCH, "BASELINE configs[3]: VGG-small (6 conv + FC) integer training step, batch 128"),
               ("train_step_vgg13", 13, 256, "BASELINE configs[4]: VGG-13 widths (10 conv + FC) integer training step, batch 256"))


# the reference's default batch size (options.py:3) and the only speeds it publishes: seconds per iteration in its
# committed training logs (results/int-vgg-small-{7,8,9}/results.log:12; data loading, display loss and host
# synchronisations included, GPU model not recorded)
TRAIN_STEPS_B256 = (("train_step_b256_vgg7", 7, 0.088), ("train_step_b256_vgg8", 8, 0.118), ("train_step_b256_vgg9", 9, 0.130))


def train_step_objects(dev, steps, warmup, graph=True, unroll=1):
    out = {}
    for name, depth, batch, workload in TRAIN_STEPS:
        try:
            ips, ms, mode = train_step_rate(dev, steps, warmup, depth, batch, graph, unroll)
            out[name] = {"workload": workload, "images_per_s": round(ips, 1), "ms_per_step": round(ms, 3), "launch_mode": mode,
                         "steps_per_graph": unroll if mode == "graph" else None,
                         "weights_state": "updated in place by every step, as in training; on the one repeated synthetic batch they "
                                          "drift towards +-127, which the conv-triple A/B (`weights`) shows to run about 7 % slower "
                                          "than seeded uniform weights"}
        except Exception as e:  # the headline line must still be printed
            out[name] = {"error": str(e)[:200]}
    for name, depth, ref_s in TRAIN_STEPS_B256:
        try:
            ips, ms, mode = train_step_rate(dev, steps, warmup, depth, 256, graph, unroll)
            out[name] = {"workload": "cifar_cfg[%d] of the reference (ti_vgg.py:10-14), integer training step at its default batch "
                                     "256 (options.py:3)" % depth,
                         "images_per_s": round(ips, 1), "ms_per_step": round(ms, 3), "launch_mode": mode,
                         "reference_published_s_per_iter": ref_s,
                         "reference_published_images_per_s": round(256 / ref_s, 1),
                         "reference_note": "results/int-vgg-small-%d/results.log:12, whole iteration (data loading, display "
                                           "loss, host synchronisations) on an unrecorded NVIDIA GPU: not the same quantity" % depth}
        except Exception as e:
            out[name] = {"error": str(e)[:200]}
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-train-step", action="store_true")
    ap.add_argument("--no-drift-ab", action="store_true",
                    help="skip timing the step without the per-step weight restore (weights drifting to +-127)")
    ap.add_argument("--no-side-workloads", action="store_true", help="skip config0 / config1 / max-pool figures")
    ap.add_argument("--sustained-seconds", type=float, default=1.0,
                    help="also replay the headline step back to back for at least this long (0: skip)")
    ap.add_argument("--train-steps-only", action="store_true",
                    help="run only the two training-step workloads and print their objects (for kernel traces of a step)")
    ap.add_argument("--side-workloads-only", action="store_true",
                    help="run only config0 / config1 / max-pool and the MFMA probe and print their objects (for kernel traces)")
    ap.add_argument("--eager", action="store_true", help="time eager launches instead of a captured HIP graph")
    ap.add_argument("--steps-per-graph", type=int, default=1,
                    help="consecutive steps captured into one HIP graph (K steps = K // U replays of it + K %% U of a one-step graph)")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run three plain 256 MiB device copies (a kernel of known traffic, to scale "
                         "rocprofv3 FETCH_SIZE / WRITE_SIZE readings)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU only (no collectives, no sharding); use --gpus 1", file=sys.stderr)
        return 2

    import torch
    import niti_amd
    niti_amd.require_library()
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        return 3
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)

    if args.calibrate_copy:
        src = torch.ones(256 << 20, dtype=torch.int8, device=dev)
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    if args.side_workloads_only:
        out = side_workloads(dev)
        out["mfma_probe"] = mfma_probe(dev)
        print(json.dumps(out))
        return 0

    if args.train_steps_only:
        print(json.dumps(train_step_objects(dev, args.steps, args.warmup, not args.eager, args.steps_per_graph)))
        return 0

    wl = ConvTriple(dev)
    runner = Runner(wl.step, args.warmup, not args.eager, args.steps_per_graph)
    mode = runner.mode
    from niti_amd import ops as _ops
    # The same step replayed back to back for a second or more.  It runs BEFORE the K timed steps: a process that has
    # just initialised the device finds it in its idle power state, and the first tens of milliseconds of work run at
    # lower clocks (K = 20 steps timed first read 5-6 % slower than the same 20 steps a second later).
    sustained = None
    if args.sustained_seconds > 0:
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        runner.run(args.steps)
        torch.cuda.synchronize()
        est_ms = (time.perf_counter() - t0) * 1e3 / args.steps
        n_rep = max(int(args.sustained_seconds * 1e3 / est_ms * 1.15), args.steps)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        runner.run(n_rep)
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        sustained = {"steps": n_rep, "seconds": round(dt, 3), "ms_per_step": round(dt * 1e3 / n_rep, 4),
                     "tops": round(wl.ops_per_step * n_rep / dt / 1e12, 2),
                     "first_steps_after_idle_ms_per_step": round(est_ms, 4)}
        if _ops.sync_timeouts(dev):
            sustained["error"] = "a grid-wide wait timed out"
        runner.run(args.warmup)     # the W untimed steps in front of the timed ones
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    runner.run(args.steps)
    torch.cuda.synchronize()
    ms_per_step = (time.perf_counter() - t0) * 1e3 / args.steps
    tops = wl.ops_per_step / (ms_per_step * 1e-3) / 1e12
    if _ops.sync_timeouts(dev):
        print("bench.py: a grid-wide wait timed out during the timed steps (the GPU was shared with other work); "
              "no result", file=sys.stderr)
        return 4

    # Dominant kernel: the MFMA implicit-GEMM convolution (forward + data-gradient launches), timed
    # per launch with HIP events on the launch stream over the same K steps run eagerly.  A device
    # sleep is queued first so that the host runs ahead of the GPU and the event pairs bracket
    # kernel execution, not host launch latency.
    torch.cuda._sleep(int(4e7))
    for _ in range(args.steps):
        wl.step(record=True)
    torch.cuda.synchronize()
    # what an event pair measures with nothing between its two records (the second marker's own processing);
    # taken off every bracket so that the figure is the kernel's duration as a kernel trace reports it
    torch.cuda._sleep(int(4e6))
    pairs = []
    for _ in range(256):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        e1.record()
        pairs.append((e0, e1))
    torch.cuda.synchronize()
    pair_ms = sorted(e0.elapsed_time(e1) for (e0, e1) in pairs)[len(pairs) // 2]
    k_ms = sum(max(ev[0].elapsed_time(ev[1]) - pair_ms, 0.0) for ev in wl.events)
    k_ops = sum(ev[2] for ev in wl.events)
    n_launch = len(wl.events)
    achieved = k_ops / (k_ms * 1e-3) / 1e12
    # per layer and direction: average bracket over the K eager steps (a weight-gradient bracket holds its two kernels)
    per_layer = []
    for i, (c, k, hw) in enumerate(LAYERS):
        row = {"layer": "%d->%d@%d" % (c, k, hw)}
        for direction, evs in (("fprop", wl.events), ("dgrad", wl.events), ("wgrad", wl.wgrad_events)):
            sel = [ev for ev in evs if ev[3] == i and ev[4] == direction]
            if not sel:
                continue
            us = sum(max(ev[0].elapsed_time(ev[1]) - pair_ms, 0.0) for ev in sel) * 1e3 / len(sel)
            t = sel[0][2] / (us * 1e-6) / 1e12
            row[direction] = {"us": round(us, 2), "tops": round(t, 1), "frac": round(t / INT8_MFMA_PEAK_TOPS, 4)}
        per_layer.append(row)
    # HBM bytes per launch of this kernel as the counters of an earlier rocprofv3 run gave them (the summary states
    # the figure on a line of its own); null when the summary is not there
    traffic = wgrad_traffic = None
    tpath = os.path.join(ROOT, "profiles", "conv_triple_hbm_traffic.txt")
    traffic_source = None
    if os.path.exists(tpath):
        traffic_source = "profiles/conv_triple_hbm_traffic.txt (rocprofv3 FETCH_SIZE / WRITE_SIZE of an earlier run of this command, " \
                         "scaled by a plain copy; counters cannot be read inside this run)"
        with open(tpath) as f:
            for line in f:
                if line.startswith("traffic_bytes_per_launch:"):
                    traffic = int(line.split(":", 1)[1].split()[0])
                if line.startswith("wgrad_traffic_bytes_per_launch:"):
                    wgrad_traffic = int(line.split(":", 1)[1].split()[0])
    # the weight-gradient family (layers 2-6: wgrad3x3_narrow_kernel with its finishing pass inside), same brackets
    wsel = [ev for ev in wl.wgrad_events if ev[3] > 0]
    w_ms = sum(max(ev[0].elapsed_time(ev[1]) - pair_ms, 0.0) for ev in wsel)
    w_ops = sum(ev[2] for ev in wsel)
    w_achieved = w_ops / (w_ms * 1e-3) / 1e12 if w_ms > 0 else 0.0
    w_alg_bytes = sum(BATCH * hw * hw * (c + k) + 3 * k * 9 * c for (c, k, hw) in LAYERS[1:]) / (len(LAYERS) - 1)
    roofline_wgrad = {"bound": "mfma", "achieved": round(w_achieved, 2), "peak": INT8_MFMA_PEAK_TOPS, "unit": "TFLOP/s",
                      "frac": round(w_achieved / INT8_MFMA_PEAK_TOPS, 4), "traffic": wgrad_traffic,
                      "traffic_source": traffic_source,
                      "kernel": "wgrad3x3_narrow_kernel<..., true> (weight gradient + gradient rounding + weight update + "
                                "filter copy, one launch; layers 2-6)",
                      "launches": len(wsel), "avg_launch_us": round(w_ms * 1e3 / max(len(wsel), 1), 2),
                      "ops_per_launch_avg": w_ops / max(len(wsel), 1), "algorithmic_bytes_per_launch_avg": int(w_alg_bytes),
                      "note": "algorithmic bytes = |x| + |err| + 3 |w| (weights read and written, kernel-ready filter copy written)"}
    roofline = {"bound": "mfma", "achieved": round(achieved, 2), "peak": INT8_MFMA_PEAK_TOPS, "unit": "TFLOP/s",
                "frac": round(achieved / INT8_MFMA_PEAK_TOPS, 4), "traffic": traffic, "traffic_source": traffic_source,
                "kernel": "conv3x3_halo_kernel<..., true, *> (convolution + requantisation)", "launches": n_launch,
                "avg_launch_us": round(k_ms * 1e3 / max(n_launch, 1), 2), "event_pair_overhead_us": round(pair_ms * 1e3, 2),
                "ops_per_launch_avg": k_ops / max(n_launch, 1),
                "note": "int8 multiply-accumulate counted as 2 ops; unit is tera-ops/s"}

    out = {"metric": "int8 TOPS, conv fwd/bwd (VGG-small conv stack triple, 1 GPU)", "value": round(tops, 2), "unit": "TOPS",
           "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms_per_step, 4),
           "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "int8 x int8 -> int32",
           "data": "synthetic",
           "config": {"workload": "BASELINE configs[2]: conv layer triple (fprop + act requant, dgrad + err requant, "
                                  "wgrad + grad rounding + weight update) over the six VGG-small conv shapes, batch 128, "
                                  "3x3 pad 1, uniform int8 inputs, Laplace int8 errors",
                      "ops_per_step": wl.ops_per_step, "batch": BATCH},
           "launch_mode": mode, "steps_per_graph": runner.unroll if mode == "graph" else None,
           "pct_int8_mfma_peak": round(100.0 * tops / INT8_MFMA_PEAK_TOPS, 2),
           "roofline": roofline, "roofline_wgrad": roofline_wgrad, "per_layer": per_layer}
    out["weights"] = {"state": "every step starts from the seeded uniform int8 weights: all weights and kernel-ready filter copies "
                               "are restored from a pristine copy by one device copy inside the timed step, which also zeroes the sync words (the "
                               "step's only fill)",
                      "restored_bytes_per_step": wl.restore_bytes}
    if not args.no_drift_ab:
        # the same step without the restore: the weights drift (the same gradient every step drives them to +-127)
        try:
            wl2 = ConvTriple(dev, restore_weights=False)
            r2 = Runner(wl2.step, args.warmup, not args.eager, args.steps_per_graph)
            r2.run(500)                    # saturates the weights, as a long run would
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            r2.run(args.steps)
            torch.cuda.synchronize()
            drift_ms = (time.perf_counter() - t0) * 1e3 / args.steps
            runner.run(args.steps)         # and the restored form again, right after it
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            runner.run(args.steps)
            torch.cuda.synchronize()
            fresh_ms = (time.perf_counter() - t0) * 1e3 / args.steps
            out["weights"].update({"fresh_ms_per_step": round(fresh_ms, 4), "drifted_ms_per_step": round(drift_ms, 4),
                                   "drifted_note": "no restore, weights updated in place for 500+ steps with the same inputs "
                                                   "(nearly all at +-127); timed back to back with the restored form"})
            del wl2, r2
        except Exception as e:
            out["weights"]["drift_ab_error"] = str(e)[:200]
    try:
        probe = mfma_probe(dev)
        out["mfma_probe"] = probe
        roofline["frac_of_random_operand_probe"] = round(achieved / probe["random_operands_tops"], 4)
        out["pct_of_random_operand_probe"] = round(100.0 * tops / probe["random_operands_tops"], 2)
    except Exception as e:
        out["mfma_probe"] = {"error": str(e)[:200]}
    if sustained is not None:
        out["sustained"] = sustained
    if not args.no_side_workloads:
        try:
            out.update(side_workloads(dev))
        except Exception as e:  # the headline line must still be printed
            out["side_workloads_error"] = str(e)[:300]
    if not args.no_train_step:
        out.update(train_step_objects(dev, max(args.steps, 5), max(args.warmup, 2), True, args.steps_per_graph))
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline()
        try:
            cb = cpu_baseline_train_step()
            out["cpu_baseline_train_step"] = cb
            if "images_per_s" in out.get("train_step", {}):
                out["train_step"]["vs_cpu_baseline"] = round(out["train_step"]["images_per_s"] / cb["value"], 1)
        except Exception as e:
            out["cpu_baseline_train_step"] = {"error": str(e)[:200]}
    print(json.dumps(out))
    return 0


if __name__ == "__main__":
    sys.exit(main())
