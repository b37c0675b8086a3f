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

    def __init__(self, dev, seed=1236):
        import torch
        import torch.nn.functional as F
        from niti_amd import ops
        self.torch, self.ops, self.dev = torch, ops, dev
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
        # one buffer, hence one fill per step: the sync words, then (256-byte aligned) the ranges of the two-pass paths
        sync_words = (max(off, 1) + 63) // 64 * 64
        self.zeroed = torch.zeros(sync_words + 3 * len(LAYERS), dtype=torch.int32, device=dev)
        self.sync = self.zeroed[:sync_words]
        self.absmax = self.zeroed[sync_words:]
        self.ws = ops.scratch(256 << 20, dev)    # shared by all weight-gradient launches
        self.exp0 = torch.zeros(1, dtype=torch.int32, device=dev)
        self.ops_per_step = sum(conv_ops(BATCH, hw, c, k) * (2 if i == 0 else 3) for i, (c, k, hw) in enumerate(LAYERS))
        self.main_kernel_ops = []     # algorithmic ops of every launch bracketed by events, in launch order
        self.events = []

    def step(self, record=False):
        torch, ops = self.torch, self.ops
        import torch.nn.functional as F
        self.zeroed.zero_()
        for i, L in enumerate(self.layers):
            c, k, hw = L["c"], L["k"], L["hw"]
            am = self.absmax[3 * i: 3 * i + 3]
            if L.get("wp") is None or not c % 16:
                L["w16"] = F.pad(L["w"], (0, 16 - c % 16)).contiguous() if c % 16 else L["w"]
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
                self.events.append((e0, e1, conv_ops(BATCH, hw, c, k)))
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
                    self.events.append((e0, e1, conv_ops(BATCH, hw, c, k)))
                if not sn:
                    ops.requant(dx, am[1:2], 7, "round")
            # weight gradient + gradient rounding + weight update
            so, sn = L["sync_w"]
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


def make_runner(step_fn, warmup, use_graph=True):
    """Warm up eagerly, then capture one step into a HIP graph (launch-bound chains of small kernels
    replay without per-launch host cost).  Returns (callable, "graph" | "eager")."""
    import torch
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(max(warmup, 3)):
            step_fn()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    if not use_graph:
        return step_fn, "eager"
    try:
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            step_fn()
        for _ in range(2):
            g.replay()
        torch.cuda.synchronize()
        return g.replay, "graph"
    except Exception as e:  # capture refused: keep measuring, say so
        print("bench.py: graph capture failed (%s); timing eager launches" % e, file=sys.stderr)
        torch.cuda.synchronize()
        return step_fn, "eager"


def cpu_baseline(min_seconds=10.0):
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


def train_step_rate(dev, steps, warmup, depth=7, batch=BATCH, graph=True):
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
    x = torch.randint(-127, 128, (batch, 32, 32, 3), generator=g, dtype=torch.int8).to(dev)
    target = torch.randint(0, 10, (batch,), generator=g).to(dev)
    ti_torch.TRAINING = True
    ti_torch.GRAD_BITWIDTH = 5

    def one():
        net.forward_int8(x, 0)
        net.backward(target)

    run, mode = make_runner(one, warmup, graph)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        run()
    torch.cuda.synchronize()
    dt = (time.perf_counter() - t0) / steps
    return batch / dt, dt * 1e3, mode


TRAIN_STEPS = (("train_step", 7, BATCH, "BASELINE configs[3]: VGG-small (6 conv + FC) integer training step, batch 128"),
               ("train_step_vgg13", 13, 256, "BASELINE configs[4]: VGG-13 widths (10 conv + FC) integer training step, batch 256"))


def train_step_objects(dev, steps, warmup, graph=True):
    out = {}
    for name, depth, batch, workload in TRAIN_STEPS:
        try:
            ips, ms, mode = train_step_rate(dev, steps, warmup, depth, batch, graph)
            out[name] = {"workload": workload, "images_per_s": round(ips, 1), "ms_per_step": round(ms, 3), "launch_mode": mode}
        except Exception as e:  # the headline line must still be printed
            out[name] = {"error": str(e)[:200]}
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-train-step", action="store_true")
    ap.add_argument("--train-steps-only", action="store_true",
                    help="run only the two training-step workloads and print their objects (for kernel traces of a step)")
    ap.add_argument("--eager", action="store_true", help="time eager launches instead of a captured HIP graph")
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

    if args.train_steps_only:
        print(json.dumps(train_step_objects(dev, args.steps, args.warmup, not args.eager)))
        return 0

    wl = ConvTriple(dev)
    run, mode = make_runner(wl.step, args.warmup, not args.eager)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        run()
    torch.cuda.synchronize()
    ms_per_step = (time.perf_counter() - t0) * 1e3 / args.steps
    tops = wl.ops_per_step / (ms_per_step * 1e-3) / 1e12

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
    k_ms = sum(max(e0.elapsed_time(e1) - pair_ms, 0.0) for (e0, e1, _) in wl.events)
    k_ops = sum(o for (_, _, o) in wl.events)
    n_launch = len(wl.events)
    achieved = k_ops / (k_ms * 1e-3) / 1e12
    # HBM bytes per launch of this kernel as the counters of an earlier rocprofv3 run gave them (the summary states
    # the figure on a line of its own); null when the summary is not there
    traffic = None
    tpath = os.path.join(ROOT, "profiles", "conv_triple_hbm_traffic.txt")
    if os.path.exists(tpath):
        with open(tpath) as f:
            for line in f:
                if line.startswith("traffic_bytes_per_launch:"):
                    traffic = int(line.split(":", 1)[1].split()[0])
    roofline = {"bound": "mfma", "achieved": round(achieved, 2), "peak": INT8_MFMA_PEAK_TOPS, "unit": "TFLOP/s",
                "frac": round(achieved / INT8_MFMA_PEAK_TOPS, 4), "traffic": traffic,
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
           "launch_mode": mode,
           "pct_int8_mfma_peak": round(100.0 * tops / INT8_MFMA_PEAK_TOPS, 2),
           "roofline": roofline}
    if not args.no_train_step:
        out.update(train_step_objects(dev, max(args.steps, 5), max(args.warmup, 2)))
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline()
    print(json.dumps(out))
    return 0


if __name__ == "__main__":
    sys.exit(main())
