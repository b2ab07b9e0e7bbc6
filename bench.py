#!/usr/bin/env python3
"""Benchmark of the LIF fire forward+backward hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload cfg2|cfg3|cfg5|cfg5_bf16|cfg1|t96|t100|t120]
                    [--no-cpu-baseline] [--no-extra-legs]
    python bench.py --workload train_step [--steps K] [--warmup W]     (context figure, see below)
    python bench.py --workload cifar_step [--steps K] [--warmup W]     (context figure, see below)
    python bench.py --workload bn_fire    [--steps K] [--warmup W]     (next-row op, see below)
    python bench.py --workload bn         [--steps K] [--warmup W]     (next-row op, see below)
    python bench.py --workload policy_sweep                            (kernel rates over shapes, see below)

One "step" is one forward (spikes from the input current) plus one backward (input gradient from
the saved input current and the spike gradient) over one synthetic batch that is already resident
in HBM.  The default workload is the headline configuration ``T=8, B=64, C=128, 32x32`` fp32.
Exactly one JSON line is printed on stdout.

The timed region, and with it ``value``, ``ms_per_step`` and the top level of ``roofline``, is the path
a user of the reference's interface gets: the step loop calls ``snnlib.fire_s_fp(x, alpha, thresh)`` and
``snnlib.fire_bp(x, g, alpha, thresh, beta, interval)`` of the pybind module (the two calls of
``snnlib_func.FireFunc``), outputs come from PyTorch's caching allocator inside the calls, and no cache
hint is passed (the reference's interface has no way to express one), so tensors of more than 32 MiB run
the *streamed* kernels.  The loop rotates over several independent (x, g) sets, all forwards of a round
first, then all backwards, so that several times the capacity of the 256 MB memory-side cache passes
between a batch's forward and its backward, as the other layers of a network would put there: every
byte comes from HBM.

* ``value``      neuron-steps per second over the K timed steps (wall clock between two device
                 synchronisations).
* ``roofline``   the streamed backward kernel (the dominant one): algorithmic bytes per launch
                 (12 B x neuron-steps in fp32: read x, read grad_spike, write grad_x) divided by its
                 mean time in the timed region, against the 8 TB/s HBM peak.  Every dispatch of the timed
                 region carries a stop event on the launch stream; a kernel's time is the interval from
                 the completion of the kernel before it to its own (no stream-time overhead, and the
                 intervals add up to the wall clock: kernel duration plus a dispatch gap of about 1 us).  ``fwd`` and ``fwd_bwd`` give the same figure for the
                 forward kernel (8 B) and for the pair (20 B); ``module`` repeats the leg's wall-clock
                 figures and compares them with ``cabi_streamed``.
* ``roofline.cabi_streamed`` the same rotation through the C ABI (ctypes, pre-allocated outputs,
                 SNNLIF_STREAM_SPATIAL): what the module adds on top of the kernels shows as the difference.
* ``roofline.same_tensors`` the module again, one tensor set, backward straight after the forward step
                 after step (the pattern of the reference's test_fire.py): still the streamed kernels.
* ``roofline.kept`` the C ABI with the SNNLIF_KEEP_SPATIAL hint on one tensor set: the caller declares that
                 the backward follows the forward on the same input current, ``x`` is loaded with the
                 default cache policy and stays in the memory-side cache, and the launch shape is the
                 one that serves cache hits best.  Only a caller of the C ABI can ask for this.
* ``cpu_baseline`` the pure-PyTorch restatement of the reference's gold path
                 (``oracle/gold_fire.py``) on the host cores, forward + autograd backward on the same
                 inputs, best of 3 after a warm-up; its outputs also serve as the parity check of
                 this very run (``parity``).

``--workload train_step`` is not the headline metric: it runs one SGD step of a small synthetic
spiking CNN on CIFAR-shaped random data (conv / linear / pooling on PyTorch-ROCm, the four LIF layers
through ``snnlib_op.Fire``) and reports the end-to-end step time and the share of it spent in the
fire kernels, measured with events around the ``snnlib.fire_s_fp`` / ``snnlib.fire_bp`` calls.

``--workload cifar_step`` is a context figure too: one SGD step of the reference's CIFAR model
(snnlib/example/models.py:8-61: nine 3x3 convolutions of 128 / 256 / 512 channels, 8192-1024-512 fully
connected, every layer but the first a batch norm + fire fused with the dense op that follows) assembled from
this package's ``snnlib_op`` layers, with the batch size, window and optimiser of the reference's training
script (snnlib/example/train_test_cifar.py:19, 32: 64 images, SGD lr 1e-2 momentum 0.9; 6 steps) on random
CIFAR-shaped data.  Reports the step time and the GPU time inside each native op of the ``snnlib`` module
(events around the calls; a fused op's time includes its MIOpen / rocBLAS half).

``--workload bn_fire`` times the batch-norm + fire layer's training step (``snnlif_bn_stats``,
``snnlif_bn_fire_s_fp``, ``snnlif_bn_fire_bp``) at the headline shape through the C ABI: 4 B per
neuron-step for the batch statistics, 8 B forward, 20 B backward (two sweeps over x and the spike
gradient, one write of the input gradient), checked against the CPU oracle on a sample of channels.

``--workload policy_sweep`` lists forward / backward kernel rates in both cache policies over some twenty
shapes (the reference's callers, window lengths, tensor sizes, odd row pitches, odd neuron counts).

``--workload bn`` does the same for the plain batch norm (``snnlif_bn_stats``, ``snnlif_bn_fp``,
``snnlif_bn_bp``): 4 + 8 + 20 B per element.
"""
import argparse
import json
import os
import sys
import time

REPO = os.path.dirname(os.path.abspath(__file__))
if REPO not in sys.path:
    sys.path.insert(0, REPO)

HBM_PEAK_GBPS = 8000.0
ALPHA, THRESH, BETA, INTERVAL = 0.25, 0.5, 1.0, 0.5
SEED = 0

# name -> (shape [T,B,C,H,W], input mean, input std, storage dtype name)
WORKLOADS = {
    "cfg1": ((4, 8, 16, 8, 8), 0.5, 1.0, "float32"),
    "cfg2": ((8, 64, 128, 32, 32), 0.5, 1.0, "float32"),
    "cfg3": ((32, 32, 256, 16, 16), 0.3, 0.8, "float32"),
    "cfg5": ((16, 128, 512, 16, 16), 0.5, 1.0, "float32"),
    "cfg5_bf16": ((16, 128, 512, 16, 16), 0.5, 1.0, "bfloat16"),
    # no configuration of the reference: a 96-step window, the longest range of the backward that
    # still recomputes the whole window in registers (67 239 936 neuron-steps, 257 MiB per tensor)
    "t96": ((96, 4, 171, 32, 32), 0.5, 1.0, "float32"),
    # ... a 100-step one, which the backward runs as a 96-step body with a 4-step head (67 174 400
    # neuron-steps) ...
    "t100": ((100, 4, 164, 32, 32), 0.5, 1.0, "float32"),
    # ... and a 120-step one, which it cuts into a 32-step segment and an 88-step tail window (67 338 240
    # neuron-steps)
    "t120": ((120, 4, 137, 32, 32), 0.5, 1.0, "float32"),
}
# HBM bytes per launch of the backward kernel, measured with rocprofv3 --pmc FETCH_SIZE and WRITE_SIZE runs
# of this file (each counter scaled by its reading for a plain device copy of the same tensor:
# --copy-calibration).  Counters cannot be read from inside this process, so the figures are read from the
# tracked profile summary they were written to; a workload without one reports null.
TRAFFIC_PROFILES = {
    "cfg2": "profiles/pmc_fetch_write_fire_fwd_bwd_cfg2_f32.txt",
    "cfg3": "profiles/pmc_fetch_write_fire_fwd_bwd_cfg3_f32.txt",
    "cfg5": "profiles/pmc_fetch_write_fire_fwd_bwd_cfg5_f32.txt",
    "cfg5_bf16": "profiles/pmc_fetch_write_fire_fwd_bwd_cfg5_bf16.txt",
    "t96": "profiles/pmc_fetch_write_fire_fwd_bwd_t96_f32.txt",
    "t100": "profiles/pmc_fetch_write_fire_fwd_bwd_t100_f32.txt",
    "t120": "profiles/pmc_fetch_write_fire_fwd_bwd_t120_f32.txt",
    "bn_fire": "profiles/pmc_fetch_write_bn_fire_fwd_bwd_cfg2_f32.txt",
    "bn": "profiles/pmc_fetch_write_bn_fwd_bwd_cfg2_f32.txt",
}


def measured_traffic(workload):
    """{"source": path, "<pass>, <policy>": bytes, ...} from the "Scaled HBM traffic" table of the
    workload's PMC summary (lines `  <name> : <bytes> B = ...`), or {} when there is none."""
    import re
    rel = TRAFFIC_PROFILES.get(workload)
    path = os.path.join(REPO, rel) if rel else None
    if not path or not os.path.exists(path):
        return {}
    out = {"source": rel}
    in_table = False
    for line in open(path):
        if line.startswith("Scaled HBM traffic"):
            in_table = True
            continue
        if in_table:
            m = re.match(r"\s+([^:]+?)\s*:\s*(\d+) B\b", line)
            if m:
                out[" ".join(m.group(1).split())] = int(m.group(2))
            elif line.strip() and not line.startswith(" "):
                in_table = False
    return out


HEADLINE = "cfg2"
METRIC = "LIF fwd+bwd neuron-steps/s + HBM GB/s (% of peak), T=8,B=64,C=128,32x32"


def metric_name(workload, shape, dtype_name):
    """The headline configuration carries the metric's published name; every other workload says
    which shape it ran."""
    if workload == HEADLINE:
        return METRIC
    T, B, C, H, W = shape
    return f"LIF fwd+bwd neuron-steps/s + HBM GB/s (% of peak), T={T},B={B},C={C},{H}x{W} {dtype_name} ({workload})"


def backward_kernel_name(T, esize, lif_cabi):
    """Which kernel the library launches for a backward window of T steps (fp32 arithmetic: fp32 or bf16
    storage).  One register window (a multiple of 8 steps, or that plus a head of up to 7 steps) up to
    111 steps (bf16 with a head: up to 63), 32-step segments up to 1024, the workspace stream beyond."""
    if T > lif_cabi.BP_NO_WORKSPACE_MAX_T:
        return "lif_backward_stream_kernel"
    body = T // 8 * 8
    whole = T <= lif_cabi.BP_FUSED_MAX_T or (T == body and T <= 104)
    headed = body <= 104 and (esize == 4 or body + 7 <= 64)
    return "lif_backward_fused_kernel" if whole or headed else "lif_backward_segmented_kernel"


def make_inputs(torch, shape, mean, std, dtype):
    """Seeded on the CPU so the host baseline and the GPU see identical bits."""
    gen = torch.Generator().manual_seed(SEED)
    x = torch.randn(shape, generator=gen).mul_(std).add_(mean).to(dtype)
    g = torch.randn(shape, generator=gen).to(dtype)
    return x, g


def cpu_baseline(torch, x, g, repeats=3):
    """Time oracle/gold_fire.py (forward + autograd backward) on the host; return timing + outputs."""
    from oracle import gold_fire

    xf, gf = x.float(), g.float()
    threads = torch.get_num_threads()
    best = None
    outs = None
    for it in range(repeats + 1):  # first pass is the warm-up
        xr = xf.clone().requires_grad_(True)
        t0 = time.perf_counter()
        u, s = gold_fire.gold_fire(xr, ALPHA, THRESH, BETA, INTERVAL)
        t1 = time.perf_counter()
        s.backward(gf)
        t2 = time.perf_counter()
        if it > 0 and (best is None or (t2 - t0) < best[0]):
            best = (t2 - t0, t1 - t0, t2 - t1)
        outs = (s.detach(), xr.grad.detach())
        del u, s, xr
    return best, threads, outs


def tensor_sets(tensor_bytes):
    """How many independent tensor sets the rotating legs cycle through: four (two for tensors beyond
    512 MiB), more for small tensors so that a cycle moves at least 2 GiB of inputs."""
    sets = 4 if tensor_bytes <= (512 << 20) else 2
    while sets * 2 * tensor_bytes < (2 << 30):
        sets *= 2
    return min(sets, 64)


def rotation_leg(torch, lif_cabi, sets, steps, warmup, forward, backward, bytes_fwd, bytes_bwd,
                 neuron_steps, instrumented=None):
    """K steps over `sets` independent tensor sets in rounds: forward(j) for every set j of the round,
    then backward(j) for every set, so that between a set's forward and its backward lie the other
    sets' forwards and backwards, several times the capacity of the memory-side cache.  A round holds
    `sets` steps (the last one what is left of K).

    Every dispatch of the timed region carries a stop event (snnlif_time_next_kernel with no start
    event: the completion of the kernel on the launch stream); a kernel's time is the interval from the
    completion of the kernel before it to its own.  A stop event alone adds nothing to the stream
    (measured: the wall clock per step is the same with and without), the intervals add up to the wall
    clock, and in a saturated stream they are the kernels' durations plus the dispatch gap of about a
    microsecond -- what a kernel costs in a sequence of launches.  (A start event as well costs 4-5 us
    of stream time per dispatch, and on a dispatch that follows an un-instrumented one that time falls
    inside the bracket.)"""
    def run(n, events):
        k = i = 0
        while k < n:
            r = min(sets, n - k)
            for fn in (forward, backward):
                for j in range(r):
                    if events is not None:
                        lif_cabi.time_next_kernel(None, events[i][1])
                        events[i][0] = fn is forward
                        i += 1
                    fn(j)
            k += r
        return time.perf_counter()

    run(max(warmup, sets), None)
    events = [[None, torch.cuda.Event(enable_timing=True)] for _ in range(2 * steps)]
    begin = torch.cuda.Event(enable_timing=True)
    for e in events:   # create them on the device side before handing out their handles
        e[1].record()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    begin.record()
    t_enqueued = run(steps, events)
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    wall = t1 - t0
    # intervals between consecutive completions; the first one starts at a stream marker, not at a
    # kernel's completion, and is left out
    spans = [(events[i][0], events[i - 1][1].elapsed_time(events[i][1])) for i in range(1, len(events))]
    fwd = [ms for is_fwd, ms in spans if is_fwd]
    bwd = [ms for is_fwd, ms in spans if not is_fwd]
    fwd_ms, bwd_ms = sum(fwd) / len(fwd), sum(bwd) / len(bwd)
    rate = lambda nbytes, ms: nbytes / (ms * 1e-3) / 1e9
    return {
        "sets": sets, "steps": steps, "launches_timed": len(spans),
        "ms_per_step": wall / steps * 1e3,
        "host_enqueue_ms_per_step": (t_enqueued - t0) / steps * 1e3,
        "neuron_steps_per_s": neuron_steps * steps / wall,
        "fwd": {"kernel": "lif_forward_kernel", "algorithmic_bytes_per_launch": bytes_fwd, "avg_launch_ms": fwd_ms,
                "achieved": rate(bytes_fwd, fwd_ms), "frac": rate(bytes_fwd, fwd_ms) / HBM_PEAK_GBPS},
        "bwd": {"algorithmic_bytes_per_launch": bytes_bwd, "avg_launch_ms": bwd_ms,
                "achieved": rate(bytes_bwd, bwd_ms), "frac": rate(bytes_bwd, bwd_ms) / HBM_PEAK_GBPS},
        "fwd_bwd": {"algorithmic_bytes": bytes_fwd + bytes_bwd, "kernel_ms": fwd_ms + bwd_ms,
                    "achieved": rate(bytes_fwd + bytes_bwd, fwd_ms + bwd_ms),
                    "frac": rate(bytes_fwd + bytes_bwd, fwd_ms + bwd_ms) / HBM_PEAK_GBPS},
    }


def build_synthetic_snn(torch, fire_factory, seed=0):
    """conv3x3(3->128)-LIF-conv3x3(128->256)-LIF-avgpool2-conv3x3(256->256)-LIF-avgpool2-
    linear(256*8*8->1024)-LIF-linear(1024->10) on [T, B, ...] tensors; output averaged over T.
    Convolutions and linears see T folded into the batch.  Kaiming-normal weights, zero biases."""
    nn = torch.nn

    class TimeFolded(nn.Module):
        def __init__(self, layer):
            super().__init__()
            self.layer = layer

        def forward(self, x):
            T, B = x.shape[0], x.shape[1]
            y = self.layer(x.reshape(T * B, *x.shape[2:]))
            return y.reshape(T, B, *y.shape[1:])

    class Flatten(nn.Module):
        def forward(self, x):
            return x.reshape(x.shape[0], x.shape[1], -1)

    torch.manual_seed(seed)
    net = nn.Sequential(
        TimeFolded(nn.Conv2d(3, 128, 3, padding=1)), fire_factory(),
        TimeFolded(nn.Conv2d(128, 256, 3, padding=1)), fire_factory(),
        TimeFolded(nn.AvgPool2d(2)),
        TimeFolded(nn.Conv2d(256, 256, 3, padding=1)), fire_factory(),
        TimeFolded(nn.AvgPool2d(2)),
        Flatten(),
        TimeFolded(nn.Linear(256 * 8 * 8, 1024)), fire_factory(),
        TimeFolded(nn.Linear(1024, 10)),
    )
    for m in net.modules():
        if isinstance(m, (nn.Conv2d, nn.Linear)):
            nn.init.kaiming_normal_(m.weight)
            nn.init.zeros_(m.bias)
    return net


def synthetic_batch(torch, T=8, B=64, seed=0):
    gen = torch.Generator().manual_seed(seed)
    images = torch.rand((B, 3, 32, 32), generator=gen)
    labels = torch.randint(0, 10, (B,), generator=gen)
    return images.unsqueeze(0).repeat(T, 1, 1, 1, 1), labels


def run_train_step(args):
    import torch
    from snn_gpu_training_bptt_amd import snnlib_func as sf
    from snn_gpu_training_bptt_amd import snnlib_op as sop

    if not torch.cuda.is_available():
        sys.exit("bench.py: no ROCm GPU visible")
    dev = torch.device("cuda:0")
    sf.alpha, sf.thresh, sf.beta, sf.interval = ALPHA, THRESH, BETA, INTERVAL
    T, B = 8, 64
    net = build_synthetic_snn(torch, sop.Fire).to(dev)
    opt = torch.optim.SGD(net.parameters(), lr=0.1)
    crit = torch.nn.CrossEntropyLoss()
    x, labels = synthetic_batch(torch, T, B)
    x, labels = x.to(dev), labels.to(dev)

    # events around the native fire calls: a proxy in place of the module object snnlib_func uses
    native = sf.snnlib
    spans = []

    class TimedOps:
        def __getattr__(self, name):
            fn = getattr(native, name)

            def timed(*a):
                e0 = torch.cuda.Event(enable_timing=True)
                e1 = torch.cuda.Event(enable_timing=True)
                e0.record()
                out = fn(*a)
                e1.record()
                spans.append((name, a[0].numel(), e0, e1))
                return out
            return timed

    def one_step():
        opt.zero_grad(set_to_none=True)
        out = net(x).mean(dim=0)
        loss = crit(out, labels)
        loss.backward()
        opt.step()
        return loss

    for _ in range(args.warmup):
        one_step()
    torch.cuda.synchronize()
    sf.snnlib = TimedOps()
    try:
        t0 = time.perf_counter()
        for _ in range(args.steps):
            loss = one_step()
        torch.cuda.synchronize()
        t1 = time.perf_counter()
    finally:
        sf.snnlib = native
    step_ms = (t1 - t0) / args.steps * 1e3
    lif_ms = sum(e0.elapsed_time(e1) for _, _, e0, e1 in spans) / args.steps
    lif_ns = sum(n for _, n, _, _ in spans) // (2 * args.steps)   # each layer appears in fwd and bwd
    print(json.dumps({
        "metric": "synthetic SNN training step (context figure, not the headline metric)",
        "value": step_ms, "unit": "ms/step", "higher_is_better": False, "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": step_ms, "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": "train_step: conv3x3(3-128)-LIF-conv3x3(128-256)-LIF-pool-conv3x3(256-256)-"
                               "LIF-pool-fc(16384-1024)-LIF-fc(1024-10), T=8 B=64 CIFAR-shaped random data, "
                               "SGD lr 0.1, CE on the time-averaged output"},
        "lif_ms_per_step": lif_ms, "lif_share": lif_ms / step_ms,
        "lif_neuron_steps_per_step": lif_ns,
        "lif_algorithmic_GBps": 20 * lif_ns / (lif_ms * 1e-3) / 1e9,
        "final_loss": float(loss.item()),
    }), flush=True)


def run_cifar_step(args):
    import torch
    from snn_gpu_training_bptt_amd import snnlib_func as sf
    from snn_gpu_training_bptt_amd import snnlib_op as sop

    if not torch.cuda.is_available():
        sys.exit("bench.py: no ROCm GPU visible")
    dev = torch.device("cuda:0")
    T, B = 6, 64
    sf.time_step = T

    class Cifar(torch.nn.Module):
        def __init__(self):
            super().__init__()
            s1, s2, p = (1, 1), (2, 2), (1, 1)
            self.conv1_1 = sop.Conv(3, 128, kernel_size=(3, 3), stride=s1, padding=p)
            self.conv1_2 = sop.BnFireConv(128, 128, kernel_size=(3, 3), stride=s1, padding=p)
            self.conv1_3 = sop.BnFireConv(128, 128, kernel_size=(3, 3), stride=s2, padding=p)
            self.conv2_1 = sop.BnFireConv(128, 256, kernel_size=(3, 3), stride=s1, padding=p)
            self.conv2_2 = sop.BnFireConv(256, 256, kernel_size=(3, 3), stride=s1, padding=p)
            self.conv2_3 = sop.BnFireConv(256, 256, kernel_size=(3, 3), stride=s2, padding=p)
            self.conv3_1 = sop.BnFireConv(256, 512, kernel_size=(3, 3), stride=s1, padding=p)
            self.conv3_2 = sop.BnFireConv(512, 512, kernel_size=(3, 3), stride=s1, padding=p)
            self.conv3_3 = sop.BnFireConv(512, 512, kernel_size=(3, 3), stride=s2, padding=p)
            self.fc1 = sop.BnFireFc(4 * 4 * 512, 1024, dim_bn=(0, 1, 3, 4), cin_bn=512)
            self.fc2 = sop.BnFireFc(1024, 512, dim_bn=(0, 1))
            self.bn = sop.BnFire(512, dim_bn=(0, 1))
            self.fc3 = torch.nn.Linear(512, 10)
            self.stack = ("conv1_1", "conv1_2", "conv1_3", "conv2_1", "conv2_2", "conv2_3", "conv3_1",
                          "conv3_2", "conv3_3", "fc1", "fc2", "bn")

        def forward(self, images):
            x = torch.stack([images for _ in range(T)], dim=0)
            for name in self.stack:
                x = getattr(self, name)(x)
            return self.fc3(x.mean(dim=0))

    torch.manual_seed(SEED)
    net = Cifar().to(dev)
    gen = torch.Generator().manual_seed(SEED)
    images = torch.rand((B, 3, 32, 32), generator=gen).to(dev)
    labels = torch.randint(0, 10, (B,), generator=gen).to(dev)
    opt = torch.optim.SGD([q for n, q in net.named_parameters() if "running" not in n], lr=1e-2, momentum=0.9)
    crit = torch.nn.CrossEntropyLoss()

    native = sf.snnlib
    spans = []

    class TimedOps:
        def __getattr__(self, name):
            fn = getattr(native, name)

            def timed(*a):
                e0 = torch.cuda.Event(enable_timing=True)
                e1 = torch.cuda.Event(enable_timing=True)
                e0.record()
                out = fn(*a)
                e1.record()
                spans.append((name, e0, e1))
                return out
            return timed

    def one_step():
        opt.zero_grad(set_to_none=True)
        loss = crit(net(images), labels)
        loss.backward()
        opt.step()
        return loss

    for _ in range(max(args.warmup, 2)):     # (MIOpen picks its algorithms during the first steps)
        one_step()
    torch.cuda.synchronize()
    sf.snnlib = TimedOps()
    try:
        t0 = time.perf_counter()
        for _ in range(args.steps):
            loss = one_step()
        torch.cuda.synchronize()
        t1 = time.perf_counter()
    finally:
        sf.snnlib = native
    step_ms = (t1 - t0) / args.steps * 1e3
    per_op = {}
    for name, e0, e1 in spans:
        per_op[name] = per_op.get(name, 0.0) + e0.elapsed_time(e1) / args.steps
    fused_free = sum(v for k, v in per_op.items() if k in ("bn_stats", "bn_fire_s_fp", "bn_fire_bp"))
    print(json.dumps({
        "metric": "CIFAR_BN training step (context figure, not the headline metric)",
        "value": step_ms, "unit": "ms/step", "higher_is_better": False, "n_gpus": 1,
        "steps": args.steps, "warmup": max(args.warmup, 2), "ms_per_step": step_ms, "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": "cifar_step: the reference's CIFAR_BN model (models.py:8-61) from snnlib_op layers, "
                               f"T={T} B={B}, random CIFAR-shaped batch, SGD lr 1e-2 momentum 0.9, cross entropy"},
        "images_per_s": B / (step_ms * 1e-3),
        "native_op_ms_per_step": {k: round(v, 4) for k, v in sorted(per_op.items(), key=lambda kv: -kv[1])},
        "native_ops_ms_per_step": sum(per_op.values()),
        "ops_without_a_dense_half_ms_per_step": fused_free,
        "final_loss": float(loss.item()),
    }), flush=True)


def run_bn(args, plain):
    """The training step of a batch-norm layer at the headline shape through the C ABI: batch statistics,
    forward, backward.  plain = False: batch norm folded into the fire recurrence (snnlif_bn_fire_*);
    plain = True: the batch norm on its own (snnlif_bn_fp / snnlif_bn_bp)."""
    import numpy as np
    import torch
    from snn_gpu_training_bptt_amd import lif_cabi

    if not torch.cuda.is_available():
        sys.exit("bench.py: no ROCm GPU visible")
    lif_cabi.load()
    dev = torch.device("cuda:0")
    shape = (8, 64, 128, 32, 32)
    T, B, C, HW = shape[0], shape[1], shape[2], shape[3] * shape[4]
    ns = T * B * C * HW
    eps = 1e-5
    name = "bn" if plain else "bn_fire"
    gen = torch.Generator(device=dev).manual_seed(SEED)
    x = 0.5 + torch.randn(shape, generator=gen, device=dev)
    g = torch.randn(shape, generator=gen, device=dev)
    weight = 0.5 + torch.rand(C, generator=gen, device=dev)
    bias = 0.2 * torch.randn(C, generator=gen, device=dev)
    var, mean = torch.empty_like(weight), torch.empty_like(weight)
    stats_ws = torch.empty(lif_cabi.bn_stats_workspace_bytes(lif_cabi.DTYPE_F32, T, B, C, HW),
                           dtype=torch.uint8, device=dev)
    lif_cabi.bn_stats_into(x, mean, var, stats_ws)
    ivar, out = torch.empty_like(var), torch.empty_like(x)
    gx, gw, gb = torch.empty_like(x), torch.empty_like(weight), torch.empty_like(weight)
    ws_bytes = (lif_cabi.bn_bp_workspace_bytes if plain else lif_cabi.bn_fire_bp_workspace_bytes)(
        lif_cabi.DTYPE_F32, T, B, C, HW)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)

    def stats(xk=x):
        lif_cabi.bn_stats_into(xk, mean, var, stats_ws)

    def fwd(xk=x, outk=out, keep=True):
        if plain:
            lif_cabi.bn_fp_into(xk, weight, bias, var, mean, ivar, outk, eps)
        else:
            # step loop: the backward follows straight on the same tensors, x is worth keeping in the
            # cache; cold leg: no hint, as the layer calls it
            lif_cabi.bn_fire_s_fp_into(xk, weight, bias, var, mean, ivar, outk, eps, ALPHA, THRESH,
                                       keep_spatial=True if keep else None)

    def bwd(xk=x, gk=g, gxk=gx):
        if plain:
            lif_cabi.bn_bp_into(xk, weight, ivar, mean, gk, gxk, gw, gb, ws)
        else:
            lif_cabi.bn_fire_bp_into(xk, weight, bias, ivar, mean, gk, gxk, gw, gb, ALPHA, THRESH, BETA,
                                     INTERVAL, ws)

    for _ in range(args.warmup):
        stats()
        fwd()
        bwd()
    if args.copy_calibration:      # plain device copies of known size, to scale PMC readings by
        torch.cuda.synchronize()
        scratch_copy = torch.empty_like(x)
        for _ in range(3):
            scratch_copy.copy_(x)
        torch.cuda.synchronize()
        del scratch_copy
    # a step is what the layer does in training: batch statistics, forward, backward.  The statistics
    # and the backward are several kernels each: stream markers around each pass (dispatch gaps included)
    ev = [[torch.cuda.Event(enable_timing=True) for _ in range(4)] for _ in range(args.steps)]
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for k in range(args.steps):
        ev[k][0].record()
        stats()
        ev[k][1].record()
        fwd()
        ev[k][2].record()
        bwd()
        ev[k][3].record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    stats_ms = sum(e[0].elapsed_time(e[1]) for e in ev) / args.steps
    fwd_ms = sum(e[1].elapsed_time(e[2]) for e in ev) / args.steps
    bwd_ms = sum(e[2].elapsed_time(e[3]) for e in ev) / args.steps

    traffic = measured_traffic(name)
    bwd_traffic = [v for k, v in traffic.items() if k.startswith("backward")]
    rate = lambda nbytes, ms: nbytes / (ms * 1e-3) / 1e9
    if plain:
        title = "Bn statistics+fwd+bwd elements/s (next-row op, not the headline metric)"
        what = f"bn: plain batch norm fwd+bwd, [T,B,C,H,W]={list(shape)} float32, batch statistics, eps={eps}"
        kernels = "bn_plain_sums_wave_kernel + bn_channel_reduce_finalize_kernel + bn_plain_input_kernel"
        fwd_kernel = "bn_plain_forward_kernel"
    else:
        title = "BnFire statistics+fwd+bwd neuron-steps/s (next-row op, not the headline metric)"
        what = (f"bn_fire: batch-norm + LIF fire fwd+bwd, [T,B,C,H,W]={list(shape)} float32, batch statistics, "
                f"eps={eps}, alpha={ALPHA} thresh={THRESH} beta={BETA} interval={INTERVAL}")
        kernels = "lif_bn_backward_partial_kernel + bn_channel_reduce/finalize + lif_bn_backward_input_kernel"
        fwd_kernel = "lif_bn_forward_kernel"
    result = {
        "metric": title,
        "value": ns * args.steps / wall, "unit": "elements/s" if plain else "neuron-steps/s", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": wall / args.steps * 1e3,
        "higher_is_better": True, "dtype": "f32", "data": "synthetic",
        "config": {"workload": what},
        "roofline": {"kernel": kernels,
                     "policy": "step loop on one tensor set (statistics, forward, backward back to back)",
                     "bound": "hbm", "algorithmic_bytes_per_launch": 20 * ns, "avg_launch_ms": bwd_ms,
                     "achieved": rate(20 * ns, bwd_ms), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": rate(20 * ns, bwd_ms) / HBM_PEAK_GBPS,
                     "traffic": sum(bwd_traffic) if bwd_traffic else None,
                     "traffic_source": traffic.get("source"),
                     "fwd": {"kernel": fwd_kernel, "algorithmic_bytes_per_launch": 8 * ns, "avg_launch_ms": fwd_ms,
                             "achieved": rate(8 * ns, fwd_ms), "frac": rate(8 * ns, fwd_ms) / HBM_PEAK_GBPS},
                     "stats": {"kernel": "bn_stats_wave_kernel + bn_stats_finalize_kernel",
                               "algorithmic_bytes_per_launch": 4 * ns, "avg_launch_ms": stats_ms,
                               "achieved": rate(4 * ns, stats_ms), "frac": rate(4 * ns, stats_ms) / HBM_PEAK_GBPS}},
    }
    if not args.no_extra_legs:
        # the layer with nothing cached between its forward and its backward: four tensor sets, all
        # (statistics + forward), then all backwards; events bracket each operation (for the
        # statistics and the backward: all of their kernels, dispatch gaps included)
        sets, rounds = 4, 5
        xs = [x] + [x.clone() for _ in range(sets - 1)]
        gs = [g] + [g.clone() for _ in range(sets - 1)]
        outs = [torch.empty_like(x) for _ in range(sets)]
        gxs = [torch.empty_like(x) for _ in range(sets)]
        cev = [[[torch.cuda.Event(enable_timing=True) for _ in range(6)] for _ in range(sets)] for _ in range(rounds + 1)]
        for per_round in cev:
            for per_set in per_round:
                for e in per_set:
                    e.record()
        torch.cuda.synchronize()
        for r in range(rounds + 1):
            for k in range(sets):
                e = cev[r][k]
                lif_cabi.time_next_kernel(e[0], e[1])
                stats(xs[k])
                lif_cabi.time_next_kernel(e[2], e[3])
                fwd(xs[k], outs[k], keep=False)
            for k in range(sets):
                e = cev[r][k]
                lif_cabi.time_next_kernel(e[4], e[5])
                bwd(xs[k], gs[k], gxs[k])
        torch.cuda.synchronize()
        timed = [e for per_round in cev[1:] for e in per_round]
        avg = lambda a, b: sum(e[a].elapsed_time(e[b]) for e in timed) / len(timed)
        cs, cf, cb = avg(0, 1), avg(2, 3), avg(4, 5)
        result["roofline"]["cold"] = {
            "what": f"{sets} independent tensor sets, all (statistics + forward) then all backwards, {rounds} timed "
                    "rounds after one untimed; events bracket each operation",
            "policy": "no hint, as the layer calls the ops; every byte of the backward from HBM",
            "stats": {"avg_ms": cs, "achieved": rate(4 * ns, cs), "frac": rate(4 * ns, cs) / HBM_PEAK_GBPS},
            "fwd": {"avg_ms": cf, "achieved": rate(8 * ns, cf), "frac": rate(8 * ns, cf) / HBM_PEAK_GBPS},
            "stats_fwd": {"avg_ms": cs + cf, "achieved": rate(12 * ns, cs + cf),
                          "frac": rate(12 * ns, cs + cf) / HBM_PEAK_GBPS},
            "bwd": {"avg_ms": cb, "achieved": rate(20 * ns, cb), "frac": rate(20 * ns, cb) / HBM_PEAK_GBPS},
            "outputs_equal_across_sets": bool(all(torch.equal(o, outs[0]) for o in outs[1:])
                                              and all(torch.equal(q, gxs[0]) for q in gxs[1:])),
        }
        if plain:
            # the bias gradient of a layer that ends in a convolution, the same reduction without the squares:
            # snnlif_channel_sum against the framework's torch.sum over the same axes, both cold
            total = torch.empty_like(weight)
            sev = [[[torch.cuda.Event(enable_timing=True) for _ in range(4)] for _ in range(sets)]
                   for _ in range(rounds + 1)]
            for per_round in sev:   # (torch only reads an event it has recorded itself once)
                for per_set in per_round:
                    per_set[0].record()
                    per_set[1].record()
            torch.cuda.synchronize()
            for r in range(rounds + 1):
                for k in range(sets):
                    lif_cabi.time_next_kernel(sev[r][k][0], sev[r][k][1])
                    lif_cabi.channel_sum_into(gs[k], total, stats_ws)
                for k in range(sets):
                    sev[r][k][2].record()
                    framework_total = torch.sum(gs[k], dim=(0, 1, 3, 4))
                    sev[r][k][3].record()
            torch.cuda.synchronize()
            timed = [e for per_round in sev[1:] for e in per_round]
            ours = sum(e[0].elapsed_time(e[1]) for e in timed) / len(timed)
            framework = sum(e[2].elapsed_time(e[3]) for e in timed) / len(timed)
            exact = gs[0].double().sum(dim=(0, 1, 3, 4))
            result["roofline"]["cold"]["channel_sum"] = {
                "kernel": "bn_stats_wave_kernel + bn_stats_finalize_kernel (sums only)",
                "avg_ms": ours, "achieved": rate(4 * ns, ours), "frac": rate(4 * ns, ours) / HBM_PEAK_GBPS,
                "framework_sum_avg_ms": framework,
                "max_error_vs_float64": float((total.double() - exact).abs().max()),
                "framework_max_error_vs_float64": float((framework_total.double() - exact).abs().max())}
        del xs, gs, outs, gxs

    if not args.no_cpu_baseline:
        # CPU leg: the scalar C loops of the oracle on a bounded sample (channels are independent given
        # their statistics; the backward's means are those of the sample), one host thread.  Its
        # forward outputs double as the parity check of this run.
        from oracle import c_oracle
        pick = [0, 1, C // 2, C - 1]
        take = lambda t: t[:, :8, pick].contiguous().cpu().numpy()
        p = lambda t: t[pick].cpu().numpy()
        xs, gs = take(x), take(g)
        t0 = time.perf_counter()
        if plain:
            ivar_o, out_o = c_oracle.bn_forward(xs, p(weight), p(bias), p(var), p(mean), eps)
            t1 = time.perf_counter()
            c_oracle.bn_backward(xs, p(weight), ivar_o, p(mean), gs)
        else:
            ivar_o, _, out_o = c_oracle.bn_fire_forward(xs, p(weight), p(bias), p(var), p(mean), eps, ALPHA, THRESH)
            t1 = time.perf_counter()
            c_oracle.bn_fire_backward(xs, p(weight), p(bias), ivar_o, p(mean), gs, ALPHA, THRESH, BETA, INTERVAL)
        t2 = time.perf_counter()
        result["cpu_baseline"] = {
            "value": xs.size / (t2 - t0), "unit": result["unit"], "cores": 1, "kind": "port",
            "sample": f"channels {pick} of batch entries [0, 8) ({xs.size} elements), forward + backward of "
                      "oracle/lif_oracle.c (scalar C loops), single run",
            "fwd_s": t1 - t0, "bwd_s": t2 - t1}
        result["parity"] = {("sampled_output_bit_exact" if plain else "sampled_spikes_bit_exact"):
                            bool(np.array_equal(take(out), out_o)),
                            "sampled_ivar_bit_exact": bool(np.array_equal(p(ivar), ivar_o))}
    print(json.dumps(result), flush=True)


# Shapes of the policy sweep: the reference's own callers of Fire, window lengths 4-32 at about 256 MiB,
# tensor sizes 8 MiB - 1 GiB at 8 steps, row pitches that are an odd multiple of 4 KiB, neuron counts
# that are not a multiple of the workgroup size.
SWEEP_SHAPES = [
    ((6, 64, 4096), "Alexnet_BN_DIST.fire (models.py:78,100)"),
    ((6, 64, 512, 7, 7), "Resnet_DIST.fire (models.py:145,183)"),
    ((4, 64, 256, 32, 32), "T=4, 256 MiB"),
    ((6, 64, 128, 32, 32), "T=6, 192 MiB"),
    ((8, 64, 128, 32, 32), "T=8, 256 MiB (configuration 2)"),
    ((12, 64, 64, 32, 32), "T=12, 192 MiB"),
    ((16, 64, 64, 32, 32), "T=16, 256 MiB"),
    ((24, 32, 64, 32, 32), "T=24, 192 MiB"),
    ((32, 32, 256, 16, 16), "T=32, 256 MiB (configuration 3)"),
    ((8, 64, 4, 32, 32), "T=8, 8 MiB"),
    ((8, 64, 16, 32, 32), "T=8, 32 MiB"),
    ((8, 64, 32, 32, 32), "T=8, 64 MiB"),
    ((8, 64, 64, 32, 32), "T=8, 128 MiB"),
    ((8, 64, 256, 32, 32), "T=8, 512 MiB"),
    ((8, 64, 512, 32, 32), "T=8, 1 GiB"),
    ((16, 128, 512, 16, 16), "T=16, 1 GiB (configuration 5)"),
    ((8, 63, 127, 32, 32), "T=8, row pitch 8001 x 4 KiB"),
    ((16, 65, 63, 32, 32), "T=16, row pitch 4095 x 4 KiB"),
    ((32, 33, 61, 32, 32), "T=32, row pitch 2013 x 4 KiB"),
    ((8, 63, 127, 31, 33), "T=8, N = 8185023 (odd)"),
    ((6, 50, 100, 17, 19), "T=6, N = 1615000, 37 MiB"),
    ((20, 32, 64, 32, 32), "T=20, 160 MiB"),
    ((26, 40, 64, 32, 32), "T=26 (24-step body + 2-step head), 260 MiB"),
    ((40, 16, 100, 32, 32), "T=40, 250 MiB"),
    ((100, 4, 164, 32, 32), "T=100 (96-step body + 4-step head), 256 MiB"),
    ((120, 4, 137, 32, 32), "T=120 (segmented backward), 257 MiB"),
]


def run_policy_sweep(args):
    """Forward and backward kernel rates in both cache policies over shapes the launch policy was not
    tuned on.  Streamed: rotation over independent tensor sets (cold cache), SNNLIF_STREAM_SPATIAL; kept:
    one tensor set, backward straight after the forward, SNNLIF_KEEP_SPATIAL.  Kernel durations from
    events attached to the dispatches.  `no_hint` names the policy the library picks by itself."""
    import torch
    from snn_gpu_training_bptt_amd import lif_cabi

    if not torch.cuda.is_available():
        sys.exit("bench.py: no ROCm GPU visible")
    lif_cabi.load()
    dev = torch.device("cuda:0")
    rows = []
    for shape, what in SWEEP_SHAPES:
        T = shape[0]
        ns = 1
        for d in shape:
            ns *= d
        gen = torch.Generator(device=dev).manual_seed(SEED)
        x = 0.5 + torch.randn(shape, generator=gen, device=dev)
        g = torch.randn(shape, generator=gen, device=dev)
        tensor_bytes = ns * 4
        sets = tensor_sets(tensor_bytes)
        xs = [x] + [x.clone() for _ in range(sets - 1)]
        gs = [g] + [g.clone() for _ in range(sets - 1)]
        spikes = [torch.empty_like(x) for _ in range(sets)]
        gxs = [torch.empty_like(x) for _ in range(sets)]
        steps = max(sets * 3, 12)
        streamed = rotation_leg(
            torch, lif_cabi, sets, steps, sets,
            lambda j: lif_cabi.fire_s_fp_into(xs[j], spikes[j], ALPHA, THRESH, keep_spatial=False),
            lambda j: lif_cabi.fire_bp_into(xs[j], gs[j], gxs[j], ALPHA, THRESH, BETA, INTERVAL, keep_spatial=False),
            8 * ns, 12 * ns, ns)
        s_ref, gx_ref = spikes[0].clone(), gxs[0].clone()
        kept = rotation_leg(
            torch, lif_cabi, 1, 24, 4,
            lambda j: lif_cabi.fire_s_fp_into(x, spikes[0], ALPHA, THRESH, keep_spatial=True),
            lambda j: lif_cabi.fire_bp_into(x, g, gxs[0], ALPHA, THRESH, BETA, INTERVAL, keep_spatial=True),
            8 * ns, 12 * ns, ns)
        same = bool(torch.equal(spikes[0], s_ref) and torch.equal(gxs[0], gx_ref))
        rows.append({"shape": list(shape), "what": what, "tensor_MiB": round(tensor_bytes / 2**20, 1),
                     "row_pitch_bytes": ns // T * 4, "no_hint": "kept" if tensor_bytes <= (32 << 20) else "streamed",
                     "streamed": {"fwd_us": streamed["fwd"]["avg_launch_ms"] * 1e3, "fwd_frac": streamed["fwd"]["frac"],
                                  "bwd_us": streamed["bwd"]["avg_launch_ms"] * 1e3, "bwd_frac": streamed["bwd"]["frac"],
                                  "pair_frac": streamed["fwd_bwd"]["frac"]},
                     "kept": {"fwd_us": kept["fwd"]["avg_launch_ms"] * 1e3, "fwd_frac": kept["fwd"]["frac"],
                              "bwd_us": kept["bwd"]["avg_launch_ms"] * 1e3, "bwd_frac": kept["bwd"]["frac"],
                              "pair_frac": kept["fwd_bwd"]["frac"]},
                     "policies_agree_bit_for_bit": same})
        print(f"{str(list(shape)):24s} {rows[-1]['tensor_MiB']:7.1f} MiB | streamed fwd {rows[-1]['streamed']['fwd_frac']:.3f} "
              f"bwd {rows[-1]['streamed']['bwd_frac']:.3f} | kept fwd {rows[-1]['kept']['fwd_frac']:.3f} "
              f"bwd {rows[-1]['kept']['bwd_frac']:.3f} | {what}", file=sys.stderr, flush=True)
        del xs, gs, spikes, gxs, x, g, s_ref, gx_ref
        torch.cuda.empty_cache()
    print(json.dumps({"metric": "LIF fire kernel rates over shapes (fraction of the 8 TB/s HBM peak of algorithmic bytes; "
                                "not the headline metric)", "unit": "fraction of peak", "n_gpus": 1, "dtype": "f32",
                      "data": "synthetic", "config": {"workload": "policy_sweep"}, "rows": rows}), flush=True)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--workload", default="cfg2", choices=sorted(WORKLOADS) + ["train_step", "cifar_step", "bn_fire", "bn", "policy_sweep"])
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-extra-legs", "--no-cold-leg", dest="no_extra_legs", action="store_true",
                    help="run the timed region only (fire workloads: no cabi_streamed / same_tensors / kept "
                         "blocks; bn_fire, bn: no cold-cache leg)")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run three plain device copies of the input tensor (known size: one "
                         "read + one write of it) so that rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE "
                         "readings can be scaled to bytes")
    args = ap.parse_args()

    if args.gpus != 1:
        sys.exit("bench.py: this build measures one GPU only (the fire op needs no communication; "
                 "neurons shard across GPUs with zero exchange). Run with --gpus 1.")

    if args.workload == "cifar_step":
        if args.steps == 200:
            args.steps = 10
        if args.warmup == 20:
            args.warmup = 3
        return run_cifar_step(args)
    if args.workload == "train_step":
        if args.steps == 200:
            args.steps = 10
        if args.warmup == 20:
            args.warmup = 3
        return run_train_step(args)

    if args.workload == "policy_sweep":
        return run_policy_sweep(args)

    if args.workload in ("bn_fire", "bn"):
        return run_bn(args, plain=args.workload == "bn")

    import torch
    from snn_gpu_training_bptt_amd import lif_cabi
    from snn_gpu_training_bptt_amd._loader import load_snnlib

    if not torch.cuda.is_available():
        sys.exit("bench.py: no ROCm GPU visible")
    lif_cabi.load()          # raises if the HIP library has not been built
    snnlib = load_snnlib()   # the pybind module the reference's autograd functions call; raises likewise
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)

    shape, mean, std, dtype_name = WORKLOADS[args.workload]
    dtype = getattr(torch, dtype_name)
    T = shape[0]
    n_steps_total = 1
    for d in shape:
        n_steps_total *= d  # neuron-steps per pass
    esize = torch.empty((), dtype=dtype).element_size()
    bytes_fwd = 2 * esize * n_steps_total
    bytes_bwd = 3 * esize * n_steps_total
    traffic = measured_traffic(args.workload)

    x_cpu, g_cpu = make_inputs(torch, shape, mean, std, dtype)
    x = x_cpu.to(dev)
    g = g_cpu.to(dev)
    sets = tensor_sets(x.numel() * esize)
    xs = [x] + [x.clone() for _ in range(sets - 1)]
    gs = [g] + [g.clone() for _ in range(sets - 1)]

    if args.copy_calibration:
        scratch_copy = torch.empty_like(x)
        for _ in range(3):
            scratch_copy.copy_(x)
        torch.cuda.synchronize()
        del scratch_copy

    # ---- the timed region: the module's two calls, rotating over the tensor sets ----
    # The outputs of a round stay referenced until the next round replaces them (a network keeps a
    # layer's spikes for the next layer), so the allocator hands out distinct blocks within a round.
    spikes, gxs = [None] * sets, [None] * sets

    def module_forward(j):
        spikes[j] = snnlib.fire_s_fp(xs[j], ALPHA, THRESH)

    def module_backward(j):
        gxs[j] = snnlib.fire_bp(xs[j], gs[j], ALPHA, THRESH, BETA, INTERVAL)

    head = rotation_leg(torch, lif_cabi, sets, args.steps, args.warmup, module_forward, module_backward,
                        bytes_fwd, bytes_bwd, n_steps_total)
    spike, gx = spikes[0], gxs[0]
    same_across_sets = all(torch.equal(sp, spike) for sp in spikes[1:] if sp is not None) and \
        all(torch.equal(q, gx) for q in gxs[1:] if q is not None)
    spikes, gxs = [spike], [gx]   # release the other sets' outputs
    spike_rate = float(spike.float().mean().item())
    bwd_kernel = backward_kernel_name(T, esize, lif_cabi)

    result = {
        "metric": metric_name(args.workload, shape, dtype_name),
        "value": head["neuron_steps_per_s"],
        "unit": "neuron-steps/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": head["ms_per_step"],
        "host_enqueue_ms_per_step": head["host_enqueue_ms_per_step"],
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32" if dtype == torch.float32 else "bf16-storage/f32-arithmetic",
        "data": "synthetic",
        "config": {
            "workload": f"{args.workload}: LIF fire fwd+bwd, [T,B,C,H,W]={list(shape)} {dtype_name}, "
                        f"x~N({mean},{std}) g~N(0,1) seed {SEED}, alpha={ALPHA} thresh={THRESH} "
                        f"beta={BETA} interval={INTERVAL}",
            "neuron_steps_per_step": n_steps_total,
            "spike_rate": round(spike_rate, 4),
            "path": "snnlib.fire_s_fp + snnlib.fire_bp (pybind module, outputs from the caching allocator, "
                    f"no cache hint), {sets} tensor sets in rotation: all forwards of a round, then all backwards",
        },
        "roofline": {
            "kernel": bwd_kernel,
            "policy": "streamed (no hint: what the module launches for tensors beyond 32 MiB; every byte from HBM)"
                      if x.numel() * esize > (32 << 20) else "kept (no hint: tensors of at most 32 MiB)",
            "bound": "hbm",
            "achieved": head["bwd"]["achieved"],
            "peak": HBM_PEAK_GBPS,
            "unit": "GB/s",
            "frac": head["bwd"]["frac"],
            "traffic": traffic.get("backward, streamed"),
            "traffic_source": traffic.get("source"),
            "algorithmic_bytes_per_launch": bytes_bwd,
            "avg_launch_ms": head["bwd"]["avg_launch_ms"],
            "timing": f"completion-to-completion intervals of stop events attached to every dispatch of the timed "
                      f"region ({head['launches_timed']} intervals over {args.steps} steps; they add up to the wall clock)",
            "fwd": head["fwd"],
            "fwd_bwd": head["fwd_bwd"],
            "module": {"policy": "streamed", "ms_per_step": head["ms_per_step"],
                       "host_enqueue_ms_per_step": head["host_enqueue_ms_per_step"],
                       "kernel_ms_per_step": head["fwd_bwd"]["kernel_ms"],
                       "neuron_steps_per_s": head["neuron_steps_per_s"],
                       "outputs_equal_across_sets": bool(same_across_sets)},
        },
    }

    if not args.no_extra_legs:
        code = {torch.float32: lif_cabi.DTYPE_F32, torch.bfloat16: lif_cabi.DTYPE_BF16}[dtype]
        ws_bytes = lif_cabi.fire_bp_workspace_bytes(code, T, n_steps_total // T)
        ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev) if ws_bytes else None
        extra_steps = min(args.steps, 100)

        # the same rotation through the C ABI: pre-allocated outputs, the streamed kernels asked for by name
        c_spikes = [torch.empty_like(x) for _ in range(sets)]
        c_gxs = [torch.empty_like(x) for _ in range(sets)]
        cabi = rotation_leg(
            torch, lif_cabi, sets, extra_steps, sets,
            lambda j: lif_cabi.fire_s_fp_into(xs[j], c_spikes[j], ALPHA, THRESH, keep_spatial=False),
            lambda j: lif_cabi.fire_bp_into(xs[j], gs[j], c_gxs[j], ALPHA, THRESH, BETA, INTERVAL, workspace=ws,
                                            keep_spatial=False),
            bytes_fwd, bytes_bwd, n_steps_total)
        cabi["policy"] = "streamed (SNNLIF_STREAM_SPATIAL), C ABI through ctypes, pre-allocated outputs"
        cabi["outputs_equal_to_module"] = bool(torch.equal(c_spikes[0], spike) and torch.equal(c_gxs[0], gx))
        cabi["bwd"]["traffic"] = traffic.get("backward, streamed")
        del c_spikes, c_gxs
        result["roofline"]["cabi_streamed"] = cabi
        result["roofline"]["module"]["wall_vs_cabi_streamed"] = head["ms_per_step"] / cabi["ms_per_step"]
        result["roofline"]["module"]["kernels_vs_cabi_streamed"] = \
            head["fwd_bwd"]["kernel_ms"] / cabi["fwd_bwd"]["kernel_ms"]

        # the module on one tensor set, backward straight after the forward, step after step
        one = {}

        def same_forward(j):
            one["spike"] = snnlib.fire_s_fp(x, ALPHA, THRESH)

        def same_backward(j):
            one["gx"] = snnlib.fire_bp(x, g, ALPHA, THRESH, BETA, INTERVAL)

        same = rotation_leg(torch, lif_cabi, 1, extra_steps, 5, same_forward, same_backward, bytes_fwd,
                            bytes_bwd, n_steps_total)
        same["policy"] = ("streamed kernels (no hint), one tensor set: the backward runs straight after the "
                          "forward on the same input current, step after step")
        one.clear()
        result["roofline"]["same_tensors"] = same

        # the C ABI with the caller's promise that x is read again soon
        k_spike, k_gx = torch.empty_like(x), torch.empty_like(x)
        kept = rotation_leg(
            torch, lif_cabi, 1, extra_steps, 5,
            lambda j: lif_cabi.fire_s_fp_into(x, k_spike, ALPHA, THRESH, keep_spatial=True),
            lambda j: lif_cabi.fire_bp_into(x, g, k_gx, ALPHA, THRESH, BETA, INTERVAL, workspace=ws,
                                            keep_spatial=True),
            bytes_fwd, bytes_bwd, n_steps_total)
        kept["policy"] = ("kept (SNNLIF_KEEP_SPATIAL), C ABI through ctypes, one tensor set, backward straight after "
                          "the forward: x stays in the 256 MB memory-side cache, so part of the bytes never "
                          "come from HBM; not reachable through the reference's interface")
        kept["outputs_equal_to_module"] = bool(torch.equal(k_spike, spike) and torch.equal(k_gx, gx))
        kept["bwd"]["traffic"] = traffic.get("backward, kept")
        del k_spike, k_gx
        result["roofline"]["kept"] = kept

    del xs, gs

    if not args.no_cpu_baseline:
        best, threads, (s_ref, gx_ref) = cpu_baseline(torch, x_cpu, g_cpu)
        # per-core figure: one thread on the first eighth of the batch
        b8 = max(1, shape[1] // 8)
        torch.set_num_threads(1)
        best_1t, _, _ = cpu_baseline(torch, x_cpu[:, :b8].contiguous(), g_cpu[:, :b8].contiguous(), repeats=2)
        torch.set_num_threads(threads)
        ns_1t = n_steps_total // shape[1] * b8
        total_s, fwd_s, bwd_s = best
        s_gpu = spike.float().cpu()
        gx_gpu = gx.float().cpu()
        if dtype != torch.float32:  # storage rounding of the outputs is the only difference
            gx_ref_cmp = gx_ref.to(dtype).float()
        else:
            gx_ref_cmp = gx_ref
        denom = gx_ref_cmp.abs().clamp_min(1e-30)
        result["cpu_baseline"] = {
            "value": n_steps_total / total_s,
            "unit": "neuron-steps/s",
            "cores": threads,
            "kind": "port",
            "sample": f"the full {args.workload} tensor, forward + autograd backward of "
                      f"oracle/gold_fire.py (pure PyTorch, fp32) on the host, 1 warm-up then best of 3",
            "fwd_s": fwd_s,
            "bwd_s": bwd_s,
            "host_cpus": os.cpu_count(),
            "one_thread": {"value": ns_1t / best_1t[0], "unit": "neuron-steps/s", "cores": 1,
                           "sample": f"batch entries [0, {b8}) of the same tensor, best of 2"},
        }
        result["parity"] = {
            "what": "outputs of the timed region (module path, set 0) against the CPU gold path",
            "spikes_bit_exact": bool(torch.equal(s_gpu, s_ref)),
            "spike_mismatches": int((s_gpu != s_ref).sum().item()),
            "grad_bit_exact": bool(torch.equal(gx_gpu, gx_ref_cmp)),
            "grad_max_rel_err": float(((gx_gpu - gx_ref_cmp).abs() / denom).max().item()),
        }

    print(json.dumps(result), flush=True)


if __name__ == "__main__":
    main()
