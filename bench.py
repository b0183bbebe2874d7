#!/usr/bin/env python3
"""
Benchmark of the gated linear scan on one MI355X.

A step is one forward + one backward scan over one batch of the Mamba-like
configuration, fp32 [B=8, C=2048, T=4096] (a = sigmoid(N(0,1)), b, grad_h ~
N(0,1), seed 0), with every tensor already resident in HBM and every output
pre-allocated. The headline value is the achieved HBM bandwidth of the step in
algorithmic bytes (32 B per element: forward reads a, b and writes h = 12 B;
backward reads a, h, grad_h and writes grad_a, grad_b = 20 B).

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu] [--no-configs] [--workload N]
                    [--channels-last BxTxC[:dtype]] [--launch-shapes]

--workload runs another of the synthetic configurations (1, 3, 4, 4f16, 5; or `long`, `long16`, `short70`) through the same timed
region instead of configuration 2 (used for the rocprofv3 summaries under profiles/).

Prints ONE JSON line. Besides the contract fields it carries
  roofline      the dominant kernel (backward) against the 8 TB/s HBM peak, its
                duration measured with HIP events on the launch stream, bound to
                the kernel itself (start and end of the kernel on the GPU): the
                average over ten launches of the timed region, and in
                `after_region` median, minimum and mean over 50 or more further
                launches that all carry events;
  roofline_fwd  the same for the forward kernel;
  cpu_baseline  the reference's single-threaded CPU loop on the same tensors,
                timed on this host (oracle/_ref if it was built, else the C
                restatement in oracle/); every entry of `configs` carries the
                same for its own tensors;
  kernel_time   median over the launches after the region of forward + backward
                kernel time per step, as GB/s (steadier than the wall-clock value);
  host_library  the package's own loop for CPU tensors on the same tensors
                (not the baseline: several rows side by side, several threads);
  long_rows     many rows of 16K to 96K elements (long-context shapes);
  odd_lengths   row lengths that are no multiple of a 128-byte line or of the
                16-byte vector;
  channels_last contiguous [B, T, C] tensors scanned along T (the reference's
                transposed kernels): its timing shape, many channels, many batch
                elements, channel counts off the 128-byte line and below a wave,
                fp32 and bf16, with the launch plan each direction takes;
  autograd_op   the same step through the op a model calls,
                scanscam_amd.scan(a, b).backward(grad_h), outputs allocated per call;
  configs       forward and forward+backward GB/s of the other four synthetic
                configurations and of configuration 2's bytes in float64
                ([8, 2048, 2048]) (buffer sets rotated so that the 256 MB
                Infinity Cache cannot serve them; timed as batches of
                back-to-back launches, gaps included). Where a launch is
                shorter than the host's call (under 25 us), the *_graph_*
                fields give the same launches replayed from a HIP graph.
"""
import argparse
import json
import os
import statistics
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0
# HBM bytes per launch at configs[1] come from rocprofv3 FETCH_SIZE + WRITE_SIZE, scaled by what the same
# counters read for a copy kernel of known size. They are read from this summary, which names the
# kernel sources it was taken with (a digest); with other sources the figure is reported as null.
TRAFFIC_PROFILE = os.path.join("profiles", "scan_row_f32_fwd_bwd_8x2048x4096_pmc_traffic.txt")
KERNEL_SOURCES = ("scan_kernels.hpp", "scan_launch.hpp", "scan_api.hip", "scan_f32.hip")
METRIC = "scan HBM GB/s and % of MI355X peak, fwd and fwd+bwd, fp32 [B,C,T]"
FWD_BYTES = {8: 24, 4: 12, 2: 6}
BWD_BYTES = {8: 40, 4: 20, 2: 10}
# Launches shorter than this are paced by the host's call; they are also timed replaying from a HIP graph.
GRAPH_BELOW_MS = 0.025


def kernel_sources_digest():
    """sha256 over the sources the row kernels are built from (what a traffic profile is valid for)."""
    import hashlib

    d = hashlib.sha256()
    for name in KERNEL_SOURCES:
        with open(os.path.join(ROOT, "scanscam_amd", "csrc", name), "rb") as f:
            d.update(f.read())
    return d.hexdigest()


def measured_traffic():
    """({"fwd": bytes, "bwd": bytes}, source) from the committed counter summary, or nulls if it is stale.

    The summary carries two machine-readable lines:
        traffic_bytes_per_launch fwd=<int> bwd=<int>
        kernel_sources_sha256 <hex>
    """
    none = {"fwd": None, "bwd": None}
    try:
        with open(os.path.join(ROOT, TRAFFIC_PROFILE)) as f:
            lines = f.read().splitlines()
    except OSError:
        return none, {"file": TRAFFIC_PROFILE, "state": "missing"}
    vals, digest = None, None
    for line in lines:
        w = line.split()
        if len(w) == 3 and w[0] == "traffic_bytes_per_launch":
            vals = {k: int(v) for k, v in (x.split("=") for x in w[1:])}
        if len(w) == 2 and w[0] == "kernel_sources_sha256":
            digest = w[1]
    if vals is None or digest is None:
        return none, {"file": TRAFFIC_PROFILE, "state": "no machine-readable figures"}
    if digest != kernel_sources_digest():
        return none, {"file": TRAFFIC_PROFILE, "state": "stale: taken with other kernel sources"}
    return vals, {"file": TRAFFIC_PROFILE, "state": "taken with these kernel sources", "kernel_sources_sha256": digest}


# --workload: name -> (configuration number for make_config, description)
WORKLOADS = {
    "1": (1, "configs[0]: fp32 scan, [B=4, C=256, T=1024], a ~ U(0,1), b ~ N(0,1), seed 0 (forward + backward timed)"),
    "2": (2, "configs[1]: forward + backward fp32 scan, [B=8, C=2048, T=4096], a=sigmoid(N(0,1)), "
             "b, grad_h ~ N(0,1), seed 0"),
    "3": (3, "configs[2]: forward + backward fp32 scan, long rows [B=1, C=64, T=1048576], a ~ U(0.9,1), b ~ N(0,1)"),
    "4": (4, "configs[3]: forward + backward scan, bf16 storage / fp32 arithmetic, [B=16, C=1024, T=2048], "
             "a=sigmoid(N(2,1)), b ~ N(0,0.5)"),
    "4f16": (40, "configs[3]: forward + backward scan, fp16 storage / fp32 arithmetic, [B=16, C=1024, T=2048], "
                 "a=sigmoid(N(2,1)), b ~ N(0,0.5)"),
    "5": (5, "configs[4]: forward + backward fp32 scan, many short rows [B=256, C=512, T=64], a ~ U(0,1), b ~ N(0,1)"),
    "long16": (60, "long-context shape in bf16 storage / fp32 arithmetic (not one of the five configurations): "
                   "forward + backward scan, [B=1, C=2048, T=32768], a=sigmoid(N(0,1)), b ~ N(0,1)"),
    "short70": (7, "short rows of odd length (not one of the five configurations): forward + backward fp32 scan, "
                   "[958698, 70], a ~ U(0,1), b ~ N(0,1)"),
    "long": (6, "long-context shape (not one of the five configurations): forward + backward fp32 scan, "
                "[B=1, C=2048, T=32768], a=sigmoid(N(0,1)), b ~ N(0,1)"),
}


def make_config(n, torch):
    """Inputs of synthetic configuration n (1-based), on the CPU generator, seed 0."""
    torch.manual_seed(0)
    dtype = torch.float32
    if n == 1:
        shape = (4, 256, 1024)
        a, b = torch.rand(shape), torch.randn(shape)
    elif n == 2:
        shape = (8, 2048, 4096)
        a, b = torch.sigmoid(torch.randn(shape)), torch.randn(shape)
    elif n == 3:
        shape = (1, 64, 1 << 20)
        a, b = 0.9 + 0.1 * torch.rand(shape), torch.randn(shape)
    elif n in (4, 40):
        shape = (16, 1024, 2048)
        a, b = torch.sigmoid(2 + torch.randn(shape)), 0.5 * torch.randn(shape)
        dtype = torch.bfloat16 if n == 4 else torch.float16
    elif n == 5:
        shape = (256, 512, 64)
        a, b = torch.rand(shape), torch.randn(shape)
    elif n in (6, 60):
        shape = (1, 2048, 32768)
        a, b = torch.sigmoid(torch.randn(shape)), torch.randn(shape)
        dtype = torch.float32 if n == 6 else torch.bfloat16
    elif n == 7:
        shape = (958698, 70)
        a, b = torch.rand(shape), torch.randn(shape)
    elif n == 20:  # configuration 2's bytes in float64 (the reference's other storage type): half its T
        shape = (8, 2048, 2048)
        a, b = torch.sigmoid(torch.randn(shape)), torch.randn(shape)
        dtype = torch.float64
    else:
        raise ValueError(n)
    gh = torch.randn(shape)
    return tuple(x.to(dtype) for x in (a, b, gh))


class DeviceSet:
    """One set of device tensors for forward + backward, flattened to [rows, T]."""

    def __init__(self, a, b, gh, dev, torch):
        T = a.shape[-1]
        self.a = a.reshape(-1, T).to(dev)
        self.b = b.reshape(-1, T).to(dev)
        self.gh = gh.reshape(-1, T).to(dev)
        self.h = torch.empty_like(self.a)
        self.ga = torch.empty_like(self.a)
        self.gb = torch.empty_like(self.a)

    def clone(self, torch):
        c = object.__new__(DeviceSet)
        for k, v in self.__dict__.items():
            setattr(c, k, v.clone())
        return c


def time_kernels(sets, steps, warmup, hip, torch):
    """Runs (forward; backward) `steps` times, rotating over `sets`.

    Returns (wall seconds per step, mean fwd kernel ms, mean bwd kernel ms,
    min fwd ms, min bwd ms). The kernel times come from HIP events on the launch
    stream that the library binds to the scan kernels themselves
    (scanscam_scan_fwd_timed / _bwd_timed): each pair holds its kernel's start and
    end on the GPU. Ten steps spread evenly over the region are sampled (a launch
    that carries events costs a few microseconds more on the stream, which the
    wall time of the region would otherwise show).
    """
    calls = [(hip.prepare_forward(s.a, s.b, s.h), hip.prepare_backward(s.a, s.h, s.gh, s.ga, s.gb)) for s in sets]
    stride = max(1, steps // 10)
    timed = {}
    for i in range(0, steps, stride):
        s = sets[i % len(sets)]
        ef, eb = hip.KernelEvents(), hip.KernelEvents()
        timed[i] = (hip.prepare_forward(s.a, s.b, s.h, events=ef),
                    hip.prepare_backward(s.a, s.h, s.gh, s.ga, s.gb, events=eb), ef, eb)
    for i in range(warmup):
        f, b = calls[i % len(calls)]
        f()
        b()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(steps):
        f, b = timed[i][:2] if i in timed else calls[i % len(calls)]
        f()
        b()
    torch.cuda.synchronize()
    wall = (time.perf_counter() - t0) / steps
    fwd = [t[2].elapsed_ms() for t in timed.values()]
    bwd = [t[3].elapsed_ms() for t in timed.values()]
    return wall, statistics.fmean(fwd), statistics.fmean(bwd), min(fwd), min(bwd)


def kernel_statistics(sets, launches, hip, torch):
    """After the timed region: `launches` more steps, every launch with its own bound events.

    Returns {"fwd": (median ms, min ms, mean ms), "bwd": ..., "step": ...} over all of them
    ("step" = forward kernel + backward kernel of the same step).
    """
    runs = []
    for i in range(launches):
        s = sets[i % len(sets)]
        ef, eb = hip.KernelEvents(), hip.KernelEvents()
        runs.append((hip.prepare_forward(s.a, s.b, s.h, events=ef),
                     hip.prepare_backward(s.a, s.h, s.gh, s.ga, s.gb, events=eb), ef, eb))
    for f, b, _, _ in runs:
        f()
        b()
    torch.cuda.synchronize()
    out = {}
    for name, k in (("fwd", 2), ("bwd", 3)):
        ms = [r[k].elapsed_ms() for r in runs]
        out[name] = (statistics.median(ms), min(ms), statistics.fmean(ms))
    both = [r[2].elapsed_ms() + r[3].elapsed_ms() for r in runs]  # kernel time of a whole step
    out["step"] = (statistics.median(both), min(both), statistics.fmean(both))
    return out


def time_batches(sets, launches, warmup, hip, torch, plan=None):
    """Mean ms per launch of each direction over `launches` back-to-back launches.

    For kernels of a few microseconds, where an event pair around every launch
    would cost as much as the launch: two events bracket the whole batch, so the
    figure includes the gaps between launches.
    """
    calls = [(hip.prepare_forward(s.a, s.b, s.h, plan=plan), hip.prepare_backward(s.a, s.h, s.gh, s.ga, s.gb, plan=plan))
             for s in sets]
    out = []
    for d in (0, 1):
        for i in range(warmup):
            calls[i % len(calls)][d]()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        e0.record()
        for i in range(launches):
            calls[i % len(calls)][d]()
        e1.record()
        torch.cuda.synchronize()
        out.append(e0.elapsed_time(e1) / launches)
    return out[0], out[1]


def time_graph(sets, replays, hip, torch, plan=None):
    """Mean ms per launch of each direction when the launches replay from a HIP graph.

    One launch per buffer set is captured (a kernel of a few microseconds is otherwise
    paced by the host's call, not by the GPU); two events bracket `replays` replays.
    """
    out = []
    for d in (0, 1):
        side = torch.cuda.Stream()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.stream(side):
            calls = [(hip.prepare_forward(s.a, s.b, s.h, plan=plan),
                      hip.prepare_backward(s.a, s.h, s.gh, s.ga, s.gb, plan=plan))[d] for s in sets]
            calls[0]()
            side.synchronize()
            with torch.cuda.graph(graph, stream=side):
                for c in calls:
                    c()
        torch.cuda.synchronize()
        graph.replay()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(replays):
            graph.replay()
        e1.record()
        torch.cuda.synchronize()
        out.append(e0.elapsed_time(e1) / (replays * len(sets)))
        del graph
    return out[0], out[1]


def autograd_step(s, shape, steps, warmup, torch):
    """Wall milliseconds per step of the op a model calls: h = scan(a, b); h.backward(grad_h).

    The same kernels as the timed region, plus what the autograd function adds per call: the
    allocation of h and of the two gradients from torch's caching allocator, the autograd graph,
    the checks and the plan look-up.
    """
    import scanscam_amd

    a = s.a.view(shape).requires_grad_()
    b = s.b.view(shape).requires_grad_()
    gh = s.gh.view(shape)

    def step():
        a.grad = b.grad = None
        scanscam_amd.scan(a, b).backward(gh)

    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        step()
    torch.cuda.synchronize()
    wall = (time.perf_counter() - t0) / steps
    a.requires_grad_(False)
    b.requires_grad_(False)
    return wall * 1e3


def reference_grid(dev, args, hip, torch):
    """The shapes the reference's own timing tests use, fp32 N(0,1) inputs.

    Row layout: scanscam/cpu_test.py:51-77 and scanscam/cuda_test.py:166-247
    ((8,256,4096), (8,256,32), (256,4096), (16384,4096)); channels-last:
    cuda_test.py:250-308 ((8,4096,512) stored [B, T, C]). Mean microseconds per
    launch over back-to-back launches on rotated buffer sets; beside them the
    reference's CPU loop on the same tensors (the CPU half of the same grid).
    """
    out = {}
    for shape in ((8, 256, 4096), (8, 256, 32), (256, 4096), (16384, 4096)):
        torch.manual_seed(0)
        x, y, z = torch.randn(shape), torch.randn(shape), torch.randn(shape)
        first = DeviceSet(x, y, z, dev, torch)
        n = x.numel()
        nsets = max(1, min(64, -(-(1 << 30) // (24 * n))))
        sets = [first] + [first.clone(torch) for _ in range(nsets - 1)]
        f_ms, b_ms = time_batches(sets, max(4 * args.steps, 4 * nsets), max(args.warmup, nsets), hip, torch)
        out["x".join(map(str, shape))] = {
            "fwd_us": round(f_ms * 1e3, 2), "bwd_us": round(b_ms * 1e3, 2),
            "fwd_GBps": round(12 * n / (f_ms * 1e-3) / 1e9, 1), "bwd_GBps": round(20 * n / (b_ms * 1e-3) / 1e9, 1),
        }
        if f_ms < GRAPH_BELOW_MS:
            gf_ms, gb_ms = time_graph(sets, max(4, 4 * args.steps // nsets), hip, torch)
            out["x".join(map(str, shape))].update(
                fwd_graph_us=round(gf_ms * 1e3, 2), bwd_graph_us=round(gb_ms * 1e3, 2),
                fwd_graph_GBps=round(12 * n / (gf_ms * 1e-3) / 1e9, 1),
                bwd_graph_GBps=round(20 * n / (gb_ms * 1e-3) / 1e9, 1))
        if not args.no_cpu:
            # The CPU half of the reference's grid (cpu_test.py:51-77): its single-threaded loop on the same
            # shapes and N(0,1) tensors, called as its tests call it (contiguous inputs, outputs allocated by the
            # caller), 1 warm-up + 3 repetitions per direction, median.
            c = cpu_baseline(x, y, z, reps=3)
            out["x".join(map(str, shape))].update(
                cpu_fwd_us=round(c["fwd_s"] * 1e6, 1), cpu_bwd_us=round(c["bwd_s"] * 1e6, 1),
                cpu_fwd_GBps=c["fwd_GBps"], cpu_bwd_GBps=c["bwd_GBps"], cpu_kind=c["kind"], cpu_cores=c["cores"])
        del sets, first
        torch.cuda.empty_cache()
    # Channels-last: logical [8, 512, 4096] stored [8, 4096, 512].
    torch.manual_seed(0)
    shape = (8, 4096, 512)
    x, y, z = (torch.randn(shape).to(dev) for _ in range(3))
    h = hip.transposed_linear_scan_forward(x, y)
    n = x.numel()
    times = []
    for fn in (lambda: hip.transposed_linear_scan_forward(x, y),
               lambda: hip.transposed_linear_scan_backward(x, h, z)):
        for _ in range(args.warmup):
            fn()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        e0.record()
        for _ in range(args.steps):
            fn()
        e1.record()
        torch.cuda.synchronize()
        times.append(e0.elapsed_time(e1) / args.steps)
    out["channels_last_8x4096x512"] = {
        "fwd_us": round(times[0] * 1e3, 2), "bwd_us": round(times[1] * 1e3, 2),
        "fwd_GBps": round(12 * n / (times[0] * 1e-3) / 1e9, 1), "bwd_GBps": round(20 * n / (times[1] * 1e-3) / 1e9, 1),
        "note": "includes the wrapper's output allocation; working set fits the Infinity Cache",
    }
    return out


def long_rows(dev, args, hip, torch):
    """Many rows of 8K to 128K elements (long-context shapes), 64 M elements each, fp32 and bf16.

    From two tiles per row on these run on the look-back kernel with its tiles handed out row after row;
    mean microseconds per launch over back-to-back launches (each tensor is 268 MB / 134 MB, beyond the
    Infinity Cache).
    """
    shapes = ((4096, 16384), (2048, 32768), (1365, 49152), (682, 98304))
    return shape_table(dev, args, hip, torch, [(r, t, d) for d in (torch.float32, torch.bfloat16) for r, t in shapes])


def odd_lengths(dev, args, hip, torch):
    """Row lengths that are no multiple of a 128-byte line, or of the 16-byte vector; about 64 M elements each.

    3000 and 9000: rows start inside a line (chunks are laid out from the line border before the row);
    4097 and 70, and the 16-bit lengths that are no multiple of 8: rows start at any element
    (element-aligned vectors, partial first and last ones).
    """
    shapes = [(22369, 3000, torch.float32), (7456, 9000, torch.float32), (16380, 4097, torch.float32),
              (958698, 70, torch.float32), (16380, 4097, torch.bfloat16), (67040, 1001, torch.bfloat16),
              (134216, 500, torch.bfloat16), (32752, 2049, torch.bfloat16), (2013, 33333, torch.bfloat16)]
    return shape_table(dev, args, hip, torch, shapes)


def shape_table(dev, args, hip, torch, shapes):
    """{shape: microseconds per launch, fraction of peak, plans} for (rows, T, dtype) triples, one buffer set each."""
    out = {}
    for rows, T, dtype in shapes:
        g = torch.Generator(device=dev).manual_seed(0)
        a = torch.rand((rows, T), generator=g, device=dev).to(dtype)
        b = torch.randn((rows, T), generator=g, device=dev).to(dtype)
        gh = torch.randn((rows, T), generator=g, device=dev).to(dtype)
        s = object.__new__(DeviceSet)
        s.a, s.b, s.gh = a, b, gh
        s.h, s.ga, s.gb = (torch.empty_like(a) for _ in range(3))
        f_ms, b_ms = time_batches([s], max(20, args.steps // 2), max(3, args.warmup // 2), hip, torch)
        n, esize = a.numel(), a.element_size()
        out[f"{rows}x{T}_{str(dtype).replace('torch.', '')}"] = {
            "fwd_us": round(f_ms * 1e3, 1), "bwd_us": round(b_ms * 1e3, 1),
            "fwd_frac": round(FWD_BYTES[esize] * n / (f_ms * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4),
            "bwd_frac": round(BWD_BYTES[esize] * n / (b_ms * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4),
            "plan_fwd": repr(hip.resolve_plan(rows, T, dtype, hip.FORWARD)),
            "plan_bwd": repr(hip.resolve_plan(rows, T, dtype, hip.BACKWARD)),
        }
        del s, a, b, gh
        torch.cuda.empty_cache()
    return out


def strided_views(dev, args, hip, torch):
    """Views scanned in place against copy-then-scan (what the reference's wrappers do, cuda.py:36-37).

    Row layout: the halves of one fused projection x[8, 2*2048, 4096] (a, b = x.chunk(2, dim=1)), i.e.
    config 2's shape with two levels of row strides. Channels-last: the halves of x[64, 2048, 2*1024].
    Mean microseconds per call, output allocation included on both sides.
    """
    def mean_us(fn):
        for _ in range(max(3, args.warmup // 2)):
            fn()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        e0.record()
        for _ in range(args.steps):
            fn()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / args.steps * 1e3

    out = {}
    torch.manual_seed(0)
    for name, shape, dim, to_logical in (
            ("rows_halves_of_8x4096x4096", (8, 4096, 4096), 1, lambda t: t),
            ("channels_last_halves_of_64x2048x2048", (64, 2048, 2048), 2, lambda t: t.mT)):
        x = torch.randn(shape, device=dev)
        g = torch.randn(shape, device=dev)
        half = shape[dim] // 2
        x.narrow(dim, 0, half).sigmoid_()
        a, b = (to_logical(t) for t in x.chunk(2, dim=dim))
        gh = to_logical(g.narrow(dim, half, half))
        h = hip.scan_forward(a, b)
        n = a.numel()
        dense = (lambda t: t.contiguous()) if dim == 1 else (lambda t: t.mT.contiguous().mT)
        f_us = mean_us(lambda: hip.scan_forward(a, b))
        b_us = mean_us(lambda: hip.scan_backward(a, h, gh))
        fc_us = mean_us(lambda: hip.scan_forward(dense(a), dense(b)))
        bc_us = mean_us(lambda: hip.scan_backward(dense(a), h, dense(gh)))
        out[name] = {
            "fwd_us": round(f_us, 1), "bwd_us": round(b_us, 1),
            "fwd_frac": round(12 * n / (f_us * 1e-6) / 1e9 / HBM_PEAK_GBPS, 4),
            "bwd_frac": round(20 * n / (b_us * 1e-6) / 1e9 / HBM_PEAK_GBPS, 4),
            "copy_first_fwd_us": round(fc_us, 1), "copy_first_bwd_us": round(bc_us, 1),
        }
        del x, g, a, b, gh, h
        torch.cuda.empty_cache()
    return out


def launch_shapes(args, hip, torch):
    """--launch-shapes: configuration 1 ([1024, 1024] fp32) under every launch shape of the row kernel.

    Microseconds per launch, launched one by one and replayed from a HIP graph (64 buffer sets in rotation),
    and the same for a scan of [4, 64] elements, which is the cost of a launch with nothing to stream.
    Prints one JSON line; its summary is kept under profiles/.
    """
    dev = torch.device("cuda:0")
    a, b, gh = make_config(1, torch)
    first = DeviceSet(a, b, gh, dev, torch)
    sets = [first] + [first.clone(torch) for _ in range(63)]
    out = {"workload": WORKLOADS["1"][1], "shapes": []}
    shapes = [None] + [hip.Plan(mode=hip.MODE_ROW, vec=4, unroll=u, waves=w, waves_per_row=r) for u, w, r in
                       ((4, 4, 1), (4, 2, 1), (4, 1, 1), (4, 8, 1), (2, 4, 2), (2, 2, 2), (2, 8, 2), (1, 4, 4), (1, 8, 4),
                        (1, 16, 4), (2, 16, 2), (1, 2, 2), (3, 4, 1))]
    for plan in shapes:
        f_ms, b_ms = time_batches(sets, 256, 64, hip, torch, plan=plan)
        gf_ms, gb_ms = time_graph(sets, 20, hip, torch, plan=plan)
        out["shapes"].append({"plan": repr(plan) if plan is not None else "automatic: " + repr(hip.resolve_plan(1024, 1024, a.dtype, hip.FORWARD)),
                              "fwd_us": round(f_ms * 1e3, 2), "fwd_graph_us": round(gf_ms * 1e3, 2),
                              "bwd_us": round(b_ms * 1e3, 2), "bwd_graph_us": round(gb_ms * 1e3, 2)})
    tiny = []
    for _ in range(64):
        s = object.__new__(DeviceSet)
        s.a, s.b, s.gh = (torch.rand((4, 64), device=dev) for _ in range(3))
        s.h, s.ga, s.gb = (torch.empty_like(s.a) for _ in range(3))
        tiny.append(s)
    f_ms, b_ms = time_batches(tiny, 256, 64, hip, torch)
    gf_ms, gb_ms = time_graph(tiny, 20, hip, torch)
    out["launch_floor_4x64"] = {"fwd_us": round(f_ms * 1e3, 2), "fwd_graph_us": round(gf_ms * 1e3, 2),
                                "bwd_us": round(b_ms * 1e3, 2), "bwd_graph_us": round(gb_ms * 1e3, 2)}
    print(json.dumps(out))


def time_channels_last(B, T, C, dtype, steps, warmup, hip, torch):
    """Forward and backward over contiguous [B, T, C] tensors (scanned along T): milliseconds per launch, buffer sets.

    Buffer sets rotate over >= 1 GiB; mean over back-to-back launches.
    """
    dev = torch.device("cuda:0")
    g = torch.Generator(device=dev).manual_seed(0)
    n = B * T * C
    esize = torch.empty(0, dtype=dtype).element_size()
    nsets = max(1, min(16, -(-(1 << 30) // (6 * n * esize))))
    fwd, bwd = [], []
    for _ in range(nsets):
        a = torch.rand((B, T, C), generator=g, device=dev).to(dtype)
        b = torch.randn((B, T, C), generator=g, device=dev).to(dtype)
        gh = torch.randn((B, T, C), generator=g, device=dev).to(dtype)
        h, ga, gb = (torch.empty_like(a) for _ in range(3))
        fwd.append(hip.prepare_forward_cl(a, b, h))
        bwd.append(hip.prepare_backward_cl(a, h, gh, ga, gb))
    ms = []
    for calls in (fwd, bwd):
        for i in range(max(warmup, nsets)):
            calls[i % nsets]()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        e0.record()
        for i in range(steps):
            calls[i % nsets]()
        e1.record()
        torch.cuda.synchronize()
        ms.append(e0.elapsed_time(e1) / steps)
    del fwd, bwd
    torch.cuda.empty_cache()
    return ms[0], ms[1], nsets


def channels_last_workload(spec, args, hip, torch):
    """--channels-last BxTxC[:dtype]: forward and backward over contiguous [B, T, C] tensors (scanned along T).

    Used for the rocprofv3 summaries of the channels-last kernels under profiles/; prints its own JSON line.
    """
    shape_s, _, dtype_s = spec.partition(":")
    B, T, C = (int(v) for v in shape_s.lower().split("x"))
    dtype = {"": torch.float32, "f32": torch.float32, "bf16": torch.bfloat16, "f16": torch.float16,
             "f64": torch.float64}[dtype_s]
    f_ms, b_ms, nsets = time_channels_last(B, T, C, dtype, args.steps, args.warmup, hip, torch)
    n = B * T * C
    esize = torch.empty(0, dtype=dtype).element_size()
    print(json.dumps({
        "workload": f"channels-last [B={B}, T={T}, C={C}] {str(dtype).replace('torch.', '')}, a ~ U(0,1), b, grad_h ~ N(0,1)",
        "buffer_sets": nsets, "steps": args.steps,
        "fwd_us": round(f_ms * 1e3, 2), "bwd_us": round(b_ms * 1e3, 2),
        "fwd_frac": round(FWD_BYTES[esize] * n / (f_ms * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4),
        "bwd_frac": round(BWD_BYTES[esize] * n / (b_ms * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4),
        "fwd_bytes": FWD_BYTES[esize] * n, "bwd_bytes": BWD_BYTES[esize] * n,
    }))


def channels_last_table(args, hip, torch):
    """Contiguous [B, T, C] tensors scanned along T (the layout of the reference's transposed kernels,
    scanscam/cuda.py:69-95): its timing shape, many-channel and many-batch shapes in fp32 and bf16, channel
    counts that are no whole 128-byte lines or fewer than a wave. Rotated buffer sets, prepared calls."""
    shapes = [(8, 4096, 512, torch.float32), (8, 4096, 2048, torch.float32), (64, 2048, 1024, torch.float32),
              (256, 1024, 1024, torch.float32), (8, 4096, 512, torch.bfloat16), (8, 4096, 2048, torch.bfloat16),
              (64, 2048, 1024, torch.bfloat16), (256, 1024, 1024, torch.bfloat16), (8, 4096, 1000, torch.float32),
              (64, 2048, 1001, torch.float32), (64, 2048, 1001, torch.bfloat16), (2048, 512, 40, torch.float32),
              (2048, 512, 40, torch.bfloat16)]
    out = {}
    for B, T, C, dtype in shapes:
        f_ms, b_ms, nsets = time_channels_last(B, T, C, dtype, max(20, args.steps // 2), max(3, args.warmup // 2), hip, torch)
        n, esize = B * T * C, torch.empty(0, dtype=dtype).element_size()
        short = lambda p: f"mode={p.mode} vec={p.vec} steps={p.unroll} waves={p.waves}"
        out[f"{B}x{T}x{C}_{str(dtype).replace('torch.', '')}"] = {
            "fwd_us": round(f_ms * 1e3, 1), "bwd_us": round(b_ms * 1e3, 1),
            "fwd_frac": round(FWD_BYTES[esize] * n / (f_ms * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4),
            "bwd_frac": round(BWD_BYTES[esize] * n / (b_ms * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4),
            "buffer_sets": nsets,
            "plan_fwd": short(hip.resolve_plan_cl(B, T, C, dtype, hip.FORWARD)),
            "plan_bwd": short(hip.resolve_plan_cl(B, T, C, dtype, hip.BACKWARD)),
        }
    return out


def cpu_baseline(a, b, gh, reps):
    """The reference's CPU loop on the same tensors, one thread."""
    import numpy as np
    import torch

    import oracle

    T = a.shape[-1]
    n = a.numel()
    ext = oracle.ref_ext()
    if ext is not None:
        kind = "reference"
        a2, b2, gh2 = (x.reshape(-1, T).contiguous() for x in (a, b, gh))
        h, ga, gb = torch.empty_like(a2), torch.empty_like(a2), torch.empty_like(a2)

        def fwd():
            ext.simple_linear_scan_cpu(a2, b2, h)

        def bwd():
            ext.simple_linear_scan_backward_cpu(a2, h, gh2, ga, gb)
    else:
        kind = "port"
        a2, b2, gh2 = (np.ascontiguousarray(x.reshape(-1, T).numpy()) for x in (a, b, gh))
        state = {}

        def fwd():
            state["h"] = oracle.fwd(a2, b2)

        def bwd():
            oracle.bwd(a2, state["h"], gh2)

    times = {"fwd": [], "bwd": []}
    for rep in range(reps + 1):
        for name, fn in (("fwd", fwd), ("bwd", bwd)):
            t0 = time.perf_counter()
            fn()
            dt = time.perf_counter() - t0
            if rep > 0:  # first pass is the warm-up
                times[name].append(dt)
    tf, tb = statistics.median(times["fwd"]), statistics.median(times["bwd"])
    return {
        "value": round(32 * n / (tf + tb) / 1e9, 3),
        "unit": "GB/s",
        "cores": 1,
        "kind": kind,
        "sample": f"the full workload ({n} elements), 1 warm-up + {reps} repetitions per direction, median",
        "fwd_GBps": round(12 * n / tf / 1e9, 3),
        "bwd_GBps": round(20 * n / tb / 1e9, 3),
        "fwd_s": round(tf, 7),
        "bwd_s": round(tb, 7),
        "elements_per_s": round(n / (tf + tb)),
        "host_cpus": os.cpu_count(),
    }


def host_library(a, b, gh, reps):
    """The package's own loop for CPU tensors (libscanscam_cpu.so) on the same tensors.

    Bit-identical to the reference's loop per row; 8 rows side by side per thread, slabs of rows over
    threads. Outputs pre-allocated and touched, as for cpu_baseline. Reported beside it, not part of it.
    """
    import torch

    from scanscam_amd import cpu

    if not cpu.has_cpu_ops:
        return None
    T = a.shape[-1]
    n = a.numel()
    a2, b2, gh2 = (x.reshape(-1, T).contiguous() for x in (a, b, gh))
    rows = a2.shape[0]
    h, ga, gb = torch.zeros_like(a2), torch.zeros_like(a2), torch.zeros_like(a2)
    suffix = cpu._SUFFIX[a2.dtype]
    f, g = getattr(cpu._lib, f"scanscam_cpu_fwd_{suffix}"), getattr(cpu._lib, f"scanscam_cpu_bwd_{suffix}")
    times = {"fwd": [], "bwd": []}
    for rep in range(reps + 1):
        for name, fn, tensors in (("fwd", f, (a2, b2, h)), ("bwd", g, (a2, h, gh2, ga, gb))):
            t0 = time.perf_counter()
            cpu._run(fn, tensors, rows, T)
            dt = time.perf_counter() - t0
            if rep > 0:
                times[name].append(dt)
    tf, tb = statistics.median(times["fwd"]), statistics.median(times["bwd"])
    return {
        "value": round(32 * n / (tf + tb) / 1e9, 3),
        "unit": "GB/s",
        "threads": len(cpu._slabs(rows, T)),
        "fwd_s": round(tf, 7),
        "bwd_s": round(tb, 7),
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-configs", action="store_true", help="skip the other four configurations")
    ap.add_argument("--workload", default="2", choices=sorted(WORKLOADS),
                    help="synthetic configuration the timed region runs (default 2, the one the metric is quoted on)")
    ap.add_argument("--channels-last", metavar="BxTxC[:dtype]", default=None,
                    help="time the channels-last kernels on this shape instead (dtype f32, bf16, f16 or f64) and exit")
    ap.add_argument("--launch-shapes", action="store_true",
                    help="time configuration 1 under every launch shape, one by one and from a HIP graph, and exit")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on one GPU only (rows are independent, so more GPUs would "
                 "just split the rows with no communication); use --gpus 1")

    import torch

    if not os.path.exists(os.path.join(ROOT, "scanscam_amd", "libscanscam_hip.so")):
        import __graft_entry__

        __graft_entry__.build()  # nothing built yet; otherwise what is built is what runs
    from scanscam_amd import hip

    if not hip.has_hip_ops:
        sys.exit("bench.py: scanscam_amd/libscanscam_hip.so does not load; no other implementation is timed")
    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible")
    dev = torch.device("cuda:0")
    if args.channels_last:
        channels_last_workload(args.channels_last, args, hip, torch)
        return
    if args.launch_shapes:
        launch_shapes(args, hip, torch)
        return

    cfg, label = WORKLOADS[args.workload]
    a, b, gh = make_config(cfg, torch)
    n = a.numel()
    esize = a.element_size()
    first = DeviceSet(a, b, gh, dev, torch)
    # Working sets that would fit the 256 MB Infinity Cache are rotated over >= 1 GiB of buffer sets.
    nsets = max(1, min(64, -(-(1 << 30) // (6 * n * esize)))) if 6 * n * esize < (1 << 30) else 1
    sets = [first] + [first.clone(torch) for _ in range(nsets - 1)]
    wall, fwd_ms, bwd_ms, fwd_min, bwd_min = time_kernels(sets, args.steps, max(args.warmup, nsets), hip, torch)
    stats = kernel_statistics(sets, max(50, args.steps), hip, torch)
    step_bytes = FWD_BYTES[esize] + BWD_BYTES[esize]
    fwd_gbps = FWD_BYTES[esize] * n / (fwd_ms * 1e-3) / 1e9
    bwd_gbps = BWD_BYTES[esize] * n / (bwd_ms * 1e-3) / 1e9
    step_gbps = step_bytes * n / wall / 1e9
    rows, T = first.a.shape
    plan_f = hip.resolve_plan(rows, T, a.dtype, hip.FORWARD)
    family = {hip.MODE_SMALL: "scan_small_kernel", hip.MODE_ROW: "scan_row_kernel",
              hip.MODE_LOOKBACK: "scan_lookback_kernel", hip.MODE_FLAT: "scan_flat_kernel"}[plan_f.mode]
    storage = {"float32": "float", "bfloat16": "__bf16", "float16": "_Float16"}[str(a.dtype).replace("torch.", "")]
    kernel = f"{family}<{storage}, {plan_f.vec}, {plan_f.unroll}, REV=%s>"
    traffic, traffic_source = measured_traffic() if args.workload == "2" else ({"fwd": None, "bwd": None}, None)

    out = {
        "metric": METRIC,
        "value": round(step_gbps, 1),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(wall * 1e3, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",  # arithmetic type; storage is named in config.workload
        "data": "synthetic",
        "config": {
            "workload": label + f"; value = {step_bytes} B/element * elements / step time",
            "elements": n,
            "buffer_sets": nsets,
            "plan": repr(plan_f),
            "library": os.path.relpath(hip.LIB_PATH, ROOT),  # the build that ran (SCANSCAM_HIP_LIB may name another)
        },
        "frac_of_peak": round(step_gbps / HBM_PEAK_GBPS, 4),
        # The steadier figure: median over the launches after the region of (forward + backward kernel
        # time) per step, from events bound to the kernels (no gaps between launches in it).
        "kernel_time": {"launches": max(50, args.steps), "fwd_bwd_median_ms": round(stats["step"][0], 4),
                        "GBps": round(step_bytes * n / (stats["step"][0] * 1e-3) / 1e9, 1),
                        "frac": round(step_bytes * n / (stats["step"][0] * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4)},
        "elements_per_s": round(n / wall),
        "fwd": {"ms": round(fwd_ms, 4), "min_ms": round(fwd_min, 4), "GBps": round(fwd_gbps, 1),
                "frac": round(fwd_gbps / HBM_PEAK_GBPS, 4)},
        "fwd_bwd": {"ms": round(fwd_ms + bwd_ms, 4),
                    "GBps": round(step_bytes * n / ((fwd_ms + bwd_ms) * 1e-3) / 1e9, 1),
                    "frac": round(step_bytes * n / ((fwd_ms + bwd_ms) * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4)},
        "roofline": {
            "kernel": kernel % "true" + " (backward)",
            "bound": "hbm",
            "achieved": round(bwd_gbps, 1),
            "peak": HBM_PEAK_GBPS,
            "unit": "GB/s",
            "frac": round(bwd_gbps / HBM_PEAK_GBPS, 4),
            "traffic": traffic["bwd"],
            "traffic_source": traffic_source,
            "bytes_per_launch": BWD_BYTES[esize] * n,
            "avg_ms": round(bwd_ms, 4),
            "min_ms": round(bwd_min, 4),
            "after_region": {"launches": max(50, args.steps), "median_ms": round(stats["bwd"][0], 4),
                             "min_ms": round(stats["bwd"][1], 4), "mean_ms": round(stats["bwd"][2], 4)},
        },
        "roofline_fwd": {
            "kernel": kernel % "false" + " (forward)",
            "bound": "hbm",
            "achieved": round(fwd_gbps, 1),
            "peak": HBM_PEAK_GBPS,
            "unit": "GB/s",
            "frac": round(fwd_gbps / HBM_PEAK_GBPS, 4),
            "traffic": traffic["fwd"],
            "traffic_source": traffic_source,
            "bytes_per_launch": FWD_BYTES[esize] * n,
            "avg_ms": round(fwd_ms, 4),
            "min_ms": round(fwd_min, 4),
            "after_region": {"launches": max(50, args.steps), "median_ms": round(stats["fwd"][0], 4),
                             "min_ms": round(stats["fwd"][1], 4), "mean_ms": round(stats["fwd"][2], 4)},
        },
    }
    op_ms = autograd_step(first, tuple(a.shape), args.steps, args.warmup, torch)
    out["autograd_op"] = {
        "call": "scanscam_amd.scan(a, b).backward(grad_h), outputs allocated per call",
        "ms_per_step": round(op_ms, 4),
        "GBps": round(step_bytes * n / (op_ms * 1e-3) / 1e9, 1),
        "frac": round(step_bytes * n / (op_ms * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4),
    }
    del sets, first

    if not args.no_configs:
        others = {}
        for key, cfg in (("1", 1), ("3", 3), ("4_bf16", 4), ("4_f16", 40), ("5", 5), ("2_f64_half_T", 20)):
            ca, cb, cgh = make_config(cfg, torch)
            esize = ca.element_size()
            cn = ca.numel()
            first = DeviceSet(ca, cb, cgh, dev, torch)
            # Enough distinct buffer sets that a pass cannot be served from the
            # 256 MB Infinity Cache: at least 1 GiB of tensors in rotation.
            per_set = 6 * cn * esize
            nsets = max(1, min(64, -(-(1 << 30) // per_set)))
            csets = [first] + [first.clone(torch) for _ in range(nsets - 1)]
            f_ms, b_ms = time_batches(csets, max(4 * args.steps, 4 * nsets), max(args.warmup, nsets), hip, torch)
            rows, T = first.a.shape
            others[key] = {
                "shape": list(ca.shape),
                "dtype": str(ca.dtype).replace("torch.", ""),
                "plan": repr(hip.resolve_plan(rows, T, ca.dtype, hip.FORWARD)),
                "buffer_sets": nsets,
                "fwd_ms": round(f_ms, 4),
                "fwd_GBps": round(FWD_BYTES[esize] * cn / (f_ms * 1e-3) / 1e9, 1),
                "fwd_frac": round(FWD_BYTES[esize] * cn / (f_ms * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4),
                "fwd_bwd_ms": round(f_ms + b_ms, 4),
                "fwd_bwd_GBps": round((FWD_BYTES[esize] + BWD_BYTES[esize]) * cn / ((f_ms + b_ms) * 1e-3) / 1e9, 1),
                "fwd_bwd_frac": round((FWD_BYTES[esize] + BWD_BYTES[esize]) * cn / ((f_ms + b_ms) * 1e-3) / 1e9
                                      / HBM_PEAK_GBPS, 4),
                "elements_per_s_fwd_bwd": round(cn / ((f_ms + b_ms) * 1e-3)),
            }
            if f_ms < GRAPH_BELOW_MS:
                # Launch-bound from the host: the same launches replayed from a HIP graph.
                gf_ms, gb_ms = time_graph(csets, max(4, 4 * args.steps // nsets), hip, torch)
                others[key].update(
                    fwd_graph_ms=round(gf_ms, 4),
                    fwd_graph_frac=round(FWD_BYTES[esize] * cn / (gf_ms * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4),
                    fwd_bwd_graph_ms=round(gf_ms + gb_ms, 4),
                    fwd_bwd_graph_frac=round((FWD_BYTES[esize] + BWD_BYTES[esize]) * cn / ((gf_ms + gb_ms) * 1e-3)
                                             / 1e9 / HBM_PEAK_GBPS, 4))
            if not args.no_cpu and ca.dtype != torch.float64:
                # The reference's loop on this configuration's own tensors (16-bit storage: on the fp32 upcast).
                c = cpu_baseline(ca.float(), cb.float(), cgh.float(), reps=2)
                others[key]["cpu_baseline"] = {k: c[k] for k in ("value", "unit", "cores", "kind", "fwd_GBps",
                                                                 "bwd_GBps", "sample")}
            del csets, first
            torch.cuda.empty_cache()
        out["configs"] = others

    if not args.no_configs:
        out["reference_grid"] = reference_grid(dev, args, hip, torch)
        out["strided_views"] = strided_views(dev, args, hip, torch)
        out["long_rows"] = long_rows(dev, args, hip, torch)
        out["odd_lengths"] = odd_lengths(dev, args, hip, torch)
        out["channels_last"] = channels_last_table(args, hip, torch)

    if not args.no_cpu:
        # 16-bit workloads: the reference has no 16-bit path, so its loop runs on the exact fp32 upcast.
        out["cpu_baseline"] = cpu_baseline(a.float(), b.float(), gh.float(), reps=5)
        out["host_library"] = host_library(a.float(), b.float(), gh.float(), reps=5)

    print(json.dumps(out))


if __name__ == "__main__":
    main()
