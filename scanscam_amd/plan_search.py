"""
Time the library's automatic launch plan for a shape against a set of forced plans.

    python -m scanscam_amd.plan_search rows 8192x4096 2047x16385:bf16 ...
    python -m scanscam_amd.plan_search cl 8x4096x512:bf16 64x2048x1001 ...
    python -m scanscam_amd.plan_search --suite cl-a | cl-b | cl-odd | rows-23 | rows-25 | rows-26
    python -m scanscam_amd.plan_search --random 40 --seed 3      (channels-last shapes drawn at random, and the
                                                                  distribution of automatic / best over them)
    python -m scanscam_amd.plan_search rows --random 30 --seed 1 (the same for the row layout)

``rows`` shapes are contiguous ``[rows, T]`` tensors scanned along ``T`` (the layout of
``simple_linear_scan`` and its siblings, ``scanscam/cuda.py:16-66`` in the reference), ``cl`` shapes are
contiguous ``[batch, T, C]`` tensors scanned along ``T`` (``transposed_linear_scan``, ``cuda.py:69-95``).
dtype is f32 (default), bf16, f16 or f64.

One line per shape and dtype: the automatic plan's forward / backward microseconds and fraction of the 8 TB/s
HBM peak in algorithmic bytes (3 and 5 elements per scanned element), then the fastest plan of the set for each
direction, and a mark where the automatic plan (shown in brackets: mode, vec, unroll, waves, waves per row) is
more than 8 % behind it. The automatic plan is timed first
and again last and the faster of the two is kept, so that warm-up does not count against it. Buffer sets rotate
over at least 512 MiB so that the 256 MB Infinity Cache does not serve them. A plan the library rejects for a
shape is skipped.

The same search serves a caller who wants the best plan for one fixed shape: pass the printed plan to the
``plan=`` argument of the calls in ``scanscam_amd.hip`` (``struct scanscam_plan`` in the C interface).
"""
import argparse
import random
import sys

import torch

from . import hip

P = hip.Plan
DTYPES = {"": torch.float32, "f32": torch.float32, "bf16": torch.bfloat16, "f16": torch.float16, "f64": torch.float64}
HBM_PEAK_GBPS = 8000.0

SUITES = {
    "cl-a": ("cl", [(8, 4096, 512), (64, 2048, 1024), (256, 1024, 256), (32, 2048, 2048), (16, 8192, 512),
                    (128, 1024, 768), (4, 32768, 512), (512, 512, 512), (24, 2048, 1536), (96, 1024, 1280),
                    (12, 4096, 3072), (2, 65536, 1024), (1024, 256, 384), (48, 4096, 640), (200, 1024, 896),
                    (20, 8192, 256), (320, 1024, 512), (6, 16384, 2048), (40, 2048, 4096), (700, 512, 192)]),
    "cl-b": ("cl", [(1024, 1024, 64), (300, 2048, 128), (2000, 128, 256), (64, 512, 4096), (16, 2048, 8192),
                    (100, 3000, 300), (256, 333, 1000), (512, 700, 200), (28, 4096, 1024), (72, 2048, 768),
                    (3, 50000, 640), (5, 30000, 1280), (1, 100000, 1024), (150, 1500, 448), (4096, 256, 32),
                    (260, 4000, 48), (520, 2000, 96), (130, 8000, 64), (66, 3000, 1344), (10, 12000, 1600)]),
    "cl-odd": ("cl", [(64, 2048, 1001), (256, 1024, 1001), (128, 1024, 1003), (32, 4096, 999), (512, 512, 333),
                      (300, 1000, 77), (1000, 500, 130), (20, 8192, 250), (48, 2048, 1500), (8, 4096, 1000),
                      (90, 2048, 514), (700, 300, 257), (16, 4096, 2050), (260, 2000, 66)]),
}


def _row_suite(log_n):
    n = 1 << log_n
    lengths = (32, 70, 128, 256, 300, 512, 800, 1024, 1600, 2048, 3000, 4096, 6000, 8192, 10000, 16384, 20000,
               32768, 50000, 65536, 100000)
    shapes = [(n // t, t) for t in lengths]
    shapes += [(n >> 17, 1 << 17), (n >> 18, 1 << 18), (n >> 19, 1 << 19), (n >> 20, 1 << 20), (n >> 22, 1 << 22)]
    shapes += [(r * n >> 25, t) for r, t in ((131071, 255), (43690, 767), (9999, 3333), (2047, 16385), (513, 65537),
                                              (70000, 480), (26000, 1290), (7000, 4800), (1200, 28000))]
    return "rows", [s for s in shapes if s[0] >= 1]


for _log_n in (23, 25, 26):
    SUITES[f"rows-{_log_n}"] = _row_suite(_log_n)


def row_plans(dtype, T):
    """Forced plans for the row layout: workgroups of whole rows, time-split tiles, and for short rows the others."""
    full = 16 // torch.empty(0, dtype=dtype).element_size()
    out = [P(mode=hip.MODE_ROW, vec=full, unroll=u, waves=w, waves_per_row=r)
           for u, w, r in ((4, 4, 1), (4, 4, 4), (2, 4, 1), (4, 8, 8), (4, 16, 16), (2, 8, 8), (4, 4, 2), (1, 4, 1),
                           (2, 4, 2), (3, 3, 3), (4, 2, 2), (8, 4, 4), (4, 12, 12), (2, 16, 16))]
    out += [P(mode=hip.MODE_LOOKBACK, vec=full, unroll=u, waves=w)
            for u, w in ((4, 8), (4, 4), (8, 8), (4, 16), (2, 8), (4, 6))]
    if T <= 64 * full:
        out += [P(mode=hip.MODE_SMALL, vec=full, unroll=u, waves=4) for u in (1, 2, 4)]
        out += [P(mode=hip.MODE_FLAT, vec=full, unroll=4, waves=4), P(mode=hip.MODE_FLAT, vec=full, unroll=2, waves=8)]
    return out


def cl_plans(dtype, C):
    """Forced plans for channels-last storage: every lane width over a few tile shapes, whole-T walks and time-split tiles."""
    esize = torch.empty(0, dtype=dtype).element_size()
    full = 16 // esize
    half, narrow = max(1, full // 2), (2 if esize == 2 else 1)
    walk, split = hip.MODE_ROW, hip.MODE_LOOKBACK
    most = 16 if full == 4 else 8  # waves that the kernels' LDS arrays allow with 16-byte lanes
    out = [P(vec=v, unroll=s, waves=w, mode=walk)
           for v, s, w in ((full, 4, most), (full, 4, 4), (half, 8, 8), (half, 8, 4), (half, 16, 8), (half, 16, 4),
                           (narrow, 8, 8 * (3 - narrow)), (narrow, 16, 8), (1, 8, 16), (1, 16, 8)) if C % v == 0]
    if C % full != 0:  # lanes wider than the channel count divides: taken where a time step fills a wave of them
        out += [P(vec=v, unroll=s, waves=w, mode=walk)
                for v, s, w in ((full, 4, most), (full, 4, 4), (half, 8, 8), (half, 8, 4), (2, 16, 8), (2, 8, 8))
                if C % v != 0 and C > 32 * v]
    out += [P(vec=v, unroll=s, waves=w, mode=split)
            for v, s, w in ((narrow, 16, 8), (half, 16, 8), (half, 8, 8), (1, 16, 8)) if C % v == 0]
    return out


def cl_plans_all(dtype, C):
    """Every launch plan of the channels-last kernels worth timing on a shape: each lane width (whole or
    element-aligned), a walk of all of T or tiles over time, every number of steps per wave, 2 to 16 waves.
    The set that --dump records, from which the constants of the library's cost model are fitted."""
    esize = torch.empty(0, dtype=dtype).element_size()
    full = 16 // esize
    widths = sorted({1, full, max(1, full // 2)} | ({2} if esize == 2 else set()))
    out = []
    for v in widths:
        if C % v != 0 and C <= 32 * v:
            continue  # element-aligned lanes need more than half a wave of them per time step
        for s in ((2, 4, 8) if v == full else (4, 8, 16)):
            for w in (2, 4, 8, 16):
                out.append(P(vec=v, unroll=s, waves=w, mode=hip.MODE_ROW))
                if C % v == 0:
                    out.append(P(vec=v, unroll=s, waves=w, mode=hip.MODE_LOOKBACK))
    return out


def random_cl_shapes(n, seed):
    """n shapes [batch, T, C]: C from 8 to 5000 and T from 64 to 16384, both log-uniform, half of the channel counts
    rounded to multiples of 8; 8 M to 190 M elements; batch what that leaves, 1 to 8192."""
    rng = random.Random(seed)
    out = []
    while len(out) < n:
        C = int(round(2 ** rng.uniform(3, 12.3)))
        if rng.random() < 0.5:
            C = max(8, (C + 4) // 8 * 8)
        T = int(round(2 ** rng.uniform(6, 14)))
        batch = int(2 ** rng.uniform(23, 27.5) / (T * C))
        if 1 <= batch <= 8192:
            out.append((batch, T, C))
    return out


def random_row_shapes(n, seed):
    """n shapes [rows, T]: T from 4 to 2^20 log-uniform, four in ten rounded to multiples of 8; 8 M to 190 M elements."""
    rng = random.Random(seed)
    out = []
    while len(out) < n:
        T = int(round(2 ** rng.uniform(2, 20)))
        if rng.random() < 0.4:
            T = max(4, (T + 4) // 8 * 8)
        rows = int(2 ** rng.uniform(23, 27.5) / T)
        if 1 <= rows <= 1 << 22:
            out.append((rows, T))
    return out


def _time(calls, reps, warm):
    n = len(calls)
    for i in range(max(warm, 1)):
        calls[i % n]()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    e0.record()
    for i in range(reps):
        calls[i % n]()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) / reps * 1e3


def _short(plan):
    if plan is None:
        return "auto"
    s = f"m{plan.mode} v{plan.vec} u{plan.unroll} w{plan.waves}"
    return s + (f" r{plan.waves_per_row}" if plan.waves_per_row else "")


def search(layout, shape, dtype, reps=24, warm=4, out=sys.stdout, every=False, dump=None):
    """Time every plan of the set on ``shape``; returns {direction: (auto_us, best_us, best_plan)}.
    With ``dump`` (an open text file) the set is every plan of ``cl_plans_all`` and each timing is written there as
    one line ``batch T C dtype direction mode vec unroll waves microseconds`` (mode 0 = the automatic plan)."""
    dev = torch.device("cuda:0")
    esize = torch.empty(0, dtype=dtype).element_size()
    n = 1
    for d in shape:
        n *= d
    nsets = max(1, min(8, -(-(1 << 29) // (6 * n * esize))))
    g = torch.Generator(device=dev).manual_seed(0)
    sets = []
    for _ in range(nsets):
        a = (0.9 + 0.1 * torch.rand(shape, generator=g, device=dev)).to(dtype)
        b, gh = (torch.randn(shape, generator=g, device=dev).to(dtype) for _ in range(2))
        sets.append((a, b, gh, torch.empty_like(a), torch.empty_like(a), torch.empty_like(a)))
    if layout == "rows":
        plans, fwd, bwd = row_plans(dtype, shape[-1]), hip.prepare_forward, hip.prepare_backward
    else:
        plans, fwd, bwd = cl_plans(dtype, shape[-1]), hip.prepare_forward_cl, hip.prepare_backward_cl
        if dump is not None:
            plans = cl_plans_all(dtype, shape[-1])
    times = {"fwd": [], "bwd": []}
    for plan in [None] + plans + [None]:
        try:
            f = [fwd(a, b, h, plan=plan) for a, b, gh, h, ga, gb in sets]
            f[0]()  # fills h for the backward pass, and shows whether the library takes this plan here
            r = [bwd(a, h, gh, ga, gb, plan=plan) for a, b, gh, h, ga, gb in sets]
            r[0]()
        except RuntimeError:
            continue
        times["fwd"].append((_time(f, reps, warm), plan))
        times["bwd"].append((_time(r, reps, warm), plan))
        if dump is not None:
            for name in ("fwd", "bwd"):
                q = plan if plan is not None else P()
                print(*shape, str(dtype).replace("torch.", ""), name, q.mode, q.vec, q.unroll, q.waves,
                      f"{times[name][-1][0]:.2f}", file=dump, flush=True)
    res, text = {}, []
    if layout == "rows":
        chosen = [hip.resolve_plan(*shape, dtype, d) for d in (hip.FORWARD, hip.BACKWARD)]
    else:
        chosen = [hip.resolve_plan_cl(*shape, dtype, d) for d in (hip.FORWARD, hip.BACKWARD)]
    for (name, per_elem), auto_plan in zip((("fwd", 3), ("bwd", 5)), chosen):
        auto = min(t for t, p in times[name] if p is None)
        best, best_plan = min(times[name], key=lambda tp: tp[0])
        res[name] = (auto, best, best_plan)
        frac = per_elem * esize * n / (auto * 1e-6) / 1e9 / HBM_PEAK_GBPS
        text.append(f"{name} auto [{_short(auto_plan):16s}] {auto:7.1f} us {100 * frac:4.1f} %  best {best:7.1f} {_short(best_plan):16s}"
                    + (" BEHIND" if auto > 1.08 * best else "       "))
    label = "x".join(str(d) for d in shape) + ":" + str(dtype).replace("torch.", "")
    print(f"{layout} {label:26s} {len(times['fwd']) - 2:2d} plans | " + " | ".join(text), file=out, flush=True)
    if every:
        for (tf, plan), (tb, _) in zip(times["fwd"], times["bwd"]):
            print(f"    {_short(plan):18s} fwd {tf:7.1f} us  bwd {tb:7.1f} us", file=out, flush=True)
    return res


def main(argv=None):
    ap = argparse.ArgumentParser(description=__doc__.split("\n\n")[0])
    ap.add_argument("layout", nargs="?", choices=("rows", "cl"))
    ap.add_argument("shapes", nargs="*", metavar="SHAPE[:dtype]")
    ap.add_argument("--suite", choices=sorted(SUITES), help="a fixed list of shapes, each in f32 and bf16")
    ap.add_argument("--random", type=int, metavar="N",
                    help="N shapes drawn at random (channels-last, or rows when that layout is named), each in f32 and bf16")
    ap.add_argument("--seed", type=int, default=0, help="seed of --random")
    ap.add_argument("--dtypes", default="f32,bf16", help="storage types of --suite and --random shapes (f32, bf16, f16, f64)")
    ap.add_argument("--reps", type=int, default=24)
    ap.add_argument("--every", action="store_true", help="also print every plan's timings")
    ap.add_argument("--dump", metavar="FILE", help="channels-last: time every plan of the full set and append each "
                    "timing to FILE (the data the cost model's constants are fitted to)")
    args = ap.parse_intermixed_args(argv)  # options may stand between the layout and the shapes
    if not hip.has_hip_ops:
        sys.exit("plan_search: libscanscam_hip.so does not load")
    if not torch.cuda.is_available():
        sys.exit("plan_search: no GPU visible")
    jobs = []
    if args.suite:
        layout, shapes = SUITES[args.suite]
        jobs = [(layout, s, DTYPES[dt]) for s in shapes for dt in args.dtypes.split(",")]
    elif args.random:
        layout = args.layout or "cl"
        shapes = (random_row_shapes if layout == "rows" else random_cl_shapes)(args.random, args.seed)
        jobs = [(layout, s, DTYPES[dt]) for s in shapes for dt in args.dtypes.split(",")]
    elif args.layout is None:
        ap.error("give a layout and shapes, --suite or --random")
    for spec in args.shapes:
        shape_s, _, dtype_s = spec.partition(":")
        shape = tuple(int(v) for v in shape_s.lower().split("x"))
        if len(shape) != (2 if args.layout == "rows" else 3):
            ap.error(f"{spec}: a {args.layout} shape has {2 if args.layout == 'rows' else 3} sizes")
        jobs.append((args.layout, shape, DTYPES[dtype_s]))
    ratios = []
    dump = open(args.dump, "a") if args.dump else None
    for layout, shape, dtype in jobs:
        res = search(layout, shape, dtype, reps=args.reps, every=args.every, dump=dump if layout == "cl" else None)
        ratios += [auto / best for auto, best, _ in res.values()]
    behind = sum(r > 1.08 for r in ratios)
    print(f"{2 * len(jobs)} timings, automatic plan more than 8 % behind the set's best in {behind}", flush=True)
    if args.random and ratios:
        ratios.sort()
        print(f"automatic / best: median {ratios[len(ratios) // 2]:.3f}, mean {sum(ratios) / len(ratios):.3f}, "
              f"above 1.15 in {sum(r > 1.15 for r in ratios)}, above 1.3 in {sum(r > 1.3 for r in ratios)}, "
              f"largest {ratios[-1]:.2f}", flush=True)


if __name__ == "__main__":
    main()
