"""
Fit the constants of the channels-last cost model to measured timings.

    python -m scanscam_amd.plan_search --random 40 --seed 11 --dump timings.txt     (on the GPU; any shapes, any number of files)
    python -m scanscam_amd.plan_fit timings.txt [more.txt ...] [--held-out other.txt] > scanscam_amd/csrc/scan_cl_model.inc

The library chooses the launch plan of a channels-last call by estimating every candidate plan's duration
(``scanscam_amd/csrc/scan_cl_plan.hpp``: ``cl_predict_us``) and taking the smallest. This tool holds the same
formula (``predict`` below; ``tests/test_host.py`` checks the two against each other through
``scanscam_predict_cl``), fits its constants to the dumped timings by least squares on the logarithm of the
duration -- plans within 2.5 times of a shape's best only, weighted towards the best -- and prints the table the
library is compiled with. To stderr it reports how far the plan the fitted model would pick is behind the best
measured plan, per (shape, storage type, direction), on the training files and on ``--held-out`` files that took no
part in the fit.

A dump line is ``batch T C dtype direction mode vec unroll waves microseconds`` (mode 2 = a workgroup walks all
of T, 3 = tiles of time over workgroups, 0 = the library's automatic plan at the time of the dump).
"""
import argparse
import collections
import math
import sys

import numpy as np

ESIZE = {"float32": 4, "bfloat16": 2, "float16": 2, "float64": 8}
KERNELS, STORAGE, LANES = (0, 1, 2), (2, 4, 8), (2, 4, 8, 16)
SCALARS = ["latency", "latency_w8", "issue", "issue_bwd", "issue_16", "issue_ragged", "launch", "launch_split", "carry",
           "fill_alpha", "chain", "issue_shared", "line_2", "line_4", "line_8", "line_16"]
START = [1.0, 0.5, 0.04, 1.4, 0.6, 0.6, 3.0, 0.5, 6.0, 0.2, 1.0, 0.5, 0.5, 0.5, 0.5, 0.5]
LOWER = [0.2, 0.0, 0.001, 0.8, 0.3, 0.0, 0.0, 0.0, 0.0, 0.0, 0.0, 0.0, 0.0, 0.0, 0.0, 0.0]
UPPER = [10.0, 5.0, 0.3, 4.0, 4.0, 3.0, 15.0, 20.0, 20.0, 1.0, 10.0, 10.0, 5.0, 5.0, 5.0, 5.0]
N_RATE = len(KERNELS) * len(STORAGE) * len(LANES) * 2 * 2
WAVE, CUS = 64, 256


def rate_index(kernel, esize, lane, rev, whole=False):
    return (((kernel * len(STORAGE) + STORAGE.index(esize)) * len(LANES) + LANES.index(max(lane, 2))) * 2 + int(rev)) * 2 + int(whole)


def pow2_ceil(v):
    p = 1
    while p < v:
        p <<= 1
    return p


def describe(batch, T, C, esize, rev, mode, vec, steps, waves):
    """What cl_complete() and the first lines of cl_predict_us() derive from (shape, plan)."""
    kind = 2 if mode == 3 else 0
    G = -(-C // (WAVE * vec))
    group = WAVE
    if kind == 0 and G == 1:
        g = pow2_ceil(-(-C // vec))
        if g < WAVE:
            group = g
    sub = WAVE // group
    tile_steps = waves * steps * sub
    return dict(batch=batch, T=T, C=C, esize=esize, rev=rev, vec=vec, steps=steps, waves=waves, kind=kind, G=G,
                group=group, sub=sub, ragged=C % vec != 0, lane=vec * esize, RG=batch * G, tiles=-(-T // tile_steps),
                fill=C / (G * WAVE * vec) if group == WAVE else C / (group * vec),
                bytes=batch * T * C * esize * (5 if rev else 3))


def registers(d):
    per = (3.8 if d["rev"] else 2.8) if d["esize"] == 2 else (3.0 if d["rev"] else 2.1)
    base = 34.0 if d["kind"] == 2 else 24.0
    if d["group"] < WAVE:
        base, per = (36.0, 5.7) if d["rev"] else (32.0, 4.6)
    return base + d["steps"] * d["vec"] * per * (2.0 if d["esize"] == 8 else 1.0)


def predict(d, p):
    """cl_predict_us() of scan_cl_plan.hpp, term for term."""
    q = dict(zip(SCALARS, p[N_RATE:]))
    regs = registers(d)
    cap = 256.0 if d["vec"] > 1 and d["steps"] >= 8 else 128.0  # the kernels' launch bounds: 512 or 1024 threads
    spills = regs > cap
    regs = min(regs, cap)
    occupancy = max(1, min(8, int(512.0 / regs)))
    resident_max = max(1, (4 * occupancy) // d["waves"])
    busy = (q["issue"] * d["steps"] * d["vec"] * (d["waves"] / 4.0 if d["waves"] > 4 else 1.0) *
            (q["issue_bwd"] if d["rev"] else 1.0) * (q["issue_16"] if d["esize"] == 2 else 1.0))
    if spills:
        busy *= 2.0
    if d["group"] < WAVE:
        busy *= 1.0 + q["issue_shared"] * math.log2(d["sub"])
    if d["ragged"]:
        busy *= 1.0 + q["issue_ragged"]
    workgroups = d["RG"] * d["tiles"] if d["kind"] == 2 else d["RG"]
    resident = min(math.ceil(workgroups / CUS), resident_max)
    tile_us = q["latency"] + q["latency_w8"] * d["waves"] / 8.0 + busy + (q["carry"] if d["kind"] == 2 else 0.0)
    rounds = math.ceil(workgroups / (CUS * resident_max))
    latency_us = rounds * (1 if d["kind"] == 2 else d["tiles"]) * max(tile_us, resident * busy)
    kernel = 1 if d["group"] < WAVE else d["kind"]
    rate = p[rate_index(kernel, d["esize"], d["lane"], d["rev"], (d["C"] * d["esize"]) % 128 == 0)] * 1e6
    step_bytes = d["C"] * d["esize"]
    line = q["line_%d" % max(2, d["lane"])]
    if d["group"] < WAVE:
        span = d["sub"] * step_bytes
        lines = 1.0 + line * (128 - math.gcd(span, 128)) / span
    else:
        a = math.gcd(math.gcd(step_bytes, WAVE * d["lane"]), 128)
        lines = 1.0 + line * d["G"] * (128 - a) / step_bytes
    stream_us = d["bytes"] / d["fill"] ** q["fill_alpha"] / rate * lines
    chain_us = q["chain"] * d["tiles"] / d["waves"] if d["kind"] == 2 else 0.0
    return q["launch"] + (q["launch_split"] if d["kind"] == 2 else 0.0) + stream_us + latency_us + chain_us


FIELDS = ("steps", "vec", "waves", "rev", "esize", "group", "sub", "ragged", "kind", "RG", "tiles", "lane", "C", "G", "fill",
          "bytes")


def columns(ds):
    """The descriptions of many (shape, plan) pairs as arrays, for predict_many()."""
    cols = {k: np.array([float(d[k]) for d in ds]) for k in FIELDS}
    cols["regs"] = np.array([registers(d) for d in ds])
    cols["cap"] = np.array([256.0 if d["vec"] > 1 and d["steps"] >= 8 else 128.0 for d in ds])
    cols["rate_index"] = np.array([rate_index(1 if d["group"] < WAVE else d["kind"], d["esize"], d["lane"], d["rev"],
                                              (d["C"] * d["esize"]) % 128 == 0) for d in ds])
    step_bytes = [d["C"] * d["esize"] for d in ds]
    cols["lines_extra"] = np.array([
        (128 - math.gcd(d["sub"] * sb, 128)) / (d["sub"] * sb) if d["group"] < WAVE
        else d["G"] * (128 - math.gcd(math.gcd(sb, WAVE * d["lane"]), 128)) / sb for d, sb in zip(ds, step_bytes)])
    return cols


def predict_many(c, p):
    """predict() over the arrays of columns(): the same arithmetic, vectorised (the fit calls it millions of times)."""
    q = dict(zip(SCALARS, p[N_RATE:]))
    spills = c["regs"] > c["cap"]
    regs = np.minimum(c["regs"], c["cap"])
    occupancy = np.clip(np.floor(512.0 / regs), 1, 8)
    resident_max = np.maximum(1, np.floor(4 * occupancy / c["waves"]))
    packed, split, rev = c["group"] < WAVE, c["kind"] == 2, c["rev"] > 0
    busy = (q["issue"] * c["steps"] * c["vec"] * np.where(c["waves"] > 4, c["waves"] / 4.0, 1.0) *
            np.where(rev, q["issue_bwd"], 1.0) * np.where(c["esize"] == 2, q["issue_16"], 1.0))
    busy = busy * np.where(spills, 2.0, 1.0) * np.where(packed, 1.0 + q["issue_shared"] * np.log2(c["sub"]), 1.0)
    busy = busy * np.where(c["ragged"] > 0, 1.0 + q["issue_ragged"], 1.0)
    workgroups = np.where(split, c["RG"] * c["tiles"], c["RG"])
    resident = np.minimum(np.ceil(workgroups / CUS), resident_max)
    tile_us = q["latency"] + q["latency_w8"] * c["waves"] / 8.0 + busy + np.where(split, q["carry"], 0.0)
    rounds = np.ceil(workgroups / (CUS * resident_max))
    latency_us = rounds * np.where(split, 1.0, c["tiles"]) * np.maximum(tile_us, resident * busy)
    rate = p[c["rate_index"]] * 1e6
    line = np.choose(np.log2(np.maximum(c["lane"], 2)).astype(int) - 1, [q["line_2"], q["line_4"], q["line_8"], q["line_16"]])
    lines = 1.0 + line * c["lines_extra"]
    stream_us = c["bytes"] / c["fill"] ** q["fill_alpha"] / rate * lines
    chain_us = np.where(split, q["chain"] * c["tiles"] / c["waves"], 0.0)
    return q["launch"] + np.where(split, q["launch_split"], 0.0) + stream_us + latency_us + chain_us


def load(paths):
    """{(batch, T, C, esize, rev): [(description or None for the automatic plan, microseconds), ...]}"""
    by = collections.defaultdict(list)
    for path in paths:
        for line in open(path):
            f = line.split()
            if len(f) != 10:
                continue
            batch, T, C, esize, rev = int(f[0]), int(f[1]), int(f[2]), ESIZE[f[3]], f[4] == "bwd"
            mode, vec, steps, waves, us = int(f[5]), int(f[6]), int(f[7]), int(f[8]), float(f[9])
            d = describe(batch, T, C, esize, rev, mode, vec, steps, waves) if mode else None
            by[(batch, T, C, esize, rev)].append((d, us))
    return by


def candidate(d):
    """A plan the library's own choice considers (cl_choose): 4 or 8 waves (a walk also 16), no 16-byte 16-bit lanes in
    a time split."""
    waves = (4, 8, 16) if d["kind"] == 0 else (4, 8)
    return d["waves"] in waves and not (d["kind"] == 2 and d["esize"] == 2 and d["vec"] == 8)


def regret(by, p, out, label):
    picks, autos = [], []
    for key, timings in by.items():
        plans = [(d, us) for d, us in timings if d is not None]
        cands = [(d, us) for d, us in plans if candidate(d)]
        # cl_choose passes over a walk with fewer workgroups than half the compute units when the time can be split
        wide = [(d, us) for d, us in cands if not (d["kind"] == 0 and 2 * d["RG"] < CUS)]
        cands = wide or cands
        if not cands:
            continue
        best = min(us for _, us in plans)
        picks.append(min(cands, key=lambda t: predict(t[0], p))[1] / best)
        auto = [us for d, us in timings if d is None]
        if auto:
            autos.append(min(auto) / best)
    for name, x in (("model's pick", np.array(picks)), ("automatic plan of the dump", np.array(autos))):
        if len(x):
            print(f"{label}: {name} / best measured plan over {len(x)} cases: median {np.median(x):.3f}, mean {x.mean():.3f}, "
                  f"above 1.15 in {(x > 1.15).sum()}, above 1.3 in {(x > 1.3).sum()}, largest {x.max():.2f}", file=out)


def fit(by, evaluations=200):
    from scipy.optimize import least_squares

    rows, weights, case = [], [], []
    for number, (key, timings) in enumerate(by.items()):
        plans = [(d, us) for d, us in timings if d is not None and d["waves"] in (4, 8, 16)]
        if not plans:
            continue
        best = min(us for _, us in plans)
        for d, us in plans:
            if us < 2.5 * best:
                rows.append((d, math.log(us)))
                weights.append(1.0 / (1.0 + 3.0 * math.log(us / best)))
                case.append(number)
    weights = np.array(weights)
    target = np.array([y for _, y in rows])
    case = np.array(case)
    case_weight = np.maximum(np.bincount(case, weights=weights), 1e-9)
    cols = columns([d for d, _ in rows])
    # Only the rates that some timing exercises are free; the others stay at the start value (emit() says so).
    seen = sorted(set(int(i) for i in cols["rate_index"]))
    free = np.array(seen + list(range(N_RATE, N_RATE + len(SCALARS))))
    full0 = np.concatenate([np.full(N_RATE, 5.5), START])
    lo = np.concatenate([np.full(N_RATE, 1.0), LOWER])[free]
    hi = np.concatenate([np.full(N_RATE, 8.0), UPPER])[free]

    def expand(x):
        p = full0.copy()
        p[free] = x
        return p

    # What the choice needs is the order of one shape's plans, not the level of its durations: 0.7 of a case's
    # (weighted) mean error is taken out of each of its residuals, so an error common to all plans of a shape
    # counts for little and the constants go where they tell plans apart.
    def residual(x):
        r = np.log(np.maximum(predict_many(cols, expand(x)), 1e-3)) - target
        common = np.bincount(case, weights=weights * r) / case_weight
        return (r - 0.7 * common[case]) * weights

    sol = least_squares(residual, full0[free], bounds=(lo, hi), loss="soft_l1", f_scale=0.1, max_nfev=evaluations)
    p = expand(sol.x)
    # The vectorised form and the term-for-term one are the same function.
    for i in range(0, len(rows), max(1, len(rows) // 200)):
        one = predict(rows[i][0], p)
        assert abs(one - predict_many({k: v[i:i + 1] for k, v in cols.items()}, p)[0]) <= 1e-6 * one
    return p, float(np.sqrt((residual(sol.x) ** 2).mean())), set(seen), len(rows)


def emit(p, seen, note, out):
    print("// Constants of the channels-last cost model (ClModel, scan_cl_plan.hpp). Printed by", file=out)
    print(f"//   python -m scanscam_amd.plan_fit {note}", file=out)
    print("// from timings written by `python -m scanscam_amd.plan_search --dump` on one MI355X; do not edit by hand.", file=out)
    print("// rate[kernel][storage][lane][direction][time steps are whole 128-byte lines]; a variant that no timing exercised", file=out)
    print("// (marked *) holds the mean of the exercised ones of its kernel and storage size.", file=out)
    print("const ClModel kClModel = {", file=out)
    print("    {", file=out)
    per = len(LANES) * 4
    for k in KERNELS:
        print("        {", file=out)
        for e in STORAGE:
            cells = []
            for lane in LANES:
                pairs = []
                for rev in (0, 1):
                    vals = []
                    for whole in (0, 1):
                        i = rate_index(k, e, lane, rev, whole)
                        v = p[i]
                        if i not in seen:
                            same = [p[j] for j in seen if j // per == i // per] or [p[j] for j in seen]
                            v = float(np.mean(same))
                        vals.append(f"{v:.3f}" + ("" if i in seen else " /* * */"))
                    pairs.append("{" + ", ".join(vals) + "}")
                cells.append("{" + ", ".join(pairs) + "}")
            print(f"            {{{', '.join(cells)}}},  // kernel {k}, {e}-byte storage: lanes of 2, 4, 8, 16 bytes x (forward, backward) x (part lines, whole lines)", file=out)
        print("        },", file=out)
    print("    },", file=out)
    q = dict(zip(SCALARS, p[N_RATE:]))
    for name in SCALARS[:12]:
        print(f"    {q[name]:.4f},  // {name}", file=out)
    print("    {" + ", ".join(f"{q['line_%d' % b]:.4f}" for b in LANES) + "},  // line: lanes of 2, 4, 8, 16 bytes", file=out)
    print("};", file=out)


def read_table(path):
    """The constants of a scan_cl_model.inc as the vector predict() takes (the inverse of emit())."""
    import re

    body = open(path).read().split("const ClModel kClModel")[1]
    body = re.sub(r"/\*.*?\*/", "", body)
    body = re.sub(r"//[^\n]*", "", body)
    nums = [float(x) for x in re.findall(r"-?\d+\.\d+(?:e-?\d+)?", body)]
    assert len(nums) == N_RATE + len(SCALARS), (len(nums), N_RATE + len(SCALARS))
    return np.array(nums)


def main(argv=None):
    ap = argparse.ArgumentParser(description=__doc__.split("\n\n")[0])
    ap.add_argument("dumps", nargs="+", help="files written by plan_search --dump")
    ap.add_argument("--held-out", nargs="*", default=[], help="dumps that take no part in the fit, for the report")
    ap.add_argument("--evaluations", type=int, default=200)
    args = ap.parse_args(argv)
    by = load(args.dumps)
    p, rms, seen, n = fit(by, args.evaluations)
    print(f"fitted {N_RATE + len(SCALARS)} constants ({len(seen)} of {N_RATE} rates exercised) to {n} timings of "
          f"{len(by)} cases; rms error of log(duration) {rms:.3f}", file=sys.stderr)
    regret(by, p, sys.stderr, "training files")
    if args.held_out:
        regret(load(args.held_out), p, sys.stderr, "held-out files")
    emit(p, seen, " ".join(a.split("/")[-1] for a in args.dumps), sys.stdout)


if __name__ == "__main__":
    main()
