"""
Fit the constants of the channels-last cost model to measured timings.

    python -m scanscam_amd.plan_search --random 40 --seed 11 --dump timings.txt     (on the GPU; any shapes, any number of files)
    python -m scanscam_amd.plan_fit timings.txt [more.txt ...] [--held-out other.txt] > scanscam_amd/csrc/scan_cl_model.inc

The library chooses the launch plan of a channels-last call by estimating every candidate plan's duration
(``scanscam_amd/csrc/scan_cl_plan.hpp``: ``cl_predict_us``) and taking the smallest. This tool holds the same
formula (``predict`` below; ``tests/test_host.py`` checks the two against each other through
``scanscam_predict_cl``), fits its constants to the dumped timings by least squares on the logarithm of the
duration -- plans within 2.5 times of a shape's best only, weighted towards the best. What that formula leaves
unexplained (about 7 % rms, against 1 % of run-to-run noise) a small network then learns from the same timings
(``fit_residual``: 24 inputs that describe shape and plan, two hidden layers, the logarithm of measured over
estimated duration as the target; scikit-learn trains it, the library only evaluates it), and the tool prints both
tables, which the library is compiled with. To stderr it reports how far the plan the fitted model would pick is behind the best
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


N_FEATURES, HIDDEN, RESIDUAL_LIMIT = 24, (64, 32), 0.7


def features(d, physical_us):
    """cl_features() of scan_cl_plan.hpp: what the learned correction sees of a (shape, plan) pair."""
    step_bytes = d["C"] * d["esize"]
    workgroups = d["RG"] * d["tiles"] if d["kind"] == 2 else d["RG"]
    return [math.log2(d["RG"]), math.log2(d["tiles"]), math.log2(d["T"]), math.log2(d["C"]), math.log2(d["batch"]),
            d["fill"], float(d["steps"]), float(d["vec"]), float(d["waves"]), float(d["kind"]), float(d["esize"]),
            float(d["rev"]), float(d["group"] < WAVE), math.log2(d["sub"]), float(d["ragged"]), registers(d),
            math.log2(workgroups), ((workgroups - 1) % CUS + 1) / float(CUS), float(step_bytes % 128 == 0),
            float(step_bytes % 16 == 0), math.log2(d["bytes"]), math.log(physical_us), math.log2(d["lane"]),
            min(workgroups / float(CUS), 8.0)]


class Residual:
    """The learned correction: ln(measured / physical estimate) as a function of features(), clipped to
    +-RESIDUAL_LIMIT; inputs are clipped to the range the training timings covered, so it never extrapolates."""

    def __init__(self, lo, hi, mean, scale, w1, b1, w2, b2, w3, b3):
        self.parts = [np.asarray(a, dtype=np.float64) for a in (lo, hi, mean, scale, w1, b1, w2, b2, w3)] + [float(b3)]

    @classmethod
    def zero(cls):
        n, (h1, h2) = N_FEATURES, HIDDEN
        return cls(np.full(n, -1e30), np.full(n, 1e30), np.zeros(n), np.ones(n), np.zeros((n, h1)), np.zeros(h1),
                   np.zeros((h1, h2)), np.zeros(h2), np.zeros(h2), 0.0)

    def correct(self, x):
        """x: [rows, N_FEATURES] (or one row) -> the correction of ln(duration) per row."""
        lo, hi, mean, scale, w1, b1, w2, b2, w3, b3 = self.parts
        z = (np.clip(np.atleast_2d(np.asarray(x, dtype=np.float64)), lo, hi) - mean) / scale
        y = np.tanh(np.tanh(z @ w1 + b1) @ w2 + b2) @ w3 + b3
        return np.clip(y, -RESIDUAL_LIMIT, RESIDUAL_LIMIT)

    def flat(self):
        return np.concatenate([np.ravel(a) for a in self.parts[:-1]] + [[self.parts[-1]]])


def estimate(d, p, r):
    """cl_predict_us(): the physical estimate times the learned correction."""
    physical = predict(d, p)
    return physical * math.exp(float(r.correct(features(d, physical))[0]))


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


def regret(by, p, out, label, r=None):
    cost = (lambda d: estimate(d, p, r)) if r is not None else (lambda d: predict(d, p))
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
        picks.append(min(cands, key=lambda t: cost(t[0]))[1] / best)
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


def fit_residual(by, p, seed=0, max_iter=600):
    """Trains the correction on what the fitted formula leaves: ln(measured / physical estimate) of every timed plan
    within 4 times of its shape's best. Returns (Residual, rms before, rms after) over those timings."""
    from sklearn.neural_network import MLPRegressor
    from sklearn.preprocessing import StandardScaler

    x, y = [], []
    for key, timings in by.items():
        plans = [(d, us) for d, us in timings if d is not None and d["waves"] in (4, 8, 16)]
        if not plans:
            continue
        best = min(us for _, us in plans)
        for d, us in plans:
            if us < 4.0 * best:
                physical = predict(d, p)
                x.append(features(d, physical))
                y.append(math.log(us / physical))
    x, y = np.array(x), np.array(y)
    scaler = StandardScaler().fit(x)
    net = MLPRegressor(hidden_layer_sizes=HIDDEN, activation="tanh", alpha=1e-3, max_iter=max_iter, random_state=seed,
                       early_stopping=True, n_iter_no_change=25)
    net.fit(scaler.transform(x), y)
    r = Residual(x.min(0), x.max(0), scaler.mean_, scaler.scale_, net.coefs_[0], net.intercepts_[0], net.coefs_[1],
                 net.intercepts_[1], net.coefs_[2][:, 0], net.intercepts_[2][0])
    after = y - r.correct(x)
    return r, float(np.sqrt((y ** 2).mean())), float(np.sqrt((after ** 2).mean()))


def emit(p, seen, note, out, r=None):
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
    r = r if r is not None else Residual.zero()
    lo, hi, mean, scale, w1, b1, w2, b2, w3, b3 = r.parts

    def row(a):
        return "{" + ", ".join(f"{v:.9g}" for v in a) + "}"

    print("", file=out)
    print("// The learned correction (ClResidual): ln(measured / estimate above) from cl_features(); trained by the same", file=out)
    print("// command on the same timings. lo, hi: the range of each input in the training timings (inputs are clipped to it).", file=out)
    print("const ClResidual kClResidual = {", file=out)
    for name, a in (("lo", lo), ("hi", hi), ("mean", mean), ("scale", scale)):
        print(f"    {row(a)},  // {name}", file=out)
    print("    {  // w1[input][hidden 1]", file=out)
    for a in w1:
        print(f"        {row(a)},", file=out)
    print("    },", file=out)
    print(f"    {row(b1)},  // b1", file=out)
    print("    {  // w2[hidden 1][hidden 2]", file=out)
    for a in w2:
        print(f"        {row(a)},", file=out)
    print("    },", file=out)
    print(f"    {row(b2)},  // b2", file=out)
    print(f"    {row(w3)},  // w3", file=out)
    print(f"    {b3:.9g},  // b3", file=out)
    print("};", file=out)


def read_table(path):
    """The constants of a scan_cl_model.inc as the vector predict() takes (the inverse of emit())."""
    import re

    body = open(path).read().split("const ClModel kClModel")[1].split("\n};")[0]
    body = re.sub(r"/\*.*?\*/", "", body)
    body = re.sub(r"//[^\n]*", "", body)
    nums = [float(x) for x in re.findall(r"-?\d+\.\d+(?:e-?\d+)?", body)]
    assert len(nums) == N_RATE + len(SCALARS), (len(nums), N_RATE + len(SCALARS))
    return np.array(nums)


def read_residual(path):
    """The learned correction of a scan_cl_model.inc (the inverse of emit()'s second table)."""
    import re

    body = open(path).read().split("const ClResidual kClResidual")[1].split("\n};")[0]
    body = re.sub(r"//[^\n]*", "", body)
    nums = [float(x) for x in re.findall(r"-?(?:\d+\.?\d*|\.\d+)(?:[eE][-+]?\d+)?", body)]
    n, (h1, h2) = N_FEATURES, HIDDEN
    sizes = [n, n, n, n, n * h1, h1, h1 * h2, h2, h2, 1]
    assert len(nums) == sum(sizes), (len(nums), sum(sizes))
    parts, at = [], 0
    for size in sizes:
        parts.append(np.array(nums[at:at + size]))
        at += size
    parts[4], parts[6] = parts[4].reshape(n, h1), parts[6].reshape(h1, h2)
    return Residual(*parts[:9], parts[9][0])


def main(argv=None):
    ap = argparse.ArgumentParser(description=__doc__.split("\n\n")[0])
    ap.add_argument("dumps", nargs="+", help="files written by plan_search --dump")
    ap.add_argument("--held-out", nargs="*", default=[], help="dumps that take no part in the fit, for the report")
    ap.add_argument("--evaluations", type=int, default=200)
    ap.add_argument("--no-residual", action="store_true", help="fit the formula only; the correction is printed as zero")
    args = ap.parse_args(argv)
    by = load(args.dumps)
    p, rms, seen, n = fit(by, args.evaluations)
    print(f"fitted {N_RATE + len(SCALARS)} constants ({len(seen)} of {N_RATE} rates exercised) to {n} timings of "
          f"{len(by)} cases; rms error of log(duration) {rms:.3f}", file=sys.stderr)
    held = load(args.held_out) if args.held_out else None
    regret(by, p, sys.stderr, "training files, formula alone")
    if held:
        regret(held, p, sys.stderr, "held-out files, formula alone")
    r = None
    if not args.no_residual:
        r, before, after = fit_residual(by, p)
        print(f"learned correction ({N_FEATURES} inputs, hidden layers of {HIDDEN[0]} and {HIDDEN[1]}): rms of ln(measured / "
              f"estimate) over the plans within 4 times of the best {before:.3f} -> {after:.3f}", file=sys.stderr)
        regret(by, p, sys.stderr, "training files, with the correction", r)
        if held:
            regret(held, p, sys.stderr, "held-out files, with the correction", r)
    emit(p, seen, " ".join(a.split("/")[-1] for a in args.dumps), sys.stdout, r)

if __name__ == "__main__":
    main()
