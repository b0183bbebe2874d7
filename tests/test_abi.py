"""
The C-ABI library loads here (no GPU needed), exports every function that
include/scanscam_hip.h declares, and rejects bad arguments before launching
anything. No kernel is launched in this file.
"""
import ctypes
import os
import re

import numpy as np
import pytest
import torch

from scanscam_amd import hip

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "scanscam_hip.h")

E_OK, E_INVAL, E_DTYPE, E_ALIGN, E_PLAN, E_WORKSPACE, E_LAUNCH = range(7)


def declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(scanscam_[a-z0-9_]+)\s*\(", text)))


def test_library_is_built_and_loads():
    assert os.path.exists(hip.LIB_PATH), "build with `make -C scanscam_amd/csrc`"
    assert hip.has_hip_ops
    assert hip.lib().scanscam_abi_version() == hip.ABI_VERSION


def test_every_declared_symbol_is_exported():
    names = declared_functions()
    assert "scanscam_scan_fwd" in names and "scanscam_scan_bwd" in names and len(names) == 23
    raw = ctypes.CDLL(hip.LIB_PATH)
    for name in names:
        assert hasattr(raw, name), f"{name} declared in scanscam_hip.h but not exported"


def test_header_is_plain_c():
    import subprocess
    import tempfile

    with tempfile.TemporaryDirectory() as d:
        src = os.path.join(d, "t.c")
        open(src, "w").write('#include "scanscam_hip.h"\nint main(void) { scanscam_plan p = {0}; return p.mode; }\n')
        subprocess.run(["gcc", "-std=c99", "-Wall", "-Werror", "-I", os.path.join(ROOT, "include"), "-c", src,
                        "-o", os.path.join(d, "t.o")], check=True)


def test_strerror_covers_every_code():
    seen = set()
    for code in range(8):
        msg = hip.strerror(code)
        assert msg and msg not in seen
        seen.add(msg)
    assert "unknown" in hip.strerror(99)


def test_plan_struct_layout_matches_header():
    assert ctypes.sizeof(hip.Plan) == 24
    assert [f[0] for f in hip.Plan._fields_] == ["mode", "vec", "unroll", "waves", "waves_per_row", "spin_limit"]


def test_argument_errors_are_reported_before_any_launch():
    L = hip.lib()
    fake = 0x10000  # never dereferenced: every call below must fail validation first
    assert L.scanscam_scan_fwd(fake, fake, fake, 4, 8, 7, None, 0, None) == E_DTYPE
    assert L.scanscam_scan_fwd(fake, fake, fake, -1, 8, 0, None, 0, None) == E_INVAL
    assert L.scanscam_scan_fwd(fake, fake, fake, 4, 2**31, 0, None, 0, None) == E_INVAL
    assert L.scanscam_scan_fwd(None, fake, fake, 4, 8, 0, None, 0, None) == E_INVAL
    assert L.scanscam_scan_bwd(fake, fake, fake, None, fake, 4, 8, 0, None, 0, None) == E_INVAL
    assert L.scanscam_scan_fwd(fake + 2, fake, fake, 4, 8, 0, None, 0, None) == E_ALIGN
    assert L.scanscam_scan_fwd(fake + 1, fake, fake, 4, 8, 1, None, 0, None) == E_ALIGN
    # Long rows need a workspace.
    assert hip.workspace_bytes(4, 1 << 20, torch.float32) > 0
    assert L.scanscam_scan_fwd(fake, fake, fake, 4, 1 << 20, 0, None, 0, None) == E_WORKSPACE
    assert L.scanscam_scan_fwd(fake, fake, fake, 4, 1 << 20, 0, fake, 64, None) == E_WORKSPACE
    # Bad explicit plans.
    for bad in (hip.Plan(mode=9), hip.Plan(vec=3), hip.Plan(mode=hip.MODE_ROW, unroll=5),
                hip.Plan(mode=hip.MODE_ROW, unroll=8, waves=9), hip.Plan(mode=hip.MODE_ROW, waves=4, waves_per_row=3),
                hip.Plan(mode=hip.MODE_SMALL), hip.Plan(waves=17)):
        rc = L.scanscam_scan_fwd_plan(fake, fake, fake, 4, 4096, 0, None, 0, None, ctypes.byref(bad))
        assert rc == E_PLAN, bad
    # Rows of fewer than four vectors can use the 16-byte vector only if they start on 16-byte borders.
    v4 = hip.Plan(vec=4)
    assert L.scanscam_scan_fwd_plan(fake, fake, fake, 4, 5, 0, None, 0, None, ctypes.byref(v4)) == E_PLAN
    assert L.scanscam_scan_fwd_plan(fake + 4, fake, fake, 4, 12, 0, None, 0, None, ctypes.byref(v4)) == E_PLAN
    # ... and element-aligned long rows only with 2 or 4 chunks per wave.
    v4u8 = hip.Plan(vec=4, unroll=8)
    assert L.scanscam_scan_fwd_plan(fake, fake, fake, 4, 1025, 0, None, 0, None, ctypes.byref(v4u8)) == E_PLAN


def test_strided_calls_check_their_arguments():
    L = hip.lib()
    fake = ctypes.c_void_p(0x1000)
    S = hip.Strides
    assert ctypes.sizeof(S) == 16
    dense = ctypes.byref(S(4096, 64))
    neg = ctypes.byref(S(-1, 64))
    # negative strides, negative sizes and a row count that overflows are rejected before any launch
    assert L.scanscam_scan_fwd_strided(fake, fake, fake, neg, dense, dense, 4, 64, 64, 0, None, 0, None, None) == E_INVAL
    assert L.scanscam_scan_fwd_strided(fake, fake, fake, dense, dense, dense, -1, 64, 64, 0, None, 0, None, None) == E_INVAL
    assert L.scanscam_scan_fwd_strided(fake, fake, fake, None, None, None, 1 << 40, 1 << 40, 64, 0, None, 0, None,
                                       None) == E_INVAL
    assert L.scanscam_scan_bwd_strided(fake, fake, fake, fake, None, None, None, None, None, None, 4, 64, 64, 0, None,
                                       0, None, None) == E_INVAL
    # rows whose starts are not all 16-byte aligned cannot take a forced 16-byte vector when shorter than 4 vectors
    v4 = hip.Plan(vec=4)
    odd = ctypes.byref(S(4096, 65))
    assert L.scanscam_scan_fwd_strided(fake, fake, fake, odd, dense, dense, 4, 64, 12, 0, None, 0, None,
                                       ctypes.byref(v4)) == E_PLAN
    # channels-last: the time stride is a 32-bit quantity
    big = ctypes.byref(S(0, 1 << 31))
    assert L.scanscam_scan_fwd_cl_strided(fake, fake, fake, big, None, None, 2, 8, 64, 0, None, 0, None, None) == E_INVAL
    assert L.scanscam_scan_bwd_cl_strided(fake, fake, fake, fake, fake, neg, None, None, None, None, 2, 8, 64, 0, None,
                                          0, None, None) == E_INVAL
    # ... and a time step stays below 4 GiB / 18 (a wave addresses its steps with 32-bit offsets)
    wide = ctypes.byref(S(0, 60_000_000))
    assert L.scanscam_scan_fwd_cl_strided(fake, fake, fake, wide, None, None, 1, 8, 64, 0, None, 0, None, None) == E_INVAL
    assert L.scanscam_scan_fwd_cl(fake, fake, fake, 1, 8, 60_000_000, 0, None, 0, None, None) == E_INVAL
    # empty problems succeed without touching anything
    assert L.scanscam_scan_fwd_strided(None, None, None, None, None, None, 0, 5, 64, 0, None, 0, None, None) == E_OK
    assert L.scanscam_scan_fwd_cl_strided(None, None, None, None, None, None, 3, 0, 64, 0, None, 0, None, None) == E_OK


def test_empty_inputs_are_a_successful_noop():
    L = hip.lib()
    assert L.scanscam_scan_fwd(None, None, None, 0, 128, 0, None, 0, None) == E_OK
    assert L.scanscam_scan_fwd(None, None, None, 5, 0, 0, None, 0, None) == E_OK
    assert L.scanscam_scan_bwd(None, None, None, None, None, 0, 0, 0, None, 0, None) == E_OK


@pytest.mark.parametrize(
    "rows,T,dtype,mode,vec",
    [
        (1024, 1024, torch.float32, hip.MODE_ROW, 4),       # forward-only config
        (16384, 4096, torch.float32, hip.MODE_ROW, 4),      # Mamba-like config
        (64, 1 << 20, torch.float32, hip.MODE_LOOKBACK, 4), # long sequence
        (16384, 2048, torch.bfloat16, hip.MODE_ROW, 8),     # 16-bit storage
        (16384, 2048, torch.float16, hip.MODE_ROW, 8),
        (131072, 64, torch.float32, hip.MODE_SMALL, 4),     # many short rows
        (32, 1025, torch.float32, hip.MODE_ROW, 4),         # odd length: element-aligned 16-byte vectors
        (32, 5, torch.float32, hip.MODE_FLAT, 4),           # short rows of any length, dense: one flat stream
        (200000, 70, torch.float32, hip.MODE_FLAT, 4),
        (200000, 48, torch.float32, hip.MODE_FLAT, 4),      # 12 vectors: no power-of-two group of lanes
        (32, 70, torch.float32, hip.MODE_FLAT, 4),
        (32, 61, torch.float32, hip.MODE_SMALL, 4),         # ... up to 32 MiB per tensor, rows that fill their lane group: element-aligned vectors, several rows per wave
        (200000, 61, torch.float32, hip.MODE_FLAT, 4),
        (32, 3, torch.float32, hip.MODE_SMALL, 1),          # shorter than a vector
        (200000, 100, torch.bfloat16, hip.MODE_FLAT, 8),
        (200000, 104, torch.bfloat16, hip.MODE_SMALL, 8),   # 16-bit storage keeps groups that are at least 0.6 full
        (3, 5, torch.float32, hip.MODE_SMALL, 1),           # too few rows for a whole number of vectors
    ],
)
def test_automatic_plan_per_regime(rows, T, dtype, mode, vec):
    for direction in (hip.FORWARD, hip.BACKWARD):
        plan = hip.resolve_plan(rows, T, dtype, direction)
        assert (plan.mode, plan.vec) == (mode, vec), plan
        ws = hip.workspace_bytes(rows, T, dtype, direction)
        assert (ws > 0) == (mode == hip.MODE_LOOKBACK)


def test_lookback_workspace_size_formula():
    plan = hip.Plan(mode=hip.MODE_LOOKBACK, vec=4, unroll=2, waves=2)
    # tile = 2 waves * 2 chunks * 256 elements = 1024 elements; 5 tiles per row of 4100;
    # one ticket counter (a 16-word line) per row; fp32: 1 word per tile (its pair), 2 per super-tile of 64 tiles (its
    # pair and its end value); fp64: 4 and 6 (a word per 32-bit half).
    assert hip.workspace_bytes(3, 4100, torch.float32, hip.FORWARD, plan) == (3 * 16 + 3 * 5 * 1 + 3 * 1 * 2) * 8
    plan64 = hip.Plan(mode=hip.MODE_LOOKBACK, vec=2, unroll=2, waves=2)  # tile = 512 float64 elements: 9 tiles
    assert hip.workspace_bytes(3, 4100, torch.float64, hip.FORWARD, plan64) == (3 * 16 + 3 * 9 * 4 + 3 * 1 * 6) * 8


def test_every_automatic_plan_is_a_valid_plan():
    # The rules that pick the launch shape (rows per workgroup, waves fitted to the row, chunks per wave by
    # storage type, kernel family by direction) must never produce a shape the library then refuses:
    # sizes on both sides of every rule's borders, all storage types, both directions, with and without
    # one element per lane forced.
    L = hip.lib()
    lengths = list(range(1, 70)) + [100, 127, 128, 129, 255, 256, 257, 500, 511, 512, 513, 1000, 1001, 1023, 1024,
                                    1025, 1280, 1500, 2047, 2048, 2049, 3000, 4096, 4097, 4100, 5000, 8191, 8192,
                                    8640, 8704, 10000, 10001, 12223, 12288, 12289, 14271, 14336, 16320, 16384,
                                    16640, 20000, 33333, 65536, 65537, 100000, 131072, 1000001, 1 << 22]
    checked = 0
    for dtype in (torch.float32, torch.bfloat16, torch.float16, torch.float64):
        code = hip._dtype_code(dtype)
        for rows in (1, 3, 16, 255, 256, 700, 5000, 100000):
            for T in lengths:
                for direction in (hip.FORWARD, hip.BACKWARD):
                    for vec in (0, 1):
                        plan, out = hip.Plan(vec=vec), hip.Plan()
                        rc = L.scanscam_resolve_plan(rows, T, code, direction, ctypes.byref(plan), ctypes.byref(out))
                        assert rc == 0, (dtype, rows, T, direction, vec, hip.strerror(rc))
                        assert 1 <= out.waves <= 16 and out.unroll in (1, 2, 3, 4, 8) and out.mode in (1, 2, 3, 4)
                        if out.mode == 2:
                            assert out.waves_per_row >= 1 and out.waves % out.waves_per_row == 0
                        checked += 1
    assert checked > 10000
    # Hints without a mode: the automatic choice may only pick a family that accepts them (dense short rows
    # prefer the flat kernel, which has 2 or 4 chunks per wave; the small kernel takes the other counts).
    for dtype, T in ((torch.float32, 68), (torch.float64, 34), (torch.bfloat16, 136)):
        for plan in (hip.Plan(unroll=1), hip.Plan(unroll=8), hip.Plan(unroll=8, waves=8), hip.Plan(unroll=2),
                     hip.Plan(waves=3), hip.Plan(unroll=4, waves=16)):
            for direction in (hip.FORWARD, hip.BACKWARD):
                out = hip.Plan()
                rc = L.scanscam_resolve_plan(200000, T, hip._dtype_code(dtype), direction, ctypes.byref(plan), ctypes.byref(out))
                assert rc == 0, (dtype, T, plan, hip.strerror(rc))
                assert out.mode == (hip.MODE_FLAT if plan.unroll in (0, 2, 4) else hip.MODE_SMALL), (dtype, T, plan, out)


WALK, TILES = hip.MODE_ROW, hip.MODE_LOOKBACK


CL_SHAPES = [(8, 4096, 512), (64, 2048, 1024), (256, 1024, 1024), (8, 4096, 2048), (256, 4096, 64), (4096, 256, 64),
             (2048, 512, 40), (512, 4096, 8), (128, 8192, 16), (90, 2048, 514), (64, 2048, 1001), (300, 1000, 77),
             (476, 1998, 113), (4526, 65, 432), (1, 262144, 256), (24, 2048, 3072), (2000, 1000, 65), (3, 107, 197),
             (5, 6113, 107), (40, 2048, 4096)]
CL_DTYPES = (torch.float32, torch.bfloat16, torch.float16, torch.float64)


def _forced_cl_plans(dtype):
    full = 16 // torch.empty(0, dtype=dtype).element_size()
    widths = sorted({1, full, max(1, full // 2)} | ({2} if full == 8 else set()))
    return [hip.Plan(mode=m, vec=v, unroll=s, waves=w) for v in widths for m in (WALK, TILES)
            for s in ((2, 4, 8) if v == full else (4, 8, 16)) for w in ((4, 8, 16) if m == WALK else (4, 8))]


def test_the_automatic_channels_last_plan_is_the_cheapest_by_the_cost_model():
    """The choice is an argmin and nothing else: no candidate plan has a smaller estimate than the automatic one.
    Two kinds of plan are not candidates: 16-byte lanes of 16-bit storage in a time split (they spill), and a walk
    with fewer workgroups than half the compute units where the time can be split instead."""
    checked = thin = 0
    for shape in CL_SHAPES:
        for dtype in CL_DTYPES:
            for direction in (hip.FORWARD, hip.BACKWARD):
                auto = hip.resolve_plan_cl(*shape, dtype, direction)
                auto_us = hip.predict_cl(*shape, dtype, direction)
                assert auto_us > 0 and abs(hip.predict_cl(*shape, dtype, direction, auto) - auto_us) <= 1e-9 * auto_us
                for plan in _forced_cl_plans(dtype):
                    if plan.mode == TILES and plan.vec == 8:
                        continue
                    try:
                        us = hip.predict_cl(*shape, dtype, direction, plan)
                        got = hip.resolve_plan_cl(*shape, dtype, direction, plan)
                    except RuntimeError:
                        continue  # not a plan the kernels can run on this shape
                    if (got.mode, got.waves) != (plan.mode, plan.waves):
                        continue  # (a forced split of a single tile falls back to the walk)
                    lanes = 64 * plan.vec
                    if plan.mode == WALK and auto.mode == TILES and 2 * shape[0] * -(-shape[2] // lanes) < 256:
                        thin += 1
                        continue
                    assert us >= auto_us * (1 - 1e-9), (shape, dtype, direction, auto, plan, us, auto_us)
                    checked += 1
    assert checked > 2000 and 0 < thin < checked // 4


def test_the_fitting_tool_and_the_library_hold_the_same_cost_model():
    """scanscam_amd/plan_fit.py fits the constants with its own copy of the formula and of the learned correction; each
    pair must be one function."""
    from scanscam_amd import plan_fit

    inc = os.path.join(ROOT, "scanscam_amd", "csrc", "scan_cl_model.inc")
    table, residual = plan_fit.read_table(inc), plan_fit.read_residual(inc)
    rng = np.random.default_rng(5)
    checked = 0
    for _ in range(400):
        dtype = CL_DTYPES[rng.integers(4)]
        esize = torch.empty(0, dtype=dtype).element_size()
        batch, T = int(2 ** rng.uniform(0, 12)), int(2 ** rng.uniform(0, 15))
        C = int(2 ** rng.uniform(0, 12.5))
        if rng.random() < 0.5:
            C = max(16, C // 16 * 16)  # lanes of every width are whole here (dense tensors: the alignment follows C)
        plans = _forced_cl_plans(dtype)
        plan = plans[rng.integers(len(plans))]
        direction = int(rng.integers(2))
        try:
            got = hip.predict_cl(batch, T, C, dtype, direction, plan)
            back = hip.resolve_plan_cl(batch, T, C, dtype, direction, plan)
        except RuntimeError:
            continue
        if (back.mode, back.waves) != (plan.mode, plan.waves):
            continue
        d = plan_fit.describe(batch, T, C, esize, direction == hip.BACKWARD, plan.mode, plan.vec, plan.unroll, plan.waves)
        want = plan_fit.estimate(d, table, residual)
        assert abs(got - want) <= 1e-6 * want, (batch, T, C, dtype, direction, plan, got, want)
        # ... and the learned part is a bounded factor on the formula
        assert abs(np.log(want / plan_fit.predict(d, table))) <= plan_fit.RESIDUAL_LIMIT + 1e-9
        checked += 1
    assert checked > 150


def test_no_unexplained_cliffs_between_neighbouring_channels_last_shapes():
    """Where two shapes differ by 8 channels or a few time steps or batch elements, the plan of one costs the other at
    most 15 % more than its own by the model -- or a quantity of the model is what changes between them under that
    plan or under the shape's own: the kernel variant (lanes per time step, whole or element-aligned lanes), the fill of the lanes, the lines a
    wave touches, the rounds of workgroups, or whether a walk would occupy half the compute units (the one occupancy
    guard on the candidates). No choice moves because any other threshold was crossed."""
    from scanscam_amd import plan_fit

    def quantities(batch, T, C, esize, rev, plan):
        d = plan_fit.describe(batch, T, C, esize, rev, plan.mode, plan.vec, plan.unroll, plan.waves)
        cols = plan_fit.columns([d])
        wgs = d["RG"] * (d["tiles"] if d["kind"] == 2 else 1)
        thin = tuple(2 * batch * -(-C // (64 * v)) < 256 for v in (1, 16 // esize))
        return (d["group"], d["ragged"], round(d["fill"], 1), round(float(cols["lines_extra"][0]), 1), -(-wgs // 256), thin)

    checked = explained = 0
    for batch, T, C in CL_SHAPES + [(100, 3000, 300), (32, 2048, 2048), (1024, 256, 384), (700, 300, 257)]:
        for dtype in (torch.float32, torch.bfloat16):
            esize = torch.empty(0, dtype=dtype).element_size()
            for direction in (hip.FORWARD, hip.BACKWARD):
                own_us = hip.predict_cl(batch, T, C, dtype, direction)
                for nb, nT, nC in ((batch, T, C + 8), (batch, T, max(8, C - 8)), (batch + 1, T, C), (batch, T + 16, C),
                                   (max(1, batch - 1), T, C)):
                    theirs = hip.resolve_plan_cl(nb, nT, nC, dtype, direction)
                    try:
                        us = hip.predict_cl(batch, T, C, dtype, direction, theirs)
                        back = hip.resolve_plan_cl(batch, T, C, dtype, direction, theirs)
                    except RuntimeError:
                        continue
                    if back.mode != theirs.mode:
                        continue
                    checked += 1
                    if us > 1.15 * own_us:
                        rev = direction == hip.BACKWARD
                        mine = hip.resolve_plan_cl(batch, T, C, dtype, direction)
                        differs = False
                        for plan in (theirs, mine):  # under their plan, or under the one this shape takes itself
                            try:
                                here = quantities(batch, T, C, esize, rev, plan)
                                there = quantities(nb, nT, nC, esize, rev, plan)
                            except (ValueError, ZeroDivisionError):
                                differs = True  # the plan does not exist on the other shape
                                break
                            differs = differs or here != there
                        assert differs, ((batch, T, C), (nb, nT, nC), dtype, direction, theirs, mine, us, own_us)
                        explained += 1
    assert checked > 300 and explained < checked // 10


def test_every_automatic_channels_last_plan_is_a_valid_plan():
    # Every plan the channels-last choice arrives at must be one the library accepts when it is forced,
    # with the workspace the automatic call asks for being enough for it.
    L = hip.lib()
    channels = list(range(1, 70)) + [77, 96, 100, 127, 128, 129, 130, 200, 250, 256, 257, 300, 320, 333, 384, 448, 500,
                                     511, 512, 513, 514, 640, 768, 1000, 1001, 1003, 1004, 1016, 1024, 1280, 1500, 1501,
                                     2001, 2048, 2050, 4001, 4096, 8192]
    checked = 0
    for dtype in (torch.float32, torch.bfloat16, torch.float16, torch.float64):
        code = hip._dtype_code(dtype)
        for batch in (1, 8, 36, 64, 100, 128, 160, 256, 300, 400, 1024, 5000):
            for T in (1, 50, 512, 1024, 4096):
                for C in channels:
                    for direction in (hip.FORWARD, hip.BACKWARD):
                        out, again = hip.Plan(), hip.Plan()
                        rc = L.scanscam_resolve_plan_cl(batch, T, C, code, direction, None, ctypes.byref(out))
                        assert rc == 0, (dtype, batch, T, C, direction, hip.strerror(rc))
                        assert out.mode in (WALK, TILES) and out.unroll in (2, 4, 8, 16) and 1 <= out.waves <= 16
                        assert out.vec in (1, 2, 4, 8) and out.vec * torch.empty(0, dtype=dtype).element_size() <= 16
                        rc = L.scanscam_resolve_plan_cl(batch, T, C, code, direction, ctypes.byref(out), ctypes.byref(again))
                        assert rc == 0, (dtype, batch, T, C, direction, out, hip.strerror(rc))
                        assert (again.vec, again.unroll, again.waves) == (out.vec, out.unroll, out.waves), (out, again)
                        need = L.scanscam_workspace_bytes_cl(batch, T, C, code, direction, ctypes.byref(out))
                        assert need <= hip.workspace_bytes_cl(batch, T, C, dtype, direction), (dtype, batch, T, C, out)
                        checked += 1
    assert checked > 10000
