"""
The C-ABI library loads here (no GPU needed), exports every function that
include/scanscam_hip.h declares, and rejects bad arguments before launching
anything. No kernel is launched in this file.
"""
import ctypes
import os
import re

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
    assert "scanscam_scan_fwd" in names and "scanscam_scan_bwd" in names and len(names) == 22
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


@pytest.mark.parametrize(
    "shape,dtype,fwd,bwd",
    [
        # (mode, channels per lane, time steps per wave, waves) forwards and backwards
        ((8, 4096, 2048), torch.float32, (WALK, 1, 8, 16), (WALK, 1, 8, 16)),     # 256 workgroups of single channels
        ((64, 2048, 1024), torch.float32, (WALK, 2, 8, 8), (WALK, 2, 8, 8)),      # 8-byte lanes give 512 workgroups
        ((8, 4096, 512), torch.float32, (TILES, 2, 16, 8), (TILES, 1, 16, 8)),    # too few for a walk: tiles over time
        ((8, 4096, 2048), torch.bfloat16, (WALK, 1, 16, 16), (TILES, 4, 16, 8)),
        ((256, 4096, 64), torch.bfloat16, (WALK, 1, 16, 16), (WALK, 1, 16, 16)),  # 64 channels: a wave of single channels
        ((4096, 256, 64), torch.bfloat16, (WALK, 1, 16, 8), (WALK, 1, 16, 8)),    # ... 8 waves from two workgroups per CU on
        ((4096, 128, 64), torch.bfloat16, (WALK, 1, 16, 8), (WALK, 2, 8, 4)),     # ... short rows keep pairs backwards
        ((512, 1024, 256), torch.bfloat16, (WALK, 2, 16, 8), (WALK, 2, 16, 8)),   # narrow 16-bit lanes: 16 steps from 512 steps on
        ((2048, 256, 256), torch.bfloat16, (WALK, 2, 8, 8), (WALK, 2, 8, 8)),
        ((512, 2048, 192), torch.bfloat16, (WALK, 1, 16, 8), (WALK, 1, 16, 8)),   # three whole waves of single channels
        ((24, 2048, 3072), torch.bfloat16, (TILES, 2, 16, 8), (TILES, 4, 16, 8)), # 288 workgroups: tiles, pairs forwards
        ((520, 2000, 96), torch.bfloat16, (WALK, 2, 16, 8), (WALK, 2, 16, 8)),    # ... not where the pairs leave a wave 25 % empty
        ((128, 1024, 1003), torch.bfloat16, (WALK, 4, 8, 8), (WALK, 4, 8, 8)),    # element-aligned 8-byte lanes, 512 workgroups
        ((256, 1024, 1001), torch.bfloat16, (WALK, 8, 4, 8), (WALK, 8, 4, 8)),    # ... 16-byte lanes from 400 workgroups on
        ((96, 1024, 1003), torch.float32, (WALK, 4, 4, 4), (WALK, 4, 4, 4)),      # fp32 keeps its 16-byte lanes
        ((300, 1024, 256), torch.float32, (TILES, 2, 16, 8), (WALK, 2, 8, 4)),    # 600 workgroups: 0.78 of three rounds
        ((300, 1000, 77), torch.bfloat16, (WALK, 1, 16, 8), (TILES, 1, 16, 8)),
        ((2048, 512, 40), torch.float32, (WALK, 1, 16, 8), (WALK, 4, 4, 4)),      # 33 to 63 channels, two workgroups per CU or more
        ((2048, 512, 40), torch.bfloat16, (WALK, 1, 16, 8), (WALK, 4, 8, 4)),
        ((540, 4225, 8), torch.float32, (WALK, 4, 4, 4), (WALK, 4, 4, 4)),        # several time steps per instruction
        ((306, 6590, 16), torch.float32, (WALK, 2, 8, 8), (WALK, 4, 4, 4)),
        ((128, 8192, 16), torch.bfloat16, (WALK, 2, 16, 8), (WALK, 2, 16, 8)),    # ... walked from 100 workgroups on
        ((64, 16384, 16), torch.bfloat16, (TILES, 1, 16, 8), (TILES, 1, 16, 8)),
        ((209, 221, 1370), torch.bfloat16, (WALK, 4, 8, 8), (WALK, 4, 8, 8)),     # short rows, element-aligned: 8-byte lanes
        ((476, 1998, 157), torch.float32, (TILES, 1, 16, 8), (TILES, 1, 16, 8)),  # fp32 off whole lines: tiles (forwards from 1900 steps)
        ((90, 2048, 514), torch.float32, (TILES, 2, 16, 8), (TILES, 2, 8, 8)),
        ((986, 969, 157), torch.float32, (WALK, 1, 8, 16), (TILES, 1, 16, 8)),
        ((4526, 65, 432), torch.float32, (WALK, 1, 16, 5), (WALK, 1, 8, 9)),       # rows of one or two tiles: evenly filled tiles
        ((506, 75, 943), torch.bfloat16, (WALK, 4, 8, 4), (WALK, 4, 8, 4)),        # ... three tiles of 4 waves for lanes of 8 bytes
        ((512, 512, 333), torch.float32, (WALK, 2, 16, 8), (WALK, 2, 16, 8)),     # ... element-aligned pairs only from 2048 steps
        ((476, 1998, 113), torch.bfloat16, (WALK, 2, 8, 8), (WALK, 2, 8, 8)),      # 65-127 channels, an odd count: one wave of element-aligned pairs
        ((2000, 1000, 65), torch.float32, (WALK, 2, 8, 8), (WALK, 2, 8, 8)),
        ((15, 6680, 188), torch.bfloat16, (TILES, 2, 16, 8), (TILES, 4, 16, 8)),   # 16-bit backward tiles: four-channel lanes from 53 % fill
        ((71, 1910, 257), torch.bfloat16, (TILES, 1, 16, 8), (WALK, 2, 16, 8)),   # 213 workgroups of element-aligned pairs backwards
        ((128, 512, 2048), torch.float32, (WALK, 2, 16, 8), (WALK, 4, 4, 4)),     # 2048 or more fp32 channels
        ((256, 1024, 256), torch.float64, (WALK, 1, 8, 8), (WALK, 1, 8, 8)),      # float64: its 8-byte lane is one channel
        ((8, 4096, 512), torch.float64, (TILES, 1, 16, 8), (TILES, 1, 8, 8)),
        ((24, 2048, 4096), torch.float32, (WALK, 2, 16, 4), (WALK, 4, 4, 4)),
    ],
)
def test_automatic_channels_last_plan_per_regime(shape, dtype, fwd, bwd):
    for direction, want in ((hip.FORWARD, fwd), (hip.BACKWARD, bwd)):
        plan = hip.resolve_plan_cl(*shape, dtype, direction)
        assert (plan.mode, plan.vec, plan.unroll, plan.waves) == want, (direction, plan)
        ws = hip.workspace_bytes_cl(*shape, dtype, direction)
        assert ws > 0 or want[0] != TILES  # (the size covers tensors of any alignment, so it may be non-zero for a walk)


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
