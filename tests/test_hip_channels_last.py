"""
Parity of the channels-last kernels ([batch, T, C] storage, scanned along T)
with the CPU oracle, through the C ABI. Shapes and the N(0,1) gates follow the
reference's tests of its transposed kernels (scanscam/cuda_test.py:129-163); the
oracle sees the same values as contiguous [batch, C, T] arrays.
"""
import ctypes
import itertools

import numpy as np
import pytest
import torch

import oracle
from criteria import assert_reference_allclose
from scanscam_amd import hip

pytestmark = pytest.mark.gpu

REFERENCE_SHAPES = [(8, 4096, 512), (512, 4096, 8), (3, 107, 197), (3, 293, 283), (5, 6113, 107)]


def row_norm_err(x, ref):
    x = np.asarray(x, np.float64).reshape(-1, x.shape[-1])
    ref = np.asarray(ref, np.float64).reshape(-1, ref.shape[-1])
    scale = np.maximum(np.max(np.abs(ref), axis=1), 1.0)
    return float(np.max(np.max(np.abs(x - ref), axis=1) / scale))


def rel_err(x, ref, floor=None):
    x, ref = np.asarray(x, np.float64), np.asarray(ref, np.float64)
    den = np.maximum(np.abs(ref), 1.0)
    if floor is not None:
        den = np.maximum(den, floor)
    return float(np.max(np.abs(x - ref) / den))


def prev_abs(h):
    h = np.abs(np.asarray(h, np.float64))
    out = np.zeros_like(h)
    out[..., 1:] = h[..., :-1]
    return out


def as_rows(t):
    """[batch, T, C] torch tensor -> contiguous [batch, C, T] numpy array (float64 stays, else float32)."""
    t = t.detach().cpu()
    t = t if t.dtype == torch.float64 else t.float()
    return t.mT.contiguous().numpy()


@pytest.mark.parametrize("shape", REFERENCE_SHAPES)
@pytest.mark.parametrize("channels_per_block", [1, 32])
def test_reference_shapes(gpu, shape, channels_per_block):
    g = torch.Generator().manual_seed(sum(shape))
    x = torch.randn(shape, generator=g)
    y = torch.randn(shape, generator=g)
    gh = torch.randn(shape, generator=g)
    print(f"case channels_last shape={shape}", flush=True)
    out = hip.transposed_linear_scan_forward(x.to(gpu), y.to(gpu), channels_per_block)
    assert out.shape == x.shape and out.is_contiguous()
    want = oracle.fwd(as_rows(x), as_rows(y))
    assert row_norm_err(as_rows(out), want) <= 1e-4
    # The reference tests' own criterion, element by element (scanscam/cuda_test.py:141, 163).
    assert_reference_allclose(as_rows(out), want, lambda: oracle.fwd_acc64(as_rows(x), as_rows(y)), f"h {shape}")
    hs = torch.from_numpy(want).mT.contiguous()  # the oracle's output, stored [batch, T, C]
    ga, gb = hip.transposed_linear_scan_backward(x.to(gpu), hs.to(gpu), gh.to(gpu), channels_per_block)
    wga, wgb = oracle.bwd(as_rows(x), want, as_rows(gh))
    assert row_norm_err(as_rows(gb), wgb) <= 1e-4
    assert row_norm_err(as_rows(ga), wga) <= 1e-4
    exact = lambda: oracle.bwd_acc64(as_rows(x), want, as_rows(gh))  # noqa: E731
    assert_reference_allclose(as_rows(gb), wgb, lambda: exact()[1], f"grad_b {shape}")
    assert_reference_allclose(as_rows(ga), wga, lambda: exact()[0], f"grad_a {shape}")


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64, torch.bfloat16, torch.float16])
def test_forced_plans(gpu, dtype):
    full = 16 // torch.empty(0, dtype=dtype).element_size()
    bar = {torch.float32: 1e-5, torch.float64: 1e-13}.get(dtype, 1e-2)
    g = torch.Generator().manual_seed(17)
    cases = []
    for shape in [(3, 301, 64 * full + full), (2, 77, 3 * full), (1, 1500, 256), (2, 5, 130), (4, 64, 33)]:
        a = torch.rand(shape, generator=g, dtype=torch.float64).to(dtype)
        b = torch.randn(shape, generator=g, dtype=torch.float64).to(dtype)
        gh = torch.randn(shape, generator=g, dtype=torch.float64).to(dtype)
        h = oracle.fwd(as_rows(a), as_rows(b))
        hs = torch.from_numpy(h).mT.contiguous().to(dtype)
        ga, gb = oracle.bwd(as_rows(a), as_rows(hs), as_rows(gh))
        cases.append((shape, a.to(gpu), b.to(gpu), gh.to(gpu), hs.to(gpu), h, ga, gb, prev_abs(as_rows(hs))))
    n = 0
    # Lanes of 16 bytes, of 8 bytes (two fp32 channels, four 16-bit ones), of two 16-bit channels, of one channel.
    for vec in {8: (8, 4, 2, 1), 4: (4, 2, 1), 2: (2, 1)}[full]:
        for steps in ((2, 4, 8) if vec == full else (4, 8, 16)):
            csize = 8 if dtype == torch.float64 else 4
            max_waves = min(16, 65536 // (4 * vec * 64 * csize), (512 if (vec > 1 and steps >= 8) else 1024) // 64)
            shapes_plans = [hip.Plan(vec=vec, unroll=steps, waves=waves, mode=hip.MODE_ROW) for waves in sorted({1, 3, max_waves})]
            # Time split over workgroups: tiles with a look-back chain per channel (7 LDS arrays).
            lb_waves = min(max_waves, 65536 // (7 * vec * 64 * csize))
            shapes_plans += [hip.Plan(vec=vec, unroll=steps, waves=waves, mode=hip.MODE_LOOKBACK)
                             for waves in sorted({1, 2, lb_waves})]
            for plan in shapes_plans:
                for shape, a, b, gh, hs, h, ga, gb, hp in cases:
                    if vec != 1 and shape[-1] % vec != 0:
                        continue
                    print(f"case cl forced {dtype} shape={shape} {plan}", flush=True)
                    got_h = hip.transposed_linear_scan_forward(a, b, plan=plan)
                    got_ga, got_gb = hip.transposed_linear_scan_backward(a, hs, gh, plan=plan)
                    assert rel_err(as_rows(got_h), h) <= bar, (plan, shape)
                    assert rel_err(as_rows(got_gb), gb) <= bar, (plan, shape)
                    assert rel_err(as_rows(got_ga), ga, hp) <= bar, (plan, shape)
                    n += 1
    assert n > 90


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64, torch.bfloat16, torch.float16])
def test_element_aligned_lanes(gpu, dtype):
    """Wide lanes where C is no multiple of the lane's channels, or the tensors start at any element."""
    full = 16 // torch.empty(0, dtype=dtype).element_size()
    bar = {torch.float32: 1e-5, torch.float64: 1e-13}.get(dtype, 1e-2)
    g = torch.Generator().manual_seed(23)
    n = 0
    for shape in [(3, 107, 64 * full + 1), (2, 70, 64 * full + full - 1), (5, 33, 130 * full + 3), (2, 50, 401),
                  (3, 85, 67), (2, 60, 127), (4, 40, 32 * full + 1)]:  # (more than half a wave of lanes per time step is enough)
        a = torch.rand(shape, generator=g, dtype=torch.float64).to(dtype)
        b = torch.randn(shape, generator=g, dtype=torch.float64).to(dtype)
        gh = torch.randn(shape, generator=g, dtype=torch.float64).to(dtype)
        h = oracle.fwd(as_rows(a), as_rows(b))
        hs = torch.from_numpy(h).mT.contiguous().to(dtype)
        ga, gb = oracle.bwd(as_rows(a), as_rows(hs), as_rows(gh))
        hp = prev_abs(as_rows(hs))
        numel = a.numel()
        for offset in (0, 1):  # views that start one element into their allocation
            def view_of(t):
                buf = torch.full((numel + 8,), float("nan"), dtype=dtype, device=gpu)
                v = buf[offset:offset + numel].view(shape)
                v.copy_(t)
                return v
            da, db, dgh, dhs = view_of(a), view_of(b), view_of(gh), view_of(hs)
            for vec in {8: (8, 4, 2), 4: (4, 2), 2: (2,)}[full]:
                if shape[-1] <= 32 * vec:
                    continue
                for steps in ((2, 4, 8) if vec == full else (4, 8, 16)):
                    plan = hip.Plan(vec=vec, unroll=steps, waves=3, mode=hip.MODE_ROW)
                    print(f"case cl element-aligned {dtype} shape={shape} offset={offset} {plan}", flush=True)
                    got_h = hip.transposed_linear_scan_forward(da, db, plan=plan)
                    got_ga, got_gb = hip.transposed_linear_scan_backward(da, dhs, dgh, plan=plan)
                    assert rel_err(as_rows(got_h), h) <= bar, (plan, shape)
                    assert rel_err(as_rows(got_gb), gb) <= bar, (plan, shape)
                    assert rel_err(as_rows(got_ga), ga, hp) <= bar, (plan, shape)
                    n += 1
    assert n >= 20
    # The automatic choice takes such lanes where they still give 256 workgroups ...
    shape = (260, 40, 64 * full + 5)
    a = torch.rand(shape, generator=g, dtype=torch.float64).to(dtype)
    b = torch.randn(shape, generator=g, dtype=torch.float64).to(dtype)
    want = oracle.fwd(as_rows(a), as_rows(b))
    assert rel_err(as_rows(hip.transposed_linear_scan_forward(a.to(gpu), b.to(gpu))), want) <= bar
    # ... and a forced wide lane is refused where a time step fills no more than half a wave of them.
    small = torch.rand(2, 8, 32 * full - 3, device=gpu).to(dtype)
    with pytest.raises(RuntimeError, match="plan"):
        hip.transposed_linear_scan_forward(small, small, plan=hip.Plan(vec=full, mode=hip.MODE_ROW))


def test_matches_row_layout_kernels(gpu):
    # Same data through both layouts: the two kernel families must agree closely
    # (each is within 1e-5 of the oracle; they differ only in association order).
    g = torch.Generator(device=gpu).manual_seed(9)
    x = torch.rand((4, 2048, 1024), generator=g, device=gpu)
    y = torch.randn((4, 2048, 1024), generator=g, device=gpu)
    cl = hip.transposed_linear_scan_forward(x, y)
    rows = hip.blocked_linear_scan_forward(x.mT.contiguous(), y.mT.contiguous())
    assert float((cl.mT - rows).abs().max()) <= 2e-5
    ga, gb = hip.transposed_linear_scan_backward(x, cl, y)
    rga, rgb = hip.blocked_linear_scan_backward(x.mT.contiguous(), cl.mT.contiguous(), y.mT.contiguous())
    assert float((gb.mT - rgb).abs().max()) <= 2e-5
    assert float((ga.mT - rga).abs().max() / rga.abs().max().clamp(min=1)) <= 2e-5


def test_empty_and_argument_checks(gpu):
    for shape in [(0, 4, 8), (2, 0, 8), (2, 4, 0)]:
        z = torch.zeros(shape, device=gpu)
        assert hip.transposed_linear_scan_forward(z, z).shape == z.shape
        ga, gb = hip.transposed_linear_scan_backward(z, z, z)
        assert ga.shape == z.shape and gb.shape == z.shape
    x = torch.zeros(2, 8, 16, device=gpu)
    with pytest.raises(AssertionError):
        hip.transposed_linear_scan_forward(x, x[:, :4])
    with pytest.raises(AssertionError):
        hip.transposed_linear_scan_forward(x.mT, x.mT)  # not contiguous as [batch, T, C]
    with pytest.raises(AssertionError):
        hip.transposed_linear_scan_forward(x[0], x[0])  # not 3-D
    with pytest.raises(RuntimeError):
        hip.transposed_linear_scan_forward(x, x, plan=hip.Plan(vec=4, unroll=3))


def test_time_split_is_chosen_for_few_channels_and_is_reproducible(gpu):
    # [8, 4096, 512]: 16 (batch element, channel group) pairs would leave most of the GPU idle,
    # so the automatic plan cuts time into tiles over workgroups; results must not depend on timing.
    g = torch.Generator(device=gpu).manual_seed(23)
    x = torch.rand((8, 4096, 512), generator=g, device=gpu)
    y = torch.randn((8, 4096, 512), generator=g, device=gpu)
    assert hip.lib().scanscam_workspace_bytes_cl(8, 4096, 512, 0, 0, None) > 0
    first = hip.transposed_linear_scan_forward(x, y)
    whole = hip.transposed_linear_scan_forward(x, y, plan=hip.Plan(mode=hip.MODE_ROW))
    assert float((first - whole).abs().max()) <= 2e-5
    for _ in range(3):
        assert torch.equal(hip.transposed_linear_scan_forward(x, y), first)
    ga0, gb0 = hip.transposed_linear_scan_backward(x, first, y)
    ga1, gb1 = hip.transposed_linear_scan_backward(x, first, y)
    assert torch.equal(ga0, ga1) and torch.equal(gb0, gb1)


@pytest.mark.parametrize("dtype,shape,vec", [
    (torch.float32, (9, 700, 2059), 1),    # 297 (batch element, channel group) pairs: runs of 38 and 37 per XCD
    (torch.float32, (131, 300, 100), 1),   # 131 pairs of two steps' worth of tiles
    (torch.bfloat16, (17, 600, 515), 1),   # 153 pairs
    (torch.bfloat16, (43, 500, 772), 4),   # 172 pairs of four-channel lanes, time steps of 1544 bytes
    (torch.float32, (3, 900, 300), 1),     # 15 pairs: too few for runs, dealt round-robin
])
def test_time_split_with_pairs_that_are_no_multiple_of_eight(gpu, dtype, shape, vec):
    # Time steps that are no whole 128-byte lines: each XCD takes a contiguous run of the (batch element, channel group)
    # pairs and every tile of them; with a pair count that is no multiple of 8 the runs differ in length and the grid
    # is padded, so some workgroups have nothing to do. Every tile of every pair must still be handed out exactly once.
    bar = 1e-5 if dtype == torch.float32 else 1e-2
    g = torch.Generator().manual_seed(sum(shape))
    a = torch.rand(shape, generator=g, dtype=torch.float64).to(dtype)
    b = torch.randn(shape, generator=g, dtype=torch.float64).to(dtype)
    gh = torch.randn(shape, generator=g, dtype=torch.float64).to(dtype)
    h = oracle.fwd(as_rows(a), as_rows(b))
    hs = torch.from_numpy(h).mT.contiguous().to(dtype)
    ga, gb = oracle.bwd(as_rows(a), as_rows(hs), as_rows(gh))
    hp = prev_abs(as_rows(hs))
    for waves in (2, 8):
        plan = hip.Plan(vec=vec, unroll=16, waves=waves, mode=hip.MODE_LOOKBACK)
        print(f"case cl time split {dtype} shape={shape} {plan}", flush=True)
        for _ in range(2):
            got_h = hip.transposed_linear_scan_forward(a.to(gpu), b.to(gpu), plan=plan)
            got_ga, got_gb = hip.transposed_linear_scan_backward(a.to(gpu), hs.to(gpu), gh.to(gpu), plan=plan)
            assert rel_err(as_rows(got_h), h) <= bar
            assert rel_err(as_rows(got_gb), gb) <= bar
            assert rel_err(as_rows(got_ga), ga, hp) <= bar


def test_expired_wait_is_reported_and_every_wave_exits(gpu):
    # One poll allowed: the launch must still complete; either all waits succeeded in that poll or
    # word 1 of the workspace is raised and the poisoned outputs are NaN.
    import ctypes

    B, T, C = 1, 4096, 64
    g = torch.Generator(device=gpu).manual_seed(29)
    x = torch.rand((B, T, C), generator=g, device=gpu)
    y = torch.randn((B, T, C), generator=g, device=gpu)
    good = hip.transposed_linear_scan_forward(x, y, plan=hip.Plan(mode=hip.MODE_LOOKBACK, vec=1, unroll=4, waves=2))
    plan = hip.Plan(mode=hip.MODE_LOOKBACK, vec=1, unroll=4, waves=2, spin_limit=1)
    L = hip.lib()
    n = L.scanscam_workspace_bytes_cl(B, T, C, 0, 0, ctypes.byref(plan))
    assert n > 0
    ws = torch.empty(n, dtype=torch.uint8, device=gpu)
    out = torch.empty_like(x)
    rc = L.scanscam_scan_fwd_cl(x.data_ptr(), y.data_ptr(), out.data_ptr(), B, T, C, 0, ws.data_ptr(), n,
                                torch.cuda.current_stream().cuda_stream, ctypes.byref(plan))
    assert rc == 0
    torch.cuda.synchronize()
    if int(ws.view(torch.int64)[1].item()) != 0:
        assert bool(torch.isnan(out).any())
    else:
        assert torch.equal(out, good)
    assert torch.equal(hip.transposed_linear_scan_forward(x, y, plan=hip.Plan(mode=hip.MODE_LOOKBACK, vec=1, unroll=4, waves=2)), good)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64, torch.bfloat16])
def test_few_channels_packed_kernel(gpu, dtype):
    # C <= 32 with enough batch elements: a wave holds several consecutive time steps per instruction and
    # scans across them with lane shuffles. Every lane-group width (1 ... 32 lanes per step), channel
    # counts that do not fill the group, 16-byte and single-channel lanes, lengths that end inside an
    # instruction, inside a wave's span and inside a tile.
    full = 16 // torch.empty(0, dtype=dtype).element_size()
    bar = {torch.float32: 1e-5, torch.float64: 1e-13}.get(dtype, 1e-2)
    g = torch.Generator().manual_seed(23)
    for C, T in [(1, 700), (2, 129), (3, 1000), (5, 64), (8, 4097), (12, 333), (16, 2048), (24, 515), (31, 77), (32, 1030)]:
        shape = (257, T, C)
        a = torch.rand(shape, generator=g, dtype=torch.float64).to(dtype)
        b = torch.randn(shape, generator=g, dtype=torch.float64).to(dtype)
        gh = torch.randn(shape, generator=g, dtype=torch.float64).to(dtype)
        h = oracle.fwd(as_rows(a), as_rows(b))
        hs = torch.from_numpy(h).mT.contiguous().to(dtype)
        ga, gb = oracle.bwd(as_rows(a), as_rows(hs), as_rows(gh))
        plans = [None]
        if C % full == 0:
            plans += [hip.Plan(vec=full, unroll=4, mode=hip.MODE_ROW), hip.Plan(vec=full, unroll=2, waves=3, mode=hip.MODE_ROW)]
        plans += [hip.Plan(vec=1, unroll=16, waves=2, mode=hip.MODE_ROW)]
        for plan in plans:
            print(f"case cl packed {dtype} shape={shape} {plan}", flush=True)
            got_h = hip.transposed_linear_scan_forward(a.to(gpu), b.to(gpu), plan=plan)
            got_ga, got_gb = hip.transposed_linear_scan_backward(a.to(gpu), hs.to(gpu), gh.to(gpu), plan=plan)
            assert rel_err(as_rows(got_h), h) <= bar, (plan, shape)
            assert rel_err(as_rows(got_gb), gb) <= bar, (plan, shape)
            assert rel_err(as_rows(got_ga), ga, prev_abs(as_rows(hs))) <= bar, (plan, shape)


# (dtype, [batch, T, C], slice of C taken from a wider buffer or None). Shapes at the borders where the automatic
# launch plan changes -- lane width, a walk of all of T or tiles of time over workgroups, steps per wave, waves,
# several time steps per instruction -- and where the kernels' special cases sit: time steps that are not whole
# 128-byte lines (dense, and views whose rows are whole lines but start inside one), numbers of (batch element,
# channel group) pairs that are and are not multiples of 8, channel counts on and off every lane's multiple, rows of
# one or two tiles, a single time step, very wide time steps. Whatever plan the cost model picks there, the result
# has to agree with the oracle.
MANY_WORKGROUPS = [
    (torch.float32, (37, 300, 1000), None),
    (torch.float32, (67, 90, 1000), None),
    (torch.bfloat16, (130, 60, 1096), None),
    (torch.float32, (70, 129, 264), None),
    (torch.float32, (65, 64, 1001), None),
    (torch.float32, (67, 90, 520), None),
    (torch.bfloat16, (33, 200, 1096), None),
    (torch.float16, (64, 130, 1001), None),
    (torch.float64, (40, 100, 500), None),
    (torch.float32, (20, 150, 1000), (8, 1056)),
    (torch.bfloat16, (24, 140, 1024), (16, 1088)),
    (torch.float32, (8, 2100, 500), None),
    (torch.bfloat16, (8, 1500, 1000), None),
    (torch.float32, (80, 200, 1024), None),
    (torch.bfloat16, (260, 130, 64), None),
    (torch.bfloat16, (260, 130, 96), None),
    (torch.float16, (300, 100, 40), None),
    (torch.bfloat16, (257, 64, 256), None),
    (torch.bfloat16, (9, 3000, 64), None),
    (torch.bfloat16, (16, 1100, 1024), None),
    (torch.float32, (260, 60, 256), None),
    (torch.bfloat16, (130, 70, 1024), None),
    (torch.float32, (130, 70, 512), None),
    (torch.float16, (64, 100, 1016), None),
    (torch.bfloat16, (64, 90, 1001), None),
    (torch.float32, (70, 50, 501), None),
    (torch.float32, (300, 100, 40), None),
    (torch.float32, (257, 64, 96), None),
    (torch.float32, (300, 200, 8), None),
    (torch.float32, (260, 90, 64), None),
    (torch.bfloat16, (300, 200, 8), None),
    (torch.float16, (300, 100, 24), None),
    (torch.float32, (8, 2100, 512), None),
    (torch.bfloat16, (8, 1500, 1024), None),
    (torch.float16, (8, 1100, 2048), None),
    (torch.float32, (36, 1100, 512), None),
    (torch.bfloat16, (36, 1100, 1024), None),
    (torch.float32, (260, 50, 320), None),
    (torch.float32, (50, 1100, 512), None),
    (torch.float32, (260, 1100, 48), None),
    (torch.bfloat16, (260, 1100, 48), None),
    (torch.bfloat16, (400, 60, 200), None),
    (torch.float16, (300, 50, 320), None),
    (torch.bfloat16, (130, 70, 1003), None),
    (torch.float16, (96, 70, 1501), None),
    (torch.bfloat16, (130, 70, 1004), None),
    (torch.float32, (300, 600, 256), None),
    (torch.float32, (300, 600, 77), None),
    (torch.bfloat16, (300, 600, 77), None),
    (torch.float32, (260, 70, 333), None),
    (torch.bfloat16, (260, 70, 333), None),
    (torch.float16, (130, 1030, 601), None),
    (torch.bfloat16, (260, 130, 256), None),
    (torch.bfloat16, (32, 1100, 4096), None),
    (torch.float64, (260, 70, 256), None),
    (torch.float64, (8, 1100, 256), None),
    (torch.float32, (2, 40, 65536), None),
    (torch.bfloat16, (1, 7, 100001), None),
    (torch.float16, (300, 1, 1000), None),
    (torch.float32, (20, 300, 2048), None),
    (torch.float32, (10, 200, 4096), None),
    (torch.float32, (600, 65, 432), None),
    (torch.bfloat16, (520, 67, 85), None),
    (torch.float32, (700, 99, 64), None),
    (torch.bfloat16, (300, 75, 943), None),
    (torch.float32, (1200, 330, 21), None),
    (torch.float32, (600, 500, 40), None),
    (torch.bfloat16, (600, 520, 40), None),
    (torch.float32, (520, 300, 8), None),
    (torch.float32, (100, 1300, 24), None),
    (torch.bfloat16, (64, 2100, 16), None),
    (torch.float32, (260, 600, 113), None),
    (torch.float32, (60, 2000, 113), None),
    (torch.float32, (14, 1100, 2539), None),
    (torch.bfloat16, (71, 600, 257), None),
    (torch.bfloat16, (39, 125, 4806), None),
    (torch.float32, (350, 300, 65), None),
    (torch.bfloat16, (350, 300, 113), None),
    (torch.float16, (400, 67, 127), None),
    (torch.float32, (345, 520, 93), None),
    (torch.bfloat16, (15, 1100, 188), None),
    (torch.float16, (13, 900, 400), None),
]


@pytest.mark.parametrize("dtype,shape,window", MANY_WORKGROUPS)
def test_automatic_plans_on_many_workgroups(gpu, dtype, shape, window):
    bar = {torch.float32: 1e-5, torch.float64: 1e-13}.get(dtype, 1e-2)
    B, T, C = shape
    g = torch.Generator().manual_seed(T + C)

    def place(t):
        t = t.to(dtype).to(gpu)
        if window is None:
            return t
        first, width = window
        buf = torch.full((B, T, width), float("nan"), dtype=dtype, device=gpu)
        buf[..., first:first + C] = t
        return buf[..., first:first + C]

    a = place(torch.rand(shape, generator=g, dtype=torch.float64))
    b = place(torch.randn(shape, generator=g, dtype=torch.float64))
    gh = place(torch.randn(shape, generator=g, dtype=torch.float64))
    print(f"case cl many workgroups {dtype} shape={shape} window={window}", flush=True)
    h = oracle.fwd(as_rows(a), as_rows(b))
    got_h = hip.scan_forward(a.mT, b.mT)
    assert got_h.shape == a.mT.shape and got_h.mT.is_contiguous()
    assert rel_err(as_rows(got_h.mT), h) <= bar
    hs = place(torch.from_numpy(h).mT)
    ga, gb = oracle.bwd(as_rows(a), as_rows(hs), as_rows(gh))
    got_ga, got_gb = hip.scan_backward(a.mT, hs.mT, gh.mT)
    assert rel_err(as_rows(got_gb.mT), gb) <= bar
    assert rel_err(as_rows(got_ga.mT), ga, prev_abs(as_rows(hs))) <= bar


def _large_shapes():
    from scanscam_amd import plan_search

    shapes = [s for s in plan_search.random_cl_shapes(60, 101) if s[0] * s[1] * s[2] <= 24 << 20][:8]
    return [(dtype, s) for s in shapes for dtype in (torch.float32, torch.bfloat16)]


@pytest.mark.parametrize("dtype,shape", _large_shapes())
def test_automatic_plans_on_large_shapes(gpu, dtype, shape):
    """The automatic plan of shapes of the size the plan search times (8 M to 24 M elements, drawn like its random
    audit's): at that size the cost model picks plans (16-wave walks, tiles in wide lanes) that the small shapes of
    the other tests never reach. Against the oracle, the bars of the other tests."""
    bar = 1e-5 if dtype == torch.float32 else 1e-2
    B, T, C = shape
    g = torch.Generator().manual_seed(B + T + C)
    a = torch.rand(shape, generator=g, dtype=torch.float32).to(dtype).to(gpu)
    b = torch.randn(shape, generator=g, dtype=torch.float32).to(dtype).to(gpu)
    gh = torch.randn(shape, generator=g, dtype=torch.float32).to(dtype).to(gpu)
    plans = [hip.resolve_plan_cl(B, T, C, dtype, d) for d in (hip.FORWARD, hip.BACKWARD)]
    print(f"case cl large {dtype} shape={shape} plans={plans}", flush=True)
    h = oracle.fwd(as_rows(a), as_rows(b))
    got_h = hip.scan_forward(a.mT, b.mT)
    assert rel_err(as_rows(got_h.mT), h) <= bar
    hs = torch.from_numpy(h).mT.to(dtype).to(gpu).contiguous()  # [B, T, C], rounded to the storage type
    ga, gb = oracle.bwd(as_rows(a), as_rows(hs), as_rows(gh))
    got_ga, got_gb = hip.scan_backward(a.mT, hs.mT, gh.mT)
    assert rel_err(as_rows(got_gb.mT), gb) <= bar
    assert rel_err(as_rows(got_ga.mT), ga, prev_abs(as_rows(hs))) <= bar


CHANNEL_EDGES = [1, 2, 3, 5, 8, 24, 31, 32, 33, 40, 63, 64, 65, 66, 77, 96, 100, 127, 128, 129, 130, 192, 200, 250, 256,
                 257, 300, 320, 333, 384, 448, 500, 511, 512, 513, 514, 600, 601, 640, 768, 777, 896, 1000, 1001, 1002,
                 1003, 1004, 1016, 1024, 1100]


@pytest.mark.parametrize("block", range(8))
def test_random_channels_last_shapes(gpu, block):
    """
    Seeded random [batch, T, C] shapes, storage types and windows: batch sizes on both sides of 256 workgroups
    for every lane width, channel counts on and off every lane's multiple and the 128-byte line, windows of a
    wider buffer that start at any element. Whatever lies around a window holds NaN, inputs and outputs alike, so a
    lane that reads or writes a channel it does not own shows either in the result or in the surroundings.
    """
    rng = np.random.default_rng(5000 + block)
    g = torch.Generator().manual_seed(6000 + block)
    for i in range(24):
        dtype = [torch.float32, torch.bfloat16, torch.float16, torch.float32, torch.bfloat16, torch.float64][rng.integers(6)]
        C = int(CHANNEL_EDGES[rng.integers(len(CHANNEL_EDGES))]) if rng.random() < 0.8 else int(rng.integers(1, 1200))
        regime = rng.integers(3)  # many batch elements and few steps, a few of each, few batch elements and many steps
        B = int([rng.integers(200, 600), rng.integers(16, 200), rng.integers(1, 16)][regime])
        budget = (1 << 22) // (B * C)
        T = int(rng.integers(1, max(2, min([160, 1200, 6000][regime], budget))))
        first, extra = (int(rng.integers(0, 9)), int(rng.integers(0, 9))) if rng.random() < 0.5 else (0, 0)
        width = first + C + extra
        bar = {torch.float32: 1e-5, torch.float64: 1e-13}.get(dtype, 1e-2)
        print(f"case cl random block={block} i={i} {dtype} B={B} T={T} C={C} window=({first}, {width})", flush=True)

        def place(values):
            buf = torch.full((B, T, width), float("nan"), dtype=dtype, device=gpu)
            buf[..., first:first + C] = values.to(dtype).to(gpu)
            return buf, buf[..., first:first + C]

        def surroundings_are_nan(buf):
            return bool(torch.isnan(buf[..., :first]).all()) and bool(torch.isnan(buf[..., first + C:]).all())

        shape = (B, T, C)
        _, a = place(torch.rand(shape, generator=g, dtype=torch.float64))
        _, b = place(torch.randn(shape, generator=g, dtype=torch.float64))
        _, gh = place(torch.randn(shape, generator=g, dtype=torch.float64))
        want_h = oracle.fwd(as_rows(a), as_rows(b))
        got_h = hip.scan_forward(a.mT, b.mT)
        assert rel_err(as_rows(got_h.mT), want_h) <= bar, "forward"
        _, hs = place(torch.from_numpy(want_h).mT)
        want_ga, want_gb = oracle.bwd(as_rows(a), as_rows(hs), as_rows(gh))
        got_ga, got_gb = hip.scan_backward(a.mT, hs.mT, gh.mT)
        assert rel_err(as_rows(got_gb.mT), want_gb) <= bar, "grad of value"
        assert rel_err(as_rows(got_ga.mT), want_ga, prev_abs(as_rows(hs))) <= bar, "grad of gate"
        # The same through the C ABI's strided calls with the outputs inside NaN-filled buffers of their own.
        L = hip.lib()
        code = hip._dtype_code(dtype)
        outs = [place(torch.zeros(shape, dtype=torch.float64)) for _ in range(3)]
        st = hip.Strides(outer=T * width, row=width)
        # (the workspace size the library reports covers every alignment a window may turn out to have)
        ws_n = max(hip.workspace_bytes_cl(B, T, C, dtype, d) for d in (hip.FORWARD, hip.BACKWARD))
        ws = torch.empty(max(ws_n, 8), dtype=torch.uint8, device=gpu)
        stream = torch.cuda.current_stream().cuda_stream
        refs = [ctypes.byref(st)] * 5
        rc = L.scanscam_scan_fwd_cl_strided(a.data_ptr(), b.data_ptr(), outs[0][1].data_ptr(), refs[0], refs[1], refs[2],
                                            B, T, C, code, ws.data_ptr(), ws.numel(), stream, None)
        assert rc == 0, hip.strerror(rc)
        rc = L.scanscam_scan_bwd_cl_strided(a.data_ptr(), hs.data_ptr(), gh.data_ptr(), outs[1][1].data_ptr(),
                                            outs[2][1].data_ptr(), refs[0], refs[1], refs[2], refs[3], refs[4],
                                            B, T, C, code, ws.data_ptr(), ws.numel(), stream, None)
        assert rc == 0, hip.strerror(rc)
        torch.cuda.synchronize()
        assert rel_err(as_rows(outs[0][1]), want_h) <= bar, "forward into a window"
        assert rel_err(as_rows(outs[2][1]), want_gb) <= bar, "grad of value into a window"
        assert rel_err(as_rows(outs[1][1]), want_ga, prev_abs(as_rows(hs))) <= bar, "grad of gate into a window"
        for buf, _ in outs:
            assert surroundings_are_nan(buf), "a store outside the window"


def test_plan_search_runs_and_reports_both_directions(gpu):
    # The tuning tool on two small shapes: every plan it keeps is one the library ran, the automatic plan is among them.
    import io

    from scanscam_amd import plan_search

    for layout, shape in (("cl", (4, 300, 96)), ("rows", (64, 1000))):
        text = io.StringIO()
        res = plan_search.search(layout, shape, torch.float32, reps=3, warm=1, out=text, every=True)
        assert set(res) == {"fwd", "bwd"}
        for auto_us, best_us, _ in res.values():
            assert 0 < best_us <= auto_us
        lines = text.getvalue().splitlines()
        assert lines[0].startswith(layout) and sum(line.strip().startswith("auto") for line in lines[1:]) == 2
