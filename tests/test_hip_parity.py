"""
Parity of the HIP kernels (through the C ABI) with the CPU oracle on identical
seeded inputs.

Bars:
  * fp32: max |x - ref| / max(|ref|, 1) <= 1e-5 for h and grad_b on the
    benchmark configurations (gates in [0, 1]); for grad_a = grad_b * h[t-1] the
    denominator is max(|ref|, |h[t-1]|, 1), i.e. the same bar carried through
    the product (see prev_abs); on the reference's own test
    grid, whose gates are N(0, 1), the reference's bar
    allclose(atol=1e-4, rtol=1e-5) (scanscam/cuda_test.py:26-34) applied to the
    normwise error of each row;
  * 16-bit storage: <= 1e-2 against the fp32 oracle on the upcast inputs.
The GPU result is not expected to be bit-identical to the oracle: the kernels
use FMAs and a parallel association order, the oracle a sequential mul + add.
"""
import itertools

import numpy as np
import pytest
import torch

import oracle
from criteria import assert_reference_allclose
from scanscam_amd import hip

pytestmark = pytest.mark.gpu

FP32_BAR = 1e-5
FP64_BAR = 1e-13
HALF_BAR = 1e-2


def rel_err(x, ref, floor=None):
    """max |x - ref| / max(|ref|, 1 [, floor]) over all elements."""
    x = np.asarray(x, dtype=np.float64)
    ref = np.asarray(ref, dtype=np.float64)
    if x.size == 0:
        return 0.0
    den = np.maximum(np.abs(ref), 1.0)
    if floor is not None:
        den = np.maximum(den, floor)
    return float(np.max(np.abs(x - ref) / den))


def prev_abs(h):
    """|h[t-1]| with h[-1] = 0: the factor that turns grad_b into grad_a.

    grad_a[t] = grad_b[t] * h[t-1], so an error of 1e-5 * max(|grad_b|, 1) in
    grad_b is an error of 1e-5 * max(|grad_a|, |h[t-1]|) in grad_a; the bar for
    grad_a therefore uses |h[t-1]| as an additional floor of the denominator.
    """
    h = np.abs(np.asarray(h, dtype=np.float64))
    out = np.zeros_like(h)
    out[..., 1:] = h[..., :-1]
    return out


def row_norm_err(x, ref):
    """max over rows of max|x - ref| / max(1, max|ref|) -- scale-free per row."""
    x = np.asarray(x, dtype=np.float64).reshape(-1, x.shape[-1])
    ref = np.asarray(ref, dtype=np.float64).reshape(-1, ref.shape[-1])
    if x.size == 0:
        return 0.0
    scale = np.maximum(np.max(np.abs(ref), axis=1), 1.0)
    return float(np.max(np.max(np.abs(x - ref), axis=1) / scale))


def to_np(t):
    t = t.detach().cpu()
    return (t if t.dtype == torch.float64 else t.float()).numpy()


def upcast(t):
    """The oracle's view of a tensor: float64 stays, everything else is exactly upcast to float32."""
    return (t if t.dtype == torch.float64 else t.float()).numpy()


def full_vec(dtype):
    return 16 // torch.empty(0, dtype=dtype).element_size()


def bar_for(dtype):
    return {torch.float32: FP32_BAR, torch.float64: FP64_BAR}.get(dtype, HALF_BAR)


def run_fwd(gpu, a, b, plan=None):
    return hip.linear_scan_forward(a.to(gpu), b.to(gpu), plan)


def run_bwd(gpu, a, h, gh, plan=None):
    return hip.linear_scan_backward(a.to(gpu), h.to(gpu), gh.to(gpu), plan)


def seeded(seed):
    return torch.Generator().manual_seed(seed)


# ---------------------------------------------------------------------------
# The reference's own test grid (scanscam/cuda_test.py:19-126), N(0,1) gates.
# ---------------------------------------------------------------------------
REFERENCE_GRID = [
    (32, 5), (16, 2, 5), (32, 64), (32, 128), (32, 256), (32, 512), (32, 513), (1, 1024), (32, 1024),
    (32, 1025), (1, 1025), (32, 4095), (32, 4096), (32, 4097), (32, 4100), (32, 16384), (32, 16388),
]


@pytest.mark.parametrize("shape", REFERENCE_GRID)
@pytest.mark.parametrize("permute", [False, True])
def test_reference_grid(gpu, shape, permute):
    g = seeded(100 + sum(shape))
    a = torch.randn(shape, generator=g)
    b = torch.randn(shape, generator=g)
    gh = torch.randn(shape, generator=g)
    if permute:
        a = a.mT.contiguous().mT
    print(f"case reference_grid shape={shape} permute={permute}", flush=True)
    h = run_fwd(gpu, a, b)
    assert h.shape == a.shape and h.dtype == a.dtype
    want = oracle.fwd(a.numpy(), b.numpy())
    assert row_norm_err(to_np(h), want) <= 1e-4
    # The reference tests' own criterion, element by element (scanscam/cuda_test.py:80).
    assert_reference_allclose(to_np(h), want, lambda: oracle.fwd_acc64(a.numpy(), b.numpy()), f"h {shape}")
    # Backward as a pure function of (gate, output, out_grad), as the reference tests it.
    hs = torch.from_numpy(want)
    if permute:
        hs = hs.mT.contiguous().mT
    ga, gb = run_bwd(gpu, a, hs, gh)
    wga, wgb = oracle.bwd(a.numpy(), hs.numpy(), gh.numpy())
    assert row_norm_err(to_np(gb), wgb) <= 1e-4
    assert row_norm_err(to_np(ga), wga) <= 1e-4
    # The reference tests' own criterion, element by element, on both gradients
    # (scanscam/cuda_test.py:100-103, 123-126).
    exact = lambda: oracle.bwd_acc64(a.numpy(), hs.numpy(), gh.numpy())  # noqa: E731
    assert_reference_allclose(to_np(gb), wgb, lambda: exact()[1], f"grad_b {shape}")
    assert_reference_allclose(to_np(ga), wga, lambda: exact()[0], f"grad_a {shape}")


# ---------------------------------------------------------------------------
# The five benchmark configurations at full size.
# ---------------------------------------------------------------------------
def config_inputs(n):
    torch.manual_seed(0)
    if n == 1:
        shape = (4, 256, 1024)
        a, b = torch.rand(shape), torch.randn(shape)
    elif n == 2:
        shape = (8, 2048, 4096)
        a, b = torch.sigmoid(torch.randn(shape)), torch.randn(shape)
    elif n == 3:
        shape = (1, 64, 1 << 20)
        a, b = 0.9 + 0.1 * torch.rand(shape), torch.randn(shape)
    elif n == 4:
        shape = (16, 1024, 2048)
        a, b = torch.sigmoid(2 + torch.randn(shape)), 0.5 * torch.randn(shape)
    elif n == 5:
        shape = (256, 512, 64)
        a, b = torch.rand(shape), torch.randn(shape)
    gh = torch.randn(shape)
    return a, b, gh


def report_line(name, got, ref, floor=None):
    """max abs error, elementwise and normwise relative error, and the reference tests' allclose."""
    got, ref = np.asarray(got, np.float64), np.asarray(ref, np.float64)
    max_abs = float(np.max(np.abs(got - ref)))
    normwise = max_abs / max(float(np.max(np.abs(ref))), 1e-300)
    close = bool(np.allclose(got, ref, atol=1e-4, rtol=1e-5))
    return (f"    {name:34s} max|x-ref| {max_abs:.3e}  elementwise {rel_err(got, ref, floor):.3e}  "
            f"normwise {normwise:.3e}  allclose(1e-4, 1e-5) {close}")


@pytest.mark.parametrize("n", [1, 2, 3, 5])
def test_benchmark_config_fp32(gpu, n):
    a, b, gh = config_inputs(n)
    print(f"case config{n} shape={tuple(a.shape)}", flush=True)
    h = run_fwd(gpu, a, b)
    want_h = oracle.fwd(a.numpy(), b.numpy())
    e_h = rel_err(to_np(h), want_h)
    # The backward pass is fed the oracle's h, so its error is its own.
    hs = torch.from_numpy(want_h)
    ga, gb = run_bwd(gpu, a, hs, gh)
    wga, wgb = oracle.bwd(a.numpy(), want_h, gh.numpy())
    hp = prev_abs(want_h)
    e_ga, e_gb = rel_err(to_np(ga), wga, hp), rel_err(to_np(gb), wgb)
    # Reassociation report: GPU and CPU fp32 against the recurrences carried in float64.
    h64 = oracle.fwd_acc64(a.numpy(), b.numpy())
    ga64, gb64 = oracle.bwd_acc64(a.numpy(), want_h, gh.numpy())
    print(f"parity report, configuration {n}, fp32 {tuple(a.shape)} (elementwise = max |x-ref| / max(|ref|, 1); "
          f"for grad_a also |h[t-1]| in the denominator)")
    print(report_line("h       GPU vs CPU fp32", to_np(h), want_h))
    print(report_line("grad_b  GPU vs CPU fp32", to_np(gb), wgb))
    print(report_line("grad_a  GPU vs CPU fp32", to_np(ga), wga, hp))
    print(report_line("h       GPU vs float64 recurrence", to_np(h), h64))
    print(report_line("h       CPU fp32 vs float64", want_h, h64))
    print(report_line("grad_b  GPU vs float64 recurrence", to_np(gb), gb64))
    print(report_line("grad_b  CPU fp32 vs float64", wgb, gb64))
    print(report_line("grad_a  GPU vs float64 recurrence", to_np(ga), ga64, hp))
    print(report_line("grad_a  CPU fp32 vs float64", wga, ga64, hp), flush=True)
    assert e_h <= FP32_BAR and e_ga <= FP32_BAR and e_gb <= FP32_BAR
    # Beside the bars above (of which grad_a's has |h[t-1]| in its denominator: with max(|ref|, 1) alone the
    # reference's own fp32 loop misses 1e-5 against float64 at configuration 3), the criterion the reference's
    # tests apply, element by element, to all three tensors (scanscam/cpu_test.py:25, 46-48).
    for name, got, ref in (("h", h, want_h), ("grad_a", ga, wga), ("grad_b", gb, wgb)):
        assert np.allclose(to_np(got), ref, atol=1e-4, rtol=1e-5), f"configuration {n}: {name} fails allclose(1e-4, 1e-5)"
    del h64, ga64, gb64


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_benchmark_config_16bit(gpu, dtype):
    a32, b32, gh32 = config_inputs(4)
    a, b, gh = (x.to(dtype) for x in (a32, b32, gh32))
    print(f"case config4 dtype={dtype}", flush=True)
    h = run_fwd(gpu, a, b)
    assert h.dtype == dtype
    want_h = oracle.fwd(a.float().numpy(), b.float().numpy())
    assert rel_err(to_np(h), want_h) <= HALF_BAR
    # Feed both sides the same 16-bit saved output, so that its storage rounding
    # is not charged to the backward kernel.
    hs = h.cpu()
    ga, gb = run_bwd(gpu, a, hs, gh)
    wga, wgb = oracle.bwd(a.float().numpy(), hs.float().numpy(), gh.float().numpy())
    hp = prev_abs(hs.float().numpy())
    # Against the all-fp32 chain (inputs never rounded to 16 bits): what the storage type costs in total.
    h_all32 = oracle.fwd(a32.numpy(), b32.numpy())
    print(f"parity report, configuration 4, {str(dtype).replace('torch.', '')} storage / fp32 arithmetic {tuple(a.shape)}")
    print(report_line("h       GPU vs fp32 CPU on upcast inputs", to_np(h), want_h))
    print(report_line("grad_b  GPU vs fp32 CPU on upcast inputs", to_np(gb), wgb))
    print(report_line("grad_a  GPU vs fp32 CPU on upcast inputs", to_np(ga), wga, hp))
    print(report_line("h       GPU vs all-fp32 chain", to_np(h), h_all32), flush=True)
    assert rel_err(to_np(gb), wgb) <= HALF_BAR
    assert rel_err(to_np(ga), wga, hp) <= HALF_BAR


# ---------------------------------------------------------------------------
# Every kernel family / vector width / unroll / workgroup shape, forced on
# small inputs with ragged rows and lengths.
# ---------------------------------------------------------------------------
def plans_for(dtype):
    full = full_vec(dtype)
    out = []
    for vec in (full, 1):
        unrolls = (1, 2, 4, 8) if vec == full else (1, 4)
        for unroll in unrolls:
            max_waves = 16 if unroll <= 4 else 8
            for waves in sorted({1, 4, max_waves}):
                for wpr in sorted({1, 2, waves} & {1, 2, 4, 8, 16}):
                    if waves % wpr == 0:
                        out.append(hip.Plan(mode=hip.MODE_ROW, vec=vec, unroll=unroll, waves=waves, waves_per_row=wpr))
                out.append(hip.Plan(mode=hip.MODE_LOOKBACK, vec=vec, unroll=unroll, waves=waves))
    # Workgroups fitted to a row: any number of waves per row, several such rows per workgroup.
    for waves, wpr in ((3, 3), (9, 9), (13, 13), (15, 5), (12, 3), (6, 2)):
        out.append(hip.Plan(mode=hip.MODE_ROW, vec=full, unroll=4, waves=waves, waves_per_row=wpr))
        out.append(hip.Plan(mode=hip.MODE_ROW, vec=1, unroll=1, waves=waves, waves_per_row=wpr))
    return out


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64, torch.bfloat16, torch.float16])
def test_forced_plans_row_and_lookback(gpu, dtype):
    full = full_vec(dtype)
    bar = bar_for(dtype)
    g = seeded(7)
    cases = {}
    for rows, T in [(5, 8 * full * 37), (3, 64 * full * 5 + full), (1, 64 * full * 33), (7, 1037), (2, 64 * full)]:
        a = torch.rand((rows, T), generator=g, dtype=torch.float64).to(dtype)
        b = torch.randn((rows, T), generator=g, dtype=torch.float64).to(dtype)
        gh = torch.randn((rows, T), generator=g, dtype=torch.float64).to(dtype)
        h = oracle.fwd(upcast(a), upcast(b))
        hs = torch.from_numpy(h).to(dtype)
        ga, gb = oracle.bwd(upcast(a), upcast(hs), upcast(gh))
        cases[(rows, T)] = (a.to(gpu), b.to(gpu), gh.to(gpu), hs.to(gpu), h, ga, gb, prev_abs(upcast(hs)))
    n = 0
    for plan in plans_for(dtype):
        for (rows, T), (a, b, gh, hs, h, ga, gb, hp) in cases.items():
            if plan.vec != 1 and T % full != 0 and (T <= 64 * full or plan.unroll not in (2, 4)):
                continue  # element-aligned rows take the full vector only when longer than a chunk, U = 2 or 4
            print(f"case forced {dtype} rows={rows} T={T} {plan}", flush=True)
            got_h = hip.linear_scan_forward(a, b, plan)
            got_ga, got_gb = hip.linear_scan_backward(a, hs, gh, plan)
            assert rel_err(to_np(got_h), h) <= bar, (plan, rows, T)
            assert rel_err(to_np(got_gb), gb) <= bar, (plan, rows, T)
            assert rel_err(to_np(got_ga), ga, hp) <= bar, (plan, rows, T)
            n += 1
    assert n > 100


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64, torch.bfloat16])
def test_forced_plans_small(gpu, dtype):
    full = full_vec(dtype)
    bar = bar_for(dtype)
    g = seeded(8)
    n = 0
    for vec, unroll, waves in itertools.product((full, 1), (1, 2, 4, 8), (1, 4)):
        if vec == 1 and unroll not in (1, 4):
            continue
        lengths = [vec * k for k in (1, 2, 3, 4, 7, 8, 16, 31, 33, 64)] if vec > 1 else [1, 2, 3, 5, 8, 17, 32, 63, 64]
        if vec > 1 and unroll in (2, 4):  # element-aligned rows of 4 vectors to one chunk: 16-byte lanes, last one partial
            lengths += [4 * vec + 1, 7 * vec + vec - 1, 33 * vec + 1, 64 * vec - 1]
        for T in lengths:
            for rows in (1, 37, 515):
                plan = hip.Plan(mode=hip.MODE_SMALL, vec=vec, unroll=unroll, waves=waves)
                a = torch.rand((rows, T), generator=g, dtype=torch.float64).to(dtype)
                b = torch.randn((rows, T), generator=g, dtype=torch.float64).to(dtype)
                gh = torch.randn((rows, T), generator=g, dtype=torch.float64).to(dtype)
                print(f"case small {dtype} rows={rows} T={T} {plan}", flush=True)
                h = oracle.fwd(upcast(a), upcast(b))
                hs = torch.from_numpy(h).to(dtype)
                ga, gb = oracle.bwd(upcast(a), upcast(hs), upcast(gh))
                got_h = run_fwd(gpu, a, b, plan)
                got_ga, got_gb = run_bwd(gpu, a, hs, gh, plan)
                assert rel_err(to_np(got_h), h) <= bar, (plan, rows, T)
                assert rel_err(to_np(got_gb), gb) <= bar, (plan, rows, T)
                assert rel_err(to_np(got_ga), ga, prev_abs(upcast(hs))) <= bar, (plan, rows, T)
                n += 1
    assert n > 100


# ---------------------------------------------------------------------------
# Edge cases and properties.
# ---------------------------------------------------------------------------
def test_empty_inputs(gpu):
    for shape in [(0, 16), (4, 0), (0, 0), (2, 0, 8)]:
        a = torch.zeros(shape, device=gpu)
        h = hip.linear_scan_forward(a, a)
        assert h.shape == a.shape
        ga, gb = hip.linear_scan_backward(a, a, a)
        assert ga.shape == a.shape and gb.shape == a.shape


@pytest.mark.parametrize("T", [1, 2, 3, 4, 63, 64, 65, 229, 231, 250, 255, 256, 257, 260])
@pytest.mark.parametrize("rows", [1, 2, 129])
def test_short_rows_automatic(gpu, rows, T):
    g = seeded(rows * 1000 + T)
    a = torch.rand((rows, T), generator=g)
    b = torch.randn((rows, T), generator=g)
    gh = torch.randn((rows, T), generator=g)
    h = oracle.fwd(a.numpy(), b.numpy())
    assert rel_err(to_np(run_fwd(gpu, a, b)), h) <= FP32_BAR
    ga, gb = oracle.bwd(a.numpy(), h, gh.numpy())
    got_ga, got_gb = run_bwd(gpu, a, torch.from_numpy(h), gh)
    assert rel_err(to_np(got_gb), gb) <= FP32_BAR
    assert rel_err(to_np(got_ga), ga, prev_abs(h)) <= FP32_BAR


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float64])
@pytest.mark.parametrize("T", [29, 57, 59, 461, 463, 500, 511])
def test_short_element_aligned_rows_other_types(gpu, dtype, T):
    # Rows of odd length around the border (nine tenths of a chunk: 461 elements of 16-bit storage, 116 of
    # float64... the float64 lengths here are 29, 57, 59) from which 16-byte lanes with a masked end take
    # over from one element per lane.
    rows = 131
    g = seeded(4000 + T)
    a = torch.rand((rows, T), generator=g, dtype=torch.float64).to(dtype)
    b = torch.randn((rows, T), generator=g, dtype=torch.float64).to(dtype)
    gh = torch.randn((rows, T), generator=g, dtype=torch.float64).to(dtype)
    bar = bar_for(dtype)
    h = oracle.fwd(upcast(a), upcast(b))
    assert rel_err(to_np(run_fwd(gpu, a, b)), h) <= bar
    hs = torch.from_numpy(h).to(dtype)
    ga, gb = oracle.bwd(upcast(a), upcast(hs), upcast(gh))
    got_ga, got_gb = run_bwd(gpu, a, hs, gh)
    assert rel_err(to_np(got_gb), gb) <= bar
    assert rel_err(to_np(got_ga), ga, prev_abs(upcast(hs))) <= bar


# One shape per branch of the automatic plan for rows longer than a chunk: (rows, T) -> the
# (mode, waves per row, chunks per wave) the library reports for it, forward and backward.
ROW, LOOKBACK = hip.MODE_ROW, hip.MODE_LOOKBACK
AUTO_REGIMES = [
    (2048, 1280, (ROW, 4, 2), None),
    (2048, 4100, (ROW, 5, 4), None),          # 17 chunks: one step of a 5-wave workgroup
    (2048, 10000, (ROW, 10, 4), (LOOKBACK, 0, 4)),  # 40 chunks: forward one workgroup of 10 waves, backward 2 tiles of 5 waves
    (2048, 12501, (LOOKBACK, 0, 4), None),    # element-aligned rows, 50 chunks = 2 tiles of 7 waves, row-major order
    (700, 20000, (LOOKBACK, 0, 4), None),     # 3 tiles per row, 2100 tiles
    (256, 131072, (ROW, 16, 4), (LOOKBACK, 0, 4)),  # 16 tiles per row: only the backward pass gains
    (600, 20000, (ROW, 10, 4), None),         # 1800 tiles: too small for the look-back launch; 79 chunks = 2 steps of 10 waves
    (300, 81920, (LOOKBACK, 0, 4), None),     # 10 tiles per row
    (512, 81920, (LOOKBACK, 0, 4), None),     # also where the row kernel's workgroups come out in full rounds
    (300, 4100, (ROW, 5, 4), None),
    (270, 140000, (LOOKBACK, 0, 4), None),    # 18 tiles per row, 270 rows on 256 CUs: tile-major look-back
    (512, 140000, (ROW, 16, 4), None),        # 18 tiles per row in full rounds: the row kernel
    (300, 16640, (ROW, 9, 4), None),          # few rows, 65 chunks: 2 steps of 9 waves
    (255, 16640, (LOOKBACK, 0, 4), None),     # fewer than 256 rows: tiles in tile-major order
    (12, 300000, (LOOKBACK, 0, 8), (LOOKBACK, 0, 4)),  # up to 16 rows: forward tiles of 8 waves x 8 chunks
    (48, 100000, (LOOKBACK, 0, 8), (LOOKBACK, 0, 4)),  # ... and 17 to 64 rows of a problem of 8 M elements or less
]


@pytest.mark.parametrize("rows,T,expect,expect_bwd", AUTO_REGIMES)
def test_automatic_plan_regimes(gpu, rows, T, expect, expect_bwd):
    if (rows, T) == (2048, 10000):
        # Tiles and row workgroups are fitted to the row: 40 chunks are 2 look-back tiles of 5 waves
        # (backward), or one workgroup of 10 waves (forward; 16-bit storage takes the tiles there too).
        assert hip.resolve_plan(rows, T, torch.float32, hip.BACKWARD).waves == 5
        fwd = hip.resolve_plan(rows, T, torch.float32, hip.FORWARD)
        assert (fwd.waves, fwd.waves_per_row, fwd.unroll) == (10, 10, 4)
        assert hip.resolve_plan(rows, 2 * T, torch.bfloat16, hip.FORWARD).mode == LOOKBACK
    plan = hip.resolve_plan(rows, T, torch.float32, hip.FORWARD)
    assert (plan.mode, plan.waves_per_row, plan.unroll) == expect, plan
    plan = hip.resolve_plan(rows, T, torch.float32, hip.BACKWARD)
    assert (plan.mode, plan.waves_per_row, plan.unroll) == (expect_bwd or expect), plan
    g = seeded(rows + T)
    a = torch.rand((rows, T), generator=g)
    b = torch.randn((rows, T), generator=g)
    gh = torch.randn((rows, T), generator=g)
    h = oracle.fwd(a.numpy(), b.numpy())
    assert rel_err(to_np(run_fwd(gpu, a, b)), h) <= FP32_BAR
    ga, gb = oracle.bwd(a.numpy(), h, gh.numpy())
    got_ga, got_gb = run_bwd(gpu, a, torch.from_numpy(h), gh)
    assert rel_err(to_np(got_gb), gb) <= FP32_BAR
    assert rel_err(to_np(got_ga), ga, prev_abs(h)) <= FP32_BAR


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float64])
def test_rows_that_start_inside_a_cache_line(gpu, dtype):
    # Rows of a length that is a multiple of 16 bytes but not of 128: every row starts at another place
    # inside a 128-byte line, and the row and look-back kernels lay their chunks out from the line
    # border before it (slots before the row's start are masked). Dense tensors and views at every
    # 16-byte offset of a line, both directions, automatic and forced plans.
    full = full_vec(dtype)
    bar = bar_for(dtype)
    g = seeded(91)
    chunk = 64 * full
    plans = [None, hip.Plan(mode=hip.MODE_ROW, vec=full, unroll=2, waves=3, waves_per_row=3),
             hip.Plan(mode=hip.MODE_ROW, vec=1, unroll=4, waves=4, waves_per_row=2),
             hip.Plan(mode=hip.MODE_LOOKBACK, vec=full, unroll=1, waves=2),
             hip.Plan(mode=hip.MODE_LOOKBACK, vec=full, unroll=4, waves=5)]
    for rows, T in [(37, 4 * chunk + 5 * full), (9, 11 * chunk + full), (300, 40 * chunk + 3 * full), (3, 130 * chunk - full)]:
        for off in (0, full, 3 * full, 7 * full):
            def view(fn):
                buf = fn((rows * T + 8 * full,), generator=g, dtype=torch.float64).to(dtype).to(gpu)
                return buf[off:off + rows * T].view(rows, T)
            a, b, gh = view(torch.rand), view(torch.randn), view(torch.randn)
            h = oracle.fwd(upcast(a.cpu()), upcast(b.cpu()))
            hs = torch.from_numpy(h).to(dtype).to(gpu)
            ga, gb = oracle.bwd(upcast(a.cpu()), upcast(hs.cpu()), upcast(gh.cpu()))
            hp = prev_abs(upcast(hs.cpu()))
            for plan in plans:
                if rows >= 300 and plan is not None and plan.vec == 1:
                    continue
                print(f"case lines {dtype} rows={rows} T={T} offset={off} {plan}", flush=True)
                assert rel_err(to_np(hip.linear_scan_forward(a, b, plan)), h) <= bar
                got_ga, got_gb = hip.linear_scan_backward(a, hs, gh, plan)
                assert rel_err(to_np(got_gb), gb) <= bar
                assert rel_err(to_np(got_ga), ga, hp) <= bar


def test_unaligned_base_pointers(gpu):
    # Views that start 4 bytes into an allocation: the library must fall back to
    # element-wise loads, not fault or misread.
    g = seeded(21)
    rows, T = 9, 512
    a = torch.rand((rows, T), generator=g)
    b = torch.randn((rows, T), generator=g)
    gh = torch.randn((rows, T), generator=g)

    def offset_copy(x):
        return torch.empty(rows * T + 1, device=gpu)[1:].view(rows, T).copy_(x)

    da, db, dgh = offset_copy(a), offset_copy(b), offset_copy(gh)
    assert da.data_ptr() % 16 == 4
    out = torch.empty(rows * T + 1, device=gpu)[1:].view(rows, T)
    hip.scan_forward_out(da, db, out)
    h = oracle.fwd(a.numpy(), b.numpy())
    assert rel_err(to_np(out), h) <= FP32_BAR
    oga = torch.empty(rows * T + 1, device=gpu)[1:].view(rows, T)
    ogb = torch.empty(rows * T + 1, device=gpu)[1:].view(rows, T)
    hip.scan_backward_out(da, out, dgh, oga, ogb)
    ga, gb = oracle.bwd(a.numpy(), to_np(out), gh.numpy())
    assert rel_err(to_np(ogb), gb) <= FP32_BAR and rel_err(to_np(oga), ga, prev_abs(to_np(out))) <= FP32_BAR


def test_closed_forms_at_full_size(gpu):
    # Size-independent properties at the Mamba-like shape [8, 2048, 4096].
    shape = (8, 2048, 4096)
    g = torch.Generator(device=gpu).manual_seed(3)
    b = torch.randn(shape, generator=g, device=gpu)
    zero, one = torch.zeros_like(b), torch.ones_like(b)
    # gate 0: h = b exactly; backward: gb = gh exactly, ga[..., 0] = 0.
    assert torch.equal(hip.linear_scan_forward(zero, b), b)
    ga, gb = hip.linear_scan_backward(zero, b, b)
    assert torch.equal(gb, b)
    assert torch.equal(ga[..., 0], torch.zeros_like(ga[..., 0]))
    assert torch.equal(ga[..., 1:], b[..., 1:] * b[..., :-1])
    # value 0: h = 0 exactly.
    assert torch.equal(hip.linear_scan_forward(torch.rand_like(b), zero), zero)
    # gate 1: running sum (compare with a float64 cumsum).
    h = hip.linear_scan_forward(one, b)
    want = torch.cumsum(b.double(), dim=-1)
    assert float((h.double() - want).abs().max()) <= 2e-3
    ga, gb = hip.linear_scan_backward(one, b, b)
    want = torch.flip(torch.cumsum(torch.flip(b.double(), [-1]), dim=-1), [-1])
    assert float((gb.double() - want).abs().max()) <= 2e-3
    # Linearity in the value: scan(a, b1 + 2*b2) = scan(a, b1) + 2*scan(a, b2).
    a = torch.rand_like(b)
    b2 = torch.randn(shape, generator=g, device=gpu)
    lhs = hip.linear_scan_forward(a, b + 2 * b2)
    rhs = hip.linear_scan_forward(a, b) + 2 * hip.linear_scan_forward(a, b2)
    assert float((lhs - rhs).abs().max()) <= 1e-4


def test_long_rows_restart_property(gpu):
    # Scanning [0, k) and then [k, T) from the carried state equals scanning [0, T):
    # h[k:] = scan(a[k:], b[k:] with b[k] += a[k] * h[k-1]). Exercises the look-back
    # chain at 2^20 +- 1 without the CPU in the loop.
    g = torch.Generator(device=gpu).manual_seed(4)
    for T in ((1 << 20) - 1, 1 << 20, (1 << 20) + 4):
        a = 0.9 + 0.1 * torch.rand((3, T), generator=g, device=gpu)
        b = torch.randn((3, T), generator=g, device=gpu)
        full = hip.linear_scan_forward(a, b)
        k = 300000
        b_tail = b[:, k:].clone()
        b_tail[:, 0] += a[:, k] * full[:, k - 1]
        tail = hip.linear_scan_forward(a[:, k:].contiguous(), b_tail)
        assert float((tail - full[:, k:]).abs().max()) <= 1e-4


def test_results_do_not_depend_on_timing(gpu):
    # Same launch twice: bit-identical, look-back included.
    g = torch.Generator(device=gpu).manual_seed(5)
    a = 0.9 + 0.1 * torch.rand((5, 300001), generator=g, device=gpu)
    b = torch.randn(a.shape, generator=g, device=gpu)
    for plan in (None, hip.Plan(mode=hip.MODE_LOOKBACK, vec=1, unroll=1, waves=1)):
        first = hip.linear_scan_forward(a, b, plan)
        for _ in range(3):
            assert torch.equal(hip.linear_scan_forward(a, b, plan), first)
        ga0, gb0 = hip.linear_scan_backward(a, first, b, plan)
        ga1, gb1 = hip.linear_scan_backward(a, first, b, plan)
        assert torch.equal(ga0, ga1) and torch.equal(gb0, gb1)


def test_nonfinite_rows_do_not_leak_into_other_rows(gpu):
    a = torch.rand(6, 1024)
    b = torch.randn(6, 1024)
    b[2, 100] = float("inf")
    b[4, 7] = float("nan")
    h = to_np(run_fwd(gpu, a, b))
    want = oracle.fwd(a.numpy(), b.numpy())
    for r in (0, 1, 3, 5):
        assert np.all(np.isfinite(h[r])) and rel_err(h[r], want[r]) <= FP32_BAR
    assert np.all(np.isfinite(h[2, :100])) and not np.any(np.isfinite(h[2, 100:110]))
    assert np.all(np.isnan(h[4, 7:]))


@pytest.mark.parametrize("T,plan", [
    (64, None),                                                         # small kernel
    (1024, None),                                                       # row kernel, one wave per row
    (20000, None),                                                      # row kernel, 16 waves per row
    (20000, hip.Plan(mode=hip.MODE_LOOKBACK, vec=4, unroll=1, waves=2)),  # look-back, 40 tiles per row
])
def test_backward_nonfinite_gradients_follow_the_reference(gpu, T, plan):
    # The reference forms grad_a[0] as grad_b[0] * 0.0, a multiplication (src/scanscam_cpu.hpp:70-74: h[-1] is
    # the value 0, not a skipped term), so an infinite or NaN grad_b[0] gives NaN there, and an infinite
    # upstream gradient reaches every earlier time step through the gates. Gates just below 1 keep the
    # sign of everything and keep products of gates over any span away from underflow (a parallel scan
    # multiplies an infinite carry by the product of a whole span's gates, and 0 * inf would be NaN where
    # the sequential loop, gate by gate, keeps inf), so the pattern of inf / NaN is fixed by the recurrence,
    # not by the order of association; finite elements must still meet the fp32 bar. Gates 1 - x with
    # x up to 2e-6: in fp32 the product (1 - x)(1 - y) loses its x*y term whenever that is below half the
    # spacing 6e-8 of the numbers under 1, always in the same direction, so products of many gates that
    # close to 1 come out low. A scan over pairs, which multiplies gates with each other, then ends a sum
    # of 20 000 positive terms low by 1e-5 (relative) for x up to 2e-5 and by 3e-5 for x up to 1e-4 -- a
    # plain Hillis-Steele scan in numpy does the same -- while the sequential loop never multiplies two
    # gates. With x up to 2e-6 the effect is below 2e-6.
    g = seeded(1200 + T)
    rows = 6
    a = 1.0 - 2e-6 * torch.rand((rows, T), generator=g)
    b = torch.randn((rows, T), generator=g)
    gh = torch.randn((rows, T), generator=g).abs()
    gh[1, T // 2] = float("inf")     # everything at and before T/2 becomes +inf; grad_a[1, 0] = inf * 0 = NaN
    gh[3, 0] = float("inf")          # only t = 0: grad_b = inf, grad_a = NaN
    gh[4, T - 1] = float("nan")      # the whole row
    h = oracle.fwd(a.numpy(), b.numpy())
    wga, wgb = oracle.bwd(a.numpy(), h, gh.numpy())
    ga, gb = (to_np(x) for x in run_bwd(gpu, a, torch.from_numpy(h), gh, plan))
    for got, want in ((gb, wgb), (ga, wga)):
        assert np.array_equal(np.isnan(got), np.isnan(want))
        assert np.array_equal(np.isposinf(got), np.isposinf(want))
        assert np.array_equal(np.isneginf(got), np.isneginf(want))
    assert np.isnan(wga[1, 0]) and np.isnan(wga[3, 0]) and np.isposinf(wgb[3, 0]) and np.all(np.isnan(wgb[4]))
    # Finite values against the float64 recurrence: with gates this close to 1 a row is nearly a running
    # sum of T positive terms, which the fp32 sequential loop itself only holds to a few 1e-5.
    h64 = h.astype(np.float64)
    xga, xgb = oracle.bwd(a.double().numpy(), h64, gh.double().numpy())
    for r in (0, 2, 5):
        assert rel_err(gb[r], xgb[r]) <= FP32_BAR
        assert rel_err(ga[r], xga[r], prev_abs(h)[r]) <= FP32_BAR
    fin = np.isfinite(wgb[1])
    assert rel_err(gb[1][fin], xgb[1][fin]) <= FP32_BAR


@pytest.mark.parametrize("shape", [(32, 1025), (32, 4100), (3, 300001), (4, 64), (16, 2, 5)])
def test_float64(gpu, shape):
    # The reference also dispatches double (src/scanscam_cpu.hpp:43): fp64 storage and arithmetic.
    g = seeded(300 + sum(shape))
    a = torch.rand(shape, generator=g, dtype=torch.float64)
    b = torch.randn(shape, generator=g, dtype=torch.float64)
    gh = torch.randn(shape, generator=g, dtype=torch.float64)
    h = run_fwd(gpu, a, b)
    assert h.dtype == torch.float64
    want = oracle.fwd(a.numpy(), b.numpy())
    assert rel_err(to_np(h), want) <= FP64_BAR
    ga, gb = run_bwd(gpu, a, torch.from_numpy(want), gh)
    wga, wgb = oracle.bwd(a.numpy(), want, gh.numpy())
    assert rel_err(to_np(gb), wgb) <= FP64_BAR
    assert rel_err(to_np(ga), wga, prev_abs(want)) <= FP64_BAR


def test_expired_wait_is_reported_and_every_wave_exits(gpu):
    # A look-back wait that gives up must not hang: with one poll allowed the launch still
    # completes, and either every tile found its predecessors in that one poll (results right)
    # or word 1 of the workspace is raised and the affected outputs are NaN.
    import ctypes

    rows, T = 2, 1 << 18
    g = torch.Generator(device=gpu).manual_seed(6)
    a = torch.rand((rows, T), generator=g, device=gpu)
    b = torch.randn((rows, T), generator=g, device=gpu)
    good = hip.linear_scan_forward(a, b, hip.Plan(mode=hip.MODE_LOOKBACK, vec=4, unroll=1, waves=1))
    plan = hip.Plan(mode=hip.MODE_LOOKBACK, vec=4, unroll=1, waves=1, spin_limit=1)
    n = hip.workspace_bytes(rows, T, torch.float32, hip.FORWARD, plan)
    ws = torch.empty(n, dtype=torch.uint8, device=gpu)
    out = torch.empty_like(a)
    rc = hip.lib().scanscam_scan_fwd_plan(a.data_ptr(), b.data_ptr(), out.data_ptr(), rows, T, 0, ws.data_ptr(), n,
                                          torch.cuda.current_stream().cuda_stream, ctypes.byref(plan))
    assert rc == 0
    torch.cuda.synchronize()  # returns: no wave is left spinning
    expired = int(ws.view(torch.int64)[1].item()) != 0
    # The library's own query of that flag says the same.
    flag = ctypes.c_int(-1)
    assert hip.lib().scanscam_workspace_timed_out(ws.data_ptr(), torch.cuda.current_stream().cuda_stream,
                                                  ctypes.byref(flag)) == 0
    assert flag.value == int(expired)
    if expired:
        assert bool(torch.isnan(out).any())
        ok = ~torch.isnan(out)
        assert torch.equal(out[ok], good[ok]) or float((out[ok] - good[ok]).abs().max()) <= 1e-4
    else:
        assert torch.equal(out, good)
    # The default limit on the same input: no expiry, right answer.
    again = hip.linear_scan_forward(a, b, hip.Plan(mode=hip.MODE_LOOKBACK, vec=4, unroll=1, waves=1))
    assert torch.equal(again, good)


def test_launch_is_split_when_a_grid_would_exceed_2_pow_32_threads(gpu):
    # 1024-thread workgroups, one row each: 2^22 workgroups is the most one launch can hold, so
    # 2^22 + 1000 rows must be issued as two launches over slabs of rows.
    rows, T = (1 << 22) + 1000, 16
    g = torch.Generator(device=gpu).manual_seed(8)
    a = torch.rand((rows, T), generator=g, device=gpu)
    b = torch.randn((rows, T), generator=g, device=gpu)
    plan = hip.Plan(mode=hip.MODE_ROW, vec=4, unroll=1, waves=16, waves_per_row=16)
    h = hip.linear_scan_forward(a, b, plan)
    want = hip.linear_scan_forward(a, b)  # automatic plan: the small-row kernel, one launch
    assert float((h - want).abs().max()) <= 1e-5
    tail = slice(rows - 2000, rows)  # rows on both sides of the slab border, against the oracle
    assert rel_err(to_np(h[tail]), oracle.fwd(to_np(a[tail]), to_np(b[tail]))) <= FP32_BAR
    ga, gb = hip.linear_scan_backward(a, h, b, plan)
    wga, wgb = hip.linear_scan_backward(a, h, b)
    assert float((gb - wgb).abs().max()) <= 1e-5 and float((ga - wga).abs().max()) <= 1e-4


def test_more_than_2_pow_32_elements(gpu):
    # Offsets beyond 32 bits. Rows are independent and the result of a row does not depend on the
    # launch it is part of, so a slab of rows scanned on its own must be bit-identical to the same
    # rows of the full tensor; slabs are taken at the start, across element 2^31, across element 2^32
    # and at the end, and one slab is also checked against the oracle.
    free, _ = torch.cuda.mem_get_info(gpu)
    rows, T = (1 << 20) + 3, 4104
    if free < 6 * rows * T * 2 + (4 << 30):
        pytest.skip("not enough free device memory for six 8.6 GB tensors")
    assert rows * T > (1 << 32)
    g = torch.Generator(device=gpu).manual_seed(11)
    a = torch.rand((rows, T), generator=g, device=gpu, dtype=torch.bfloat16)
    b = torch.randn((rows, T), generator=g, device=gpu, dtype=torch.bfloat16)
    h = hip.linear_scan_forward(a, b)
    ga, gb = hip.linear_scan_backward(a, h, b)
    r31, r32 = (1 << 31) // T, (1 << 32) // T
    for r0 in (0, r31 - 2, r32 - 2, rows - 5):
        s = slice(r0, r0 + 5)
        a_s, b_s, h_s = a[s].clone(), b[s].clone(), h[s].clone()
        assert torch.equal(hip.linear_scan_forward(a_s, b_s), h[s]), f"forward rows {r0}.."
        ga_s, gb_s = hip.linear_scan_backward(a_s, h_s, b_s)
        assert torch.equal(ga_s, ga[s]) and torch.equal(gb_s, gb[s]), f"backward rows {r0}.."
    s = slice(r32 - 2, r32 + 3)
    assert rel_err(to_np(h[s]), oracle.fwd(upcast(a[s].cpu()), upcast(b[s].cpu()))) <= HALF_BAR
    del a, b, h, ga, gb

    # The look-back kernel: 5 rows of 2^30 float32 (5.4e9 elements). Gate 0 makes the scan the
    # identity, so every element of the output names the input element it was read from; then a
    # slab against the same row scanned alone.
    rows, T = 5, 1 << 30
    if free < 3 * rows * T * 4 + (8 << 30):
        pytest.skip("not enough free device memory for three 21 GB tensors")
    b = torch.randn((rows, T), generator=g, device=gpu)
    a = torch.zeros_like(b)
    h = hip.linear_scan_forward(a, b)
    assert torch.equal(h, b)
    a.uniform_(0.9, 1.0, generator=g)
    h = hip.linear_scan_forward(a, b)
    for r in (0, 2, 4):
        assert torch.equal(hip.linear_scan_forward(a[r:r + 1].clone(), b[r:r + 1].clone()), h[r:r + 1]), f"row {r}"
    # restart property across element 2^32 of the tensor (row 4 starts at 2^32)
    k = 1 << 29
    b_tail = b[4:5, k:].clone()
    b_tail[:, 0] += a[4, k] * h[4, k - 1]
    tail = hip.linear_scan_forward(a[4:5, k:].contiguous(), b_tail)
    assert float((tail - h[4:5, k:]).abs().max()) <= 1e-4


def test_timed_entry_points(gpu):
    # The timed variants launch the same kernels (bit-identical results) and leave the kernel's own
    # duration in the caller's events: positive, and below what the whole call sequence takes.
    g = torch.Generator(device=gpu).manual_seed(12)
    for rows, T in [(1024, 4096), (2, 1 << 20), (4096, 64)]:  # row, look-back and small kernels
        a = torch.rand((rows, T), generator=g, device=gpu)
        b = torch.randn((rows, T), generator=g, device=gpu)
        gh = torch.randn((rows, T), generator=g, device=gpu)
        h, h2 = torch.empty_like(a), torch.empty_like(a)
        ga, gb, ga2, gb2 = (torch.empty_like(a) for _ in range(4))
        hip.prepare_forward(a, b, h)()
        hip.prepare_backward(a, h, gh, ga, gb)()
        ef, eb = hip.KernelEvents(), hip.KernelEvents()
        fwd = hip.prepare_forward(a, b, h2, events=ef)
        bwd = hip.prepare_backward(a, h, gh, ga2, gb2, events=eb)
        for _ in range(3):
            fwd()
            bwd()
        torch.cuda.synchronize()
        assert torch.equal(h, h2) and torch.equal(ga, ga2) and torch.equal(gb, gb2)
        tf, tb = ef.elapsed_ms(), eb.elapsed_ms()
        print(f"timed [{rows}, {T}]: forward {tf * 1e3:.1f} us, backward {tb * 1e3:.1f} us", flush=True)
        floor_ms = 12 * rows * T / 8e12 * 1e3  # no kernel is faster than the HBM peak
        assert floor_ms <= tf < 5.0 and 20 / 12 * floor_ms <= tb < 5.0


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64, torch.bfloat16, torch.float16])
def test_lookback_row_major_ticket_order(gpu, dtype):
    # From 256 rows on, rows of at most 16 tiles are handed out row after row by 4 ticket counters
    # (rows of one counter are 4 apart). Forced here with small tiles: whole and partial last tiles,
    # element-aligned rows, a row count that the counters do not divide, and two-level strided views.
    full = full_vec(dtype)
    bar = bar_for(dtype)
    g = seeded(17)
    chunk = 64 * full
    for rows, T, unroll, waves in [(259, 11 * chunk + 3, 2, 1), (257, 16 * chunk, 1, 1), (300, 7 * 8 * chunk - full, 2, 4),
                                   (256, 2 * 16 * chunk, 4, 4)]:
        plan = hip.Plan(mode=hip.MODE_LOOKBACK, vec=full, unroll=unroll, waves=waves)
        a = torch.rand((rows, T), generator=g, dtype=torch.float64).to(dtype)
        b = torch.randn((rows, T), generator=g, dtype=torch.float64).to(dtype)
        gh = torch.randn((rows, T), generator=g, dtype=torch.float64).to(dtype)
        print(f"case row-major {dtype} rows={rows} T={T} {plan}", flush=True)
        h = oracle.fwd(upcast(a), upcast(b))
        got = run_fwd(gpu, a, b, plan)
        assert rel_err(to_np(got), h) <= bar
        ga, gb = oracle.bwd(upcast(a), upcast(got.cpu()), upcast(gh))
        got_ga, got_gb = run_bwd(gpu, a, got, gh, plan)
        assert rel_err(to_np(got_gb), gb) <= bar
        assert rel_err(to_np(got_ga), ga, prev_abs(to_np(got))) <= bar
    # halves of x[3, 2*90, T]: 270 rows in two levels
    T = 6 * chunk
    x = torch.randn((3, 180, T), generator=g, dtype=torch.float64)
    x[:, :90] = torch.sigmoid(x[:, :90])
    x = x.to(dtype).to(gpu)
    a, b = x.chunk(2, dim=1)
    plan = hip.Plan(mode=hip.MODE_LOOKBACK, vec=full, unroll=1, waves=1)
    got = hip.scan_forward(a, b, plan)
    h = oracle.fwd(upcast(a.cpu()), upcast(b.cpu()))
    assert rel_err(to_np(got), h) <= bar
    ga, gb = oracle.bwd(upcast(a.cpu()), upcast(got.cpu()), upcast(b.cpu()))
    got_ga, got_gb = hip.scan_backward(a, got, b, plan)
    assert rel_err(to_np(got_gb), gb) <= bar
    assert rel_err(to_np(got_ga), ga, prev_abs(to_np(got))) <= bar
