"""
The flat kernel (dense short rows scanned as one stream with a reset at every row start) against the CPU
oracle, through the C ABI with the kernel forced (mode = MODE_FLAT) and chosen automatically.

Bars as in test_hip_parity.py: fp32 <= 1e-5 (grad_a with |h[t-1]| in the denominator), float64 <= 1e-13,
16-bit storage <= 1e-2 against the fp32 oracle on the upcast inputs.
"""
import numpy as np
import pytest
import torch

import oracle
from scanscam_amd import hip
from test_hip_parity import bar_for, full_vec, prev_abs, rel_err, seeded, to_np, upcast

pytestmark = pytest.mark.gpu


def check(gpu, a, b, gh, plan, tag):
    print(f"case flat {tag} dtype={a.dtype} shape={tuple(a.shape)} {plan}", flush=True)
    bar = bar_for(a.dtype)
    h = hip.linear_scan_forward(a.to(gpu), b.to(gpu), plan)
    want = oracle.fwd(upcast(a), upcast(b))
    assert rel_err(to_np(h), want) <= bar, tag
    hs = h.cpu()
    ga, gb = hip.linear_scan_backward(a.to(gpu), h, gh.to(gpu), plan)
    want_ga, want_gb = oracle.bwd(upcast(a), upcast(hs), upcast(gh))
    assert rel_err(to_np(gb), want_gb) <= bar, tag
    assert rel_err(to_np(ga), want_ga, prev_abs(upcast(hs))) <= bar, tag


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16, torch.float64])
def test_forced_flat_plans_over_row_lengths(gpu, dtype):
    """Every row length class: one vector, vectors straddling rows, a whole chunk; row counts that leave rows over."""
    full = full_vec(dtype)
    g = seeded(7)
    lengths = sorted({full, full + 1, 2 * full - 1, 3 * full, 5 * full + 3, 17, 63, 64, 65, 70, 33 * full, 64 * full - 1,
                      64 * full})
    for T in lengths:
        if T < full or T > 64 * full:
            continue
        for rows in (1, 2, 7, 37, 1000, 4099):
            if rows - rows % (full // np.gcd(T % full, full)) == 0:
                continue  # not one whole vector of elements: the kernel is not offered
            a = torch.rand(rows, T, generator=g).to(dtype)
            b = torch.randn(rows, T, generator=g).to(dtype)
            gh = torch.randn(rows, T, generator=g).to(dtype)
            for unroll, waves in ((4, 4), (2, 3), (2, 16)):
                check(gpu, a, b, gh, hip.Plan(mode=hip.MODE_FLAT, unroll=unroll, waves=waves), f"T={T} rows={rows}")


def test_flat_is_the_automatic_choice_for_odd_short_rows(gpu):
    # (rows that fill nine tenths of their lane group take it beyond 32 MiB per tensor only: 101 fp32 elements are 26 of 32 lanes)
    for rows, T, dtype in ((120003, 70, torch.float32), (90000, 101, torch.float32), (170000, 100, torch.bfloat16),
                           (130000, 33, torch.float64), (2048, 9, torch.float32)):
        assert hip.resolve_plan(rows, T, dtype, hip.FORWARD).mode == hip.MODE_FLAT
        assert hip.resolve_plan(rows, T, dtype, hip.BACKWARD).mode == hip.MODE_FLAT
        g = seeded(T)
        a = torch.rand(rows, T, generator=g).to(dtype)
        b = torch.randn(rows, T, generator=g).to(dtype)
        gh = torch.randn(rows, T, generator=g).to(dtype)
        check(gpu, a, b, gh, None, "automatic")


def test_flat_is_refused_where_it_cannot_run(gpu):
    flat = hip.Plan(mode=hip.MODE_FLAT)
    a = torch.rand(64, 300, device=gpu)  # longer than a chunk
    with pytest.raises(RuntimeError, match="plan"):
        hip.linear_scan_forward(a, a, flat)
    a = torch.rand(64, 3, device=gpu)    # shorter than a vector
    with pytest.raises(RuntimeError, match="plan"):
        hip.linear_scan_forward(a, a, flat)
    a = torch.rand(3, 5, device=gpu)     # 15 elements: no whole number of vectors in any number of rows below 4
    with pytest.raises(RuntimeError, match="plan"):
        hip.linear_scan_forward(a, a, flat)
    # a view with padded rows is not one dense array: automatic choice falls back, results stay right
    wide = torch.rand(64, 80, device=gpu)
    view = wide[:, :70]
    assert torch.allclose(hip.scan_forward(view, view), hip.scan_forward(view.contiguous(), view.contiguous()), rtol=1e-5,
                          atol=1e-6)


def test_rows_do_not_leak_into_each_other(gpu):
    """Non-finite values stay in their row, also where a vector or a workgroup's span straddles the row border."""
    T, rows = 70, 300
    g = seeded(3)
    a = torch.rand(rows, T, generator=g)
    b = torch.randn(rows, T, generator=g)
    gh = torch.randn(rows, T, generator=g)
    poisoned = (5, 58, 59, 117, 299)
    b[5, 3] = float("inf")
    a[58, T - 1] = float("nan")        # last element of a row: the next row starts in the same vector
    b[59, 0] = float("-inf")
    gh[117, 0] = float("inf")          # backward: first element, the row above ends in the same vector
    a[299, 10] = float("nan")
    plan = hip.Plan(mode=hip.MODE_FLAT)
    h = hip.linear_scan_forward(a.to(gpu), b.to(gpu), plan).cpu()
    clean = [r for r in range(rows) if r not in poisoned and r != 117]
    assert bool(torch.isfinite(h[clean]).all())
    assert bool(torch.isfinite(h[117]).all())  # only its incoming gradient is poisoned
    want = oracle.fwd(a.numpy(), b.numpy())
    assert rel_err(h[clean].numpy(), want[clean]) <= 1e-5
    assert np.array_equal(np.isnan(h.numpy()), np.isnan(want)) and np.array_equal(np.isinf(h.numpy()), np.isinf(want))
    # Backward on a clean forward output, with poisoned incoming gradients only.
    a2 = torch.rand(rows, T, generator=g)
    h2 = hip.linear_scan_forward(a2.to(gpu), torch.randn(rows, T, generator=g).to(gpu), plan)
    ga, gb = hip.linear_scan_backward(a2.to(gpu), h2, gh.to(gpu), plan)
    want_ga, want_gb = oracle.bwd(a2.numpy(), h2.cpu().numpy(), gh.numpy())
    others = [r for r in range(rows) if r != 117]
    assert bool(torch.isfinite(gb.cpu()[others]).all()) and bool(torch.isfinite(ga.cpu()[others]).all())
    assert rel_err(gb.cpu()[others].numpy(), want_gb[others]) <= 1e-5
    assert np.array_equal(np.isfinite(gb.cpu().numpy()), np.isfinite(want_gb))
    assert np.array_equal(np.isnan(ga.cpu().numpy()), np.isnan(want_ga))


def test_flat_is_bit_reproducible_run_to_run(gpu):
    g = seeded(11)
    a = torch.rand(5000, 101, generator=g).to(gpu)
    b = torch.randn(5000, 101, generator=g).to(gpu)
    outs = [hip.linear_scan_forward(a, b, hip.Plan(mode=hip.MODE_FLAT)) for _ in range(3)]
    assert torch.equal(outs[0], outs[1]) and torch.equal(outs[0], outs[2])


def test_forward_in_place_on_a_shape_the_flat_kernel_prefers(gpu):
    """h may share its buffer with a or b (every kernel that is chosen for such a call reads only what it is about
    to write); the flat kernel, which reads a halo of its neighbours' spans, must then not be the one chosen."""
    rows, T = 120003, 70
    assert hip.resolve_plan(rows, T, torch.float32, hip.FORWARD).mode == hip.MODE_FLAT
    g = seeded(70)
    a = torch.rand(rows, T, generator=g)
    b = torch.randn(rows, T, generator=g)
    want = oracle.fwd(a.numpy(), b.numpy())
    for alias in ("value", "gate"):
        da, db = a.to(gpu), b.to(gpu)
        out = db if alias == "value" else da
        print(f"case flat in place over {alias}", flush=True)
        hip.scan_forward_out(da, db, out)
        assert rel_err(to_np(out), want) <= 1e-5, alias
    # Forced, the flat kernel refuses an in-place call instead of racing.
    da, db = a.to(gpu), b.to(gpu)
    with pytest.raises(RuntimeError, match="plan"):
        hip.scan_forward_out(da, db, db, hip.Plan(mode=hip.MODE_FLAT))


def test_automatic_flat_choice_respects_plan_hints(gpu):
    """A plan that only names unroll or waves (mode automatic) must resolve to a kernel that accepts them:
    17 vectors per row are what the flat kernel is preferred for, and it takes 2 or 4 chunks per wave only."""
    rows, T = 120003, 68
    assert hip.resolve_plan(rows, T, torch.float32, hip.FORWARD).mode == hip.MODE_FLAT
    assert hip.resolve_plan(rows, T, torch.float32, hip.FORWARD, hip.Plan(unroll=8)).mode == hip.MODE_SMALL
    g = seeded(71)
    a = torch.rand(rows, T, generator=g)
    b = torch.randn(rows, T, generator=g)
    want = oracle.fwd(a.numpy(), b.numpy())
    for plan in (hip.Plan(unroll=1), hip.Plan(unroll=8), hip.Plan(unroll=8, waves=8), hip.Plan(unroll=2), hip.Plan(waves=2)):
        print(f"case flat hints {plan}", flush=True)
        h = hip.linear_scan_forward(a.to(gpu), b.to(gpu), plan)
        assert rel_err(to_np(h), want) <= 1e-5, plan
