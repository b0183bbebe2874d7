"""
Host-side logic that needs no GPU: the flattening decorators, the
channels-last probe, the tensor-level loop and the autograd op on CPU tensors,
each checked against the CPU oracle (shapes of scanscam/cpu_test.py:14).
"""
import numpy as np
import pytest
import torch

import oracle
import scanscam_amd
from scanscam_amd import baseline, decorator, hip, op

GRID = [(32, 5), (16, 2, 5), (32, 64), (1, 257), (3, 2, 2, 9)]


@pytest.mark.parametrize("shape", GRID)
@pytest.mark.parametrize("permute", [False, True])
def test_tensor_loop_matches_oracle(shape, permute):
    g = torch.Generator().manual_seed(11)
    a = torch.randn(shape, generator=g)
    b = torch.randn(shape, generator=g)
    gh = torch.randn(shape, generator=g)
    if permute:
        a = a.mT.contiguous().mT  # same values, not contiguous (scanscam/cpu_test.py:21-22)
        assert not a.is_contiguous() or a.shape[-1] == 1 or a.shape[-2] == 1
    h = baseline.naive_linear_scan_forward(a, b)
    assert h.shape == a.shape
    want = oracle.fwd(a.numpy(), b.numpy())
    assert np.allclose(h.numpy(), want, rtol=1e-5, atol=1e-4)
    ga, gb = baseline.naive_linear_scan_backward(a, h, gh)
    wga, wgb = oracle.bwd(a.numpy(), h.numpy(), gh.numpy())
    assert np.allclose(ga.numpy(), wga, rtol=1e-5, atol=1e-4)
    assert np.allclose(gb.numpy(), wgb, rtol=1e-5, atol=1e-4)


def test_scan_autograd_on_cpu_tensors_returns_both_gradients():
    g = torch.Generator().manual_seed(12)
    a = torch.rand((4, 3, 20), generator=g, dtype=torch.float64, requires_grad=True)
    b = torch.randn((4, 3, 20), generator=g, dtype=torch.float64, requires_grad=True)
    gh = torch.randn((4, 3, 20), generator=g, dtype=torch.float64)
    h = scanscam_amd.scan(a, b)
    h.backward(gh)
    wga, wgb = oracle.bwd(a.detach().numpy(), h.detach().numpy(), gh.numpy())
    assert np.allclose(a.grad.numpy(), wga, rtol=1e-12, atol=1e-12)
    assert np.allclose(b.grad.numpy(), wgb, rtol=1e-12, atol=1e-12)
    assert torch.autograd.gradcheck(scanscam_amd.scan, (a, b), eps=1e-6, atol=1e-6)


def test_decorators_check_shapes():
    calls = []

    @decorator.preprocess_scan_args
    def f(x, y):
        calls.append((tuple(x.shape), tuple(y.shape)))
        return x + y

    out = f(torch.zeros(2, 3, 4), torch.ones(2, 3, 4))
    assert out.shape == (2, 3, 4) and calls == [((6, 4), (6, 4))]
    with pytest.raises(AssertionError):
        f(torch.zeros(2, 3), torch.zeros(3, 2))
    with pytest.raises(AssertionError):
        f(torch.zeros(5), torch.zeros(5))

    @decorator.preprocess_backward_scan_args
    def gfn(x, y, z):
        return x * 2, z * 3

    p, q = gfn(torch.ones(2, 3, 4), torch.ones(2, 3, 4), torch.ones(2, 3, 4))
    assert p.shape == q.shape == (2, 3, 4) and float(q[0, 0, 0]) == 3.0
    with pytest.raises(AssertionError):
        gfn(torch.ones(2, 4), torch.ones(2, 4), torch.ones(2, 5))


def test_is_transpose_contig():
    x = torch.zeros(2, 5, 3)
    assert not op.is_transpose_contig(x)
    assert op.is_transpose_contig(x.mT)
    assert not op.is_transpose_contig(torch.zeros(5, 3).mT)       # 2-D never qualifies
    assert not op.is_transpose_contig(torch.zeros(2, 2, 5, 3).mT)  # nor 4-D
    assert scanscam_amd.is_transpose_contig is op.is_transpose_contig


def test_gpu_entry_points_reject_cpu_tensors_and_unknown_dtypes():
    x = torch.zeros(2, 8)
    with pytest.raises(RuntimeError, match="GPU tensor"):
        hip.blocked_linear_scan_forward(x, x)
    with pytest.raises(RuntimeError, match="GPU tensor"):
        hip.blocked_linear_scan_backward(x, x, x)
    with pytest.raises(TypeError):
        hip.resolve_plan(4, 8, torch.int32)


def test_reference_import_names_resolve_to_this_package():
    """Code written against the reference imports `scanscam...` (scanscam/cuda_test.py:7-16,
    scanscam/cpu_test.py:7-8, scanscam/op.py:5-6); every such name must lead here."""
    import scanscam
    import scanscam.cuda
    from scanscam import cpu, cuda  # noqa: F401
    from scanscam.baseline import naive_linear_scan_backward, naive_linear_scan_forward
    from scanscam.cpu import simple_linear_scan_backward, simple_linear_scan_forward
    from scanscam.cuda import (
        blocked_linear_scan_backward,
        blocked_linear_scan_forward,
        coalesced_linear_scan_forward,
        simple_linear_scan_backward as gpu_simple_backward,
        simple_linear_scan_forward as gpu_simple_forward,
        transposed_linear_scan_backward,
        transposed_linear_scan_forward,
    )
    from scanscam.decorator import preprocess_backward_scan_args, preprocess_scan_args
    from scanscam.op import Scan, is_transpose_contig, scan

    assert scanscam.scan is scanscam_amd.scan and scan is scanscam_amd.scan and Scan is op.Scan
    assert scanscam.__all__ == ["scan"]  # scanscam/__init__.py:3
    assert is_transpose_contig is op.is_transpose_contig
    assert scanscam.cuda is scanscam_amd.cuda and scanscam.cpu is scanscam_amd.cpu
    assert blocked_linear_scan_forward is hip.blocked_linear_scan_forward
    assert blocked_linear_scan_backward is hip.blocked_linear_scan_backward
    assert transposed_linear_scan_forward is hip.transposed_linear_scan_forward
    assert transposed_linear_scan_backward is hip.transposed_linear_scan_backward
    assert coalesced_linear_scan_forward is gpu_simple_forward is hip.blocked_linear_scan_forward
    assert gpu_simple_backward is hip.blocked_linear_scan_backward
    assert naive_linear_scan_forward is baseline.naive_linear_scan_forward
    assert naive_linear_scan_backward is baseline.naive_linear_scan_backward
    assert simple_linear_scan_forward is scanscam_amd.cpu.simple_linear_scan_forward
    assert simple_linear_scan_backward is scanscam_amd.cpu.simple_linear_scan_backward
    assert preprocess_scan_args is decorator.preprocess_scan_args
    assert preprocess_backward_scan_args is decorator.preprocess_backward_scan_args
    # The op itself, called through the reference's name on CPU tensors.
    g = torch.Generator().manual_seed(5)
    a, b = torch.rand((3, 4, 9), generator=g), torch.randn((3, 4, 9), generator=g)
    assert np.allclose(scanscam.scan(a, b).numpy(), oracle.fwd(a.numpy(), b.numpy()), rtol=1e-5, atol=1e-4)


def _levels(*tensors):
    return hip._two_levels(tensors[0].shape[:-1], [t.stride()[:-1] for t in tensors])


def test_views_are_described_by_at_most_two_stride_levels():
    """The host logic that lets the strided entry points take views as they are (no GPU involved)."""
    T = 12
    dense = torch.zeros(4, 6, T)
    n0, n1, st = _levels(dense)
    assert (n0, n1) == (1, 24) and (st[0].outer, st[0].row) == (0, T)       # one level: rows follow each other
    x = torch.zeros(4, 12, T)
    a, b = x.chunk(2, dim=1)                                                # halves of a fused projection
    n0, n1, st = _levels(a, b, dense)
    assert (n0, n1) == (4, 6)
    assert [(s.outer, s.row) for s in st] == [(12 * T, T), (12 * T, T), (6 * T, T)]
    sl = torch.zeros(4, 6, 20)[..., 3:3 + T]                                # a slice along time: one level, pitch 20
    n0, n1, st = _levels(sl)
    assert (n0, n1) == (1, 24) and st[0].row == 20
    bc = torch.zeros(1, 6, T).expand(4, 6, T)                               # broadcast over the batch: stride 0
    n0, n1, st = _levels(bc, dense)
    assert (n0, n1) == (4, 6) and (st[0].outer, st[0].row) == (0, T) and (st[1].outer, st[1].row) == (6 * T, T)
    assert _levels(torch.zeros(2, 6, 8, T)[:, :3, :4]) is None               # three levels: needs a copy
    assert _levels(torch.zeros(2, 1, 8, T)[:, :, :4])[:2] == (2, 4)          # size-1 dimensions do not count
    assert _levels(torch.zeros(T))[:2] == (1, 1)                            # a single row
    # size-1 dimensions merge with anything
    assert hip._joint_levels((3, 1, 5), [(40, 7, 8)]) == [(15, [8])]


def test_layout_classification_of_views():
    x = torch.zeros(2, 5, 3)
    assert hip._is_row_view(x) and not hip._is_cl_view(x)
    assert hip._is_cl_view(x.mT) and not hip._is_row_view(x.mT)
    half = torch.zeros(2, 5, 6).chunk(2, dim=-1)[0].mT                       # [2, 3, 5] stored [2, 5, 2*3]
    assert hip._is_cl_view(half) and half.stride(-1) == 6
    assert hip._is_row_view(torch.zeros(4, 9)[:, 2:7])
    assert not hip._is_row_view(torch.zeros(4, 9)[:, ::2]) and not hip._is_cl_view(torch.zeros(4, 9)[:, ::2])
    assert hip._is_row_view(torch.zeros(4, 1).expand(4, 1))                  # T == 1: any stride will do
    for bad in (torch.zeros(2, 8), ):
        with pytest.raises(RuntimeError, match="GPU tensors"):
            hip.scan_forward(bad, bad)
        with pytest.raises(RuntimeError, match="GPU tensors"):
            hip.scan_backward(bad, bad, bad)


def test_package_never_imports_the_oracle():
    import os
    import re

    root = os.path.dirname(os.path.abspath(scanscam_amd.__file__))
    for dirpath, _, files in os.walk(root):
        for f in files:
            if f.endswith((".py", ".hip", ".hpp", ".h")):
                text = open(os.path.join(dirpath, f)).read()
                assert not re.search(r"^\s*(import|from)\s+oracle\b", text, flags=re.M), f
                assert "scan_oracle" not in text, f


def test_plan_search_sets_hold_plans_the_library_knows():
    # The forced plans of scanscam_amd.plan_search: each is accepted for at least one of the search's own shapes.
    import ctypes

    from scanscam_amd import plan_search

    L = hip.lib()
    for dtype in (torch.float32, torch.bfloat16):
        code = hip._dtype_code(dtype)
        for plan in plan_search.row_plans(dtype, 64):
            out = hip.Plan()
            assert any(L.scanscam_resolve_plan(rows, T, code, hip.FORWARD, ctypes.byref(plan), ctypes.byref(out)) == 0
                       for rows, T in ((4096, 64), (4096, 4096), (16, 1 << 20))), plan
        for C in (1001, 1024):
            for plan in plan_search.cl_plans(dtype, C):
                out = hip.Plan()
                assert any(L.scanscam_resolve_plan_cl(batch, 2048, C, code, hip.FORWARD, ctypes.byref(plan), ctypes.byref(out)) == 0
                           for batch in (8, 512)), (C, plan)
    assert {"cl-a", "cl-b", "cl-odd", "rows-25"} <= set(plan_search.SUITES)
    # The random audit: the same shapes for the same seed, inside the stated bounds, and resolvable by the library.
    shapes = plan_search.random_cl_shapes(30, 3)
    assert shapes == plan_search.random_cl_shapes(30, 3) and shapes != plan_search.random_cl_shapes(30, 4)
    rows = plan_search.random_row_shapes(20, 1)
    assert rows == plan_search.random_row_shapes(20, 1) and all(1 <= r <= 1 << 22 and 4 <= T <= 1 << 20 for r, T in rows)
    for batch, T, C in shapes:
        assert 1 <= batch <= 8192 and 64 <= T <= 16384 and 8 <= C <= 5100 and batch * T * C <= 1 << 28
        for dtype in (torch.float32, torch.bfloat16):
            assert hip.resolve_plan_cl(batch, T, C, dtype, hip.BACKWARD).waves >= 1


def test_bench_refuses_more_than_one_gpu():
    # This build runs on one GPU: asking for more ends with a message that says so, before anything touches a device.
    import os
    import subprocess
    import sys

    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    done = subprocess.run([sys.executable, os.path.join(root, "bench.py"), "--gpus", "2"], capture_output=True, text=True,
                          timeout=120)
    assert done.returncode != 0
    assert "one GPU" in done.stderr and done.stdout.strip() == ""


def test_channels_last_views_with_a_far_time_stride_are_copied_first():
    """The channels-last kernels refuse time strides beyond 32-bit step offsets (4 GiB / 18); the wrapper's
    decision to copy such a view first uses the library's own bound."""
    from scanscam_amd import hip

    assert not hip._cl_step_too_far(512, 512, 4)
    assert not hip._cl_step_too_far(59_000_000, 1024, 4)        # 225 MiB steps: still addressable
    assert hip._cl_step_too_far(59_700_000, 1024, 4)            # about 227.7 MiB: beyond
    assert hip._cl_step_too_far(2 ** 31, 8, 2)
    # Exactly the library's inequality (time stride * size * 18 + C * size < 2^32).
    for stride, C, esize in ((59_652_323, 4, 4), (59_652_324, 4, 4), (119_304_646, 8, 2), (119_304_647, 2, 2)):
        assert hip._cl_step_too_far(stride, C, esize) == (stride * esize * 18 + C * esize >= 2 ** 32)


def test_the_fitting_tool_recovers_a_table_from_timings_and_writes_it_back(tmp_path):
    """plan_fit end to end on the CPU: timings generated from the shipped table (with 2 % noise), in the format
    plan_search --dump writes, are read, fitted, printed as a .inc and read back; the fitted model then orders the
    plans of each shape as the generating table does."""
    import io
    import os

    from scanscam_amd import plan_fit

    root = os.path.join(os.path.dirname(os.path.abspath(__file__)), "..")
    table = plan_fit.read_table(os.path.join(root, "scanscam_amd", "csrc", "scan_cl_model.inc"))
    rng = np.random.default_rng(11)
    dump = tmp_path / "dump.txt"
    with open(dump, "w") as f:
        for _ in range(60):
            batch, T, C = int(2 ** rng.uniform(3, 10)), int(2 ** rng.uniform(8, 13)), 64 * int(rng.integers(1, 24))
            for direction in ("fwd", "bwd"):
                for mode in (2, 3):
                    for vec, steps in ((1, 16), (2, 8), (4, 4), (4, 8)):
                        for waves in (4, 8):
                            d = plan_fit.describe(batch, T, C, 4, direction == "bwd", mode, vec, steps, waves)
                            us = plan_fit.predict(d, table) * float(np.exp(rng.normal(0, 0.02)))
                            f.write(f"{batch} {T} {C} float32 {direction} {mode} {vec} {steps} {waves} {us:.2f}\n")
    by = plan_fit.load([str(dump)])
    assert len(by) == 120
    p, rms, seen, n = plan_fit.fit(by, evaluations=60)
    assert n > 1000 and rms < 0.05, (n, rms)
    text = io.StringIO()
    plan_fit.emit(p, seen, "dump.txt", text)
    inc = tmp_path / "model.inc"
    inc.write_text(text.getvalue())
    back = plan_fit.read_table(str(inc))
    assert back.shape == table.shape
    # (printed without a learned correction, the second table is the zero one)
    assert not plan_fit.read_residual(str(inc)).flat()[4 * plan_fit.N_FEATURES:].any()
    picked, ideal = [], []
    for key, timings in by.items():
        plans = [(d, us) for d, us in timings if d is not None and plan_fit.candidate(d)]
        truth = [plan_fit.predict(d, table) for d, _ in plans]
        choice = int(np.argmin([plan_fit.predict(d, back) for d, _ in plans]))
        picked.append(truth[choice])
        ideal.append(min(truth))
    assert np.mean(np.array(picked) / np.array(ideal)) < 1.02


def test_the_learned_correction_is_trained_printed_and_read_back(tmp_path):
    """fit_residual on timings that the formula misses by a known factor per lane width: the correction learns most of
    it, stays within its limit, and survives the trip through the printed table."""
    import io
    import os

    from scanscam_amd import plan_fit

    root = os.path.join(os.path.dirname(os.path.abspath(__file__)), "..")
    table = plan_fit.read_table(os.path.join(root, "scanscam_amd", "csrc", "scan_cl_model.inc"))
    rng = np.random.default_rng(12)
    by = {}
    for _ in range(80):
        batch, T, C = int(2 ** rng.uniform(3, 10)), int(2 ** rng.uniform(8, 13)), 64 * int(rng.integers(1, 24))
        for rev in (False, True):
            timings = []
            for mode in (2, 3):
                for vec, steps in ((1, 16), (2, 8), (4, 4), (4, 8)):
                    for waves in (4, 8):
                        d = plan_fit.describe(batch, T, C, 4, rev, mode, vec, steps, waves)
                        timings.append((d, plan_fit.predict(d, table) * (1.0 + 0.1 * vec) * float(np.exp(rng.normal(0, 0.01)))))
            by[(batch, T, C, 4, rev)] = timings
    r, before, after = plan_fit.fit_residual(by, table, max_iter=300)
    assert before > 0.2 and after < 0.05, (before, after)
    text = io.StringIO()
    plan_fit.emit(table, set(range(plan_fit.N_RATE)), "synthetic", text, r)
    inc = tmp_path / "model.inc"
    inc.write_text(text.getvalue())
    back = plan_fit.read_residual(str(inc))
    d = plan_fit.describe(64, 2048, 1024, 4, False, 2, 2, 8, 8)
    x = plan_fit.features(d, plan_fit.predict(d, table))
    assert abs(float(back.correct(x)[0]) - float(r.correct(x)[0])) < 1e-6
    assert abs(float(r.correct(x)[0]) - np.log(1.2)) < 0.05
    wild = [1e9] * plan_fit.N_FEATURES
    assert abs(float(r.correct(wild)[0])) <= plan_fit.RESIDUAL_LIMIT
