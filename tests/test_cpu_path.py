"""
The host-memory path: ``libscanscam_cpu.so`` behind ``scanscam_amd/cpu.py``, the
counterpart of the reference's ``scanscam/cpu.py`` + ``src/scanscam_cpu.hpp``.

It must reproduce the reference's loop bit for bit (same operations per row,
multiply and add rounded separately), so every comparison here is
``array_equal`` against the oracle -- which ``tests/test_oracle.py`` pins bit-exactly
against the reference's own sources -- on the shapes of the reference's CPU test
(``scanscam/cpu_test.py:14``: ``(16, 2, 5)``, permuted or not) and on shapes that
cross the library's own borders (rows not a multiple of the 8 it advances
together, rows shorter than the 16-element lag between them, slabs over threads).
No GPU is involved.
"""
import ctypes
import os
import re

import numpy as np
import pytest
import torch

import oracle
import scanscam_amd
from scanscam_amd import cpu, op

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "scanscam_cpu.h")

DTYPES = [torch.float32, torch.float64]
SHAPES = [(16, 2, 5), (1, 1), (3, 1), (1, 17), (8, 16), (9, 15), (7, 130), (8, 129), (23, 1000), (64, 257), (5, 4096)]


def inputs(shape, dtype, seed):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(shape, generator=g, dtype=dtype), torch.randn(shape, generator=g, dtype=dtype),
            torch.randn(shape, generator=g, dtype=dtype))


def test_library_is_built_and_exports_what_the_header_declares():
    assert os.path.exists(cpu.LIB_PATH), "build with `make -C scanscam_amd/csrc`"
    assert cpu.has_cpu_ops
    text = re.sub(r"/\*.*?\*/", "", open(HEADER).read(), flags=re.S)
    names = sorted(set(re.findall(r"\b(scanscam_cpu_[a-z0-9_]+)\s*\(", text)))
    assert names == ["scanscam_cpu_bwd_f32", "scanscam_cpu_bwd_f64", "scanscam_cpu_fwd_f32", "scanscam_cpu_fwd_f64"]
    raw = ctypes.CDLL(cpu.LIB_PATH)
    for name in names:
        assert hasattr(raw, name), f"{name} declared in scanscam_cpu.h but not exported"


def test_header_is_plain_c():
    import subprocess
    import tempfile

    with tempfile.TemporaryDirectory() as d:
        src = os.path.join(d, "t.c")
        open(src, "w").write('#include "scanscam_cpu.h"\nint main(void) { return scanscam_cpu_fwd_f32(0, 0, 0, 0, 0); }\n')
        subprocess.run(["gcc", "-std=c99", "-Wall", "-Werror", "-I", os.path.join(ROOT, "include"), "-c", src,
                        "-o", os.path.join(d, "t.o")], check=True)


def test_plain_c_consumer():
    # tests/c_abi/cpu_abi_check: C99, no torch, no Python; built by `make -C tests/c_abi`.
    import subprocess

    binary = os.path.join(ROOT, "tests", "c_abi", "cpu_abi_check")
    assert os.path.exists(binary), "tests/c_abi/cpu_abi_check is not built: run `make -C tests/c_abi`"
    done = subprocess.run([binary], capture_output=True, text=True, timeout=120)
    assert done.returncode == 0 and "cpu_abi_check: ok" in done.stdout, done.stdout + done.stderr


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("shape", SHAPES)
def test_bit_identical_to_the_reference_loop(shape, dtype):
    a, b, gh = inputs(shape, dtype, 11 + sum(shape))
    h = cpu.simple_linear_scan_forward(a, b)
    assert h.shape == a.shape and h.dtype == dtype
    want = oracle.fwd(a.numpy(), b.numpy())
    assert np.array_equal(h.numpy(), want)
    ga, gb = cpu.simple_linear_scan_backward(a, h, gh)
    wga, wgb = oracle.bwd(a.numpy(), want, gh.numpy())
    assert np.array_equal(gb.numpy(), wgb)
    assert np.array_equal(ga.numpy(), wga)


# The reference's CPU test grid (scanscam/cpu_test.py:11-48): N(0,1) gates and values, each shape
# contiguous and with its last two dimensions transposed in memory (x.mT.contiguous().mT), forward
# against the tensor-level loop at atol 1e-4 and backward as a plain function of three unrelated
# tensors (gate, output, out_grad).
REFERENCE_CPU_GRID = [(32, 5), (16, 2, 5), (32, 64), (1, 1024), (32, 1024), (32, 1025), (1, 1025)]


@pytest.mark.parametrize("permute", [False, True])
@pytest.mark.parametrize("shape", REFERENCE_CPU_GRID)
def test_reference_cpu_grid(shape, permute):
    from scanscam_amd.baseline import naive_linear_scan_backward, naive_linear_scan_forward

    x, y, z = inputs(shape, torch.float32, 77 + sum(shape))
    if permute:
        x, y, z = (t.mT.contiguous().mT for t in (x, y, z))
        assert not x.is_contiguous() or 1 in shape[-2:]
    out = cpu.simple_linear_scan_forward(x, y)
    assert out.shape == x.shape
    assert torch.allclose(out, naive_linear_scan_forward(x, y), atol=1e-4)
    ga, gb = cpu.simple_linear_scan_backward(x, y, z)
    wa, wb = naive_linear_scan_backward(x, y, z)
    # N(0,1) gates: values grow along a row; the bar of the reference's test, scaled by the row's size.
    scale = max(1.0, float(wb.abs().max()), float(wa.abs().max()))
    assert torch.allclose(ga, wa, atol=1e-4 * scale) and torch.allclose(gb, wb, atol=1e-4 * scale)


def test_golden_vectors():
    # The fixtures written from the reference's own build (tests/golden/make_golden.py).
    z = np.load(os.path.join(ROOT, "tests", "golden", "scan_golden.npz"))
    cases = sorted({k.rsplit(".", 1)[0] for k in z.files})
    assert cases
    checked = 0
    for c in cases:
        keys = {k.rsplit(".", 1)[1]: z[k] for k in z.files if k.rsplit(".", 1)[0] == c}
        if not {"a", "b", "h"} <= set(keys):
            continue
        a, b = torch.from_numpy(keys["a"]), torch.from_numpy(keys["b"])
        if a.dtype not in DTYPES:
            continue
        h = cpu.simple_linear_scan_forward(a, b)
        assert np.array_equal(h.numpy(), keys["h"]), c
        if {"gh", "ga", "gb"} <= set(keys):
            ga, gb = cpu.simple_linear_scan_backward(a, h, torch.from_numpy(keys["gh"]))
            assert np.array_equal(ga.numpy(), keys["ga"]) and np.array_equal(gb.numpy(), keys["gb"]), c
        checked += 1
    assert checked > 0


def test_rows_over_threads_give_the_same_bits():
    # 2^21 elements: cut into several slabs of rows (a multiple of 8 each) that run side by side.
    a, b, gh = inputs((1000, 2100), torch.float32, 5)
    assert len(cpu._slabs(1000, 2100)) > 1 or torch.get_num_threads() == 1
    h = cpu.simple_linear_scan_forward(a, b)
    want = oracle.fwd(a.numpy(), b.numpy())
    assert np.array_equal(h.numpy(), want)
    ga, gb = cpu.simple_linear_scan_backward(a, h, gh)
    wga, wgb = oracle.bwd(a.numpy(), want, gh.numpy())
    assert np.array_equal(ga.numpy(), wga) and np.array_equal(gb.numpy(), wgb)


def test_multiplication_by_the_zero_before_the_row():
    # grad_a[0] = grad_b[0] * 0.0 (src/scanscam_cpu.hpp:67-74): NaN for an infinite gradient.
    a = torch.full((9, 40), 0.5)
    h = torch.ones(9, 40)
    gh = torch.ones(9, 40)
    gh[4, 0] = float("inf")
    ga, gb = cpu.simple_linear_scan_backward(a, h, gh)
    assert torch.isinf(gb[4, 0]) and torch.isnan(ga[4, 0])
    assert torch.isfinite(ga[:4]).all() and torch.isfinite(ga[5:]).all() and torch.isfinite(ga[4, 1:]).all()


def test_empty_and_bad_arguments():
    for shape in [(0, 5), (4, 0)]:
        a = torch.zeros(shape)
        assert cpu.simple_linear_scan_forward(a, a).shape == shape
        ga, gb = cpu.simple_linear_scan_backward(a, a, a)
        assert ga.shape == shape and gb.shape == shape
    L = ctypes.CDLL(cpu.LIB_PATH)
    assert L.scanscam_cpu_fwd_f32(None, None, None, ctypes.c_int64(0), ctypes.c_int64(7)) == 0
    assert L.scanscam_cpu_fwd_f32(None, None, None, ctypes.c_int64(2), ctypes.c_int64(7)) == 1
    assert L.scanscam_cpu_bwd_f64(None, None, None, None, None, ctypes.c_int64(-1), ctypes.c_int64(7)) == 1
    with pytest.raises(RuntimeError):
        cpu.simple_linear_scan_forward(torch.zeros(2, 3, dtype=torch.bfloat16), torch.zeros(2, 3, dtype=torch.bfloat16))
    with pytest.raises(RuntimeError):
        cpu.simple_linear_scan_forward(torch.zeros(2, 3), torch.zeros(2, 3, dtype=torch.float64))
    with pytest.raises(AssertionError):
        cpu.simple_linear_scan_forward(torch.zeros(2, 3), torch.zeros(2, 4))


@pytest.mark.parametrize("permute", [False, True])
def test_op_on_cpu_tensors_takes_this_path(monkeypatch, permute):
    # The reference's own CPU test (scanscam/cpu_test.py:12-48): shape (16, 2, 5), optionally
    # permuted, the op against the tensor-level loop. The reference's Scan.backward drops the
    # CPU result (op.py:52-53); here the gradients come back.
    calls = []
    real_f, real_b = cpu.simple_linear_scan_forward, cpu.simple_linear_scan_backward
    monkeypatch.setattr(cpu, "simple_linear_scan_forward", lambda *x: calls.append("f") or real_f(*x))
    monkeypatch.setattr(cpu, "simple_linear_scan_backward", lambda *x: calls.append("b") or real_b(*x))
    a, b, gh = inputs((16, 2, 5), torch.float32, 3)
    if permute:
        a, b, gh = (t.permute(1, 0, 2) for t in (a, b, gh))
    a1, b1 = a.clone().requires_grad_(), b.clone().requires_grad_()
    h = scanscam_amd.scan(a1, b1)
    h.backward(gh)
    assert calls == ["f", "b"]
    a2, b2 = a.clone().requires_grad_(), b.clone().requires_grad_()
    from scanscam_amd.baseline import naive_linear_scan_forward

    h2 = naive_linear_scan_forward(a2, b2)
    h2.backward(gh)
    assert torch.allclose(h, h2, atol=1e-4)
    assert torch.allclose(a1.grad, a2.grad, atol=1e-4) and torch.allclose(b1.grad, b2.grad, atol=1e-4)


def test_other_cpu_dtypes_take_the_tensor_level_loop(monkeypatch):
    monkeypatch.setattr(cpu, "simple_linear_scan_forward", lambda *x: pytest.fail("16-bit tensors are not the library's"))
    a = torch.rand(3, 9).to(torch.bfloat16)
    b = torch.randn(3, 9).to(torch.bfloat16)
    assert op.scan(a, b).dtype == torch.bfloat16
