"""
CPU oracle for the gated linear scan -- TEST INFRASTRUCTURE, not product code.

Only ``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of
``bench.py`` may import this package. Nothing under ``scanscam_amd/`` does.

Two checkers live here:

* ``fwd`` / ``bwd`` -- ``oracle/scan_oracle.c``, a plain C restatement of the
  reference's single-threaded loops (``src/scanscam_cpu.hpp:9-28`` forward,
  ``:54-78`` backward), loaded through ctypes and fed numpy arrays.
* ``ref_ext()`` -- the reference's own ``src/scanscam_cpu.cpp`` compiled as is
  into ``oracle/_ref/scanscam_ext.so`` by ``oracle/Makefile`` (present only if
  it was built where the reference sources are mounted).

Arrays are C-contiguous ``[rows, T]`` (any leading dims are flattened, as
``scanscam/decorator.py:18-23`` does); outputs are freshly allocated.
"""
import ctypes
import importlib.util
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libscan_oracle.so")
_REF_PATH = os.path.join(_HERE, "_ref", "scanscam_ext.so")

_lib = None
_ref = None


def build(with_ref: bool = True) -> None:
    """Compile the C restatement (and ``_ref`` when the reference is mounted)."""
    target = "all" if with_ref else "oracle"
    subprocess.run(["make", "-C", _HERE, "-B", target], check=True)


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build(with_ref=False)
        L = ctypes.CDLL(_LIB_PATH)
        p, i64 = ctypes.c_void_p, ctypes.c_int64
        for name in ("oracle_fwd_f32", "oracle_fwd_f64", "oracle_fwd_f32_acc64"):
            getattr(L, name).argtypes = [p, p, p, i64, i64]
            getattr(L, name).restype = None
        for name in ("oracle_bwd_f32", "oracle_bwd_f64", "oracle_bwd_f32_acc64"):
            getattr(L, name).argtypes = [p, p, p, p, p, i64, i64]
            getattr(L, name).restype = None
        _lib = L
    return _lib


def _prep(x, dtype):
    x = np.ascontiguousarray(x, dtype=dtype)
    if x.ndim < 2:
        raise ValueError("scan inputs need at least two dimensions")
    return x


def _rows_len(x):
    T = x.shape[-1]
    rows = x.size // T if T else 0
    return rows, T


def _ptr(x):
    return ctypes.c_void_p(x.ctypes.data)


def fwd(gate, value):
    """h[..., t] = gate[..., t] * h[..., t-1] + value[..., t], h[..., -1] = 0.

    float32 or float64 numpy arrays of equal shape; returns the same dtype.
    """
    gate = np.asarray(gate)
    dt = np.float64 if gate.dtype == np.float64 else np.float32
    gate, value = _prep(gate, dt), _prep(value, dt)
    if gate.shape != value.shape:
        raise ValueError("gate and value shapes differ")
    out = np.empty_like(gate)
    rows, T = _rows_len(gate)
    fn = lib().oracle_fwd_f64 if dt == np.float64 else lib().oracle_fwd_f32
    fn(_ptr(gate), _ptr(value), _ptr(out), rows, T)
    return out


def bwd(gate, output, out_grad):
    """Returns (gate_grad, value_grad) exactly as the reference CPU loop does."""
    gate = np.asarray(gate)
    dt = np.float64 if gate.dtype == np.float64 else np.float32
    gate, output, out_grad = _prep(gate, dt), _prep(output, dt), _prep(out_grad, dt)
    if not (gate.shape == output.shape == out_grad.shape):
        raise ValueError("gate, output and out_grad shapes differ")
    ga, gb = np.empty_like(gate), np.empty_like(gate)
    rows, T = _rows_len(gate)
    fn = lib().oracle_bwd_f64 if dt == np.float64 else lib().oracle_bwd_f32
    fn(_ptr(gate), _ptr(output), _ptr(out_grad), _ptr(ga), _ptr(gb), rows, T)
    return ga, gb


def fwd_acc64(gate, value):
    """float32 inputs, recurrence carried in float64, float64 output."""
    gate, value = _prep(gate, np.float32), _prep(value, np.float32)
    out = np.empty(gate.shape, dtype=np.float64)
    rows, T = _rows_len(gate)
    lib().oracle_fwd_f32_acc64(_ptr(gate), _ptr(value), _ptr(out), rows, T)
    return out


def bwd_acc64(gate, output, out_grad):
    gate, output, out_grad = (_prep(x, np.float32) for x in (gate, output, out_grad))
    ga = np.empty(gate.shape, dtype=np.float64)
    gb = np.empty(gate.shape, dtype=np.float64)
    rows, T = _rows_len(gate)
    lib().oracle_bwd_f32_acc64(_ptr(gate), _ptr(output), _ptr(out_grad), _ptr(ga), _ptr(gb), rows, T)
    return ga, gb


def has_ref() -> bool:
    return os.path.exists(_REF_PATH)


def ref_ext():
    """The reference's own compiled CPU extension (``None`` if it was not built).

    Exposes ``simple_linear_scan_cpu(gate, value, out)`` and
    ``simple_linear_scan_backward_cpu(gate, output, out_grad, gate_grad, value_grad)``
    on contiguous 2-D CPU torch tensors (``src/scanscam_cpu.cpp:3-8``).
    """
    global _ref
    if _ref is None and has_ref():
        import torch  # noqa: F401  (the extension links against libtorch)

        spec = importlib.util.spec_from_file_location("scanscam_ext", _REF_PATH)
        mod = importlib.util.module_from_spec(spec)
        spec.loader.exec_module(mod)
        _ref = mod
    return _ref
