"""
Binding of ``libscanscam_cpu.so`` (C ABI in ``include/scanscam_cpu.h``): the
scan for tensors that live in host memory.

Takes the place of the reference's ``scanscam/cpu.py``: ``has_cpu_ops`` is its
probe (``cpu.py:7-13``); ``simple_linear_scan_forward`` /
``simple_linear_scan_backward`` keep the names, argument order and behaviour of
``cpu.py:16-35`` (inputs made contiguous, outputs allocated with
``torch.empty_like``, any leading dimensions flattened, float32 and float64 as
in ``src/scanscam_cpu.hpp:43``). Results are bit-identical to the reference's
loop; rows are independent, so large inputs are cut into slabs of rows that run
on a few threads (the foreign call releases the interpreter lock).

Only CPU tensors come here. GPU tensors are scanned by ``scanscam_amd.hip`` or
raise; nothing in that module calls this one.
"""
import ctypes
import os
from concurrent.futures import ThreadPoolExecutor
from typing import Optional, Tuple

import torch

from .decorator import preprocess_backward_scan_args, preprocess_scan_args

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.environ.get("SCANSCAM_CPU_LIB") or os.path.join(_HERE, "libscanscam_cpu.so")

# Rows per slab are a multiple of the rows the library advances together; slabs below this many
# elements are not worth a thread.
_ROWS_TOGETHER = 8
_MIN_SLAB_ELEMENTS = 1 << 18
_SUFFIX = {torch.float32: "f32", torch.float64: "f64"}


def _bind(path: str) -> ctypes.CDLL:
    lib = ctypes.CDLL(path)
    p, i64 = ctypes.c_void_p, ctypes.c_int64
    for suffix in _SUFFIX.values():
        fwd = getattr(lib, f"scanscam_cpu_fwd_{suffix}")
        fwd.argtypes = [p, p, p, i64, i64]
        fwd.restype = ctypes.c_int
        bwd = getattr(lib, f"scanscam_cpu_bwd_{suffix}")
        bwd.argtypes = [p, p, p, p, p, i64, i64]
        bwd.restype = ctypes.c_int
    return lib


try:
    _lib: Optional[ctypes.CDLL] = _bind(LIB_PATH)
    has_cpu_ops = True
except (OSError, AttributeError):
    _lib = None
    has_cpu_ops = False

_pool: Optional[ThreadPoolExecutor] = None


def supports(t: torch.Tensor) -> bool:
    """Whether the library scans this tensor: a float32 or float64 tensor in host memory."""
    return has_cpu_ops and t.device.type == "cpu" and t.dtype in _SUFFIX


def _slabs(rows: int, T: int):
    """Row ranges [r0, r1) that run side by side."""
    threads = min(torch.get_num_threads(), os.cpu_count() or 1)
    want = min(threads, max(1, (rows * T) // _MIN_SLAB_ELEMENTS))
    per = -(-rows // want)
    per = -(-per // _ROWS_TOGETHER) * _ROWS_TOGETHER
    return [(r0, min(rows, r0 + per)) for r0 in range(0, rows, per)]


def _run(fn, tensors, rows: int, T: int) -> None:
    esize = tensors[0].element_size()
    ptrs = [t.data_ptr() for t in tensors]

    def call(r0: int, r1: int) -> int:
        off = r0 * T * esize
        return fn(*[q + off for q in ptrs], r1 - r0, T)

    slabs = _slabs(rows, T) if rows * T else []
    if len(slabs) <= 1:
        codes = [call(0, rows)]
    else:
        global _pool
        if _pool is None:
            _pool = ThreadPoolExecutor(max_workers=os.cpu_count() or 1, thread_name_prefix="scanscam_cpu")
        codes = list(_pool.map(lambda s: call(*s), slabs))
    if any(codes):
        raise RuntimeError("libscanscam_cpu: invalid argument")


def _check(*tensors: torch.Tensor) -> None:
    if _lib is None:
        raise RuntimeError(f"{LIB_PATH} is missing: build it with `make -C scanscam_amd/csrc`")
    first = tensors[0]
    if first.dtype not in _SUFFIX:
        raise RuntimeError(f"the CPU scan takes float32 or float64 tensors, got {first.dtype}")
    for t in tensors:
        if t.device.type != "cpu":
            raise RuntimeError("the CPU scan takes tensors in host memory")
        if t.dtype != first.dtype or t.shape != first.shape:
            raise RuntimeError("the CPU scan takes tensors of one dtype and shape")


@preprocess_scan_args
def simple_linear_scan_forward(x: torch.Tensor, y: torch.Tensor) -> torch.Tensor:
    """``out[r, t] = x[r, t] * out[r, t-1] + y[r, t]`` (``cpu.py:16-22`` of the reference)."""
    _check(x, y)
    x = x.contiguous()
    y = y.contiguous()
    out = torch.empty_like(x)
    rows, T = x.shape
    _run(getattr(_lib, f"scanscam_cpu_fwd_{_SUFFIX[x.dtype]}"), (x, y, out), rows, T)
    return out


@preprocess_backward_scan_args
def simple_linear_scan_backward(
    x: torch.Tensor, y: torch.Tensor, z: torch.Tensor
) -> Tuple[torch.Tensor, torch.Tensor]:
    """Gradients of gate ``x`` and value given output ``y`` and its gradient ``z`` (``cpu.py:25-35``)."""
    _check(x, y, z)
    x = x.contiguous()
    y = y.contiguous()
    z = z.contiguous()
    out_a = torch.empty_like(x)
    out_b = torch.empty_like(x)
    rows, T = x.shape
    _run(getattr(_lib, f"scanscam_cpu_bwd_{_SUFFIX[x.dtype]}"), (x, y, z, out_a, out_b), rows, T)
    return out_a, out_b
