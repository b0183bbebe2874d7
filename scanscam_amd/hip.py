"""
Binding of ``libscanscam_hip.so`` (C ABI in ``include/scanscam_hip.h``) and the
wrappers the autograd op calls.

Takes the place of the reference's ``scanscam/cuda.py``: ``has_hip_ops`` is its
``has_cuda_ops`` probe (``cuda.py:7-13``); ``blocked_linear_scan_forward`` /
``blocked_linear_scan_backward`` keep the names, argument order and behaviour of
``cuda.py:34-40`` and ``:56-66`` (inputs made contiguous, outputs allocated with
``torch.empty_like``, any leading dimensions flattened), and
``transposed_linear_scan_forward`` / ``transposed_linear_scan_backward`` those
of ``cuda.py:69-95`` (contiguous ``[batch, T, C]`` tensors). Storage types:
float32, float64, bfloat16, float16. PyTorch is used for device memory and the
current stream only; all arithmetic happens in the library's kernels. There is
no other implementation behind these functions: if the library is missing they
raise.
"""
import ctypes
import functools
import os
from typing import Optional, Tuple

import torch

from .decorator import preprocess_backward_scan_args, preprocess_scan_args

_HERE = os.path.dirname(os.path.abspath(__file__))
# SCANSCAM_HIP_LIB points at another build of the same ABI (tuning builds).
LIB_PATH = os.environ.get("SCANSCAM_HIP_LIB") or os.path.join(_HERE, "libscanscam_hip.so")

MODE_AUTO, MODE_SMALL, MODE_ROW, MODE_LOOKBACK, MODE_FLAT = 0, 1, 2, 3, 4
FORWARD, BACKWARD = 0, 1
ABI_VERSION = 3

_DTYPES = {torch.float32: 0, torch.bfloat16: 1, torch.float16: 2, torch.float64: 3}


class Plan(ctypes.Structure):
    """``scanscam_plan``: an explicit launch plan; zero fields are chosen automatically."""

    _fields_ = [
        ("mode", ctypes.c_int32),
        ("vec", ctypes.c_int32),
        ("unroll", ctypes.c_int32),
        ("waves", ctypes.c_int32),
        ("waves_per_row", ctypes.c_int32),
        ("spin_limit", ctypes.c_int32),
    ]

    def __repr__(self) -> str:
        return (
            f"Plan(mode={self.mode}, vec={self.vec}, unroll={self.unroll}, "
            f"waves={self.waves}, waves_per_row={self.waves_per_row})"
        )


class Strides(ctypes.Structure):
    """``scanscam_strides``: element strides of the two levels above the unit-stride dimension."""

    _fields_ = [("outer", ctypes.c_int64), ("row", ctypes.c_int64)]

    def __repr__(self) -> str:
        return f"Strides(outer={self.outer}, row={self.row})"


def _bind(path: str) -> ctypes.CDLL:
    lib = ctypes.CDLL(path)
    p, i64, i32, sz = ctypes.c_void_p, ctypes.c_int64, ctypes.c_int, ctypes.c_size_t
    plan_p = ctypes.POINTER(Plan)
    st_p = ctypes.POINTER(Strides)
    lib.scanscam_scan_fwd_strided.argtypes = [p, p, p, st_p, st_p, st_p, i64, i64, i64, i32, p, sz, p, plan_p]
    lib.scanscam_scan_fwd_strided.restype = i32
    lib.scanscam_scan_bwd_strided.argtypes = [p, p, p, p, p, st_p, st_p, st_p, st_p, st_p, i64, i64, i64, i32,
                                              p, sz, p, plan_p]
    lib.scanscam_scan_bwd_strided.restype = i32
    lib.scanscam_scan_fwd_cl_strided.argtypes = [p, p, p, st_p, st_p, st_p, i64, i64, i64, i32, p, sz, p, plan_p]
    lib.scanscam_scan_fwd_cl_strided.restype = i32
    lib.scanscam_scan_bwd_cl_strided.argtypes = [p, p, p, p, p, st_p, st_p, st_p, st_p, st_p, i64, i64, i64, i32,
                                                 p, sz, p, plan_p]
    lib.scanscam_scan_bwd_cl_strided.restype = i32
    lib.scanscam_scan_fwd.argtypes = [p, p, p, i64, i64, i32, p, sz, p]
    lib.scanscam_scan_fwd.restype = i32
    lib.scanscam_scan_bwd.argtypes = [p, p, p, p, p, i64, i64, i32, p, sz, p]
    lib.scanscam_scan_bwd.restype = i32
    lib.scanscam_scan_fwd_noalloc.argtypes = [p, p, p, i64, i64, i32, p]
    lib.scanscam_scan_fwd_noalloc.restype = i32
    lib.scanscam_workspace_bytes.argtypes = [i64, i64, i32, i32]
    lib.scanscam_workspace_bytes.restype = sz
    lib.scanscam_scan_fwd_plan.argtypes = [p, p, p, i64, i64, i32, p, sz, p, plan_p]
    lib.scanscam_scan_fwd_plan.restype = i32
    lib.scanscam_scan_bwd_plan.argtypes = [p, p, p, p, p, i64, i64, i32, p, sz, p, plan_p]
    lib.scanscam_scan_bwd_plan.restype = i32
    lib.scanscam_workspace_bytes_plan.argtypes = [i64, i64, i32, i32, plan_p]
    lib.scanscam_workspace_bytes_plan.restype = sz
    lib.scanscam_scan_fwd_timed.argtypes = [p, p, p, i64, i64, i32, p, sz, p, plan_p, p, p]
    lib.scanscam_scan_fwd_timed.restype = i32
    lib.scanscam_scan_bwd_timed.argtypes = [p, p, p, p, p, i64, i64, i32, p, sz, p, plan_p, p, p]
    lib.scanscam_scan_bwd_timed.restype = i32
    lib.scanscam_scan_fwd_cl.argtypes = [p, p, p, i64, i64, i64, i32, p, sz, p, plan_p]
    lib.scanscam_scan_fwd_cl.restype = i32
    lib.scanscam_scan_bwd_cl.argtypes = [p, p, p, p, p, i64, i64, i64, i32, p, sz, p, plan_p]
    lib.scanscam_scan_bwd_cl.restype = i32
    lib.scanscam_workspace_bytes_cl.argtypes = [i64, i64, i64, i32, i32, plan_p]
    lib.scanscam_workspace_bytes_cl.restype = sz
    lib.scanscam_workspace_timed_out.argtypes = [p, p, ctypes.POINTER(ctypes.c_int)]
    lib.scanscam_workspace_timed_out.restype = i32
    lib.scanscam_noalloc_timed_out.argtypes = [p, ctypes.POINTER(ctypes.c_int)]
    lib.scanscam_noalloc_timed_out.restype = i32
    lib.scanscam_resolve_plan.argtypes = [i64, i64, i32, i32, plan_p, plan_p]
    lib.scanscam_resolve_plan.restype = i32
    lib.scanscam_resolve_plan_cl.argtypes = [i64, i64, i64, i32, i32, plan_p, plan_p]
    lib.scanscam_resolve_plan_cl.restype = i32
    lib.scanscam_predict_cl.argtypes = [i64, i64, i64, i32, i32, plan_p, ctypes.POINTER(ctypes.c_double)]
    lib.scanscam_predict_cl.restype = i32
    lib.scanscam_strerror.argtypes = [i32]
    lib.scanscam_strerror.restype = ctypes.c_char_p
    lib.scanscam_abi_version.argtypes = []
    lib.scanscam_abi_version.restype = i32
    if lib.scanscam_abi_version() != ABI_VERSION:
        raise OSError(f"{path}: ABI version {lib.scanscam_abi_version()}, this binding needs {ABI_VERSION}")
    return lib


_lib: Optional[ctypes.CDLL] = None
_load_error: Optional[str] = None
try:
    _lib = _bind(LIB_PATH)
except (OSError, AttributeError) as exc:  # not built, or built for another ABI
    _load_error = str(exc)

has_hip_ops = _lib is not None


def lib() -> ctypes.CDLL:
    """The loaded library; raises if it is not there (there is no substitute)."""
    if _lib is None:
        raise RuntimeError(
            "scanscam_amd: the HIP library is not available "
            f"({_load_error}); build it with `make -C scanscam_amd/csrc` "
            "or `python -c 'import __graft_entry__ as g; g.build()'`"
        )
    return _lib


def strerror(code: int) -> str:
    return lib().scanscam_strerror(code).decode()


def resolve_plan(rows: int, T: int, dtype: torch.dtype, direction: int = FORWARD,
                 plan: Optional[Plan] = None) -> Plan:
    """The plan the library would run for this shape (no GPU needed)."""
    out = Plan()
    rc = lib().scanscam_resolve_plan(rows, T, _dtype_code(dtype), direction,
                                     ctypes.byref(plan) if plan is not None else None, ctypes.byref(out))
    if rc != 0:
        raise RuntimeError(f"scanscam_resolve_plan: {strerror(rc)}")
    return out


@functools.lru_cache(maxsize=4096)
def _workspace_bytes_auto(rows: int, T: int, code: int, direction: int) -> int:
    return int(lib().scanscam_workspace_bytes(rows, T, code, direction))


def workspace_bytes(rows: int, T: int, dtype: torch.dtype, direction: int = FORWARD,
                    plan: Optional[Plan] = None) -> int:
    if plan is None:
        return _workspace_bytes_auto(rows, T, _dtype_code(dtype), direction)
    return int(lib().scanscam_workspace_bytes_plan(rows, T, _dtype_code(dtype), direction, ctypes.byref(plan)))


def _dtype_code(dtype: torch.dtype) -> int:
    try:
        return _DTYPES[dtype]
    except KeyError:
        raise TypeError(f"scanscam_amd: unsupported dtype {dtype}; supported: float32, float64, bfloat16, float16") from None


def _check_rows(*tensors: torch.Tensor) -> None:
    first = tensors[0]
    for t in tensors:
        if t.device.type != "cuda":
            raise RuntimeError(f"scanscam_amd.hip: expected a GPU tensor, got one on {t.device}")
        if t.device != first.device:
            raise RuntimeError("scanscam_amd.hip: tensors are on different devices")
        if t.dtype != first.dtype:
            raise TypeError(f"scanscam_amd.hip: tensors differ in dtype ({first.dtype} and {t.dtype})")
        if t.shape != first.shape or t.dim() != 2:
            raise AssertionError("scanscam_amd.hip: expected 2-D tensors of one shape")
        if not t.is_contiguous():
            raise RuntimeError("scanscam_amd.hip: tensors must be contiguous")


# Kernels that wait for another workgroup's carry give up after a bounded number of polls and then
# write NaN (see ``scanscam_plan.spin_limit``); a correct launch never gets there. With checking on --
# ``SCANSCAM_DEBUG=1`` in the environment, or ``check_waits(True)`` -- every wrapper below that handed
# the library a workspace waits for its launch and raises if a wait expired, instead of returning NaN.
# ``SCANSCAM_SPIN_LIMIT`` / ``check_waits(..., spin_limit=n)`` set the poll limit of calls without a plan.
_check = os.environ.get("SCANSCAM_DEBUG", "") not in ("", "0")
_spin_limit = int(os.environ.get("SCANSCAM_SPIN_LIMIT", "0") or 0)


def check_waits(on: bool, spin_limit: int = 0) -> None:
    """Turn the check for expired carry waits on or off (it blocks the host after every such launch)."""
    global _check, _spin_limit
    _check, _spin_limit = bool(on), int(spin_limit)


def _raise_if_wait_expired(ws: Optional[torch.Tensor], what: str) -> None:
    if not _check or ws is None:
        return
    flag = ctypes.c_int(0)
    rc = lib().scanscam_workspace_timed_out(ws.data_ptr(), torch.cuda.current_stream().cuda_stream, ctypes.byref(flag))
    if rc != 0:
        raise RuntimeError(f"scanscam_workspace_timed_out: {strerror(rc)}")
    if flag.value:
        raise RuntimeError(f"{what}: a wait for another workgroup's carry expired; the affected outputs hold NaN")


def _workspace(rows: int, T: int, dtype: torch.dtype, direction: int, plan: Optional[Plan],
               device: torch.device) -> Tuple[Optional[torch.Tensor], int, int]:
    n = workspace_bytes(rows, T, dtype, direction, plan)
    if n == 0:
        return None, 0, 0
    ws = torch.empty(n, dtype=torch.uint8, device=device)
    return ws, ws.data_ptr(), n


def scan_forward_out(gate: torch.Tensor, value: torch.Tensor, out: torch.Tensor,
                     plan: Optional[Plan] = None) -> None:
    """``out[r, t] = gate[r, t] * out[r, t-1] + value[r, t]`` on contiguous 2-D GPU tensors.

    The raw call: what ``scanscam_ext.blocked_linear_scan(gate, value, output)``
    is in the reference (``src/scanscam_cuda.cu:260-263``). Asynchronous on the
    current stream.
    """
    L = lib()
    _check_rows(gate, value, out)
    rows, T = gate.shape
    code = _dtype_code(gate.dtype)
    if rows == 0 or T == 0:
        return
    with _on(gate.device):
        ws, ws_ptr, ws_n = _workspace(rows, T, gate.dtype, FORWARD, plan, gate.device)
        stream = torch.cuda.current_stream().cuda_stream
        rc = L.scanscam_scan_fwd_plan(gate.data_ptr(), value.data_ptr(), out.data_ptr(), rows, T, code,
                                      ws_ptr, ws_n, stream, _plan_ref(plan))
        if rc == 0:
            _raise_if_wait_expired(ws, "scanscam_scan_fwd")
    if rc != 0:
        raise RuntimeError(f"scanscam_scan_fwd: {strerror(rc)}")


def scan_backward_out(gate: torch.Tensor, output: torch.Tensor, out_grad: torch.Tensor,
                      gate_grad: torch.Tensor, value_grad: torch.Tensor,
                      plan: Optional[Plan] = None) -> None:
    """The raw backward call (``src/scanscam_cuda.cu:427-433`` in the reference)."""
    L = lib()
    _check_rows(gate, output, out_grad, gate_grad, value_grad)
    rows, T = gate.shape
    code = _dtype_code(gate.dtype)
    if rows == 0 or T == 0:
        return
    with _on(gate.device):
        ws, ws_ptr, ws_n = _workspace(rows, T, gate.dtype, BACKWARD, plan, gate.device)
        stream = torch.cuda.current_stream().cuda_stream
        rc = L.scanscam_scan_bwd_plan(gate.data_ptr(), output.data_ptr(), out_grad.data_ptr(),
                                      gate_grad.data_ptr(), value_grad.data_ptr(), rows, T, code,
                                      ws_ptr, ws_n, stream, _plan_ref(plan))
        if rc == 0:
            _raise_if_wait_expired(ws, "scanscam_scan_bwd")
    if rc != 0:
        raise RuntimeError(f"scanscam_scan_bwd: {strerror(rc)}")


class KernelEvents:
    """A pair of HIP events for ``prepare_forward`` / ``prepare_backward``: the timed entry points bind
    them to the scan kernel itself, so ``elapsed_ms()`` is the kernel's duration on the GPU without
    the launch gaps and event packets that a ``torch.cuda.Event`` pair around a launch includes.
    The events come straight from the HIP runtime (``libamdhip64``, already loaded by PyTorch).
    """

    _rt = None

    @classmethod
    def _runtime(cls):
        if cls._rt is None:
            rt = None
            # The events must come from the runtime instance the library launches with: the copy of
            # libamdhip64 that is already mapped into this process (PyTorch's), else the loader's choice.
            candidates = []
            try:
                with open("/proc/self/maps") as maps:
                    for line in maps:
                        path = line.split()[-1]
                        if "libamdhip64.so" in path and path not in candidates:
                            candidates.append(path)
            except OSError:
                pass
            candidates.append("libamdhip64.so")
            for path in candidates:
                try:
                    rt = ctypes.CDLL(path)
                    break
                except OSError:
                    continue
            if rt is None:
                raise RuntimeError("scanscam_amd.hip.KernelEvents: libamdhip64.so not found")
            rt.hipEventCreate.argtypes = [ctypes.POINTER(ctypes.c_void_p)]
            rt.hipEventDestroy.argtypes = [ctypes.c_void_p]
            rt.hipEventSynchronize.argtypes = [ctypes.c_void_p]
            rt.hipEventElapsedTime.argtypes = [ctypes.POINTER(ctypes.c_float), ctypes.c_void_p, ctypes.c_void_p]
            cls._rt = rt
        return cls._rt

    def __init__(self) -> None:
        rt = self._runtime()
        self.start, self.stop = ctypes.c_void_p(), ctypes.c_void_p()
        for ev in (self.start, self.stop):
            rc = rt.hipEventCreate(ctypes.byref(ev))
            if rc != 0:
                raise RuntimeError(f"hipEventCreate failed with HIP error {rc}")

    def elapsed_ms(self) -> float:
        """Duration of the last launch that recorded into this pair (waits for it to finish)."""
        rt = self._runtime()
        ms = ctypes.c_float()
        rc = rt.hipEventSynchronize(self.stop) or rt.hipEventElapsedTime(ctypes.byref(ms), self.start, self.stop)
        if rc != 0:
            raise RuntimeError(f"HIP event query failed with HIP error {rc}")
        return float(ms.value)

    def __del__(self) -> None:
        rt = type(self)._rt
        if rt is not None:
            for ev in (self.start, self.stop):
                if ev:
                    rt.hipEventDestroy(ev)


def prepare_forward(gate: torch.Tensor, value: torch.Tensor, out: torch.Tensor,
                    plan: Optional[Plan] = None, events: Optional["KernelEvents"] = None):
    """A zero-argument callable that launches this exact forward scan again and again.

    All checks, the workspace and the argument marshalling are done once, so a
    call costs one foreign-function call: for loops that re-run one shape on
    fixed buffers (benchmarks, a captured step). The tensors and the workspace
    are kept alive by the callable; launches go to the stream that is current
    when it is called, on the device that was current when it was prepared.
    The callable owns ONE workspace: launches of it that may overlap in time (two
    streams) race on it -- prepare one callable per stream.
    With ``events`` every launch records the scan kernel's own start and end
    on the GPU into them (``scanscam_scan_fwd_timed``).
    """
    L = lib()
    _check_rows(gate, value, out)
    rows, T = gate.shape
    code = _dtype_code(gate.dtype)
    ws, ws_ptr, ws_n = _workspace(rows, T, gate.dtype, FORWARD, plan, gate.device)
    args = (gate.data_ptr(), value.data_ptr(), out.data_ptr(), rows, T, code, ws_ptr, ws_n)
    plan_ref = ctypes.byref(plan) if plan is not None else None
    keep = (gate, value, out, ws, plan, events)
    current_stream = torch.cuda.current_stream
    if events is not None:
        fn, tail = L.scanscam_scan_fwd_timed, (plan_ref, events.start, events.stop)
    else:
        fn, tail = L.scanscam_scan_fwd_plan, (plan_ref,)

    def launch(_keep=keep) -> None:
        rc = fn(*args, current_stream().cuda_stream, *tail)
        if rc != 0:
            raise RuntimeError(f"scanscam_scan_fwd: {strerror(rc)}")

    return launch


def prepare_backward(gate: torch.Tensor, output: torch.Tensor, out_grad: torch.Tensor,
                     gate_grad: torch.Tensor, value_grad: torch.Tensor, plan: Optional[Plan] = None,
                     events: Optional["KernelEvents"] = None):
    """The backward counterpart of ``prepare_forward`` (one workspace: one stream at a time)."""
    L = lib()
    _check_rows(gate, output, out_grad, gate_grad, value_grad)
    rows, T = gate.shape
    code = _dtype_code(gate.dtype)
    ws, ws_ptr, ws_n = _workspace(rows, T, gate.dtype, BACKWARD, plan, gate.device)
    args = (gate.data_ptr(), output.data_ptr(), out_grad.data_ptr(), gate_grad.data_ptr(),
            value_grad.data_ptr(), rows, T, code, ws_ptr, ws_n)
    plan_ref = ctypes.byref(plan) if plan is not None else None
    keep = (gate, output, out_grad, gate_grad, value_grad, ws, plan, events)
    current_stream = torch.cuda.current_stream
    if events is not None:
        fn, tail = L.scanscam_scan_bwd_timed, (plan_ref, events.start, events.stop)
    else:
        fn, tail = L.scanscam_scan_bwd_plan, (plan_ref,)

    def launch(_keep=keep) -> None:
        rc = fn(*args, current_stream().cuda_stream, *tail)
        if rc != 0:
            raise RuntimeError(f"scanscam_scan_bwd: {strerror(rc)}")

    return launch


def linear_scan_forward(gate: torch.Tensor, value: torch.Tensor, plan: Optional[Plan] = None) -> torch.Tensor:
    """Forward scan of ``[N x ... x T]`` GPU tensors with an optional explicit plan."""

    @preprocess_scan_args
    def run(x: torch.Tensor, y: torch.Tensor) -> torch.Tensor:
        x = x.contiguous()
        y = y.contiguous()
        out = torch.empty_like(x)
        scan_forward_out(x, y, out, plan)
        return out

    return run(gate, value)


def linear_scan_backward(gate: torch.Tensor, output: torch.Tensor, out_grad: torch.Tensor,
                         plan: Optional[Plan] = None) -> Tuple[torch.Tensor, torch.Tensor]:
    """Backward scan with an optional explicit plan; returns ``(gate_grad, value_grad)``."""

    @preprocess_backward_scan_args
    def run(x: torch.Tensor, y: torch.Tensor, z: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
        x = x.contiguous()
        y = y.contiguous()
        z = z.contiguous()
        out_a = torch.empty_like(x)
        out_b = torch.empty_like(x)
        scan_backward_out(x, y, z, out_a, out_b, plan)
        return out_a, out_b

    return run(gate, output, out_grad)


def blocked_linear_scan_forward(x: torch.Tensor, y: torch.Tensor) -> torch.Tensor:
    """Drop-in for ``scanscam.cuda.blocked_linear_scan_forward`` (``cuda.py:34-40``)."""
    return linear_scan_forward(x, y)


def blocked_linear_scan_backward(
    x: torch.Tensor, y: torch.Tensor, z: torch.Tensor
) -> Tuple[torch.Tensor, torch.Tensor]:
    """Drop-in for ``scanscam.cuda.blocked_linear_scan_backward`` (``cuda.py:56-66``)."""
    return linear_scan_backward(x, y, z)


# The reference keeps two earlier kernels beside the blocked one (one thread per row, and its
# coalesced variant; cuda.py:16-31, 43-53) behind wrappers with the same contract. They compute the
# same function, so here the names lead to the one implementation.
simple_linear_scan_forward = blocked_linear_scan_forward
coalesced_linear_scan_forward = blocked_linear_scan_forward
simple_linear_scan_backward = blocked_linear_scan_backward
# The probe scanscam/op.py reads from its GPU wrapper module (cuda.py:7-13).
has_cuda_ops = has_hip_ops


@functools.lru_cache(maxsize=4096)
def _workspace_bytes_cl_auto(batch: int, T: int, C: int, code: int, direction: int) -> int:
    return int(lib().scanscam_workspace_bytes_cl(batch, T, C, code, direction, None))


def workspace_bytes_cl(batch: int, T: int, C: int, dtype: torch.dtype, direction: int = FORWARD,
                       plan: Optional[Plan] = None) -> int:
    if plan is None:
        return _workspace_bytes_cl_auto(batch, T, C, _dtype_code(dtype), direction)
    return int(lib().scanscam_workspace_bytes_cl(batch, T, C, _dtype_code(dtype), direction, ctypes.byref(plan)))


def resolve_plan_cl(batch: int, T: int, C: int, dtype: torch.dtype, direction: int = FORWARD,
                    plan: Optional[Plan] = None) -> Plan:
    """The plan the channels-last calls would run for dense ``[batch, T, C]`` tensors (no GPU needed)."""
    out = Plan()
    rc = lib().scanscam_resolve_plan_cl(batch, T, C, _dtype_code(dtype), direction, _plan_ref(plan), ctypes.byref(out))
    if rc != 0:
        raise RuntimeError(f"scanscam_resolve_plan_cl: {strerror(rc)}")
    return out


def predict_cl(batch: int, T: int, C: int, dtype: torch.dtype, direction: int = FORWARD,
               plan: Optional[Plan] = None) -> float:
    """Microseconds the library's cost model estimates for this channels-last call and plan (no GPU needed)."""
    us = ctypes.c_double()
    rc = lib().scanscam_predict_cl(batch, T, C, _dtype_code(dtype), direction, _plan_ref_plain(plan), ctypes.byref(us))
    if rc != 0:
        raise RuntimeError(f"scanscam_predict_cl: {strerror(rc)}")
    return float(us.value)


def _plan_ref_plain(plan: Optional[Plan]):
    return ctypes.byref(plan) if plan is not None else None


def _workspace_cl(L, batch: int, T: int, C: int, dtype: torch.dtype, direction: int, plan: Optional[Plan],
                  device: torch.device) -> Tuple[Optional[torch.Tensor], int, int]:
    n = workspace_bytes_cl(batch, T, C, dtype, direction, plan)
    if n == 0:
        return None, 0, 0
    ws = torch.empty(n, dtype=torch.uint8, device=device)
    return ws, ws.data_ptr(), n


def _check_channels_last(*tensors: torch.Tensor) -> None:
    first = tensors[0]
    for t in tensors:
        if t.shape != first.shape or t.dim() != 3:
            raise AssertionError("scanscam_amd.hip: expected 3-D [batch, T, C] tensors of one shape")
        if not t.is_contiguous():
            raise AssertionError("scanscam_amd.hip: channels-last tensors must be contiguous as [batch, T, C]")
        if t.device.type != "cuda" or t.device != first.device:
            raise RuntimeError(f"scanscam_amd.hip: expected GPU tensors on one device, got {t.device}")
        if t.dtype != first.dtype:
            raise TypeError(f"scanscam_amd.hip: tensors differ in dtype ({first.dtype} and {t.dtype})")


def transposed_linear_scan_forward(x: torch.Tensor, y: torch.Tensor, channels_per_block: int = 32,
                                   plan: Optional[Plan] = None) -> torch.Tensor:
    """Scan along T of contiguous ``[batch, T, C]`` tensors; returns ``[batch, T, C]``.

    Drop-in for ``scanscam.cuda.transposed_linear_scan_forward`` (``cuda.py:69-80``).
    ``channels_per_block`` tunes the reference's kernel and has no meaning here;
    it is accepted and ignored (``plan`` is this library's tuning hook).
    """
    L = lib()
    _check_channels_last(x, y)
    out = torch.empty_like(x)
    batch, T, C = x.shape
    if x.numel() == 0:
        return out
    plan_ref = _plan_ref(plan)
    with _on(x.device):
        ws, ws_ptr, ws_n = _workspace_cl(L, batch, T, C, x.dtype, FORWARD, plan, x.device)
        rc = L.scanscam_scan_fwd_cl(x.data_ptr(), y.data_ptr(), out.data_ptr(), batch, T, C, _dtype_code(x.dtype),
                                    ws_ptr, ws_n, torch.cuda.current_stream().cuda_stream, plan_ref)
        if rc == 0:
            _raise_if_wait_expired(ws, "scanscam_scan_fwd_cl")
    if rc != 0:
        raise RuntimeError(f"scanscam_scan_fwd_cl: {strerror(rc)}")
    return out


def transposed_linear_scan_backward(x: torch.Tensor, y: torch.Tensor, z: torch.Tensor, channels_per_block: int = 32,
                                    plan: Optional[Plan] = None) -> Tuple[torch.Tensor, torch.Tensor]:
    """``(gate_grad, value_grad)`` for contiguous ``[batch, T, C]`` gate ``x``, output ``y``, output grad ``z``.

    Drop-in for ``scanscam.cuda.transposed_linear_scan_backward`` (``cuda.py:81-95``).
    """
    L = lib()
    _check_channels_last(x, y, z)
    out_a, out_b = torch.empty_like(x), torch.empty_like(x)
    batch, T, C = x.shape
    if x.numel() == 0:
        return out_a, out_b
    plan_ref = _plan_ref(plan)
    with _on(x.device):
        ws, ws_ptr, ws_n = _workspace_cl(L, batch, T, C, x.dtype, BACKWARD, plan, x.device)
        rc = L.scanscam_scan_bwd_cl(x.data_ptr(), y.data_ptr(), z.data_ptr(), out_a.data_ptr(), out_b.data_ptr(),
                                    batch, T, C, _dtype_code(x.dtype), ws_ptr, ws_n,
                                    torch.cuda.current_stream().cuda_stream, plan_ref)
        if rc == 0:
            _raise_if_wait_expired(ws, "scanscam_scan_bwd_cl")
    if rc != 0:
        raise RuntimeError(f"scanscam_scan_bwd_cl: {strerror(rc)}")
    return out_a, out_b


def prepare_forward_cl(x: torch.Tensor, y: torch.Tensor, out: torch.Tensor, plan: Optional[Plan] = None):
    """``prepare_forward`` for contiguous ``[batch, T, C]`` tensors: a callable that launches this scan again
    (it owns one workspace: launches that may overlap on two streams need a callable each)."""
    L = lib()
    _check_channels_last(x, y, out)
    batch, T, C = x.shape
    ws, ws_ptr, ws_n = _workspace_cl(L, batch, T, C, x.dtype, FORWARD, plan, x.device)
    args = (x.data_ptr(), y.data_ptr(), out.data_ptr(), batch, T, C, _dtype_code(x.dtype), ws_ptr, ws_n)
    plan_ref = _plan_ref(plan)
    keep = (x, y, out, ws, plan)
    current_stream = torch.cuda.current_stream

    def launch(_keep=keep) -> None:
        rc = L.scanscam_scan_fwd_cl(*args, current_stream().cuda_stream, plan_ref)
        if rc != 0:
            raise RuntimeError(f"scanscam_scan_fwd_cl: {strerror(rc)}")

    return launch


def prepare_backward_cl(x: torch.Tensor, y: torch.Tensor, z: torch.Tensor, out_a: torch.Tensor, out_b: torch.Tensor,
                        plan: Optional[Plan] = None):
    """The backward counterpart of ``prepare_forward_cl`` (gate ``x``, output ``y``, output grad ``z``); one stream at a time."""
    L = lib()
    _check_channels_last(x, y, z, out_a, out_b)
    batch, T, C = x.shape
    ws, ws_ptr, ws_n = _workspace_cl(L, batch, T, C, x.dtype, BACKWARD, plan, x.device)
    args = (x.data_ptr(), y.data_ptr(), z.data_ptr(), out_a.data_ptr(), out_b.data_ptr(), batch, T, C,
            _dtype_code(x.dtype), ws_ptr, ws_n)
    plan_ref = _plan_ref(plan)
    keep = (x, y, z, out_a, out_b, ws, plan)
    current_stream = torch.cuda.current_stream

    def launch(_keep=keep) -> None:
        rc = L.scanscam_scan_bwd_cl(*args, current_stream().cuda_stream, plan_ref)
        if rc != 0:
            raise RuntimeError(f"scanscam_scan_bwd_cl: {strerror(rc)}")

    return launch


# ---------------------------------------------------------------------------
# Views without a copy. The reference's wrappers make every argument contiguous
# first (``cuda.py:36-37, 60-62``); here a view whose scan dimension (or, for
# channels-last storage, channel dimension) is unit-stride is handed to the
# kernels as it is: a half of a fused projection, a slice of a longer buffer, a
# gate broadcast over the batch.
# ---------------------------------------------------------------------------
def _joint_levels(sizes, strides_list):
    """Merge leading dimensions into as few levels as all tensors allow.

    ``sizes``: the shared sizes of the leading dimensions; ``strides_list``: their
    strides, one sequence per tensor. Two neighbouring dimensions merge when, in
    every tensor, the outer stride equals inner stride x inner size. Returns a
    list of ``(size, [stride per tensor])``, outermost first.
    """
    levels = []
    for i, n in enumerate(sizes):
        if n == 1:
            continue
        st = [s[i] for s in strides_list]
        if levels and all(p == q * n for p, q in zip(levels[-1][1], st)):
            levels[-1] = (levels[-1][0] * n, st)
        else:
            levels.append((n, st))
    return levels


def _two_levels(sizes, strides_list):
    """``(n0, n1, [Strides per tensor])`` if the leading dimensions fit two levels, else ``None``."""
    levels = _joint_levels(sizes, strides_list)
    if len(levels) > 2:
        return None
    zero = [0] * len(strides_list)
    while len(levels) < 2:
        levels.insert(0, (1, zero))
    (n0, s0), (n1, s1) = levels
    return n0, n1, [Strides(int(a), int(b)) for a, b in zip(s0, s1)]


def _is_row_view(t: torch.Tensor) -> bool:
    return t.shape[-1] == 1 or t.stride(-1) == 1


def _is_cl_view(t: torch.Tensor) -> bool:
    """``[..., C, T]`` with unit stride along C (and not along T): stored channels-last, possibly strided."""
    return t.dim() >= 2 and t.shape[-2] > 1 and t.stride(-2) == 1 and not _is_row_view(t)


def _check_same(*tensors: torch.Tensor) -> None:
    first = tensors[0]
    for t in tensors:
        if t.device.type != "cuda" or t.device != first.device:
            raise RuntimeError(f"scanscam_amd.hip: expected GPU tensors on one device, got {t.device}")
        if t.dtype != first.dtype:
            raise TypeError(f"scanscam_amd.hip: tensors differ in dtype ({first.dtype} and {t.dtype})")
        # The reference's contract for every scan (scanscam/decorator.py:19-20, 37-39).
        if t.shape != first.shape:
            raise AssertionError(
                f"scan arguments must have one shape, got {tuple(first.shape)} and {tuple(t.shape)}")
        if t.dim() < 2:
            raise AssertionError(f"scan arguments need at least 2 dimensions, got shape {tuple(t.shape)}")


def _plan_ref(plan: Optional[Plan]):
    if plan is None and _spin_limit > 0:
        plan = Plan(spin_limit=_spin_limit)
    return ctypes.byref(plan) if plan is not None else None


def _to_cl(t: torch.Tensor) -> torch.Tensor:
    """``t`` itself if it is stored channels-last, else a channels-last copy."""
    return t if _is_cl_view(t) else t.mT.contiguous().mT


class _NoSwitch:
    """Stands in for ``torch.cuda.device(...)`` when that device is already current."""

    def __enter__(self):
        return None

    def __exit__(self, *exc):
        return False


_NO_SWITCH = _NoSwitch()


def _on(device: torch.device):
    """Context that makes ``device`` current; free when it already is (the usual case)."""
    if device.index is None or device.index == torch.cuda.current_device():
        return _NO_SWITCH
    return torch.cuda.device(device)


def _run_rows(inputs, n_out: int, direction: int, plan: Optional[Plan]):
    """Row layout: ``inputs`` are views with unit stride along T; outputs are new contiguous tensors."""
    L = lib()
    first = inputs[0]
    shape = first.shape
    T = shape[-1]
    outs = [torch.empty(shape, dtype=first.dtype, device=first.device) for _ in range(n_out)]
    if first.numel() == 0:
        return outs
    tensors = list(inputs) + outs
    if all(t.is_contiguous() for t in inputs):  # the common case, kept short: one level, dense
        n0, n1, refs = 1, first.numel() // T, (None,) * len(tensors)
    else:
        lv = _two_levels(shape[:-1], [t.stride()[:-1] for t in tensors])
        if lv is None:  # more than two levels of strides: copy what is not dense
            tensors = [t.contiguous() for t in inputs] + outs
            lv = _two_levels(shape[:-1], [t.stride()[:-1] for t in tensors])
        n0, n1, st = lv
        refs = [ctypes.byref(x) for x in st]
    code = _dtype_code(first.dtype)
    with _on(first.device):
        ws, ws_ptr, ws_n = _workspace(n0 * n1, T, first.dtype, direction, plan, first.device)
        stream = torch.cuda.current_stream().cuda_stream
        ptrs = [t.data_ptr() for t in tensors]
        fn = L.scanscam_scan_fwd_strided if direction == FORWARD else L.scanscam_scan_bwd_strided
        rc = fn(*ptrs, *refs, n0, n1, T, code, ws_ptr, ws_n, stream, _plan_ref(plan))
        if rc == 0:
            _raise_if_wait_expired(ws, "scanscam_scan_fwd_strided" if direction == FORWARD else "scanscam_scan_bwd_strided")
    if rc != 0:
        raise RuntimeError(f"scanscam_scan_{'fwd' if direction == FORWARD else 'bwd'}_strided: {strerror(rc)}")
    return outs


def _cl_step_too_far(time_stride: int, C: int, esize: int) -> bool:
    """The channels-last kernels address a wave's time steps with 32-bit byte offsets from its first one (18 steps
    and the lane's channel): the library refuses time strides beyond that, and such views are copied first."""
    return time_stride * esize * 18 + C * esize >= 2 ** 32


def _run_cl(inputs, n_out: int, direction: int, plan: Optional[Plan]):
    """Channels-last: ``inputs`` are ``[..., C, T]`` views with unit stride along C; so are the outputs."""
    L = lib()
    first = inputs[0]
    shape = first.shape
    C, T = shape[-2], shape[-1]
    outs = [torch.empty(shape[:-2] + (T, C), dtype=first.dtype, device=first.device).mT for _ in range(n_out)]
    if first.numel() == 0:
        return outs
    tensors = list(inputs) + outs
    levels = _joint_levels(shape[:-2], [t.stride()[:-2] for t in tensors])
    if len(levels) > 1 or any(_cl_step_too_far(t.stride(-1), C, first.element_size()) for t in tensors):
        tensors = [t.mT.contiguous().mT for t in inputs] + outs
        levels = _joint_levels(shape[:-2], [t.stride()[:-2] for t in tensors])
    batch, sb = levels[0] if levels else (1, [0] * len(tensors))
    st = [Strides(int(b), int(t.stride(-1))) for b, t in zip(sb, tensors)]
    plan_ref = _plan_ref(plan)
    with _on(first.device):
        ws, ws_ptr, ws_n = _workspace_cl(L, batch, T, C, first.dtype, direction, plan, first.device)
        stream = torch.cuda.current_stream().cuda_stream
        ptrs = [t.data_ptr() for t in tensors]
        refs = [ctypes.byref(x) for x in st]
        fn = L.scanscam_scan_fwd_cl_strided if direction == FORWARD else L.scanscam_scan_bwd_cl_strided
        rc = fn(*ptrs, *refs, batch, T, C, _dtype_code(first.dtype), ws_ptr, ws_n, stream, plan_ref)
        if rc == 0:
            _raise_if_wait_expired(ws, "scanscam_scan_fwd_cl_strided" if direction == FORWARD else "scanscam_scan_bwd_cl_strided")
    if rc != 0:
        raise RuntimeError(f"scanscam_scan_{'fwd' if direction == FORWARD else 'bwd'}_cl_strided: {strerror(rc)}")
    return outs


def scan_forward(gate: torch.Tensor, value: torch.Tensor, plan: Optional[Plan] = None) -> torch.Tensor:
    """Forward scan along the last dimension of GPU tensors of any strides; no copy where a view will do.

    Both stored channels-last (unit stride along ``dim=-2``): the channels-last
    kernels, and the result is stored channels-last too (the rule of the
    reference's ``op.py:28-29``). Otherwise the row kernels on every tensor whose
    last dimension is unit-stride as it is (others are copied), result contiguous.
    """
    _check_same(gate, value)
    if _is_cl_view(gate) and _is_cl_view(value):
        return _run_cl([gate, value], 1, FORWARD, plan)[0]
    inputs = [t if _is_row_view(t) else t.contiguous() for t in (gate, value)]
    return _run_rows(inputs, 1, FORWARD, plan)[0]


def scan_backward(gate: torch.Tensor, output: torch.Tensor, out_grad: torch.Tensor,
                  plan: Optional[Plan] = None) -> Tuple[torch.Tensor, torch.Tensor]:
    """``(gate_grad, value_grad)`` for tensors of any strides; the counterpart of ``scan_forward``."""
    _check_same(gate, output, out_grad)
    if _is_cl_view(gate) and _is_cl_view(output):
        ga, gb = _run_cl([gate, output, _to_cl(out_grad)], 2, BACKWARD, plan)
        return ga, gb
    inputs = [t if _is_row_view(t) else t.contiguous() for t in (gate, output, out_grad)]
    ga, gb = _run_rows(inputs, 2, BACKWARD, plan)
    return ga, gb
