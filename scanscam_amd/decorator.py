"""
Batch-dimension flattening shared by every scan implementation.

Mirrors the contract of the reference's ``scanscam/decorator.py:12-46``: inputs
are ``[N x ... x T]`` tensors of one shape with at least two dimensions; the
wrapped function only ever sees ``[rows, T]`` and its results are given the
caller's shape again. Violations raise ``AssertionError`` like the reference's
``assert`` statements do, but are real checks (they survive ``python -O``).
"""
import functools
from typing import Callable, Tuple

import torch

ScanFn = Callable[[torch.Tensor, torch.Tensor], torch.Tensor]
ReverseScanFn = Callable[[torch.Tensor, torch.Tensor, torch.Tensor], Tuple[torch.Tensor, torch.Tensor]]


def _check_same_shape(*tensors: torch.Tensor) -> torch.Size:
    shape = tensors[0].shape
    for t in tensors[1:]:
        if t.shape != shape:
            raise AssertionError(f"scan arguments must have one shape, got {tuple(shape)} and {tuple(t.shape)}")
    if len(shape) < 2:
        raise AssertionError(f"scan arguments need at least 2 dimensions, got shape {tuple(shape)}")
    return shape


def _as_rows(t: torch.Tensor) -> torch.Tensor:
    rows = 1
    for d in t.shape[:-1]:
        rows *= d
    return t.reshape(rows, t.shape[-1])  # explicit row count: also valid when T == 0


def preprocess_scan_args(fn: ScanFn) -> ScanFn:
    """``fn(gate, value) -> out`` on ``[rows, T]``, lifted to any leading dims."""

    @functools.wraps(fn)
    def lifted(gate: torch.Tensor, value: torch.Tensor) -> torch.Tensor:
        shape = _check_same_shape(gate, value)
        return fn(_as_rows(gate), _as_rows(value)).reshape(shape)

    return lifted


def preprocess_backward_scan_args(fn: ReverseScanFn) -> ReverseScanFn:
    """``fn(gate, output, out_grad) -> (gate_grad, value_grad)`` lifted likewise."""

    @functools.wraps(fn)
    def lifted(
        gate: torch.Tensor, output: torch.Tensor, out_grad: torch.Tensor
    ) -> Tuple[torch.Tensor, torch.Tensor]:
        shape = _check_same_shape(gate, output, out_grad)
        gate_grad, value_grad = fn(_as_rows(gate), _as_rows(output), _as_rows(out_grad))
        return gate_grad.reshape(shape), value_grad.reshape(shape)

    return lifted
