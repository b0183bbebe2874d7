"""
The user-facing op: ``scan(gate, value)`` and its ``torch.autograd.Function``.

Same surface as the reference's ``scanscam/op.py:9-55``: ``scan`` applies
``Scan``; ``Scan.forward`` saves ``(gate, output)``; ``Scan.backward`` returns
``(grad_gate, grad_value)``. Dispatch is by device and layout as in
``op.py:27-35``: GPU tensors run the HIP kernels (the channels-last ones when the
last two dimensions are transposed in memory, the row ones otherwise),
everything else the tensor-level loop. Two
defects of the reference are not reproduced: its backward for transposed
inputs calls a three-argument wrapper with four arguments (``op.py:46-48``),
and its CPU backward drops its result (``op.py:52-53``); both return the
gradient pair here.
"""
from typing import Any, Tuple

import torch

from . import hip
from .baseline import naive_linear_scan_backward, naive_linear_scan_forward


def is_transpose_contig(x: torch.Tensor) -> bool:
    """A 3-D tensor stored channels-last: ``x`` is not contiguous but ``x.mT`` is (``op.py:9-10``)."""
    return x.dim() == 3 and not x.is_contiguous() and x.mT.is_contiguous()


def scan(gate: torch.Tensor, value: torch.Tensor) -> torch.Tensor:
    """
    Apply a first-order scan ``h[..., t] = gate[..., t] * h[..., t-1] + value[..., t]``
    with ``h[..., -1] = 0``.

    :param gate: [N x ... x T] tensor of gates
    :param value: [N x ... x T] tensor of values
    :return: an [N x ... x T] tensor of accumulated values.
    """
    return Scan.apply(gate, value)


def _is_channels_last(x: torch.Tensor) -> bool:
    """``[..., C, T]`` stored ``[..., T, C]``: the last two dimensions are transposed in memory.

    ``is_transpose_contig`` (3-D only, as in the reference) is the common case; the
    channels-last kernels take any number of leading dimensions, flattened to one
    batch dimension, so 2-D and N-D tensors of this layout are scanned in place too
    instead of being copied to row-contiguous storage first.
    """
    return x.dim() >= 2 and not x.is_contiguous() and x.mT.is_contiguous()


def _as_batch_t_c(x: torch.Tensor) -> torch.Tensor:
    """The ``[batch, T, C]`` contiguous view of a channels-last ``[..., C, T]`` tensor."""
    xt = x.mT
    return xt.reshape(-1, xt.shape[-2], xt.shape[-1])


def _on_gpu(t: torch.Tensor) -> bool:
    # PyTorch-ROCm reports AMD GPUs with device type "cuda".
    return t.device.type == "cuda"


class Scan(torch.autograd.Function):
    @staticmethod
    def forward(ctx: Any, gate: torch.Tensor, value: torch.Tensor) -> torch.Tensor:
        if _on_gpu(gate):
            # Raises if the HIP library is missing: a GPU tensor is never
            # quietly scanned any other way.
            if gate.shape == value.shape and _is_channels_last(gate) and _is_channels_last(value):
                # Stored [..., T, C]: scanned in place by the channels-last kernels
                # (op.py:28-29 of the reference); the result keeps that layout.
                out = hip.transposed_linear_scan_forward(_as_batch_t_c(gate), _as_batch_t_c(value))
                output = out.reshape(gate.mT.shape).mT
            else:
                output = hip.blocked_linear_scan_forward(gate, value)
        else:
            output = naive_linear_scan_forward(gate, value)
        ctx.save_for_backward(gate, output)
        return output

    @staticmethod
    def backward(ctx: Any, output_grad: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
        gate, output = ctx.saved_tensors
        if _on_gpu(output_grad):
            if _is_channels_last(gate) and _is_channels_last(output):
                # What op.py:45-49 of the reference means to do (its call has one argument too many).
                grads = hip.transposed_linear_scan_backward(
                    _as_batch_t_c(gate), _as_batch_t_c(output), _as_batch_t_c(output_grad.mT.contiguous().mT))
                return tuple(g.reshape(gate.mT.shape).mT for g in grads)
            return hip.blocked_linear_scan_backward(gate, output, output_grad)
        return naive_linear_scan_backward(gate, output, output_grad)
