"""
The user-facing op: ``scan(gate, value)`` and its ``torch.autograd.Function``.

Same surface as the reference's ``scanscam/op.py:9-55``: ``scan`` applies
``Scan``; ``Scan.forward`` saves ``(gate, output)``; ``Scan.backward`` returns
``(grad_gate, grad_value)``. Dispatch is by device and layout as in
``op.py:27-35``: GPU tensors run the HIP kernels (the channels-last ones when the
last two dimensions are transposed in memory, the row ones otherwise; strided
views are not copied first), float32 / float64 CPU tensors the native host loop
(``scanscam_amd/cpu.py``) when its library is built, everything else the
tensor-level loop. Two
defects of the reference are not reproduced: its backward for transposed
inputs calls a three-argument wrapper with four arguments (``op.py:46-48``),
and its CPU backward drops its result (``op.py:52-53``); both return the
gradient pair here.
"""
from typing import Any, Tuple

import torch

from . import cpu, hip
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


def _on_gpu(t: torch.Tensor) -> bool:
    # PyTorch-ROCm reports AMD GPUs with device type "cuda".
    return t.device.type == "cuda"


class Scan(torch.autograd.Function):
    @staticmethod
    def forward(ctx: Any, gate: torch.Tensor, value: torch.Tensor) -> torch.Tensor:
        if _on_gpu(gate):
            # Raises if the HIP library is missing: a GPU tensor is never quietly scanned any
            # other way. Tensors stored [..., T, C] are scanned in place by the channels-last
            # kernels and the result keeps that layout (op.py:28-29 of the reference); any number
            # of leading dimensions, and strided views of either layout, are taken as they are
            # where the reference's wrappers would copy them first (cuda.py:36-37).
            output = hip.scan_forward(gate, value)
        elif cpu.supports(gate) and cpu.supports(value):
            output = cpu.simple_linear_scan_forward(gate, value)
        else:
            output = naive_linear_scan_forward(gate, value)
        ctx.save_for_backward(gate, output)
        return output

    @staticmethod
    def backward(ctx: Any, output_grad: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
        gate, output = ctx.saved_tensors
        if _on_gpu(output_grad):
            # Channels-last when gate and output are: what op.py:45-49 of the reference means to
            # do (its call has one argument too many).
            return hip.scan_backward(gate, output, output_grad)
        if cpu.supports(gate) and cpu.supports(output) and cpu.supports(output_grad):
            return cpu.simple_linear_scan_backward(gate, output, output_grad)
        return naive_linear_scan_backward(gate, output, output_grad)
