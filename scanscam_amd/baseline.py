"""
Tensor-level loop over time, for tensors that do not live on a GPU.

This is the package's counterpart of the reference's ``scanscam/baseline.py:8-40``
(the path ``scanscam/op.py:34-35, 54-55`` takes when no native kernel applies).
It is differentiable by ``torch.autograd``. GPU tensors never come here: they
go to the HIP kernels or raise.
"""
from typing import List, Tuple

import torch

from .decorator import preprocess_backward_scan_args, preprocess_scan_args


@preprocess_scan_args
def naive_linear_scan_forward(gate: torch.Tensor, value: torch.Tensor) -> torch.Tensor:
    T = gate.shape[1]
    state = torch.zeros_like(gate[:, 0])
    states: List[torch.Tensor] = []
    for t in range(T):
        state = state * gate[:, t] + value[:, t]
        states.append(state)
    if not states:
        return torch.empty_like(gate)
    return torch.stack(states, dim=1)


@preprocess_backward_scan_args
def naive_linear_scan_backward(
    gate: torch.Tensor, output: torch.Tensor, out_grad: torch.Tensor
) -> Tuple[torch.Tensor, torch.Tensor]:
    T = gate.shape[1]
    zero = torch.zeros_like(gate[:, 0])
    running = zero
    gate_grad: List[torch.Tensor] = [zero] * T
    value_grad: List[torch.Tensor] = [zero] * T
    for t in reversed(range(T)):
        running = running + out_grad[:, t]
        value_grad[t] = running
        gate_grad[t] = running * (output[:, t - 1] if t > 0 else zero)
        running = running * gate[:, t]
    if T == 0:
        return torch.empty_like(gate), torch.empty_like(gate)
    return torch.stack(gate_grad, dim=1), torch.stack(value_grad, dim=1)
