"""
``scanscam.cuda`` is the name of the reference's module of GPU wrappers
(``scanscam/cuda.py``; PyTorch-ROCm also calls an AMD GPU's device type "cuda").
Code written against it -- ``from scanscam import cuda`` followed by
``cuda.blocked_linear_scan_forward(x, y)`` or ``cuda.has_cuda_ops`` -- finds the
same names here; every one of them is the HIP binding in ``scanscam_amd/hip.py``.
"""
from .hip import (  # noqa: F401
    blocked_linear_scan_backward,
    blocked_linear_scan_forward,
    coalesced_linear_scan_forward,
    has_cuda_ops,
    simple_linear_scan_backward,
    simple_linear_scan_forward,
    transposed_linear_scan_backward,
    transposed_linear_scan_forward,
)
