"""
scanscam_amd: the first-order gated linear scan ``h[t] = gate[t] * h[t-1] + value[t]``
and its backward pass as hand-written HIP kernels for MI355X (gfx950), behind
the Python surface of unixpickle/scanscam (``scanscam/__init__.py:1-3``).

    from scanscam_amd import scan
    h = scan(gate, value)        # [N x ... x T] tensors on an AMD GPU; differentiable
"""
from . import cpu, cuda, hip  # noqa: F401  (scanscam.cpu / scanscam.cuda of the reference, and the HIP binding)
from .op import Scan, is_transpose_contig, scan

__all__ = ["scan", "Scan", "is_transpose_contig"]
