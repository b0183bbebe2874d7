"""
``scanscam``: the import name of unixpickle/scanscam, bound to ``scanscam_amd``.

Code written against the reference -- ``import scanscam``, ``from scanscam.op
import Scan``, ``from scanscam.cuda import blocked_linear_scan_forward``,
``from scanscam.baseline import naive_linear_scan_forward`` (its own tests
import this way, ``scanscam/cuda_test.py:7-16``, ``scanscam/cpu_test.py:7-8``)
-- runs unchanged: every submodule name of the reference resolves to the module
of the same name in ``scanscam_amd``. Nothing is implemented here.
"""
import sys

import scanscam_amd
from scanscam_amd import Scan, is_transpose_contig, scan  # noqa: F401

for _name in ("op", "cuda", "cpu", "baseline", "decorator", "hip"):
    _module = __import__(f"scanscam_amd.{_name}", fromlist=[_name])
    sys.modules[f"{__name__}.{_name}"] = _module
    globals()[_name] = _module
del _name, _module

__all__ = ["scan"]
