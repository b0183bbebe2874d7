"""
Writes tests/golden/scan_golden.npz: seeded inputs and the outputs that the
REFERENCE's own CPU loops give for them.

The expected values come from oracle/_ref/scanscam_ext.so, i.e. the reference's
src/scanscam_cpu.cpp compiled unchanged by oracle/Makefile (functions
simple_linear_scan_cpu and simple_linear_scan_backward_cpu,
src/scanscam_cpu.hpp:30-52 and :80-113). Run it where the reference is mounted:

    make -C oracle ref && python tests/golden/make_golden.py

The fixture holds data only. Cases: rows x T in {3x5, 16x2x5 (N-D), 2x67, 3x1025,
1x4100} in float32 and 2x67 in float64; gates ~ N(0,1) as in the reference's
tests (scanscam/cpu_test.py:19-25) and gates ~ U(0,1).
"""
import os
import sys

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

import oracle  # noqa: E402

CASES = [
    ("f32_3x5_randn", (3, 5), np.float32, "randn"),
    ("f32_16x2x5_randn", (16, 2, 5), np.float32, "randn"),
    ("f32_2x67_randn", (2, 67), np.float32, "randn"),
    ("f32_3x1025_unit", (3, 1025), np.float32, "unit"),
    ("f32_1x4100_unit", (1, 4100), np.float32, "unit"),
    ("f64_2x67_randn", (2, 67), np.float64, "randn"),
]


def main() -> None:
    ext = oracle.ref_ext()
    if ext is None:
        raise SystemExit("oracle/_ref/scanscam_ext.so is missing: run `make -C oracle ref` first")
    rng = np.random.RandomState(20240607)
    out = {}
    for name, shape, dt, gates in CASES:
        a = rng.standard_normal(shape) if gates == "randn" else rng.uniform(0.0, 1.0, shape)
        a = a.astype(dt)
        b = rng.standard_normal(shape).astype(dt)
        gh = rng.standard_normal(shape).astype(dt)
        T = shape[-1]
        ta, tb, tgh = (torch.from_numpy(x.reshape(-1, T).copy()) for x in (a, b, gh))
        h = torch.empty_like(ta)
        ext.simple_linear_scan_cpu(ta, tb, h)
        ga, gb = torch.empty_like(ta), torch.empty_like(ta)
        ext.simple_linear_scan_backward_cpu(ta, h, tgh, ga, gb)
        out[name + ".a"], out[name + ".b"], out[name + ".gh"] = a, b, gh
        out[name + ".h"] = h.numpy().reshape(shape)
        out[name + ".ga"] = ga.numpy().reshape(shape)
        out[name + ".gb"] = gb.numpy().reshape(shape)
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "scan_golden.npz")
    np.savez_compressed(path, **out)
    print(f"wrote {path}: {len(out)} arrays, {os.path.getsize(path)} bytes")


if __name__ == "__main__":
    main()
