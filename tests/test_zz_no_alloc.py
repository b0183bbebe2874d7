"""
scanscam_scan_fwd_noalloc: the forward scan for callers that cannot allocate device memory. Its
look-back descriptors live in a fixed array inside the library instead of a caller's workspace.
Called through the C ABI and compared, bit for bit, with scanscam_scan_fwd on the same inputs
(both run the same kernels in the same association order), on calls in a row that share the array:
a large look-back shape, then a smaller one, then shapes of the other kernel families.
This file is collected last: a failure here must not hide the other GPU tests.
"""
import numpy as np
import pytest
import torch

import oracle
from scanscam_amd import hip

pytestmark = pytest.mark.gpu

E_SCRATCH = 7
SCRATCH_BYTES = 1 << 20  # SCANSCAM_NOALLOC_SCRATCH_BYTES


def _fwd_with_workspace(a, b):
    rows, T = a.shape
    h = torch.empty_like(a)
    n = hip.workspace_bytes(rows, T, a.dtype, hip.FORWARD)
    ws = torch.empty(max(n, 8), dtype=torch.uint8, device=a.device)
    rc = hip.lib().scanscam_scan_fwd(a.data_ptr(), b.data_ptr(), h.data_ptr(), rows, T, hip._dtype_code(a.dtype),
                                     ws.data_ptr() if n else None, n, torch.cuda.current_stream().cuda_stream)
    assert rc == 0, hip.strerror(rc)
    return h, n


def _fwd_noalloc(a, b):
    rows, T = a.shape
    h = torch.full_like(a, float("nan"))
    rc = hip.lib().scanscam_scan_fwd_noalloc(a.data_ptr(), b.data_ptr(), h.data_ptr(), rows, T,
                                             hip._dtype_code(a.dtype), torch.cuda.current_stream().cuda_stream)
    assert rc == 0, hip.strerror(rc)
    return h


# (rows, T, dtype): look-back shapes first large then smaller (they share the array and the second must not
# see what the first left there), then the row and small kernels (no scratch at all), then look-back again.
CASES = [
    (64, 1 << 18, torch.float32),   # look-back, tile-major, 2048 tiles
    (3, 70000, torch.float32),      # look-back, fewer and shorter rows: a smaller part of the array
    (1024, 32768, torch.bfloat16), # look-back, row-major order, 16-bit storage
    (40, 4096, torch.float32),      # row kernel
    (1000, 64, torch.float32),      # small kernel
    (2, 1 << 20, torch.float64),    # look-back, two-word descriptors
    (5, 33333, torch.float16),      # look-back, element-aligned rows
]


def test_noalloc_matches_the_workspace_entry_point_call_after_call(gpu):
    used_scratch = 0
    for i, (rows, T, dtype) in enumerate(CASES):
        print(f"case noalloc #{i} rows={rows} T={T} dtype={dtype}", flush=True)
        g = torch.Generator().manual_seed(900 + i)
        a = (0.5 + 0.5 * torch.rand((rows, T), generator=g)).to(dtype).to(gpu)
        b = torch.randn((rows, T), generator=g).to(dtype).to(gpu)
        want, ws_bytes = _fwd_with_workspace(a, b)
        got = _fwd_noalloc(a, b)
        torch.cuda.synchronize()
        assert ws_bytes <= SCRATCH_BYTES
        used_scratch += ws_bytes > 0
        assert torch.equal(got.view(torch.uint8), want.view(torch.uint8)), f"case {i}: differs from scanscam_scan_fwd"
        if i == 1:  # and against the CPU oracle, once (fp32: 1e-5)
            ref = oracle.fwd(a.cpu().numpy(), b.cpu().numpy())
            err = np.max(np.abs(got.cpu().numpy().astype(np.float64) - ref) / np.maximum(np.abs(ref), 1.0))
            assert err <= 1e-5
    assert used_scratch >= 5  # the look-back cases really went through the array
    # The same case twice in a row, with nothing in between, on a non-default stream.
    s = torch.cuda.Stream()
    with torch.cuda.stream(s):
        rows, T, dtype = CASES[1]
        a = torch.rand((rows, T), device=gpu)
        b = torch.randn((rows, T), device=gpu)
        first = _fwd_noalloc(a, b)
        second = _fwd_noalloc(a, b)
        want, _ = _fwd_with_workspace(a, b)
    s.synchronize()
    assert torch.equal(first, want) and torch.equal(second, want)
    # No wait expired in any of these calls, says the query of the array's flag word.
    import ctypes

    flag = ctypes.c_int(-1)
    assert hip.lib().scanscam_noalloc_timed_out(s.cuda_stream, ctypes.byref(flag)) == 0 and flag.value == 0
    assert hip.lib().scanscam_noalloc_timed_out(None, None) == 1


def test_noalloc_refuses_shapes_beyond_its_array_and_launches_nothing(gpu):
    a = torch.rand((4, 1024), device=gpu)
    h = torch.full_like(a, 7.0)
    # Claimed sizes far beyond the buffers: nothing may be launched, so nothing is touched.
    rows, T = 128, 1 << 26
    assert hip.workspace_bytes(rows, T, torch.float32, hip.FORWARD) > SCRATCH_BYTES
    rc = hip.lib().scanscam_scan_fwd_noalloc(a.data_ptr(), a.data_ptr(), h.data_ptr(), rows, T, 0,
                                             torch.cuda.current_stream().cuda_stream)
    assert rc == E_SCRATCH and "scratch" in hip.strerror(rc)
    torch.cuda.synchronize()
    assert bool((h == 7.0).all())
    # The usual argument errors come back as from scanscam_scan_fwd.
    assert hip.lib().scanscam_scan_fwd_noalloc(None, a.data_ptr(), h.data_ptr(), 4, 1024, 0, None) == 1
    assert hip.lib().scanscam_scan_fwd_noalloc(a.data_ptr(), a.data_ptr(), h.data_ptr(), 4, 1024, 9, None) == 2
    assert hip.lib().scanscam_scan_fwd_noalloc(a.data_ptr(), a.data_ptr(), h.data_ptr(), 0, 1024, 0, None) == 0
