"""
The autograd op end to end on the GPU: scan(gate, value) and .backward(),
N-D and non-contiguous inputs, channels-last views, and the dispatch rule that
a GPU tensor is only ever scanned by the HIP kernels.
"""
import numpy as np
import pytest
import torch

import oracle
import scanscam_amd
from scanscam_amd import hip, op

pytestmark = pytest.mark.gpu


def rel_err(x, ref, h=None):
    """max |x - ref| / max(|ref|, 1); for grad_a pass h: |h[t-1]| joins the denominator."""
    x, ref = np.asarray(x, np.float64), np.asarray(ref, np.float64)
    den = np.maximum(np.abs(ref), 1.0)
    if h is not None:
        den[..., 1:] = np.maximum(den[..., 1:], np.abs(np.asarray(h, np.float64))[..., :-1])
    return float(np.max(np.abs(x - ref) / den))


@pytest.mark.parametrize("shape", [(4, 256), (3, 5, 1024), (2, 3, 4, 68), (1, 8192)])
def test_scan_forward_backward_matches_oracle(gpu, shape):
    g = torch.Generator().manual_seed(31 + len(shape))
    a = torch.rand(shape, generator=g)
    b = torch.randn(shape, generator=g)
    gh = torch.randn(shape, generator=g)
    da = a.to(gpu).requires_grad_()
    db = b.to(gpu).requires_grad_()
    h = scanscam_amd.scan(da, db)
    assert h.shape == da.shape and h.device == da.device and h.requires_grad
    h.backward(gh.to(gpu))
    want_h = oracle.fwd(a.numpy(), b.numpy())
    assert rel_err(h.detach().cpu().numpy(), want_h) <= 1e-5
    wga, wgb = oracle.bwd(a.numpy(), h.detach().cpu().numpy(), gh.numpy())
    assert rel_err(da.grad.cpu().numpy(), wga, h.detach().cpu().numpy()) <= 1e-5
    assert rel_err(db.grad.cpu().numpy(), wgb) <= 1e-5


def test_scan_gradients_match_finite_differences(gpu):
    # Directional derivative of sum(h * w) in float32 with a coarse step.
    g = torch.Generator().manual_seed(41)
    a = torch.rand((3, 40), generator=g).to(gpu).requires_grad_()
    b = torch.randn((3, 40), generator=g).to(gpu).requires_grad_()
    w = torch.randn((3, 40), generator=g).to(gpu)
    da = torch.randn((3, 40), generator=g).to(gpu)
    db = torch.randn((3, 40), generator=g).to(gpu)
    (scanscam_amd.scan(a, b) * w).sum().backward()
    analytic = float((a.grad * da).sum() + (b.grad * db).sum())
    eps = 1e-3
    with torch.no_grad():
        up = (scanscam_amd.scan(a + eps * da, b + eps * db).double() * w).sum()
        dn = (scanscam_amd.scan(a - eps * da, b - eps * db).double() * w).sum()
    numeric = float((up - dn) / (2 * eps))
    assert abs(analytic - numeric) <= 2e-2 * max(1.0, abs(numeric))


def test_channels_last_and_noncontiguous_inputs(gpu):
    g = torch.Generator().manual_seed(51)
    base_a = torch.rand((3, 200, 24), generator=g)   # stored [B, T, C]
    base_b = torch.randn((3, 200, 24), generator=g)
    a, b = base_a.mT, base_b.mT                      # logical [B, C, T]
    assert op.is_transpose_contig(a)
    da = a.to(gpu)
    da = da.mT.contiguous().mT  # keep the channels-last strides on the device
    db = b.to(gpu).mT.contiguous().mT
    assert op.is_transpose_contig(da) and op.is_transpose_contig(db)
    da.requires_grad_()
    db.requires_grad_()
    h = scanscam_amd.scan(da, db)
    want = oracle.fwd(a.contiguous().numpy(), b.contiguous().numpy())
    assert rel_err(h.detach().cpu().numpy(), want) <= 1e-5
    gh = torch.randn((3, 24, 200), generator=g)
    h.backward(gh.to(gpu))
    wga, wgb = oracle.bwd(a.contiguous().numpy(), h.detach().cpu().numpy(), gh.numpy())
    assert rel_err(da.grad.cpu().numpy(), wga, h.detach().cpu().numpy()) <= 1e-5
    assert rel_err(db.grad.cpu().numpy(), wgb) <= 1e-5


def test_wrapper_names_of_the_reference(gpu):
    a = torch.rand(4, 128, device=gpu)
    b = torch.randn(4, 128, device=gpu)
    h = hip.blocked_linear_scan_forward(a, b)
    ga, gb = hip.blocked_linear_scan_backward(a, h, b)
    assert h.shape == ga.shape == gb.shape == (4, 128)
    with pytest.raises(AssertionError):
        hip.blocked_linear_scan_forward(a, b[:, :64])
    with pytest.raises(TypeError):
        hip.blocked_linear_scan_forward(a.long(), b.long())


def test_fewer_than_two_dimensions_are_refused_as_in_the_reference(gpu):
    # scanscam/decorator.py:19-20, 37-39: every scan asserts len(shape) >= 2. The op's GPU path, which does
    # not go through the decorators, must raise the same error as the CPU paths do.
    a = torch.rand(64, device=gpu, requires_grad=True)
    b = torch.randn(64, device=gpu)
    with pytest.raises(AssertionError):
        scanscam_amd.scan(a, b)
    with pytest.raises(AssertionError):
        hip.scan_forward(a.detach(), b)
    with pytest.raises(AssertionError):
        hip.scan_backward(a.detach(), b, b)
    with pytest.raises(AssertionError):
        scanscam_amd.scan(a.detach().cpu(), b.cpu())  # same input, CPU branch
    with pytest.raises(AssertionError):
        hip.scan_forward(a.detach().reshape(1, 64), b.reshape(2, 32))
    assert scanscam_amd.scan(a.reshape(1, 64), b.reshape(1, 64)).shape == (1, 64)


def test_reference_module_and_function_names(gpu):
    # A test written for the reference (scanscam/cuda_test.py:19-126: each wrapper of scanscam.cuda
    # against the tensor-level loop, N(0,1) inputs, atol 1e-4) runs against scanscam_amd.cuda unchanged.
    from scanscam_amd import cuda
    from scanscam_amd.baseline import naive_linear_scan_backward, naive_linear_scan_forward

    assert cuda.has_cuda_ops
    g = torch.Generator().manual_seed(5)
    x, y, z = (torch.randn((16, 2, 5), generator=g).to(gpu) for _ in range(3))
    want = naive_linear_scan_forward(x, y)
    for fn in (cuda.simple_linear_scan_forward, cuda.coalesced_linear_scan_forward, cuda.blocked_linear_scan_forward):
        assert torch.allclose(fn(x, y), want, atol=1e-4)
    wa, wb = naive_linear_scan_backward(x, y, z)
    for fn in (cuda.simple_linear_scan_backward, cuda.blocked_linear_scan_backward):
        ga, gb = fn(x, y, z)
        assert torch.allclose(ga, wa, atol=1e-4) and torch.allclose(gb, wb, atol=1e-4)
    xt, yt, zt = (t.mT.contiguous() for t in (x, y, z))  # stored [B, T, C]
    assert torch.allclose(cuda.transposed_linear_scan_forward(xt, yt, 8).mT, want, atol=1e-4)
    ga, gb = cuda.transposed_linear_scan_backward(xt, yt, zt, 8)
    assert torch.allclose(ga.mT, wa, atol=1e-4) and torch.allclose(gb.mT, wb, atol=1e-4)


def test_runs_on_the_current_stream(gpu):
    s = torch.cuda.Stream(device=gpu)
    a = torch.rand(64, 4096, device=gpu)
    b = torch.randn(64, 4096, device=gpu)
    torch.cuda.synchronize()
    with torch.cuda.stream(s):
        h = scanscam_amd.scan(a, b)
        total = h.sum()
    s.synchronize()
    want = oracle.fwd(a.cpu().numpy(), b.cpu().numpy())
    assert rel_err(h.cpu().numpy(), want) <= 1e-5
    assert np.isfinite(float(total))


def test_float64_gradcheck_on_gpu(gpu):
    # The reference dispatches float and double; with double storage the op passes
    # torch.autograd.gradcheck directly on the GPU kernels.
    g = torch.Generator().manual_seed(61)
    a = torch.rand((2, 3, 37), generator=g, dtype=torch.float64).to(gpu).requires_grad_()
    b = torch.randn((2, 3, 37), generator=g, dtype=torch.float64).to(gpu).requires_grad_()
    assert torch.autograd.gradcheck(scanscam_amd.scan, (a, b), eps=1e-6, atol=1e-7)
    # ... and through the channels-last kernels.
    a2 = torch.rand((2, 37, 5), generator=g, dtype=torch.float64).to(gpu).mT.requires_grad_()
    b2 = torch.randn((2, 37, 5), generator=g, dtype=torch.float64).to(gpu).mT.requires_grad_()
    assert op.is_transpose_contig(a2)
    assert torch.autograd.gradcheck(scanscam_amd.scan, (a2, b2), eps=1e-6, atol=1e-7)


def test_hip_graph_capture_and_replay(gpu):
    # The launch sequences (workspace clear kernel + scan kernel) contain no memset and no
    # allocation by the library, so they can be captured in a HIP graph. Replays are checked
    # against the eager result several times, with other GPU work in between.
    g = torch.Generator(device=gpu).manual_seed(71)
    shapes = [(64, 4096), (3, 200000), (512, 64)]  # row, look-back and small kernels
    ins = [(torch.rand(s, generator=g, device=gpu), torch.randn(s, generator=g, device=gpu),
            torch.randn(s, generator=g, device=gpu)) for s in shapes]
    eager = []
    for a, b, gh in ins:
        h = hip.blocked_linear_scan_forward(a, b)
        eager.append((h, *hip.blocked_linear_scan_backward(a, h, gh)))
    torch.cuda.synchronize()

    side = torch.cuda.Stream(device=gpu)
    graph = torch.cuda.CUDAGraph()
    outs = []
    with torch.cuda.stream(side):
        for a, b, gh in ins:  # warm-up on the capture stream
            hip.blocked_linear_scan_forward(a, b)
        side.synchronize()
        with torch.cuda.graph(graph, stream=side):
            for a, b, gh in ins:
                h = hip.blocked_linear_scan_forward(a, b)
                outs.append((h, *hip.blocked_linear_scan_backward(a, h, gh)))
    for replay in range(4):
        for o in outs:
            for t in o:
                t.fill_(float("nan"))
        scratch = torch.randn(1 << 20, device=gpu).cumsum(0)  # unrelated eager work between replays
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for want, got in zip(eager, outs):
            for w, x in zip(want, got):
                assert torch.equal(w, x), f"replay {replay} differs from the eager result"
        del scratch


@pytest.mark.parametrize("shape", [(300, 40), (2, 3, 129, 24), (7, 5)])
def test_transposed_storage_of_any_rank_is_scanned_in_place(gpu, shape):
    # [..., C, T] tensors whose last two dimensions are transposed in memory (the reference's
    # permute=True cases, scanscam/cpu_test.py:21-22) go to the channels-last kernels without a copy.
    g = torch.Generator().manual_seed(81 + len(shape))
    a = torch.rand(shape, generator=g)
    b = torch.randn(shape, generator=g)
    gh = torch.randn(shape, generator=g)
    da = a.to(gpu).mT.contiguous().mT.requires_grad_()
    db = b.to(gpu).mT.contiguous().mT.requires_grad_()
    assert not da.is_contiguous() and da.mT.is_contiguous()
    h = scanscam_amd.scan(da, db)
    assert h.shape == da.shape and h.stride() == da.stride()
    h.backward(gh.to(gpu))
    want = oracle.fwd(a.numpy(), b.numpy())
    assert rel_err(h.detach().cpu().numpy(), want) <= 1e-5
    wga, wgb = oracle.bwd(a.numpy(), h.detach().cpu().numpy(), gh.numpy())
    assert rel_err(da.grad.cpu().numpy(), wga, h.detach().cpu().numpy()) <= 1e-5
    assert rel_err(db.grad.cpu().numpy(), wgb) <= 1e-5


def test_concurrent_launches_on_two_streams(gpu):
    # Two long-row scans (look-back kernels, each with its own workspace) in flight at once on
    # different streams must neither disturb each other nor stall: waits only ever target
    # workgroups of the same launch that already hold a ticket.
    g = torch.Generator(device=gpu).manual_seed(91)
    xs = [(torch.rand((6, 400000), generator=g, device=gpu), torch.randn((6, 400000), generator=g, device=gpu))
          for _ in range(2)]
    want = [hip.blocked_linear_scan_forward(a, b) for a, b in xs]
    torch.cuda.synchronize()
    streams = [torch.cuda.Stream(device=gpu) for _ in range(2)]
    got = [None, None]
    for rep in range(3):
        for i, (a, b) in enumerate(xs):
            with torch.cuda.stream(streams[i]):
                got[i] = hip.blocked_linear_scan_forward(a, b)
        for s in streams:
            s.synchronize()
        for w, x in zip(want, got):
            assert torch.equal(w, x)


def test_expired_wait_raises_through_the_op_when_checking_is_on(gpu):
    """With checking on (SCANSCAM_DEBUG=1 or hip.check_waits) a carry wait that gives up is an exception from
    scan(), not NaNs in its result. One poll per wait makes expiry all but certain on 4 rows of 256 tiles; every
    kernel still runs to its end. Should every tile have found its predecessors in that one poll, the result is
    simply right."""
    g = torch.Generator(device=gpu).manual_seed(8)
    a = torch.rand((4, 1 << 22), generator=g, device=gpu)
    b = torch.randn((4, 1 << 22), generator=g, device=gpu)
    good = scanscam_amd.scan(a, b)
    hip.check_waits(True, spin_limit=1)
    try:
        print("case expired wait through scan()", flush=True)
        try:
            out = scanscam_amd.scan(a, b)
            raised = False
        except RuntimeError as exc:
            raised = True
            assert "wait" in str(exc) and "expired" in str(exc)
        torch.cuda.synchronize()  # returns: no wave is left spinning
        if not raised:
            assert not bool(torch.isnan(out).any()) and torch.equal(out, good)
        # Checking on, default limit: nothing expires, nothing raises.
        hip.check_waits(True)
        assert torch.equal(scanscam_amd.scan(a, b), good)
        # A channels-last shape whose time is split over workgroups goes through the same check.
        x = torch.rand((2, 8192, 256), generator=g, device=gpu)
        y = torch.randn((2, 8192, 256), generator=g, device=gpu)
        assert hip.resolve_plan_cl(2, 8192, 256, torch.float32).mode == hip.MODE_LOOKBACK
        good_cl = scanscam_amd.scan(x.mT, y.mT)
        hip.check_waits(True, spin_limit=1)
        try:
            out = scanscam_amd.scan(x.mT, y.mT)
            assert not bool(torch.isnan(out).any()) and torch.equal(out, good_cl)
        except RuntimeError as exc:
            assert "expired" in str(exc)
        torch.cuda.synchronize()
    finally:
        hip.check_waits(False)
