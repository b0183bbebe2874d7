"""
Strided views are scanned where they lie: no copy to contiguous storage first.

The reference's wrappers call ``.contiguous()`` on every argument
(scanscam/cuda.py:36-37, 60-62); the strided entry points of the C ABI take the
views themselves. Every case builds views of larger buffers (a half of a fused
projection, a slice, a broadcast gate), runs the HIP path on the views and the
CPU oracle on contiguous copies of the same values, and compares to the same
bars as the dense tests. Outputs written through strides are checked not to
touch the memory between rows.
"""
import ctypes

import numpy as np
import pytest
import torch

import oracle
import scanscam_amd
from scanscam_amd import hip

pytestmark = pytest.mark.gpu

FP32_BAR = 1e-5
FP64_BAR = 1e-13
HALF_BAR = 1e-2


def bar_for(dtype):
    return {torch.float32: FP32_BAR, torch.float64: FP64_BAR}.get(dtype, HALF_BAR)


def rel_err(x, ref, floor=None):
    x, ref = np.asarray(x, np.float64), np.asarray(ref, np.float64)
    if x.size == 0:
        return 0.0
    den = np.maximum(np.abs(ref), 1.0)
    if floor is not None:
        den = np.maximum(den, floor)
    return float(np.max(np.abs(x - ref) / den))


def prev_abs(h):
    h = np.abs(np.asarray(h, np.float64))
    out = np.zeros_like(h)
    out[..., 1:] = h[..., :-1]
    return out


def dense_np(t):
    """Contiguous numpy copy of a (possibly strided) tensor: float64 stays, everything else exactly upcast to float32."""
    t = t.detach().cpu().contiguous()
    return (t if t.dtype == torch.float64 else t.float()).numpy()


def check_forward_backward(a, b, gh, dtype=torch.float32, plan=None, layout="rows"):
    """a, b, gh: GPU views of one logical [..., T] shape. Compares forward and backward with the oracle."""
    bar = bar_for(dtype)
    an, bn, ghn = dense_np(a), dense_np(b), dense_np(gh)
    want_h = oracle.fwd(an, bn)
    got_h = hip.scan_forward(a, b, plan)
    assert got_h.shape == a.shape
    if layout == "rows":
        assert got_h.is_contiguous()
    else:
        assert got_h.mT.is_contiguous()
    assert rel_err(dense_np(got_h), want_h) <= bar
    # backward from the stored (rounded) forward output, as the autograd op does
    hs = got_h
    hsn = dense_np(hs)
    want_ga, want_gb = oracle.bwd(an, hsn, ghn)
    got_ga, got_gb = hip.scan_backward(a, hs, gh, plan)
    assert rel_err(dense_np(got_gb), want_gb) <= bar
    assert rel_err(dense_np(got_ga), want_ga, prev_abs(hsn)) <= bar
    return got_h


def randn(gpu, shape, seed, dtype=torch.float32, gate=False):
    g = torch.Generator().manual_seed(seed)
    t = torch.rand(shape, generator=g, dtype=torch.float64) if gate else torch.randn(shape, generator=g, dtype=torch.float64)
    return t.to(dtype).to(gpu)


# ---------------------------------------------------------------------------
# Row layout [..., T], unit stride along T.
# ---------------------------------------------------------------------------
@pytest.mark.parametrize("B,C,T", [(3, 5, 1000), (4, 64, 4096), (2, 7, 48), (64, 33, 64), (2, 2, 70000)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float64])
def test_halves_of_a_fused_projection(gpu, B, C, T, dtype):
    """a, b = x.chunk(2, dim=1) of x[B, 2C, T]: two levels of row strides (2CT between batches, T between channels)."""
    x = randn(gpu, (B, 2 * C, T), B + C + T, dtype)
    x[:, :C] = torch.sigmoid(x[:, :C].float()).to(dtype)
    a, b = x.chunk(2, dim=1)
    assert not a.is_contiguous() or B == 1
    gh = randn(gpu, (B, 2 * C, T), 7, dtype)[:, C:]
    print(f"case strided chunk B={B} C={C} T={T} {dtype}", flush=True)
    check_forward_backward(a, b, gh, dtype)


@pytest.mark.parametrize("Tfull,T", [(4100, 4096), (4099, 4096), (4099, 4097), (300, 17), (1031, 1024), (70001, 66000)])
def test_slices_along_time(gpu, Tfull, T):
    """x[..., s:s+T] of a longer buffer: the row stride exceeds T, rows start at any element."""
    rows = (6, 11) if Tfull < 10000 else (3,)
    for start in (0, 1, 3):
        if start + T > Tfull:
            continue
        a = randn(gpu, rows + (Tfull,), Tfull + start, gate=True)[..., start:start + T]
        b = randn(gpu, rows + (Tfull,), T + start)[..., start:start + T]
        gh = randn(gpu, rows + (T,), 5)
        print(f"case strided slice Tfull={Tfull} T={T} start={start}", flush=True)
        check_forward_backward(a, b, gh)


def test_gate_broadcast_over_the_batch(gpu):
    """A zero stride on an input: one gate row shared by every batch element is read in place."""
    B, C, T = 6, 40, 2048
    a = randn(gpu, (1, C, T), 1, gate=True).expand(B, C, T)
    assert a.stride(0) == 0
    b = randn(gpu, (B, C, T), 2)
    gh = randn(gpu, (B, C, T), 3)
    check_forward_backward(a, b, gh)
    # ... and a gate shared by all channels
    a2 = randn(gpu, (B, 1, T), 4, gate=True).expand(B, C, T)
    check_forward_backward(a2, b, gh)


def test_more_than_two_stride_levels_fall_back_to_a_copy(gpu):
    base = randn(gpu, (2, 6, 8, 260), 11, gate=True)
    a = base[:, :3, :4, :]
    assert hip._two_levels(a.shape[:-1], [a.stride()[:-1]]) is None
    b = randn(gpu, (2, 3, 4, 260), 12)
    gh = randn(gpu, (2, 3, 4, 260), 13)
    check_forward_backward(a, b, gh)


@pytest.mark.parametrize("mode", [hip.MODE_ROW, hip.MODE_LOOKBACK])
@pytest.mark.parametrize("T", [4096, 4099])
def test_forced_families_on_two_level_views(gpu, mode, T):
    x = randn(gpu, (3, 10, T), 21)
    x[:, :5] = torch.sigmoid(x[:, :5])
    a, b = x.chunk(2, dim=1)
    gh = randn(gpu, (3, 10, T), 22)[:, 5:]
    for unroll, waves in [(2, 2), (4, 4), (4, 16)]:
        plan = hip.Plan(mode=mode, unroll=unroll, waves=waves)
        print(f"case strided forced {plan} T={T}", flush=True)
        check_forward_backward(a, b, gh, plan=plan)


def test_small_family_on_views_of_any_alignment(gpu):
    for T, Tfull in [(64, 64), (64, 65), (20, 23), (5, 7), (256, 260)]:
        x = randn(gpu, (9, 14, Tfull), T)
        x[:, :7] = torch.sigmoid(x[:, :7])
        a, b = x[..., :T].chunk(2, dim=1)
        gh = randn(gpu, (9, 7, T), 3)
        print(f"case strided small T={T} Tfull={Tfull}", flush=True)
        check_forward_backward(a, b, gh)


def test_outputs_written_through_strides_leave_the_gaps_alone(gpu):
    """The raw C call with strided outputs: h goes into a slice of a larger buffer."""
    L = hip.lib()
    n0, n1, T, pitch = 3, 5, 1000, 1024
    a = randn(gpu, (n0, n1, T), 1, gate=True)
    b = randn(gpu, (n0, n1, T), 2)
    out = torch.full((n0, 2 * n1, pitch), -7.0, device=gpu)
    h = out[:, n1:, 8:8 + T]
    S = hip.Strides
    sh = S(h.stride(0), h.stride(1))
    rc = L.scanscam_scan_fwd_strided(a.data_ptr(), b.data_ptr(), h.data_ptr(), None, None, ctypes.byref(sh), n0, n1, T, 0,
                                     None, 0, torch.cuda.current_stream().cuda_stream, None)
    assert rc == 0, hip.strerror(rc)
    torch.cuda.synchronize()
    want = oracle.fwd(dense_np(a), dense_np(b))
    assert rel_err(dense_np(h), want) <= FP32_BAR
    mask = torch.ones_like(out, dtype=torch.bool)
    mask[:, n1:, 8:8 + T] = False
    assert bool((out[mask] == -7.0).all())

    # backward into strided gradient buffers
    gh = randn(gpu, (n0, n1, T), 3)
    hs = h.contiguous()
    grads = torch.full((2, n0, n1, pitch), -7.0, device=gpu)
    ga, gb = grads[0, :, :, :T], grads[1, :, :, 3:3 + T]   # gb's rows start off the 16-byte grid
    sga, sgb = S(ga.stride(0), ga.stride(1)), S(gb.stride(0), gb.stride(1))
    rc = L.scanscam_scan_bwd_strided(a.data_ptr(), hs.data_ptr(), gh.data_ptr(), ga.data_ptr(), gb.data_ptr(), None, None,
                                     None, ctypes.byref(sga), ctypes.byref(sgb), n0, n1, T, 0, None, 0,
                                     torch.cuda.current_stream().cuda_stream, None)
    assert rc == 0, hip.strerror(rc)
    torch.cuda.synchronize()
    want_ga, want_gb = oracle.bwd(dense_np(a), dense_np(hs), dense_np(gh))
    assert rel_err(dense_np(gb), want_gb) <= FP32_BAR
    assert rel_err(dense_np(ga), want_ga, prev_abs(dense_np(hs))) <= FP32_BAR
    assert bool((grads[0, :, :, T:] == -7.0).all()) and bool((grads[1, :, :, :3] == -7.0).all())
    assert bool((grads[1, :, :, 3 + T:] == -7.0).all())


# ---------------------------------------------------------------------------
# Channels-last [..., C, T] stored [..., T, C], unit stride along C.
# ---------------------------------------------------------------------------
@pytest.mark.parametrize("B,T,C", [(4, 300, 96), (2, 4096, 256), (64, 200, 512), (3, 107, 197), (1, 5000, 64)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_channels_last_halves_of_a_fused_projection(gpu, B, T, C, dtype):
    """a, b = x.chunk(2, dim=-1) of x[B, T, 2C], seen as [B, C, T]: the time stride is 2C."""
    x = randn(gpu, (B, T, 2 * C), B + T + C, dtype)
    x[..., :C] = torch.sigmoid(x[..., :C].float()).to(dtype)
    a, b = (t.mT for t in x.chunk(2, dim=-1))
    assert a.stride(-2) == 1 and a.stride(-1) == 2 * C
    gh = randn(gpu, (B, T, C), 9, dtype).mT
    print(f"case strided channels-last B={B} T={T} C={C} {dtype}", flush=True)
    check_forward_backward(a, b, gh, dtype, layout="cl")


def test_channels_last_batch_slices_and_lookback(gpu):
    x = randn(gpu, (6, 2500, 2 * 128), 31)
    x[..., :128] = torch.sigmoid(x[..., :128])
    a, b = (t.mT for t in x[::2].chunk(2, dim=-1))   # batch stride doubled as well
    gh = randn(gpu, (3, 2500, 128), 32).mT
    check_forward_backward(a, b, gh, layout="cl")
    for plan in (hip.Plan(mode=hip.MODE_LOOKBACK, unroll=4, waves=4), hip.Plan(mode=hip.MODE_ROW, vec=1, unroll=8)):
        print(f"case strided channels-last forced {plan}", flush=True)
        check_forward_backward(a, b, gh, plan=plan, layout="cl")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
def test_channels_last_views_on_the_8_byte_grid(gpu, dtype):
    """Views whose starts and strides are multiples of 8 bytes but not of 16: lanes of 8 bytes are the widest that fit."""
    half = 8 // torch.empty(0, dtype=dtype).element_size()   # channels of an 8-byte lane
    for B, T, C, forced in [(260, 40, 64 * half, None), (3, 300, 64 * half, hip.Plan(mode=hip.MODE_LOOKBACK, vec=half)),
                            (2, 70, 128 * half + half, hip.Plan(mode=hip.MODE_ROW, vec=half, unroll=8, waves=3))]:
        width = 2 * C + 3 * half   # time stride: a multiple of 8 bytes, not of 16
        x = randn(gpu, (B, T, width), B + T + C, dtype)
        x[..., half:half + C] = torch.sigmoid(x[..., half:half + C].float()).to(dtype)
        a, b = x[..., half:half + C].mT, x[..., half + C:half + 2 * C].mT   # start 8 bytes into a time step
        assert a.data_ptr() % 16 == 8 and (a.stride(-1) * x.element_size()) % 16 == 8
        gh = randn(gpu, (B, T, C), 5, dtype).mT
        print(f"case strided channels-last 8-byte grid B={B} T={T} C={C} {dtype} {forced}", flush=True)
        check_forward_backward(a, b, gh, dtype, plan=forced, layout="cl")


def test_channels_last_gradient_of_another_layout_is_converted(gpu):
    a = randn(gpu, (2, 50, 70), 41, gate=True).mT
    b = randn(gpu, (2, 50, 70), 42).mT
    gh = randn(gpu, (2, 70, 50), 43)     # row layout
    check_forward_backward(a, b, gh, layout="cl")


# ---------------------------------------------------------------------------
# Through the autograd op.
# ---------------------------------------------------------------------------
@pytest.mark.parametrize("layout", ["rows", "cl"])
def test_autograd_through_views(gpu, layout):
    B, C, T = 3, 24, 700
    g = torch.Generator().manual_seed(77)
    if layout == "rows":
        x_cpu = torch.randn((B, 2 * C, T), generator=g, dtype=torch.float64)
        split = lambda x: tuple(x.chunk(2, dim=1))
    else:
        x_cpu = torch.randn((B, T, 2 * C), generator=g, dtype=torch.float64)
        split = lambda x: tuple(t.mT for t in x.chunk(2, dim=-1))
    w_cpu = torch.randn((B, C, T), generator=g, dtype=torch.float64)

    def loss(x, w):
        a, b = split(x)
        return (scanscam_amd.scan(a, b) * w).sum()   # both operands are views of x

    x_ref = x_cpu.clone().requires_grad_(True)
    loss(x_ref, w_cpu).backward()           # CPU tensors: the tensor-level loop
    x_gpu = x_cpu.to(gpu).requires_grad_(True)
    loss(x_gpu, w_cpu.to(gpu)).backward()
    assert rel_err(x_gpu.grad.cpu().numpy(), x_ref.grad.numpy()) <= 1e-12
