"""
Pins the CPU oracle (oracle/scan_oracle.c) before anything is compared to it.

Sources of truth, none of which is the oracle's own formula retyped:
  * golden vectors written from the reference's own compiled CPU loops
    (tests/golden/scan_golden.npz, see make_golden.py) -- bit-exact;
  * the reference's compiled extension itself, when oracle/_ref holds it, on
    fresh seeded inputs including the reference's test grid
    (scanscam/cpu_test.py:14) -- bit-exact;
  * closed forms: gate 1 -> cumsum, gate 0 -> copy, constant gate and value 1 ->
    geometric series, T = 1;
  * brute force h_t = sum_s b_s prod_{s<u<=t} a_u on tiny inputs in float64;
  * h = P * cumsum(b / P), P = cumprod(a), in float64;
  * torch.autograd through an independent tensor-level forward for the
    backward pair (the method of scanscam/baseline_test.py:7-24).
"""
import os

import numpy as np
import pytest
import torch

import oracle

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "scan_golden.npz")
GOLDEN_CASES = [
    "f32_3x5_randn",
    "f32_16x2x5_randn",
    "f32_2x67_randn",
    "f32_3x1025_unit",
    "f32_1x4100_unit",
    "f64_2x67_randn",
]
REFERENCE_GRID = [(32, 5), (16, 2, 5), (32, 64), (1, 1024), (32, 1024), (32, 1025), (1, 1025)]


@pytest.fixture(scope="module")
def golden():
    return np.load(GOLDEN)


@pytest.mark.parametrize("name", GOLDEN_CASES)
def test_forward_matches_reference_golden_bit_exact(golden, name):
    h = oracle.fwd(golden[name + ".a"], golden[name + ".b"])
    assert h.dtype == golden[name + ".h"].dtype
    assert np.array_equal(h, golden[name + ".h"])


@pytest.mark.parametrize("name", GOLDEN_CASES)
def test_backward_matches_reference_golden_bit_exact(golden, name):
    ga, gb = oracle.bwd(golden[name + ".a"], golden[name + ".h"], golden[name + ".gh"])
    assert np.array_equal(ga, golden[name + ".ga"])
    assert np.array_equal(gb, golden[name + ".gb"])


@pytest.mark.skipif(not oracle.has_ref(), reason="oracle/_ref not built (reference sources not mounted)")
@pytest.mark.parametrize("shape", REFERENCE_GRID + [(7, 4099)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
def test_matches_compiled_reference_bit_exact(shape, dtype):
    ext = oracle.ref_ext()
    g = torch.Generator().manual_seed(1000 * sum(shape) + len(shape) + (8 if dtype == torch.float64 else 4))
    a = torch.randn(shape, generator=g, dtype=dtype)
    b = torch.randn(shape, generator=g, dtype=dtype)
    gh = torch.randn(shape, generator=g, dtype=dtype)
    T = shape[-1]
    a2, b2, gh2 = (x.reshape(-1, T).contiguous() for x in (a, b, gh))
    h_ref = torch.empty_like(a2)
    ext.simple_linear_scan_cpu(a2, b2, h_ref)
    ga_ref, gb_ref = torch.empty_like(a2), torch.empty_like(a2)
    ext.simple_linear_scan_backward_cpu(a2, h_ref, gh2, ga_ref, gb_ref)

    h = oracle.fwd(a.numpy(), b.numpy())
    ga, gb = oracle.bwd(a.numpy(), h, gh.numpy())
    assert np.array_equal(h.reshape(-1, T), h_ref.numpy())
    assert np.array_equal(ga.reshape(-1, T), ga_ref.numpy())
    assert np.array_equal(gb.reshape(-1, T), gb_ref.numpy())


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_closed_forms_forward(dtype):
    rng = np.random.RandomState(1)
    b = rng.standard_normal((4, 300)).astype(dtype)
    one, zero = np.ones_like(b), np.zeros_like(b)
    # gate 1: the scan is a running sum, accumulated left to right in dtype.
    seq = np.empty_like(b)
    acc = np.zeros(4, dtype=dtype)
    for t in range(b.shape[1]):
        acc = (acc + b[:, t]).astype(dtype)
        seq[:, t] = acc
    assert np.array_equal(oracle.fwd(one, b), seq)
    assert np.allclose(oracle.fwd(one, b), np.cumsum(b.astype(np.float64), axis=1), rtol=0, atol=1e-3)
    # gate 0: the scan is the value itself; value 0: the scan is 0.
    assert np.array_equal(oracle.fwd(zero, b), b)
    assert np.array_equal(oracle.fwd(rng.uniform(size=b.shape).astype(dtype), zero), zero)
    # constant gate c, value 1: (1 - c^(t+1)) / (1 - c).
    c = 0.75
    t = np.arange(300, dtype=np.float64)
    want = (1 - c ** (t + 1)) / (1 - c)
    got = oracle.fwd(np.full((1, 300), c, dtype=dtype), np.ones((1, 300), dtype=dtype))
    assert np.allclose(got[0], want, rtol=1e-6 if dtype == np.float32 else 1e-14, atol=0)
    # T = 1.
    assert np.array_equal(oracle.fwd(one[:, :1], b[:, :1]), b[:, :1])


def test_forward_brute_force_and_cumprod_identity():
    rng = np.random.RandomState(2)
    a = rng.uniform(0.5, 1.5, (3, 12))
    b = rng.standard_normal((3, 12))
    h = oracle.fwd(a, b)
    brute = np.zeros_like(h)
    for r in range(3):
        for t in range(12):
            brute[r, t] = sum(b[r, s] * np.prod(a[r, s + 1 : t + 1]) for s in range(t + 1))
    assert np.allclose(h, brute, rtol=1e-12, atol=1e-12)
    P = np.cumprod(a, axis=1)
    assert np.allclose(h, P * np.cumsum(b / P, axis=1), rtol=1e-12, atol=1e-12)


def test_backward_brute_force():
    # gb[t] = sum_{s>=t} gh[s] prod_{t<u<=s} a[u];  ga[t] = gb[t] * h[t-1].
    rng = np.random.RandomState(3)
    a = rng.uniform(0.5, 1.5, (2, 10))
    hsaved = rng.standard_normal((2, 10))
    gh = rng.standard_normal((2, 10))
    ga, gb = oracle.bwd(a, hsaved, gh)
    for r in range(2):
        for t in range(10):
            want = sum(gh[r, s] * np.prod(a[r, t + 1 : s + 1]) for s in range(t, 10))
            assert abs(gb[r, t] - want) < 1e-12
            prev = hsaved[r, t - 1] if t > 0 else 0.0
            assert abs(ga[r, t] - want * prev) < 1e-12


def test_backward_closed_forms():
    rng = np.random.RandomState(4)
    gh = rng.standard_normal((3, 50)).astype(np.float32)
    hsaved = rng.standard_normal((3, 50)).astype(np.float32)
    ga, gb = oracle.bwd(np.zeros_like(gh), hsaved, gh)
    assert np.array_equal(gb, gh)  # gate 0: nothing flows back
    assert np.array_equal(ga[:, 0], np.zeros(3, dtype=np.float32))
    assert np.array_equal(ga[:, 1:], gh[:, 1:] * hsaved[:, :-1])
    ga, gb = oracle.bwd(np.ones_like(gh), hsaved, gh)
    rc = np.cumsum(gh[:, ::-1].astype(np.float64), axis=1)[:, ::-1]
    assert np.allclose(gb, rc, rtol=0, atol=1e-4)  # gate 1: reverse running sum


@pytest.mark.parametrize("shape", [(8, 16), (2, 3, 33)])
def test_backward_is_the_gradient_of_forward(shape):
    # Independent tensor-level forward (torch.cumsum/cumprod free): plain loop + autograd.
    g = torch.Generator().manual_seed(5)
    a = torch.randn(shape, generator=g, dtype=torch.float64, requires_grad=True)
    b = torch.randn(shape, generator=g, dtype=torch.float64, requires_grad=True)
    gh = torch.randn(shape, generator=g, dtype=torch.float64)
    state = torch.zeros(shape[:-1], dtype=torch.float64)
    hs = []
    for t in range(shape[-1]):
        state = a[..., t] * state + b[..., t]
        hs.append(state)
    h = torch.stack(hs, dim=-1)
    (h * gh).sum().backward()
    assert np.allclose(oracle.fwd(a.detach().numpy(), b.detach().numpy()), h.detach().numpy(), rtol=1e-12, atol=1e-12)
    ga, gb = oracle.bwd(a.detach().numpy(), h.detach().numpy(), gh.numpy())
    assert np.allclose(ga, a.grad.numpy(), rtol=1e-10, atol=1e-10)
    assert np.allclose(gb, b.grad.numpy(), rtol=1e-10, atol=1e-10)


def test_backward_is_forward_on_reversed_shifted_gates():
    # gb = flip(fwd(flip(shift_left(a), a[T] := 0), flip(gh))): ties the two oracles together.
    rng = np.random.RandomState(6)
    a = rng.uniform(0, 1, (5, 40))
    gh = rng.standard_normal((5, 40))
    hsaved = rng.standard_normal((5, 40))
    shifted = np.concatenate([a[:, 1:], np.zeros((5, 1))], axis=1)
    want_gb = oracle.fwd(shifted[:, ::-1].copy(), gh[:, ::-1].copy())[:, ::-1]
    ga, gb = oracle.bwd(a, hsaved, gh)
    assert np.allclose(gb, want_gb, rtol=1e-13, atol=1e-13)
    prev = np.concatenate([np.zeros((5, 1)), hsaved[:, :-1]], axis=1)
    assert np.allclose(ga, want_gb * prev, rtol=1e-13, atol=1e-13)


def test_acc64_variants_agree_with_f64_on_upcast_inputs():
    rng = np.random.RandomState(7)
    a = rng.uniform(0, 1, (3, 200)).astype(np.float32)
    b = rng.standard_normal((3, 200)).astype(np.float32)
    gh = rng.standard_normal((3, 200)).astype(np.float32)
    h64 = oracle.fwd(a.astype(np.float64), b.astype(np.float64))
    assert np.array_equal(oracle.fwd_acc64(a, b), h64)
    h32 = oracle.fwd(a, b)
    ga64, gb64 = oracle.bwd(a.astype(np.float64), h32.astype(np.float64), gh.astype(np.float64))
    ga, gb = oracle.bwd_acc64(a, h32, gh)
    assert np.array_equal(ga, ga64) and np.array_equal(gb, gb64)


def test_empty_and_nd_shapes():
    assert oracle.fwd(np.zeros((0, 5), np.float32), np.zeros((0, 5), np.float32)).shape == (0, 5)
    assert oracle.fwd(np.zeros((3, 0), np.float32), np.zeros((3, 0), np.float32)).shape == (3, 0)
    rng = np.random.RandomState(8)
    a = rng.uniform(size=(2, 3, 4, 9)).astype(np.float32)
    b = rng.standard_normal((2, 3, 4, 9)).astype(np.float32)
    assert np.array_equal(oracle.fwd(a, b).reshape(-1, 9), oracle.fwd(a.reshape(-1, 9), b.reshape(-1, 9)))
    with pytest.raises(ValueError):
        oracle.fwd(np.zeros(5, np.float32), np.zeros(5, np.float32))
