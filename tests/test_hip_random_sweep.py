"""
Seeded random sweep of the autograd op on the GPU against the CPU oracle:
shapes, storage types and memory layouts drawn at random, so that regime
borders nobody listed by hand (rows that do not fill a workgroup, lengths one
off a chunk or tile, views with odd offsets) are crossed too. Every case goes
``scanscam_amd.scan`` -> ``.backward()`` and is compared with the oracle's
forward and backward on the same (exactly upcast) values; the bars are those of
``test_hip_parity.py``. The case is printed before it runs.
"""
import numpy as np
import pytest
import torch

import oracle
import scanscam_amd

pytestmark = pytest.mark.gpu

BARS = {torch.float32: 1e-5, torch.float64: 1e-13, torch.bfloat16: 1e-2, torch.float16: 1e-2}
EDGES = [1, 2, 3, 4, 5, 7, 8, 63, 64, 65, 127, 128, 255, 256, 257, 511, 512, 513, 1023, 1024, 1025, 2047, 2048,
         4095, 4096, 4097, 4100, 8191, 8192, 8193, 16383, 16384, 16388, 32768, 65536, 65537]


def rel_err(x, ref, h=None):
    x, ref = np.asarray(x, np.float64), np.asarray(ref, np.float64)
    if x.size == 0:
        return 0.0
    den = np.maximum(np.abs(ref), 1.0)
    if h is not None:  # grad_a = grad_b * h[t-1]: |h[t-1]| joins the denominator
        den[..., 1:] = np.maximum(den[..., 1:], np.abs(np.asarray(h, np.float64))[..., :-1])
    return float(np.max(np.abs(x - ref) / den))


def host(t):
    t = t.detach().cpu()
    return (t if t.dtype == torch.float64 else t.float()).numpy()


def draw_case(rng):
    dtype = [torch.float32, torch.float32, torch.bfloat16, torch.float16, torch.float64][rng.integers(5)]
    if rng.random() < 0.6:
        T = int(EDGES[rng.integers(len(EDGES))])
    else:
        T = int(np.exp(rng.uniform(0, np.log(70000))))
    budget = 1 << 20  # elements per tensor: the oracle is a single-threaded loop
    max_rows = max(1, min(700, budget // T))
    rows = int(rng.integers(1, max_rows + 1))
    # leading dimensions: 1, 2 or 3 of them, product = rows where it factors
    lead = [rows]
    for _ in range(int(rng.integers(0, 3))):
        d = lead[-1]
        f = [k for k in (2, 3, 4, 5, 8) if d % k == 0]
        if not f:
            break
        k = f[rng.integers(len(f))]
        lead[-1:] = [k, d // k]
    layout = ["dense", "dense", "halves", "slice", "channels_last", "permuted", "cl_halves"][rng.integers(7)]
    return dtype, tuple(lead), T, layout


def make_inputs(gpu, g, dtype, lead, T, layout):
    """(gate, value, out_grad) as GPU tensors of logical shape lead + (T,) in the drawn layout."""
    shape = lead + (T,)

    def fresh(fn, shp):
        return fn(shp, generator=g, dtype=torch.float64).to(dtype).to(gpu)

    if layout == "dense" or (layout in ("channels_last", "cl_halves", "permuted") and len(lead) < 2):
        return fresh(torch.rand, shape), fresh(torch.randn, shape), fresh(torch.randn, shape)
    if layout == "halves":  # gate and value are the two halves of one projection along dim -2
        big = lead[:-1] + (2 * lead[-1], T)
        x = fresh(torch.randn, big)
        a, b = x.chunk(2, dim=-2)
        a.copy_(torch.sigmoid(a.double()).to(dtype))
        return a, b, fresh(torch.randn, shape)
    if layout == "slice":  # a window of a longer buffer, starting at an odd element
        pad = 3
        xa, xb = fresh(torch.rand, lead + (T + 2 * pad,)), fresh(torch.randn, lead + (T + 2 * pad,))
        return xa[..., pad:pad + T], xb[..., pad:pad + T], fresh(torch.randn, shape)
    if layout == "channels_last":  # stored [..., T, C], seen as [..., C, T]
        st = lead[:-1] + (T, lead[-1])
        return fresh(torch.rand, st).mT, fresh(torch.randn, st).mT, fresh(torch.randn, st).mT
    if layout == "cl_halves":  # halves of a [..., T, 2C] projection, seen as [..., C, T]
        st = lead[:-1] + (T, 2 * lead[-1])
        x = fresh(torch.randn, st)
        a, b = x.chunk(2, dim=-1)
        a.copy_(torch.sigmoid(a.double()).to(dtype))
        return a.mT, b.mT, fresh(torch.randn, lead[:-1] + (T, lead[-1])).mT
    # "permuted": the two leading dimensions exchanged in storage
    st = (lead[1], lead[0]) + lead[2:] + (T,)
    return (fresh(torch.rand, st).transpose(0, 1), fresh(torch.randn, st).transpose(0, 1),
            fresh(torch.randn, st).transpose(0, 1))


@pytest.mark.parametrize("block", range(10))
def test_random_cases(gpu, block):
    rng = np.random.default_rng(1000 + block)
    g = torch.Generator().manual_seed(2000 + block)
    for i in range(40):
        dtype, lead, T, layout = draw_case(rng)
        print(f"case block={block} i={i} dtype={dtype} lead={lead} T={T} layout={layout}", flush=True)
        a, b, gh = make_inputs(gpu, g, dtype, lead, T, layout)
        assert a.shape == lead + (T,) and b.shape == a.shape and gh.shape == a.shape
        da, db = a.detach().requires_grad_(), b.detach().requires_grad_()
        h = scanscam_amd.scan(da, db)
        assert h.shape == a.shape and h.dtype == dtype
        h.backward(gh)
        bar = BARS[dtype]
        ha, hb, hgh, hh = host(a), host(b), host(gh), host(h)
        assert rel_err(hh, oracle.fwd(ha, hb)) <= bar, "forward"
        # The backward kernel consumes the stored (rounded) h; so does the oracle here.
        wga, wgb = oracle.bwd(ha, hh, hgh)
        assert rel_err(host(db.grad), wgb) <= bar, "grad of value"
        assert rel_err(host(da.grad), wga, hh) <= bar, "grad of gate"


@pytest.mark.parametrize("block", range(4))
def test_random_element_aligned_rows(gpu, block):
    """
    Rows that start at any element: lengths that are no multiple of the vector, bases offset by a few
    elements, row strides padded by a few elements; the buffers around and between the rows hold NaN, so a
    partial vector loaded from outside its row, or stored over it, shows.
    """
    rng = np.random.default_rng(3000 + block)
    for i in range(40):
        dtype = [torch.float32, torch.bfloat16, torch.float16, torch.float64][rng.integers(4)]
        full = 16 // torch.empty(0, dtype=dtype).element_size()
        kind = rng.integers(4)  # a group of lanes per row, a few chunks, many chunks, shorter than 4 vectors
        lo, hi = [(4 * full, 64 * full + 1), (64 * full, 1280 * full), (1280 * full, 12800 * full), (1, 4 * full)][kind]
        T = int(rng.integers(lo, hi))
        rows = int(rng.integers(1, max(2, min(2000, (1 << 20) // T))))
        offset = int(rng.integers(0, 2 * full))
        stride = T + int(rng.integers(0, 3)) * int(rng.integers(0, 2 * full))
        print(f"case ragged block={block} i={i} dtype={dtype} rows={rows} T={T} offset={offset} stride={stride}", flush=True)

        def view_of(values):
            buf = torch.full((rows * stride + offset + 64,), float("nan"), dtype=dtype, device=gpu)
            v = buf[offset:offset + rows * stride].view(rows, stride)[:, :T]
            v.copy_(torch.from_numpy(values).to(dtype))
            return buf, v

        _, a = view_of(rng.random((rows, T)))
        _, b = view_of(rng.standard_normal((rows, T)))
        _, gh = view_of(rng.standard_normal((rows, T)))
        da, db = a.detach().requires_grad_(), b.detach().requires_grad_()
        h = scanscam_amd.scan(da, db)
        h.backward(gh)
        bar = BARS[dtype]
        ha, hb, hgh, hh = (np.ascontiguousarray(host(t)) for t in (a, b, gh, h))
        assert not np.isnan(hh).any()
        assert rel_err(hh, oracle.fwd(ha, hb)) <= bar, "forward"
        wga, wgb = oracle.bwd(ha, hh, hgh)
        assert rel_err(host(db.grad), wgb) <= bar, "grad of value"
        assert rel_err(host(da.grad), wga, hh) <= bar, "grad of gate"
