"""Seeded random channel-first problems through the tile kernels and, for the same tensors, the
walking kernels (`fwd_cf_vecs` / `bwd_cf_parts` = -1): out, final_states, dx and dinitial_states
must agree bit for bit, dweight / dbias within their tolerance, and a sample of the cases is held
against the oracle.  Drawn together: dtype, width, batch, dim, a row length anywhere between 65
vectors and a dozen steps, rows as slices of wider and longer buffers (row and batch strides that
are no multiples of a vector), every tensor starting its own number of elements into its
allocation (x, dout, dx and out on different 16-byte grids), the (dim, batch, seqlen) order of
memory, states on and off, SiLU on and off."""
import ctypes

import pytest
import torch

import cabi
from helpers import DTYPES, TOL_W, assert_close, gen, make_wb
from oracle import causal_conv1d_oracle as orc

pytestmark = pytest.mark.gpu


def _draw(g, lo, hi):
    return int(torch.randint(lo, hi + 1, (1,), generator=g))


def _place(t, dev, g, batch_inner):
    """t's values on the GPU in a buffer of its own: a random start, rows a random number of
    elements apart (or the batch entries of a channel next to each other)."""
    B, D, L = t.shape
    shift, pad = _draw(g, 0, 9), _draw(g, 0, 11)
    row = L + pad
    if batch_inner:
        buf = torch.zeros(shift + D * B * row + 16, dtype=t.dtype, device=dev)
        view = buf[shift:shift + D * B * row].view(D, B, row)[:, :, :L].permute(1, 0, 2)
    else:
        buf = torch.zeros(shift + B * D * row + 16, dtype=t.dtype, device=dev)
        view = buf[shift:shift + B * D * row].view(B, D, row)[:, :, :L]
    view.copy_(t.to(dev))
    return view


def _case(seed):
    g = gen(seed)
    dtype = DTYPES[_draw(g, 0, 2)]
    vec = 16 // torch.empty(0, dtype=dtype).element_size()
    W = _draw(g, 2, 4)
    B, D = _draw(g, 1, 4), _draw(g, 1, 24)
    L = _draw(g, 64 * vec + 1, 64 * vec * (3 if _draw(g, 0, 3) else 12))
    return g, dtype, W, B, D, L


@pytest.mark.parametrize("block", range(8))
def test_forward_random(gpu_device, cc1d_lib, block):
    lib = cabi.declare(cc1d_lib)
    dev = gpu_device
    for n in range(50):
        seed = 30000 + block * 50 + n
        g, dtype, W, B, D, L = _case(seed)
        silu, states, bi = bool(_draw(g, 0, 1)), bool(_draw(g, 0, 1)), _draw(g, 0, 3) == 0
        x = torch.randn(B, D, L, generator=g).to(dtype)
        w, b = make_wb(D, W, bool(_draw(g, 0, 1)), g)
        init = torch.randn(B, W - 1, D, generator=g).to(dtype).transpose(1, 2) if states else None
        xd = _place(x, dev, g, bi)
        wd, bd = w.to(dev), None if b is None else b.to(dev)
        idev = None if init is None else init.to(dev)
        got = []
        try:
            for knob in (0, -1):
                assert lib.cc1d_set_tunable(b"fwd_cf_vecs", knob) == 0
                g2 = gen(seed)                          # the same placement for both kernels
                out = _place(torch.zeros_like(x), dev, g2, bi)
                fin = torch.empty(B, W - 1, D, dtype=dtype, device=dev).transpose(1, 2) if states else None
                p = cabi.fwd_params(xd, wd, bd, out, silu, initial_states=idev, final_states=fin)
                assert lib.cc1d_fwd(ctypes.byref(p), None) == 0
                torch.cuda.synchronize()
                got.append((out.cpu(), None if fin is None else fin.cpu()))
        finally:
            lib.cc1d_set_tunable(b"fwd_cf_vecs", 0)
        what = "seed %d %s W%d (%d, %d, %d) silu%d states%d bi%d" % (seed, str(dtype)[6:], W, B, D, L, silu, states, bi)
        assert torch.equal(got[0][0], got[1][0]), "out differs between the kernels, " + what
        if states:
            assert torch.equal(got[0][1], got[1][1]), "final_states differ, " + what
        if n % 5 == 0:
            ref = orc.fwd(x, w, b, initial_states=init, return_final_states=states, activation="silu" if silu else None)
            ref, ref_fin = ref if states else (ref, None)
            assert_close(got[0][0], ref, dtype, "out, " + what)
            if states:
                assert torch.equal(got[0][1], ref_fin), what


@pytest.mark.parametrize("block", range(8))
def test_backward_random(gpu_device, cc1d_lib, block):
    lib = cabi.declare(cc1d_lib)
    dev = gpu_device
    for n in range(50):
        seed = 40000 + block * 50 + n
        g, dtype, W, B, D, L = _case(seed)
        silu, states, bi = bool(_draw(g, 0, 1)), bool(_draw(g, 0, 1)), _draw(g, 0, 3) == 0
        x = torch.randn(B, D, L, generator=g).to(dtype)
        dout = torch.randn(B, D, L, generator=g).to(dtype)
        w, b = make_wb(D, W, bool(_draw(g, 0, 1)), g)
        init = torch.randn(B, W - 1, D, generator=g).to(dtype).transpose(1, 2) if states else None
        dfin = torch.randn(B, W - 1, D, generator=g).to(dtype).transpose(1, 2) if states else None
        xd, dd = _place(x, dev, g, bi), _place(dout, dev, g, bi)
        wd, bd = w.to(dev), None if b is None else b.to(dev)
        idev, fdev = (None, None) if init is None else (init.to(dev), dfin.to(dev))
        got = []
        try:
            for knob in (0, -1):
                assert lib.cc1d_set_tunable(b"bwd_cf_parts", knob) == 0
                g2 = gen(seed)
                dx = _place(torch.zeros_like(x), dev, g2, bi)
                dw = torch.empty(D, W, device=dev)
                db = None if b is None else torch.empty(D, device=dev)
                dinit = torch.empty(B, W - 1, D, dtype=dtype, device=dev).transpose(1, 2) if states else None
                p = cabi.bwd_params(xd, wd, bd, dd, dx, dw, db, silu, initial_states=idev, dfinal_states=fdev,
                                    dinitial_states=dinit)
                p.overwrite_dweight = 1
                need = ctypes.c_size_t()
                assert lib.cc1d_bwd_workspace_bytes(ctypes.byref(p), ctypes.byref(need)) == 0
                ws = torch.empty(max(16, need.value), dtype=torch.uint8, device=dev)
                assert lib.cc1d_bwd(ctypes.byref(p), ctypes.c_void_p(ws.data_ptr()), need, None) == 0
                torch.cuda.synchronize()
                got.append((dx.cpu(), dw.cpu(), None if db is None else db.cpu(), None if dinit is None else dinit.cpu()))
        finally:
            lib.cc1d_set_tunable(b"bwd_cf_parts", 0)
        what = "seed %d %s W%d (%d, %d, %d) silu%d states%d bi%d" % (seed, str(dtype)[6:], W, B, D, L, silu, states, bi)
        assert torch.equal(got[0][0], got[1][0]), "dx differs between the kernels, " + what
        if states:
            assert torch.equal(got[0][3], got[1][3]), "dinitial_states differ, " + what
        assert_close(got[0][1], got[1][1], what="dweight, " + what, tol=TOL_W)
        if b is not None:
            assert_close(got[0][2], got[1][2], what="dbias, " + what, tol=TOL_W)
        if n % 5 == 0:
            ref = orc.bwd(x, w, b, dout, initial_states=init, dfinal_states=dfin, activation="silu" if silu else None)
            assert_close(got[0][0], ref[0].to(dtype), dtype, "dx, " + what)
            assert_close(got[0][1], ref[1], what="dweight, " + what, tol=TOL_W)
            if states:
                assert_close(got[0][3], ref[3].to(dtype), dtype, "dinitial_states, " + what)
