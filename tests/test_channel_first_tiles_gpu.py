"""The channel-first tile kernels (rows fetched straight into LDS through per-row buffer
resources): backward for every row longer than 64 vectors, at any length and alignment; forward
for rows on the 16-byte grid of 65 to 128 whole vectors or starting on 128-byte lines, and for
rows off that grid (a length that is no whole number of vectors, a view that starts inside a
vector, out on another grid).

Checked against the CPU oracle (tolerances of test_fwd_gpu.py / test_bwd_gpu.py) and, bit for
bit, against the walking kernels, which a launch tunable brings back for the same tensors
(`bwd_cf_parts` / `fwd_cf_vecs` = -1): dx, dinitial_states, out and final_states must not depend
on which kernel produced them; dweight / dbias are sums in another order and get the oracle's
tolerance.  Lengths: one and two elements off the vector grid on either side (1001, 1023, 1025,
2047 -- rows that used to cost the backward twice the time of their neighbours), rows that end
inside a tile's first and last step, rows that end in a tail of one position per lane (516, 1025,
1032, 2049, 2113, 4099, 4161: at most 64 positions behind a whole number of steps), one tile and
several, and views that start one element into an allocation.
"""
import ctypes

import pytest
import torch

import cabi
from helpers import DTYPES, TOL_W, assert_close, gen, make_states, make_wb
from oracle import causal_conv1d_oracle as orc

pytestmark = pytest.mark.gpu


def _view(t, dev, shift):
    """The tensor's values on the GPU as a view that starts `shift` elements into its allocation."""
    flat = torch.zeros(t.numel() + 64, dtype=t.dtype, device=dev)
    flat[shift:shift + t.numel()] = t.reshape(-1).to(dev)
    return flat[shift:shift + t.numel()].view(t.shape)


def _bwd(lib, dev, x, w, b, dout, init, dfin, shift, walking):
    xd, dd = _view(x, dev, shift), _view(dout, dev, shift)
    dx = _view(torch.zeros_like(x), dev, shift)
    wd, bd = w.to(dev), b.to(dev)
    dw, db = torch.empty_like(wd), torch.empty_like(bd)
    idev = None if init is None else init.to(dev)
    fdev = None if dfin is None else dfin.to(dev)
    dinit = None if init is None else torch.empty(x.shape[0], w.shape[1] - 1, x.shape[1], dtype=x.dtype, device=dev).transpose(1, 2)
    # The parameter block holds addresses only: every operand stays referenced by a local until the
    # launch is done (a temporary would go back to the allocator and could become the workspace).
    p = cabi.bwd_params(xd, wd, bd, dd, dx, dw, db, True, initial_states=idev,
                        dfinal_states=fdev, dinitial_states=dinit)
    p.overwrite_dweight = 1
    assert lib.cc1d_set_tunable(b"bwd_cf_parts", -1 if walking else 0) == 0
    try:
        need = ctypes.c_size_t()
        assert lib.cc1d_bwd_workspace_bytes(ctypes.byref(p), ctypes.byref(need)) == 0
        ws = torch.empty(max(16, need.value), dtype=torch.uint8, device=dev)
        assert lib.cc1d_bwd(ctypes.byref(p), ctypes.c_void_p(ws.data_ptr()), need, None) == 0
        torch.cuda.synchronize()
    finally:
        lib.cc1d_set_tunable(b"bwd_cf_parts", 0)
    return dx.cpu(), dw.cpu(), db.cpu(), None if dinit is None else dinit.cpu()


@pytest.mark.parametrize("dtype", DTYPES, ids=lambda d: str(d)[6:])
@pytest.mark.parametrize("seqlen", [516, 1000, 1001, 1023, 1025, 1032, 2047, 2049, 2050, 2113, 2561, 4099, 4161])
def test_bwd_rows_of_any_length_and_alignment(gpu_device, cc1d_lib, seqlen, dtype):
    lib = cabi.declare(cc1d_lib)
    g = gen(7000 + seqlen)
    B, D, W = 3, 20, 2 + seqlen % 3
    x = torch.randn(B, D, seqlen, generator=g).to(dtype)
    dout = torch.randn(B, D, seqlen, generator=g).to(dtype)
    w, b = make_wb(D, W, True, g)
    init = make_states(B, D, W - 1, dtype, g)
    dfin = make_states(B, D, W - 1, dtype, g)
    ref = orc.bwd(x, w, b, dout, initial_states=init, dfinal_states=dfin, activation="silu")
    for shift in (0, 1, 3):
        for states in (True, False):
            i_, f_ = (init, dfin) if states else (None, None)
            tile = _bwd(lib, gpu_device, x, w, b, dout, i_, f_, shift, walking=False)
            walk = _bwd(lib, gpu_device, x, w, b, dout, i_, f_, shift, walking=True)
            what = "seqlen %d shift %d states %d" % (seqlen, shift, states)
            assert torch.equal(tile[0], walk[0]), "dx differs between the kernels, " + what
            if states:
                assert torch.equal(tile[3], walk[3]), "dinitial_states differs between the kernels, " + what
                assert_close(tile[0], ref[0].to(dtype), dtype, "dx, " + what)
                assert_close(tile[1], ref[1], what="dweight, " + what, tol=TOL_W)
                assert_close(tile[2], ref[2], what="dbias, " + what, tol=TOL_W)
                assert_close(tile[3], ref[3].to(dtype), dtype, "dinitial_states, " + what)
            else:
                assert_close(tile[1], walk[1], what="dweight, " + what, tol=TOL_W)
                assert_close(tile[2], walk[2], what="dbias, " + what, tol=TOL_W)


def test_bwd_tiles_at_a_size_that_fills_the_chip(gpu_device, cc1d_lib):
    """Rows of several tiles, more wavefronts than the chip holds at once, batch entries as
    neighbours in memory (a (dim, batch, seqlen) tensor seen as (batch, dim, seqlen))."""
    lib = cabi.declare(cc1d_lib)
    dev = gpu_device
    g = gen(7777)
    B, D, L, W = 4, 1536, 4104, 4
    x = torch.randn(D, B, L, generator=g).to(torch.bfloat16).transpose(0, 1)
    dout = torch.randn(D, B, L, generator=g).to(torch.bfloat16).transpose(0, 1)
    w, b = make_wb(D, W, True, g)

    def run(walking):
        xd, dd = x.transpose(0, 1).contiguous().to(dev).transpose(0, 1), dout.transpose(0, 1).contiguous().to(dev).transpose(0, 1)
        dx = torch.zeros(D, B, L, dtype=torch.bfloat16, device=dev).transpose(0, 1)
        dw, db = torch.empty(D, W, device=dev), torch.empty(D, device=dev)
        wd, bd = w.to(dev), b.to(dev)                  # referenced until the launch is done
        p = cabi.bwd_params(xd, wd, bd, dd, dx, dw, db, True)
        p.overwrite_dweight = 1
        assert lib.cc1d_set_tunable(b"bwd_cf_parts", -1 if walking else 0) == 0
        try:
            need = ctypes.c_size_t()
            assert lib.cc1d_bwd_workspace_bytes(ctypes.byref(p), ctypes.byref(need)) == 0
            ws = torch.empty(max(16, need.value), dtype=torch.uint8, device=dev)
            assert lib.cc1d_bwd(ctypes.byref(p), ctypes.c_void_p(ws.data_ptr()), need, None) == 0
            torch.cuda.synchronize()
        finally:
            lib.cc1d_set_tunable(b"bwd_cf_parts", 0)
        return dx.cpu(), dw.cpu(), db.cpu()

    tile, walk = run(False), run(True)
    assert torch.equal(tile[0], walk[0])
    assert_close(tile[1], walk[1], what="dweight", tol=TOL_W)
    assert_close(tile[2], walk[2], what="dbias", tol=TOL_W)
    ref = orc.bwd(x[:1, :64], w[:64], b[:64], dout[:1, :64], activation="silu")
    assert_close(tile[0][:1, :64], ref[0].to(torch.bfloat16), torch.bfloat16, "dx")


@pytest.mark.parametrize("dtype", DTYPES, ids=lambda d: str(d)[6:])
@pytest.mark.parametrize("vecs", [65, 96, 127, 128, 192, 256, 320, 520, 1032])
def test_fwd_tile_rows(pkg, gpu_device, cc1d_lib, vecs, dtype):
    """Forward rows of whole vectors on the 16-byte grid -- 65 .. 128 vectors, and longer rows that
    start on 128-byte lines (one tile, two, several; 1032 vectors end in a tail) -- tile kernel
    against the walking kernel (bit for bit) and the oracle, with and without states, rows as a
    channel slice of a wider tensor."""
    lib = cabi.declare(cc1d_lib)
    dev = gpu_device
    vec = 16 // torch.empty(0, dtype=dtype).element_size()
    L = vecs * vec
    g = gen(8000 + vecs)
    B, D, W = 3, 24, 2 + vecs % 3
    wide = torch.randn(B, D + 8, L, generator=g).to(dtype)
    x = wide[:, 4:4 + D, :]
    w, b = make_wb(D, W, True, g)
    init = make_states(B, D, W - 1, dtype, g)
    ref, ref_fin = orc.fwd(x, w, b, initial_states=init, return_final_states=True, activation="silu")
    ref_plain = orc.fwd(x, w, b, activation=None)
    xd = wide.to(dev)[:, 4:4 + D, :]
    outs = []
    try:
        for knob in (0, -1):
            assert lib.cc1d_set_tunable(b"fwd_cf_vecs", knob) == 0
            o, f = pkg.causal_conv1d_fn(xd, w.to(dev), b.to(dev), initial_states=init.to(dev),
                                        return_final_states=True, activation="silu")
            o2 = pkg.causal_conv1d_fn(xd, w.to(dev), b.to(dev), activation=None)
            outs.append((o.cpu(), f.cpu(), o2.cpu()))
    finally:
        lib.cc1d_set_tunable(b"fwd_cf_vecs", 0)
    for a, r in zip(outs[0], outs[1]):
        assert torch.equal(a, r), "tile and walking kernels differ"
    assert_close(outs[0][0], ref, dtype, "out")
    assert torch.equal(outs[0][1], ref_fin)
    assert_close(outs[0][2], ref_plain, dtype, "out without activation")


@pytest.mark.parametrize("dtype", DTYPES, ids=lambda d: str(d)[6:])
@pytest.mark.parametrize("seqlen", [513, 517, 1001, 1023, 1025, 1032, 1087, 2047, 2049, 2113, 3001])
def test_fwd_rows_off_the_grid(pkg, gpu_device, cc1d_lib, seqlen, dtype):
    """Rows that are no whole number of vectors, or start inside one: tile kernel against the
    walking kernels (bit for bit) and the oracle.  Lengths one and two elements off the grid on
    either side, rows that end in a tail of one position per lane (1025, 1032, 2049, 2113), rows
    of one tile and two, views one and three elements into their allocation, out on another
    grid than x."""
    lib = cabi.declare(cc1d_lib)
    dev = gpu_device
    vec = 16 // torch.empty(0, dtype=dtype).element_size()
    if dtype == torch.float32 and seqlen > 3 * 64 * vec:
        pytest.skip("fp32 rows this long keep the walking kernel")
    g = gen(9000 + seqlen)
    B, D, W = 3, 20, 2 + seqlen % 3
    x = torch.randn(B, D, seqlen, generator=g).to(dtype)
    w, b = make_wb(D, W, True, g)
    init = make_states(B, D, W - 1, dtype, g)
    ref, ref_fin = orc.fwd(x, w, b, initial_states=init, return_final_states=True, activation="silu")
    ref_plain = orc.fwd(x, w, b, activation=None)
    wd, bd, idev = w.to(dev), b.to(dev), init.to(dev)
    for x_shift, out_shift in ((0, 0), (1, 1), (3, 0), (0, 2)):
        xd = _view(x, dev, x_shift)
        got = []
        try:
            for knob in (0, -1):
                assert lib.cc1d_set_tunable(b"fwd_cf_vecs", knob) == 0
                out = _view(torch.zeros_like(x), dev, out_shift)
                fin = torch.empty(B, W - 1, D, dtype=dtype, device=dev).transpose(1, 2)
                p = cabi.fwd_params(xd, wd, bd, out, True, initial_states=idev, final_states=fin)
                assert lib.cc1d_fwd(ctypes.byref(p), None) == 0
                out2 = _view(torch.zeros_like(x), dev, out_shift)
                p2 = cabi.fwd_params(xd, wd, bd, out2, False)
                assert lib.cc1d_fwd(ctypes.byref(p2), None) == 0
                torch.cuda.synchronize()
                got.append((out.cpu(), fin.cpu(), out2.cpu()))
        finally:
            lib.cc1d_set_tunable(b"fwd_cf_vecs", 0)
        what = "seqlen %d x shift %d out shift %d" % (seqlen, x_shift, out_shift)
        for a, r in zip(got[0], got[1]):
            assert torch.equal(a, r), "tile and walking kernels differ, " + what
        assert_close(got[0][0], ref, dtype, "out, " + what)
        assert torch.equal(got[0][1], ref_fin), what
        assert_close(got[0][2], ref_plain, dtype, "out without activation, " + what)
