"""GPU parity of the backward kernels (dx, dweight, dbias, dinitial_states) against the CPU
oracle (autograd through the PyTorch forward), through the public autograd Function and
through the C ABI.  Grids restate tests/test_causal_conv1d.py:50-137 and :401-472 of the
reference; determinism follows :560-575.  initial/final states are also exercised for
channel-first, which the reference refuses.

Tolerances: dx / dinitial_states as the forward (fp32 1e-5 absolute, fp16 3e-3/5e-3, bf16
1e-2/5e-2); dweight / dbias rtol 1e-3, atol 1e-3 (long fp32 sums, summation order differs).
"""
import ctypes

import pytest
import torch

import cabi
from golden_io import load_case
from helpers import (DTYPES, TOL_W, assert_close, gen, make_states, make_wb, make_x, random_seq_idx,
                     to_dev_like)
from oracle import causal_conv1d_oracle as orc
from oracle import c_oracle

pytestmark = pytest.mark.gpu

SEQLENS = [1, 2, 8, 16, 32, 64, 128, 129, 130, 151, 256, 372, 512, 784, 1000, 1024, 1134, 1544, 2048, 2568, 4096]


def run_gpu(pkg, dev, x, w, b, dout, seq=None, init=None, dfin=None, act=None):
    xd = to_dev_like(x, dev).requires_grad_()
    wd = w.to(dev).requires_grad_()
    bd = b.to(dev).requires_grad_() if b is not None else None
    idev = init.to(dev).requires_grad_() if init is not None else None
    res = pkg.causal_conv1d_fn(xd, wd, bd, seq_idx=None if seq is None else seq.to(dev),
                               initial_states=idev, return_final_states=dfin is not None, activation=act)
    if dfin is not None:
        torch.autograd.backward(list(res), [to_dev_like(dout, dev), dfin.to(dev)])
    else:
        res.backward(to_dev_like(dout, dev))
    return (xd.grad, wd.grad, None if bd is None else bd.grad, None if idev is None else idev.grad)


def check(got, ref, dtype):
    names = ("dx", "dweight", "dbias", "dinitial_states")
    for name, g, r in zip(names, got, ref):
        assert (g is None) == (r is None), name
        if g is None:
            continue
        if name in ("dweight", "dbias"):
            assert g.dtype == torch.float32
            assert_close(g, r, what=name, tol=TOL_W)
        else:
            assert g.dtype == dtype
            assert_close(g, r.to(dtype), dtype, name)


def _grid():
    cases, n = [], 0
    for dim in (64, 4096 + 32):
        for seqlen in SEQLENS:
            for dtype in DTYPES:
                for channel_last in (False, True):
                    width = 2 + (n + 1) % 3
                    has_bias = (n // 3) % 2 == 0
                    silu = (n // 6) % 2 == 1
                    states = (n // 12 + n) % 4            # bit 0: initial_states, bit 1: final states
                    cases.append(pytest.param(dim, seqlen, dtype, channel_last, width, has_bias, silu, states,
                                              id=f"d{dim}-l{seqlen}-{str(dtype)[6:]}-{'cl' if channel_last else 'cf'}"
                                                 f"-w{width}-b{int(has_bias)}-s{int(silu)}-st{states}"))
                    n += 1
    return cases


@pytest.mark.parametrize("dim,seqlen,dtype,channel_last,width,has_bias,silu,states", _grid())
def test_bwd_matches_oracle(pkg, gpu_device, dim, seqlen, dtype, channel_last, width, has_bias, silu, states):
    g = gen(seqlen * 5 + dim + width)
    x = make_x(2, dim, seqlen, dtype, channel_last, g)
    w, b = make_wb(dim, width, has_bias, g)
    dout = make_x(2, dim, seqlen, dtype, channel_last, g, sliced=False)
    init = make_states(2, dim, width - 1, dtype, g) if states & 1 else None
    dfin = make_states(2, dim, width - 1, dtype, g) if states & 2 else None
    act = "silu" if silu else None
    ref = orc.bwd(x, w, b, dout, initial_states=init, dfinal_states=dfin, activation=act)
    got = run_gpu(pkg, gpu_device, x, w, b, dout, init=init, dfin=dfin, act=act)
    check(got, ref, dtype)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("seqlen", [8, 24, 40, 72, 136, 248, 256, 264, 512])
def test_bwd_channel_first_short_rows(pkg, gpu_device, seqlen, dtype):
    """Channel-first rows of at most 64 whole 16-byte vectors: several batch entries share a
    wavefront.  A batch that does not fill the last group, every vector-count class, all state
    gradients; dx and dinitial_states must also equal, bit for bit, what the same data gives
    when it sits one element off the 16-byte grid (element accesses instead of vectors)."""
    dev = gpu_device
    batch, dim, width = 5, 24, 2 + seqlen % 3
    g = gen(2000 + seqlen)
    x = torch.randn(batch, dim, seqlen, generator=g).to(dtype)
    dout = torch.randn(batch, dim, seqlen, generator=g).to(dtype)
    w, b = make_wb(dim, width, True, g)
    init = make_states(batch, dim, width - 1, dtype, g)
    dfin = make_states(batch, dim, width - 1, dtype, g)
    ref = orc.bwd(x, w, b, dout, initial_states=init, dfinal_states=dfin, activation="silu")
    got = run_gpu(pkg, dev, x, w, b, dout, init=init, dfin=dfin, act="silu")
    check(got, ref, dtype)

    def off_grid(t):                                   # same values, rows one element off the grid
        wide = torch.zeros(batch, dim, seqlen + 8, dtype=dtype)
        wide[:, :, 1:1 + seqlen] = t
        return wide[:, :, 1:1 + seqlen]
    other = run_gpu(pkg, dev, off_grid(x), w, b, off_grid(dout), init=init, dfin=dfin, act="silu")
    assert torch.equal(other[0], got[0]), "dx"
    assert torch.equal(other[3], got[3]), "dinitial_states"
    check(other, ref, dtype)
    # no states, no bias, no activation
    got = run_gpu(pkg, dev, x, w, None, dout)
    check(got, orc.bwd(x, w, None, dout), dtype)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("seqlen", [1, 2, 3, 5, 7, 9, 60, 100, 255, 500])
def test_bwd_channel_first_short_rows_of_any_length(pkg, gpu_device, seqlen, dtype):
    """Channel-first rows of at most 64 vectors that are not whole vectors share wavefronts too,
    down to one lane per batch entry.  All state gradients: in a row shorter than width-1 part of
    dfinal_states lands in dinitial_states (csrc/causal_conv1d_bwd.cu:535-561)."""
    dev = gpu_device
    batch, dim = 67, 24                                # more entries than one wavefront takes at once
    for width in (2, 3, 4):
        g = gen(4000 + seqlen * 4 + width)
        x = torch.randn(batch, dim, seqlen, generator=g).to(dtype)
        dout = torch.randn(batch, dim, seqlen, generator=g).to(dtype)
        w, b = make_wb(dim, width, True, g)
        init = make_states(batch, dim, width - 1, dtype, g)
        dfin = make_states(batch, dim, width - 1, dtype, g)
        ref = orc.bwd(x, w, b, dout, initial_states=init, dfinal_states=dfin, activation="silu")
        got = run_gpu(pkg, dev, x, w, b, dout, init=init, dfin=dfin, act="silu")
        check(got, ref, dtype)
        got = run_gpu(pkg, dev, x, w, None, dout)
        check(got, orc.bwd(x, w, None, dout), dtype)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("dim,seqlen,width,has_bias,silu", [
    (64, 8, 2, True, True), (64, 16, 3, False, True), (64, 151, 4, True, False), (64, 372, 4, True, True),
    (64, 1134, 3, True, True), (4128, 32, 4, True, True), (4128, 128, 2, False, False),
    (4128, 784, 4, True, True), (4128, 2048, 3, True, True), (4128, 4096, 4, True, True),
])
def test_bwd_seq_idx_matches_oracle(pkg, gpu_device, dim, seqlen, width, has_bias, silu, dtype):
    g = gen(seqlen + dim + width + 1)
    x = make_x(3, dim, seqlen, dtype, True, g)
    w, b = make_wb(dim, width, has_bias, g)
    dout = make_x(3, dim, seqlen, dtype, True, g, sliced=False)
    seq = random_seq_idx(3, seqlen, g)
    act = "silu" if silu else None
    ref = orc.bwd(x, w, b, dout, seq_idx=seq, activation=act)
    got = run_gpu(pkg, gpu_device, x, w, b, dout, seq=seq, act=act)
    check(got, ref, dtype)


def test_bwd_seq_idx_padding_gets_no_gradient(pkg, gpu_device):
    """The gradient of the forward as defined (exact zeros at seq_idx < 0): nothing flows
    into or out of padding tokens.  Checked against the closed-form C restatement."""
    g = gen(9)
    x = make_x(3, 64, 200, torch.float32, True, g)
    w, b = make_wb(64, 4, True, g)
    dout = make_x(3, 64, 200, torch.float32, True, g, sliced=False)
    seq = random_seq_idx(3, 200, g, pad=True)
    got = run_gpu(pkg, gpu_device, x, w, b, dout, seq=seq, act="silu")
    ref = c_oracle.bwd(x, w, b, dout, seq_idx=seq, silu=True)
    assert torch.all(got[0].cpu()[(seq < 0).unsqueeze(1).expand(3, 64, 200)] == 0)
    assert_close(got[0], ref[0].float(), torch.float32, "dx")
    assert_close(got[1], ref[1].float(), what="dweight", tol=TOL_W)
    assert_close(got[2], ref[2].float(), what="dbias", tol=TOL_W)


def test_bwd_golden_fixture(pkg, gpu_device):
    c = load_case("bwd")
    for cl in (False, True):
        lay = (lambda t: t.transpose(1, 2).contiguous().transpose(1, 2)) if cl else (lambda t: t)
        got = run_gpu(pkg, gpu_device, lay(c["x"]), c["weight"], c["bias"], lay(c["dout"]),
                      init=c["initial_states"], dfin=c["dfinal_states"], act="silu")
        check(got, (c["dx"], c["dweight"], c["dbias"], c["dinitial_states"]), torch.float32)


@pytest.mark.parametrize("channel_last", [False, True])
def test_bwd_is_bit_reproducible(pkg, gpu_device, channel_last):
    """Five runs, identical bits in dx, dweight and dbias (the reduction is a fixed-order
    two-stage sum; tests/test_causal_conv1d.py:560-575 asks this of deterministic mode)."""
    g = gen(1234)
    x = make_x(4, 1024, 2048, torch.bfloat16, channel_last, g, sliced=False)
    w, b = make_wb(1024, 4, True, g)
    dout = make_x(4, 1024, 2048, torch.bfloat16, channel_last, g, sliced=False)
    first = run_gpu(pkg, gpu_device, x, w, b, dout, act="silu")
    for _ in range(4):
        again = run_gpu(pkg, gpu_device, x, w, b, dout, act="silu")
        for a, f in zip(again[:3], first[:3]):
            assert torch.equal(a, f)
    ref = orc.bwd(x, w, b, dout, activation="silu")
    check(first, ref, torch.bfloat16)


@pytest.mark.parametrize("dtype", DTYPES)
def test_bwd_workgroup_order_does_not_change_results(pkg, gpu_device, cc1d_lib, dtype):
    """Channel-last backward: slices or chunks of runs per XCD, same bits in every gradient (the
    partial sums of dweight keep their places in the second stage's order)."""
    lib = cabi.declare(cc1d_lib)
    g = gen(13)
    x = make_x(3, 1160, 1237, dtype, True, g)
    dout = make_x(3, 1160, 1237, dtype, True, g, sliced=False)
    w, b = make_wb(1160, 4, True, g)
    outs = []
    try:
        for chunk in (-1, 0, 4, 8, 16, 64):
            assert lib.cc1d_set_tunable(b"bwd_cl_chunk_runs", chunk) == 0
            outs.append([t.cpu() for t in run_gpu(pkg, gpu_device, x, w, b, dout, act="silu")[:3]])
    finally:
        lib.cc1d_set_tunable(b"bwd_cl_chunk_runs", 0)
    for o in outs[1:]:
        for a, r in zip(o, outs[0]):
            assert torch.equal(a, r)
    check(tuple(outs[0]) + (None,), orc.bwd(x, w, b, dout, activation="silu"), dtype)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("dim,seqlen,width,has_bias,silu,extras", [
    (64, 8, 2, True, True, "seq"), (64, 151, 4, True, False, "states"), (72, 372, 3, False, True, "seq"),
    (4128, 32, 4, True, True, ""), (4128, 784, 4, True, True, "seq"), (1160, 1237, 3, True, True, "states"),
    (520, 2050, 4, False, False, ""),
])
def test_bwd_channel_last_lane_widths_agree(pkg, gpu_device, cc1d_lib, dim, seqlen, width, has_bias, silu, extras, dtype):
    """Channel-last backward on 16-bit data with 4-byte and with 8-byte lanes (the library takes
    the wider ones by itself where the rows of dx do not start on 64-byte boundaries): both match
    the oracle, and dx, a sum per element in one order, is the same bit for bit."""
    lib = cabi.declare(cc1d_lib)
    g = gen(dim + seqlen + width)
    x = make_x(3, dim, seqlen, dtype, True, g)
    dout = make_x(3, dim, seqlen, dtype, True, g, sliced=False)
    w, b = make_wb(dim, width, has_bias, g)
    seq = random_seq_idx(3, seqlen, g) if extras == "seq" else None
    init = make_states(3, dim, width - 1, dtype, g) if extras == "states" else None
    dfin = make_states(3, dim, width - 1, dtype, g) if extras == "states" else None
    act = "silu" if silu else None
    ref = orc.bwd(x, w, b, dout, seq_idx=seq, initial_states=init, dfinal_states=dfin, activation=act)
    outs = []
    try:
        for lane_bytes in (4, 8):
            assert lib.cc1d_set_tunable(b"bwd_cl_lane_bytes", lane_bytes) == 0
            outs.append(run_gpu(pkg, gpu_device, x, w, b, dout, seq=seq, init=init, dfin=dfin, act=act))
    finally:
        lib.cc1d_set_tunable(b"bwd_cl_lane_bytes", 0)
    for got in outs:
        check(got, ref, dtype)
    assert torch.equal(outs[0][0], outs[1][0])
    if outs[0][3] is not None:
        assert torch.equal(outs[0][3], outs[1][3])


def test_bwd_dx_as_column_slice_of_a_wider_tensor(gpu_device, cc1d_lib):
    """The layout of mamba_ssm's Mamba-2 backward: x and dx are column slices of tensors d_in_proj
    wide (rows that do not start on 64-byte boundaries), dout is dense; a launch large enough that
    the library picks its lane width from the alignment of dx.  Against the oracle on one batch
    entry and, bit for bit, against the same call with dense tensors."""
    lib = cabi.declare(cc1d_lib)
    dev = gpu_device
    B, L, D, d_in_proj, off = 16, 2048, 1792, 3352, 1536
    g = torch.Generator(device=dev)
    g.manual_seed(5)
    big_x = torch.randn(B, L, d_in_proj, generator=g, device=dev).to(torch.bfloat16)
    big_dx = torch.zeros(B, L, d_in_proj, device=dev, dtype=torch.bfloat16)
    x = big_x[:, :, off:off + D].transpose(1, 2)
    dx = big_dx[:, :, off:off + D].transpose(1, 2)
    dout = torch.randn(B, L, D, generator=g, device=dev).to(torch.bfloat16).transpose(1, 2)
    w, b = (t.to(dev) for t in make_wb(D, 4, True, gen(6)))
    seq = torch.zeros(B, L, dtype=torch.int32, device=dev)
    seq[:, 700:] = 1
    seq[:, 1500:] = 2
    stream = torch.cuda.current_stream().cuda_stream

    def run(xv, dxv):
        dw = torch.zeros(D, 4, device=dev)
        db = torch.zeros(D, device=dev)
        p = cabi.bwd_params(xv, w, b, dout, dxv, dw, db, True, seq_idx=seq)
        need = ctypes.c_size_t()
        assert lib.cc1d_bwd_workspace_bytes(ctypes.byref(p), ctypes.byref(need)) == 0
        ws = torch.empty(max(16, need.value), dtype=torch.uint8, device=dev)
        st = lib.cc1d_bwd(ctypes.byref(p), ws.data_ptr(), need.value, stream)
        assert st == 0, lib.cc1d_strerror(st)
        torch.cuda.synchronize()
        return dw, db

    dw, db = run(x, dx)
    assert not big_dx[:, :, :off].any() and not big_dx[:, :, off + D:].any()     # nothing outside the slice
    dense_x = x.transpose(1, 2).contiguous().transpose(1, 2)
    dense_dx = torch.empty_like(dense_x)
    dw2, db2 = run(dense_x, dense_dx)
    assert torch.equal(dx, dense_dx)
    assert_close(dw, dw2, what="dweight", tol=TOL_W)
    assert_close(db, db2, what="dbias", tol=TOL_W)
    ref = orc.bwd(x[5:6].cpu(), w.cpu(), b.cpu(), dout[5:6].cpu(), seq_idx=seq[5:6].cpu(), activation="silu")
    assert_close(dx[5:6], ref[0].to(torch.bfloat16), torch.bfloat16, "dx")


@pytest.mark.parametrize("channel_last", [False, True])
def test_bwd_c_abi_accumulates_into_dweight(gpu_device, cc1d_lib, channel_last):
    """Through the C ABI with a caller-owned workspace: dweight / dbias are added to, as the
    reference's atomicAdd / add_ do (csrc/causal_conv1d_bwd.cu:243; causal_conv1d.cpp:452)."""
    lib = cabi.declare(cc1d_lib)
    dev = gpu_device
    g = gen(77)
    x = make_x(2, 64, 500, torch.float32, channel_last, g, sliced=False)
    dout = make_x(2, 64, 500, torch.float32, channel_last, g, sliced=False)
    w, b = make_wb(64, 3, True, g)
    ref = orc.bwd(x, w, b, dout, activation="silu")
    xd, dd, wd, bd = (t.to(dev) for t in (x, dout, w, b))
    dx = torch.empty_like(xd)
    dw = torch.full((64, 3), 2.0, device=dev)
    db = torch.full((64,), -1.0, device=dev)
    p = cabi.bwd_params(xd, wd, bd, dd, dx, dw, db, True)
    need = ctypes.c_size_t()
    assert lib.cc1d_bwd_workspace_bytes(ctypes.byref(p), ctypes.byref(need)) == 0
    ws = torch.empty(max(16, need.value), dtype=torch.uint8, device=dev)
    stream = torch.cuda.current_stream().cuda_stream
    if need.value:
        assert lib.cc1d_bwd(ctypes.byref(p), ws.data_ptr(), need.value - 1, stream) == -13
    st = lib.cc1d_bwd(ctypes.byref(p), ws.data_ptr(), need.value, stream)
    assert st == 0, lib.cc1d_strerror(st)
    torch.cuda.synchronize()
    assert_close(dx, ref[0], torch.float32, "dx")
    assert_close(dw - 2.0, ref[1], what="dweight", tol=TOL_W)
    assert_close(db + 1.0, ref[2], what="dbias", tol=TOL_W)


@pytest.mark.parametrize("channel_last,dim,seqlen", [(False, 64, 500), (False, 4096, 64), (True, 64, 500),
                                                     (True, 64, 0)])
def test_bwd_c_abi_overwrite_dweight(gpu_device, cc1d_lib, channel_last, dim, seqlen):
    """overwrite_dweight = 1: dweight / dbias are plain outputs.  Whatever they held (NaN here)
    is ignored and the sums equal, bit for bit, the ones accumulated into zeros; an empty
    problem stores zeros.  dim 4096 channel-first is the path without a second stage."""
    lib = cabi.declare(cc1d_lib)
    dev = gpu_device
    g = gen(78)
    x = make_x(2, dim, seqlen, torch.bfloat16, channel_last, g, sliced=False).to(dev)
    dout = make_x(2, dim, seqlen, torch.bfloat16, channel_last, g, sliced=False).to(dev)
    w, b = (t.to(dev) for t in make_wb(dim, 4, True, g))
    stream = torch.cuda.current_stream().cuda_stream
    got = []
    for overwrite, fill in ((0, 0.0), (1, float("nan"))):
        dx = torch.empty_like(x)
        dw = torch.full((dim, 4), fill, device=dev)
        db = torch.full((dim,), fill, device=dev)
        p = cabi.bwd_params(x, w, b, dout, dx, dw, db, True)
        p.overwrite_dweight = overwrite
        need = ctypes.c_size_t()
        assert lib.cc1d_bwd_workspace_bytes(ctypes.byref(p), ctypes.byref(need)) == 0
        ws = torch.empty(max(16, need.value), dtype=torch.uint8, device=dev)
        st = lib.cc1d_bwd(ctypes.byref(p), ws.data_ptr(), need.value, stream)
        assert st == 0, lib.cc1d_strerror(st)
        torch.cuda.synchronize()
        got.append((dw, db))
    assert torch.equal(got[0][0], got[1][0]) and torch.equal(got[0][1], got[1][1])
    if seqlen == 0:
        assert not got[1][0].any() and not got[1][1].any()


def test_bwd_full_size_fp16_channel_first_with_states(pkg, gpu_device):
    """The backward configuration at full size: fp16 (4, 4096, 8192) channel-first, width 4,
    SiLU, initial_states and a gradient on final_states.  Channels are independent, so a
    handful of channels is checked exactly against the oracle at full batch and length;
    the whole dx is checked through linearity in dout."""
    import bench
    cfg = bench.config_c4()
    dev = gpu_device
    got = run_gpu(pkg, dev, cfg["x"], cfg["weight"], cfg["bias"], cfg["dout"],
                  init=cfg["initial_states"], dfin=cfg["dfinal_states"], act="silu")
    ch = torch.tensor([0, 1, 63, 64, 2047, 4095])
    ref = orc.bwd(cfg["x"][:, ch], cfg["weight"][ch], cfg["bias"][ch], cfg["dout"][:, ch],
                  initial_states=cfg["initial_states"][:, ch], dfinal_states=cfg["dfinal_states"][:, ch],
                  activation="silu")
    chd = ch.to(dev)
    sub = (got[0][:, chd], got[1][chd], got[2][chd], got[3][:, chd])
    check(sub, ref, torch.float16)
    # linearity: gradients for (2*dout, 2*dfinal) are exactly twice those for (dout, dfinal)
    got2 = run_gpu(pkg, dev, cfg["x"], cfg["weight"], cfg["bias"], cfg["dout"] * 2,
                   init=cfg["initial_states"], dfin=cfg["dfinal_states"] * 2, act="silu")
    assert_close(got2[0], got[0].float() * 2, torch.float16, "dx linearity")
    assert_close(got2[1], got[1] * 2, what="dweight linearity", tol=TOL_W)


def test_repeated_runs_are_bit_identical(pkg, gpu_device):
    """tests/test_causal_conv1d.py:342-398 of the reference hunts for races by repeating forward
    and backward on one input and demanding identical out and dx (dweight / dbias within 1e-4
    there; here they are bit-identical too, the reduction order being fixed).  10,000 repeats, as there."""
    dev = gpu_device
    g = gen(4242)
    x0 = to_dev_like(make_x(2, 4096 + 32, 2048, torch.bfloat16, True, g), dev)
    w, b = make_wb(4096 + 32, 4, True, g)
    w, b = w.to(dev).requires_grad_(), b.to(dev).requires_grad_()
    dout = to_dev_like(make_x(2, 4096 + 32, 2048, torch.bfloat16, True, g, sliced=False), dev)

    def once():
        x = x0.detach().requires_grad_()
        out = pkg.causal_conv1d_fn(x, w, b, activation="silu")
        dx, dw, db = torch.autograd.grad(out, (x, w, b), dout)
        return out.detach(), dx, dw, db

    first = once()
    same = torch.ones((), dtype=torch.bool, device=dev)
    for _ in range(10000):
        for a, f in zip(once(), first):
            same &= (a == f).all()
    assert bool(same)
