"""cc1d_bwd_noalloc, the backward entry point that allocates nothing (its partial-sum workspace is
a fixed array in the library's device image), against cc1d_bwd with a caller-owned workspace:
through the C ABI, bit for bit (same kernels, same order of additions), on two calls in a row on
the same GPU, the second on a smaller input, so the second call meets what the first left in the
shared array.  Also: the size limit is enforced before anything is launched."""
import ctypes

import pytest
import torch

import cabi
from helpers import TOL_W, assert_close, gen, make_states, make_wb, make_x, random_seq_idx
from oracle import causal_conv1d_oracle as orc

MAX_WS = 16 * 1024 * 1024
E_WORKSPACE_LIMIT = -19


def _problem(B, D, L, dtype, channel_last, seed, dev, seq_idx=False):
    g = gen(seed)
    x = make_x(B, D, L, dtype, channel_last, g, sliced=False)
    dout = make_x(B, D, L, dtype, channel_last, g, sliced=False)
    w, b = make_wb(D, 4, True, g)
    seq = random_seq_idx(B, L, g) if seq_idx else None
    init = None if seq_idx else make_states(B, D, 3, dtype, g)
    dfin = None if seq_idx else make_states(B, D, 3, dtype, g)
    host = dict(x=x, dout=dout, w=w, b=b, seq=seq, init=init, dfin=dfin)
    return host, {k: (None if v is None else v.to(dev)) for k, v in host.items()}


def _run(lib, d, dev, noalloc):
    x = d["x"]
    B, D, L = x.shape
    dx = torch.empty_like(x)
    dinit = None if d["init"] is None else torch.empty(B, 3, D, device=dev, dtype=x.dtype).transpose(1, 2)
    dw, db = torch.full((D, 4), float("nan"), device=dev), torch.full((D,), float("nan"), device=dev)
    p = cabi.bwd_params(x, d["w"], d["b"], d["dout"], dx, dw, db, True, seq_idx=d["seq"], initial_states=d["init"],
                        dfinal_states=d["dfin"], dinitial_states=dinit)
    p.overwrite_dweight = 1
    stream = torch.cuda.current_stream().cuda_stream
    need = ctypes.c_size_t()
    assert lib.cc1d_bwd_workspace_bytes(ctypes.byref(p), ctypes.byref(need)) == 0
    if noalloc:
        st = lib.cc1d_bwd_noalloc(ctypes.byref(p), stream)
    else:
        ws = torch.empty(max(16, need.value), dtype=torch.uint8, device=dev)
        st = lib.cc1d_bwd(ctypes.byref(p), ws.data_ptr(), need.value, stream)
    assert st == 0, lib.cc1d_strerror(st)
    torch.cuda.synchronize()
    return (dx, dw, db, dinit), need.value


@pytest.mark.gpu
@pytest.mark.parametrize("channel_last", [True, False], ids=["cl", "cf"])
def test_no_alloc_backward_equals_backward_with_workspace(gpu_device, cc1d_lib, channel_last):
    lib = cabi.declare(cc1d_lib)
    dev = gpu_device
    # first a larger problem, then a smaller one on the same GPU's array; both need a workspace
    # (channel-first problems of fewer than 4096 channels are cut into several parts per channel)
    shapes = [(4, 1160, 1237, torch.bfloat16, channel_last), (2, 264, 333, torch.float16, channel_last)]
    needs = []
    for i, (B, D, L, dtype, cl) in enumerate(shapes):
        host, d = _problem(B, D, L, dtype, cl, 500 + i, dev, seq_idx=cl and i == 0)
        ref, need = _run(lib, d, dev, noalloc=False)
        got, _ = _run(lib, d, dev, noalloc=True)
        needs.append(need)
        assert 0 < need <= MAX_WS
        for a, r, what in zip(got, ref, ("dx", "dweight", "dbias", "dinitial_states")):
            assert (a is None) == (r is None)
            if a is not None:
                assert torch.equal(a, r), "%s of call %d differs from cc1d_bwd" % (what, i)
        rdx, rdw, rdb, _ = orc.bwd(host["x"], host["w"], host["b"], host["dout"], seq_idx=host["seq"],
                                   initial_states=host["init"], dfinal_states=host["dfin"], activation="silu")
        assert_close(got[0], rdx, dtype, "dx")
        assert_close(got[1], rdw, what="dweight", tol=TOL_W)
        assert_close(got[2], rdb, what="dbias", tol=TOL_W)
    assert needs[1] < needs[0]


@pytest.mark.gpu
def test_no_alloc_backward_without_workspace_need(gpu_device, cc1d_lib):
    """Channel-first rows of at most 64 vectors with 4096 channels and more are one part per
    channel: no workspace at all."""
    lib = cabi.declare(cc1d_lib)
    host, d = _problem(1, 4096, 504, torch.bfloat16, False, 510, gpu_device)
    ref, need = _run(lib, d, gpu_device, noalloc=False)
    got, _ = _run(lib, d, gpu_device, noalloc=True)
    assert need == 0
    for a, r in zip(got, ref):
        assert torch.equal(a, r)


def test_no_alloc_backward_refuses_what_does_not_fit(cc1d_lib):
    """Host only: a problem that needs more than the built-in array is refused before any GPU call
    (the pointers below are never dereferenced)."""
    lib = cabi.declare(cc1d_lib)
    B, D, L = 16, 5376, 2048
    class Shaped:                                       # a tensor's shape, strides and address, no storage
        dtype, shape = torch.bfloat16, (B, D, L)
        def __init__(self, nth): self.nth = nth
        def stride(self, ax): return (L * D, 1, D)[ax]  # channel-last
        def data_ptr(self): return (1 + self.nth) << 30 # 16-byte aligned, non-NULL, one GiB apart
    x, dout, dx = Shaped(0), Shaped(1), Shaped(2)
    w, b = torch.zeros(D, 4), torch.zeros(D)
    dw, db = torch.zeros(D, 4), torch.zeros(D)
    p = cabi.bwd_params(x, w, b, dout, dx, dw, db, True)
    need = ctypes.c_size_t()
    assert lib.cc1d_bwd_workspace_bytes(ctypes.byref(p), ctypes.byref(need)) == 0
    assert need.value > MAX_WS
    assert lib.cc1d_bwd_noalloc(ctypes.byref(p), None) == E_WORKSPACE_LIMIT
    assert b"built-in" in lib.cc1d_strerror(E_WORKSPACE_LIMIT)
    assert lib.cc1d_bwd_noalloc(None, None) == -1
