"""Problems with more work items than one grid holds are cut along the batch into slices that
fit, launched back to back (the reference's grid(batch, dim) launch has no ceiling on the batch,
csrc/causal_conv1d_fwd.cu:157-167).  The real ceiling is 2^31 threads; the "launch_limit_shift"
knob lowers it so that small tensors take the sliced path.  Batch entries are independent, so the
sliced result must equal the single launch: bit for bit for out, dx, the states and conv_state;
dweight / dbias, whose order of additions follows the slices, within their tolerance and equal
to the oracle."""
import ctypes

import pytest
import torch

import cabi
from helpers import TOL_W, assert_close, gen, make_states, make_wb, make_x, random_seq_idx
from oracle import causal_conv1d_oracle as orc

pytestmark = pytest.mark.gpu

TOO_LARGE = -16                     # CC1D_ERR_TOO_LARGE (include/cc1d.h)


class _Limit:
    """Context manager: one launch holds at most 2^(31 - shift) threads."""
    def __init__(self, lib, shift):
        self.lib, self.shift = lib, shift

    def __enter__(self):
        assert self.lib.cc1d_set_tunable(b"launch_limit_shift", self.shift) == 0

    def __exit__(self, *exc):
        self.lib.cc1d_set_tunable(b"launch_limit_shift", 0)


@pytest.mark.parametrize("channel_last", [False, True], ids=["cf", "cl"])
@pytest.mark.parametrize("seqlen", [40, 700])
def test_fwd_in_batch_slices(pkg, gpu_device, cc1d_lib, channel_last, seqlen):
    lib = cabi.declare(cc1d_lib)
    dev = gpu_device
    g = gen(31 + seqlen)
    B, D = 11, 136
    x = make_x(B, D, seqlen, torch.bfloat16, channel_last, g, sliced=False).to(dev)
    w, b = (t.to(dev) for t in make_wb(D, 4, True, g))
    init = make_states(B, D, 3, torch.bfloat16, g).to(dev)
    whole, whole_fin = pkg.causal_conv1d_fn(x, w, b, initial_states=init, return_final_states=True, activation="silu")
    seq = random_seq_idx(B, seqlen, g, pad=True).to(dev) if channel_last else None
    whole_seq = pkg.causal_conv1d_fn(x, w, b, seq_idx=seq, activation="silu") if channel_last else None
    # e.g. 2^31 >> 17 = 16384 threads per launch: a handful of batch entries, or one, at a time
    for shift in ((15, 17) if seqlen == 700 else (17, 19)):
        with _Limit(lib, shift):
            got, fin = pkg.causal_conv1d_fn(x, w, b, initial_states=init, return_final_states=True, activation="silu")
            got_seq = pkg.causal_conv1d_fn(x, w, b, seq_idx=seq, activation="silu") if channel_last else None
        assert torch.equal(got, whole) and torch.equal(fin, whole_fin)
        if channel_last:
            assert torch.equal(got_seq, whole_seq)
    ref, ref_fin = orc.fwd(x.cpu(), w.cpu(), b.cpu(), initial_states=init.cpu(), return_final_states=True, activation="silu")
    assert_close(whole, ref, torch.bfloat16, "out")
    assert torch.equal(whole_fin.cpu(), ref_fin)


@pytest.mark.parametrize("overwrite", [0, 1])
@pytest.mark.parametrize("L", [300, 1100])
@pytest.mark.parametrize("channel_last", [False, True], ids=["cf", "cl"])
def test_bwd_in_batch_slices(gpu_device, cc1d_lib, channel_last, L, overwrite):
    """L = 300: channel-first rows of at most 64 vectors (short-row kernel); 1100: tile kernel, three
    steps a row, one workspace plane per batch entry."""
    lib = cabi.declare(cc1d_lib)
    dev = gpu_device
    g = gen(57 + L)
    B, D = 9, 136
    x = make_x(B, D, L, torch.bfloat16, channel_last, g, sliced=False)
    dout = make_x(B, D, L, torch.bfloat16, channel_last, g, sliced=False)
    w, b = make_wb(D, 4, True, g)
    init, dfin = make_states(B, D, 3, torch.bfloat16, g), make_states(B, D, 3, torch.bfloat16, g)
    xd, doutd, wd, bd, initd, dfind = (t.to(dev) for t in (x, dout, w, b, init, dfin))
    stream = torch.cuda.current_stream().cuda_stream

    def run(shift):
        dx = torch.empty_like(xd)
        dinit = torch.empty(B, 3, D, device=dev, dtype=xd.dtype).transpose(1, 2)
        fill = float("nan") if overwrite else 0.0
        dw, db = torch.full((D, 4), fill, device=dev), torch.full((D,), fill, device=dev)
        p = cabi.bwd_params(xd, wd, bd, doutd, dx, dw, db, True, initial_states=initd, dfinal_states=dfind,
                            dinitial_states=dinit)
        p.overwrite_dweight = overwrite
        with _Limit(lib, shift):
            need = ctypes.c_size_t()
            assert lib.cc1d_bwd_workspace_bytes(ctypes.byref(p), ctypes.byref(need)) == 0
            ws = torch.empty(max(16, need.value), dtype=torch.uint8, device=dev)
            st = lib.cc1d_bwd(ctypes.byref(p), ws.data_ptr(), need.value, stream)
        assert st == 0, lib.cc1d_strerror(st)
        torch.cuda.synchronize()
        return dx, dw, db, dinit

    whole = run(0)
    rdx, rdw, rdb, rdi = orc.bwd(x, w, b, dout, initial_states=init, dfinal_states=dfin, activation="silu")
    # L = 300, channel-last: 5120 threads per batch entry (runs of 8 rows), five entries or two to a
    # launch; channel-first: 136 wavefronts per batch entry, two entries or one to a launch
    for shift in ((16, 17) if L == 300 else (15, 16)):
        got = run(shift)
        assert torch.equal(got[0], whole[0]) and torch.equal(got[3], whole[3])
        assert_close(got[1], rdw, what="dweight", tol=TOL_W)
        assert_close(got[2], rdb, what="dbias", tol=TOL_W)
    assert_close(whole[0], rdx, torch.bfloat16, "dx")
    assert_close(whole[1], rdw, what="dweight", tol=TOL_W)


@pytest.mark.parametrize("indices", [False, True])
@pytest.mark.parametrize("unit_stride_dim", [True, False], ids=["vec", "generic"])
@pytest.mark.parametrize("circular", [False, True])
def test_update_in_batch_slices(pkg, gpu_device, cc1d_lib, circular, unit_stride_dim, indices):
    """The kernels for more than eight tokens a call (16-byte lanes) and for arbitrary strides
    number their lanes in one dimension; the decode-step kernels proper have a two-dimensional
    grid and hand batches past its reach to these."""
    lib = cabi.declare(cc1d_lib)
    dev = gpu_device
    seqlen = 12
    g = gen(77 + seqlen)
    B, D, S, SB = 37, 264, 8, 50
    x = torch.randn(B, seqlen, D, generator=g).to(torch.bfloat16).transpose(1, 2).to(dev)
    state0 = torch.randn(SB if indices else B, S, D, generator=g).to(torch.bfloat16).transpose(1, 2).to(dev)
    if not unit_stride_dim:
        x, state0 = x.contiguous(), state0.contiguous()
    w, b = (t.to(dev) for t in make_wb(D, 4, True, g))
    cs = torch.randint(0, 1000, (B,), generator=g, dtype=torch.int32).to(dev) if circular else None
    idx = None
    if indices:
        idx = torch.randperm(SB, generator=g)[:B].to(torch.int32)
        idx[5] = -1
        idx = idx.to(dev)

    def run(shift):
        st = state0.transpose(1, 2).clone().transpose(1, 2) if unit_stride_dim else state0.clone()
        with _Limit(lib, shift):
            out = pkg.causal_conv1d_update(x, st, w, b, activation="silu", cache_seqlens=cs, conv_state_indices=idx)
        return out, st

    whole = run(0)
    # vec: 33 lanes per batch entry, generic: 264; 2^31 >> 21 = 1024 and >> 22 = 512 threads per launch
    for shift in (21, 22):
        got = run(shift)
        assert torch.equal(got[0], whole[0]) and torch.equal(got[1], whole[1])


@pytest.mark.parametrize("layout", ["step", "tokens", "rowstate"])
@pytest.mark.parametrize("circular", [False, True])
def test_decode_step_in_batch_slices(pkg, gpu_device, cc1d_lib, layout, circular):
    """The decode-step launchers proper: one token on a cache with unit stride along dim (step
    kernel), four tokens (multi-token kernel), one token on a contiguous (batch, dim, state_len)
    cache (row-state kernel).  Each answers "too large" against the lowered ceiling and the
    front slices the batch; out and conv_state must equal the single launch bit for bit."""
    if layout == "rowstate" and circular:
        pytest.skip("the row-state kernel shifts its cache; ring buffers take the other kernels")
    lib = cabi.declare(cc1d_lib)
    dev = gpu_device
    g = gen(91)
    B, D, W = 37, 256, 4
    S = 4 if layout == "rowstate" else 8 if circular else 3
    seqlen = 4 if layout == "tokens" else 1
    x = torch.randn(B, seqlen, D, generator=g).to(torch.bfloat16).transpose(1, 2).to(dev)
    if layout == "rowstate":
        state0 = torch.randn(B, D, S, generator=g).to(torch.bfloat16).to(dev)
        x = x.contiguous()
    else:
        state0 = torch.randn(B, S, D, generator=g).to(torch.bfloat16).transpose(1, 2).to(dev)
    w, b = (t.to(dev) for t in make_wb(D, W, True, g))
    cs = torch.randint(0, 1000, (B,), generator=g, dtype=torch.int32).to(dev) if circular else None

    def run(shift):
        st = state0.clone() if layout == "rowstate" else state0.transpose(1, 2).clone().transpose(1, 2)
        with _Limit(lib, shift):
            out = pkg.causal_conv1d_update(x, st, w, b, activation="silu", cache_seqlens=cs)
        return out, st

    whole = run(0)
    ref_state = state0.cpu().clone()
    ref = orc.update(x.cpu(), ref_state, w.cpu(), b.cpu(), activation="silu",
                     cache_seqlens=None if cs is None else cs.cpu())
    assert_close(whole[0], ref, torch.bfloat16, "out")
    assert torch.equal(whole[1].cpu(), ref_state)
    # the whole batch is 1280 threads (step: 64 lanes x 4 channels a block row, 8 batch entries a
    # block), about as many (tokens), 5120 (row-state: 128 channels x 4 batch entries a block);
    # the ceilings leave a few blocks, or one, to a launch
    for shift in {"step": (21, 22), "tokens": (21, 22), "rowstate": (19, 20, 21)}[layout]:
        got = run(shift)
        assert torch.equal(got[0], whole[0]) and torch.equal(got[1], whole[1]), "shift %d" % shift


def test_flat_forward_in_batch_slices(pkg, gpu_device, cc1d_lib):
    """Contiguous channel-first rows that are no whole number of vectors (the flat kernel reads the
    tensor as one array): sliced along the batch against the single launch."""
    lib = cabi.declare(cc1d_lib)
    dev = gpu_device
    g = gen(92)
    B, D, L = 11, 136, 100
    x = torch.randn(B, D, L, generator=g).to(torch.bfloat16).to(dev)
    w, b = (t.to(dev) for t in make_wb(D, 4, True, g))
    whole = pkg.causal_conv1d_fn(x, w, b, activation="silu")
    for shift in (15, 17):                              # 65536 and 16384 threads to a launch; the tensor has 149600 elements
        with _Limit(lib, shift):
            got = pkg.causal_conv1d_fn(x, w, b, activation="silu")
        assert torch.equal(got, whole), "shift %d" % shift
    assert_close(whole, orc.fwd(x.cpu(), w.cpu(), b.cpu(), activation="silu"), torch.bfloat16, "out")


def test_a_batch_entry_too_large_is_refused_before_anything_runs(gpu_device, cc1d_lib):
    """When even one batch entry exceeds the ceiling no slicing can help: the call answers
    CC1D_ERR_TOO_LARGE and has launched nothing -- out, dx, dweight keep what they held."""
    lib = cabi.declare(cc1d_lib)
    dev = gpu_device
    g = gen(93)
    B, D, L = 6, 136, 700
    for channel_last in (False, True):
        x = make_x(B, D, L, torch.bfloat16, channel_last, g, sliced=False).to(dev)
        dout = make_x(B, D, L, torch.bfloat16, channel_last, g, sliced=False).to(dev)
        w, b = (t.to(dev) for t in make_wb(D, 4, True, g))
        out = torch.full_like(x, 7.0)
        dx = torch.full_like(x, 7.0)
        dw, db = torch.full((D, 4), 7.0, device=dev), torch.full((D,), 7.0, device=dev)
        pf = cabi.fwd_params(x, w, b, out, True)
        pb = cabi.bwd_params(x, w, b, dout, dx, dw, db, True)
        with _Limit(lib, 24):                           # 128 threads to a launch: less than one batch entry needs
            assert lib.cc1d_fwd(ctypes.byref(pf), None) == TOO_LARGE
            need = ctypes.c_size_t()
            st = lib.cc1d_bwd_workspace_bytes(ctypes.byref(pb), ctypes.byref(need))
            ws = torch.empty(max(16, need.value if st == 0 else 1 << 20), dtype=torch.uint8, device=dev)
            assert lib.cc1d_bwd(ctypes.byref(pb), ws.data_ptr(), ws.numel(), None) == TOO_LARGE
        torch.cuda.synchronize()
        for t in (out, dx, dw, db):
            assert bool((t == 7.0).all()), "a refused call wrote to its outputs"
