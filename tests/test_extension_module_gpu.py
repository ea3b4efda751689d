"""Callers that bypass the Python package and import `causal_conv1d_cuda` directly, with the
positional signatures of the reference's pybind module (csrc/causal_conv1d.cpp:559-563,
149-157, 260-272, 465-474), plus the pre-allocated dx route of causal_conv1d_bwd_function
(causal_conv1d/cpp_functions.py:117-160) and the prefill -> decode hand-off
(varlen final states feeding causal_conv1d_update).
"""
import pytest
import torch

from helpers import assert_close, gen, make_wb, to_dev_like
from oracle import causal_conv1d_oracle as orc

pytestmark = pytest.mark.gpu


def test_module_exports_reference_functions(pkg):
    import causal_conv1d_cuda as ext
    for name in ("causal_conv1d_fwd", "causal_conv1d_bwd", "causal_conv1d_update", "causal_conv1d_varlen_states"):
        assert callable(getattr(ext, name))


def test_direct_fwd_bwd_update_calls(pkg, gpu_device):
    import causal_conv1d_cuda as ext
    dev = gpu_device
    g = gen(41)
    B, D, L, W = 2, 128, 300, 4
    x = torch.randn(B, L, D, generator=g).to(torch.float16).transpose(1, 2)
    dout = torch.randn(B, L, D, generator=g).to(torch.float16).transpose(1, 2)
    w, b = make_wb(D, W, True, g)
    xd, dd, wd, bd = to_dev_like(x, dev), to_dev_like(dout, dev), w.to(dev), b.to(dev)

    out = torch.empty_like(xd)
    assert ext.causal_conv1d_fwd(xd, wd, bd, None, None, out, None, True) is None
    assert_close(out, orc.fwd(x, w, b, activation="silu"), torch.float16, "out")

    dx = torch.full_like(xd, float("nan"))        # every element must be overwritten
    dw = torch.zeros(D, W, device=dev)
    db = torch.zeros(D, device=dev)
    assert ext.causal_conv1d_bwd(xd, wd, bd, dd, None, None, None, dx, dw, db, None, True) is None
    ref = orc.bwd(x, w, b, dout, activation="silu")
    assert_close(dx, ref[0].to(torch.float16), torch.float16, "dx")
    assert_close(dw, ref[1], what="dweight", tol=(1e-3, 1e-3))
    assert_close(db, ref[2], what="dbias", tol=(1e-3, 1e-3))

    state = torch.randn(B, W - 1, D, generator=g).to(torch.float16).transpose(1, 2)
    xs = torch.randn(B, 1, D, generator=g).to(torch.float16).transpose(1, 2)
    sd, xsd = to_dev_like(state, dev), to_dev_like(xs, dev)
    o = torch.empty_like(xsd)
    assert ext.causal_conv1d_update(xsd, sd, wd, bd, o, True, None, None) is None
    ref_state = state.clone()
    ref_o = orc.update(xs, ref_state, w, b, activation="silu")
    assert_close(o, ref_o, torch.float16, "update out")
    assert torch.equal(sd.cpu(), ref_state)


def test_bwd_function_fills_a_caller_owned_dx(pkg, gpu_device):
    from causal_conv1d.cpp_functions import causal_conv1d_bwd_function
    dev = gpu_device
    g = gen(42)
    x = torch.randn(2, 64, 500, generator=g)
    dout = torch.randn(2, 64, 500, generator=g)
    w, b = make_wb(64, 3, True, g)
    xd, dd, wd, bd = x.to(dev), dout.to(dev), w.to(dev), b.to(dev)
    mine = torch.empty_like(xd)
    dx, dw, db, dinit = causal_conv1d_bwd_function(xd, wd, bd, dd, None, None, None, mine, False, False)
    assert dx.data_ptr() == mine.data_ptr() and dinit is None
    ref = orc.bwd(x, w, b, dout)
    assert_close(mine, ref[0], torch.float32, "dx")
    assert_close(dw, ref[1], what="dweight", tol=(1e-3, 1e-3))
    assert_close(db, ref[2], what="dbias", tol=(1e-3, 1e-3))


def test_prefill_then_decode_equals_one_long_forward(pkg, gpu_device):
    """Packed prefill with seq_idx, conv_state from causal_conv1d_varlen_states, then token by
    token causal_conv1d_update: every sequence must see exactly what one forward over its
    whole length produces (the state gather and the state shift are copies, so bit-exact)."""
    dev = gpu_device
    g = gen(43)
    D, W, S = 256, 4, 3
    lens, extra = [37, 5, 2, 120], 6
    w, b = make_wb(D, W, True, g)
    wd, bd = w.to(dev), b.to(dev)
    full = [torch.randn(1, n + extra, D, generator=g).to(torch.bfloat16).transpose(1, 2).to(dev) for n in lens]
    whole = [pkg.causal_conv1d_fn(t, wd, bd, activation="silu") for t in full]

    packed = torch.cat([t[:, :, :n] for t, n in zip(full, lens)], dim=2).transpose(1, 2).contiguous().transpose(1, 2)
    seq = torch.cat([torch.full((n,), i, dtype=torch.int32) for i, n in enumerate(lens)]).unsqueeze(0).to(dev)
    cu = torch.tensor([0] + list(torch.tensor(lens).cumsum(0)), dtype=torch.int32, device=dev)
    out = pkg.causal_conv1d_fn(packed, wd, bd, seq_idx=seq, activation="silu")
    start = 0
    for t, n in zip(whole, lens):
        assert torch.equal(out[0, :, start:start + n], t[0, :, :n])
        start += n

    state = pkg.causal_conv1d_varlen_states(packed[0].transpose(0, 1), cu, S)      # (batch, dim, S)
    for step in range(extra):
        tok = torch.stack([t[0, :, n + step] for t, n in zip(full, lens)])         # (batch, dim)
        o = pkg.causal_conv1d_update(tok, state, wd, bd, activation="silu")
        for i, (t, n) in enumerate(zip(whole, lens)):
            assert torch.equal(o[i], t[0, :, n + step])


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("seqlen", [37, 300])
def test_channel_first_outputs_on_another_16_byte_grid(pkg, gpu_device, dtype, seqlen):
    """Caller-owned out / dx whose rows sit at other offsets inside their 16-byte vectors than the
    rows of x (a slice of a wider buffer): the channel-first kernels for that case must give
    what the same-grid kernels give."""
    import causal_conv1d_cuda as ext
    dev = gpu_device
    g = gen(43 + seqlen)
    B, D, W = 2, 24, 4
    x = torch.randn(B, D, seqlen, generator=g).to(dtype)
    dout = torch.randn(B, D, seqlen, generator=g).to(dtype)
    w, b = make_wb(D, W, True, g)
    xd, dd, wd, bd = x.to(dev), dout.to(dev), w.to(dev), b.to(dev)
    wide = torch.full((B, D, seqlen + 5), float("nan"), dtype=dtype, device=dev)
    out = wide[:, :, 3:3 + seqlen]                 # rows start 3 elements into the buffer's rows
    ext.causal_conv1d_fwd(xd, wd, bd, None, None, out, None, True)
    assert_close(out, orc.fwd(x, w, b, activation="silu"), dtype, "out")
    assert torch.isnan(wide[:, :, :3]).all() and torch.isnan(wide[:, :, 3 + seqlen:]).all()

    wide_dx = torch.full((B, D, seqlen + 5), float("nan"), dtype=dtype, device=dev)
    dx = wide_dx[:, :, 1:1 + seqlen]
    dw = torch.zeros(D, W, device=dev)
    db = torch.zeros(D, device=dev)
    ext.causal_conv1d_bwd(xd, wd, bd, dd, None, None, None, dx, dw, db, None, True)
    ref = orc.bwd(x, w, b, dout, activation="silu")
    assert_close(dx, ref[0], dtype, "dx")
    assert_close(dw, ref[1], what="dweight", tol=(1e-3, 1e-3))
    assert_close(db, ref[2], what="dbias", tol=(1e-3, 1e-3))
    assert torch.isnan(wide_dx[:, :, :1]).all() and torch.isnan(wide_dx[:, :, 1 + seqlen:]).all()
