"""Taps and bias in x's own 16-bit type (a model cast to bf16 / fp16 as a whole), in fp32,
and in the other 16-bit type: forward with seq_idx, backward, and the decode step, for every
width and with and without bias.  The reference instantiates all nine type pairs
(csrc/causal_conv1d_fwd.cu:383-401, causal_conv1d_update.cu:118-136); its Python reference
computes in the weight's type, these kernels always in fp32, so the oracle is given the taps
widened to fp32 and the result is held to the tolerance of x's type."""
import pytest
import torch

from helpers import DTYPES, TOL_W, assert_close, gen, make_wb, make_x, random_seq_idx, to_dev_like
from oracle import causal_conv1d_oracle as orc

pytestmark = pytest.mark.gpu

PAIRS = [(torch.bfloat16, torch.bfloat16), (torch.float16, torch.float16), (torch.bfloat16, torch.float32),
         (torch.float32, torch.float32), (torch.float16, torch.bfloat16), (torch.float32, torch.float16)]


@pytest.mark.parametrize("width", [2, 3, 4])
@pytest.mark.parametrize("has_bias", [False, True])
@pytest.mark.parametrize("dtype,w_dtype", PAIRS)
def test_forward_backward_channel_last(pkg, gpu_device, dtype, w_dtype, has_bias, width):
    dev = gpu_device
    g = gen(width * 7 + int(has_bias))
    B, D, L = 2, 328, 300                      # 328 channels: one full and one partial wavefront of 8-byte lanes
    x = make_x(B, D, L, dtype, True, g)
    dout = make_x(B, D, L, dtype, True, g, sliced=False)
    w, b = make_wb(D, width, has_bias, g, w_dtype)
    seq = random_seq_idx(B, L, g)
    ref_out = orc.fwd_seq_idx(x, w.float(), None if b is None else b.float(), seq, activation="silu")
    ref = orc.bwd(x, w.float(), None if b is None else b.float(), dout, seq_idx=seq, activation="silu")

    xd = to_dev_like(x, dev).requires_grad_()
    wd = w.to(dev).requires_grad_()
    bd = b.to(dev).requires_grad_() if b is not None else None
    out = pkg.causal_conv1d_fn(xd, wd, bd, seq_idx=seq.to(dev), activation="silu")
    out.backward(to_dev_like(dout, dev))
    assert_close(out.detach(), ref_out, dtype, "out")
    assert_close(xd.grad, ref[0].to(dtype), dtype, "dx")
    assert wd.grad.dtype == w_dtype
    w_tol = TOL_W if w_dtype == torch.float32 else (1e-2, 5e-2)      # the gradient is rounded to the tap type
    assert_close(wd.grad.float(), ref[1], what="dweight", tol=w_tol)
    if b is not None:
        assert bd.grad.dtype == w_dtype
        assert_close(bd.grad.float(), ref[2], what="dbias", tol=w_tol)


@pytest.mark.parametrize("width", [2, 3, 4])
@pytest.mark.parametrize("has_bias", [False, True])
@pytest.mark.parametrize("circular", [False, True])
@pytest.mark.parametrize("seqlen", [1, 3, 8])
@pytest.mark.parametrize("dtype,w_dtype", PAIRS)
def test_decode_step(pkg, gpu_device, dtype, w_dtype, seqlen, circular, has_bias, width):
    dev = gpu_device
    g = gen(100 + width)
    B, D, S = 9, 328, 6
    x = torch.randn(B, D, generator=g).to(dtype) if seqlen == 1 else \
        torch.randn(B, seqlen, D, generator=g).to(dtype).transpose(1, 2)
    st = torch.randn(B, S, D, generator=g).to(dtype).transpose(1, 2)
    w, b = make_wb(D, width, has_bias, g, w_dtype)
    cs = torch.randint(0, 100, (B,), generator=g, dtype=torch.int32) if circular else None
    st_ref = st.clone()
    ref = orc.update(x, st_ref, w.float(), None if b is None else b.float(), activation="silu", cache_seqlens=cs)
    st_dev = to_dev_like(st, dev)
    got = pkg.causal_conv1d_update(to_dev_like(x, dev), st_dev, w.to(dev), None if b is None else b.to(dev), activation="silu",
                                   cache_seqlens=None if cs is None else cs.to(dev))
    assert torch.equal(st_dev.cpu(), st_ref), "conv_state must be bit-exact"
    assert_close(got, ref.to(dtype), dtype, "out")


@pytest.mark.parametrize("width,state_len", [(2, 2), (3, 3), (4, 3), (4, 4), (4, 8)])
@pytest.mark.parametrize("has_bias", [False, True])
@pytest.mark.parametrize("dtype,w_dtype", PAIRS)
def test_decode_step_contiguous_state(pkg, gpu_device, dtype, w_dtype, has_bias, width, state_len):
    """conv_state (batch, dim, state_len) contiguous (the row-state kernel): taps of every
    supported type, packed or as a strided view."""
    dev = gpu_device
    g = gen(200 + width + state_len)
    B, D = 9, 328
    x = torch.randn(B, D, generator=g).to(dtype)
    st = torch.randn(B, D, state_len, generator=g).to(dtype)
    w, b = make_wb(D, width, has_bias, g, w_dtype)
    for strided in (False, True):
        wd = w.to(dev)
        if strided:                                       # a column slice of a wider tensor: the general loader
            wide = torch.zeros(D, width + 3, dtype=w_dtype, device=dev)
            wide[:, 1:1 + width] = wd
            wd = wide[:, 1:1 + width]
        st_ref = st.clone()
        ref = orc.update(x, st_ref, w.float(), None if b is None else b.float(), activation="silu")
        st_dev = st.to(dev)
        got = pkg.causal_conv1d_update(x.to(dev), st_dev, wd, None if b is None else b.to(dev), activation="silu")
        assert torch.equal(st_dev.cpu(), st_ref), "conv_state must be bit-exact"
        assert_close(got, ref.to(dtype), dtype, "out")

