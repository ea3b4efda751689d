"""x as Mamba's in_proj leaves it: a (dim, batch, seqlen) tensor viewed as (batch, dim, seqlen), unit
stride along seqlen, the batch entries of one channel next to each other in memory
(mamba_ssm's "d (b l) -> b d l" rearrangement; the reference takes any strides with a unit one
along seqlen or dim, csrc/causal_conv1d.cpp:88-93).  The channel-first forward numbers its rows
batch-first for such tensors; results must not depend on that."""
import pytest
import torch

from helpers import DTYPES, TOL_W, assert_close, gen, make_states, make_wb
from oracle import causal_conv1d_oracle as orc

pytestmark = pytest.mark.gpu


def _view(batch, dim, seqlen, dtype, g):
    return torch.randn(dim, batch, seqlen, generator=g).to(dtype).permute(1, 0, 2)


@pytest.mark.parametrize("dtype", DTYPES, ids=["fp32", "fp16", "bf16"])
@pytest.mark.parametrize("width", [2, 4])
@pytest.mark.parametrize("batch,dim,seqlen", [(3, 40, 8), (5, 17, 100), (4, 64, 512), (2, 130, 520), (3, 96, 1001),
                                              (6, 72, 2048), (2, 33, 4104), (7, 256, 64)])
def test_forward_matches_oracle_and_the_dense_layout(pkg, gpu_device, batch, dim, seqlen, width, dtype):
    g = gen(batch * 1000 + seqlen)
    x = _view(batch, dim, seqlen, dtype, g)
    assert x.stride(2) == 1 and x.stride(0) < x.stride(1)
    w, b = make_wb(dim, width, True, g)
    init = make_states(batch, dim, width - 1, dtype, g)
    dev = gpu_device
    xd = torch.empty(dim, batch, seqlen, dtype=dtype, device=dev).permute(1, 0, 2)
    xd.copy_(x)
    assert xd.stride() == x.stride()
    ref, ref_fin = orc.fwd(x, w, b, initial_states=init, return_final_states=True, activation="silu")
    got, fin = pkg.causal_conv1d_fn(xd, w.to(dev), b.to(dev), initial_states=init.to(dev), return_final_states=True,
                                    activation="silu")
    assert got.stride() == xd.stride()
    assert_close(got, ref, dtype, "out")
    assert torch.equal(fin.cpu(), ref_fin)
    # the same numbers as from a dense (batch, dim, seqlen) copy of x, bit for bit
    dense, dense_fin = pkg.causal_conv1d_fn(xd.contiguous(), w.to(dev), b.to(dev), initial_states=init.to(dev),
                                            return_final_states=True, activation="silu")
    assert torch.equal(got, dense) and torch.equal(fin, dense_fin)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["fp32", "bf16"])
@pytest.mark.parametrize("batch,dim,seqlen", [(3, 40, 8), (4, 64, 512), (3, 96, 1001), (5, 72, 2048)])
def test_backward_matches_oracle(pkg, gpu_device, batch, dim, seqlen, dtype):
    g = gen(batch * 77 + seqlen)
    x, dout = _view(batch, dim, seqlen, dtype, g), _view(batch, dim, seqlen, dtype, g)
    w, b = make_wb(dim, 4, True, g)
    dev = gpu_device
    xd = torch.empty(dim, batch, seqlen, dtype=dtype, device=dev).permute(1, 0, 2)
    xd.copy_(x)
    doutd = torch.empty(dim, batch, seqlen, dtype=dtype, device=dev).permute(1, 0, 2)
    doutd.copy_(dout)
    rdx, rdw, rdb, _ = orc.bwd(x, w, b, dout, activation="silu")
    xg, wg, bg = xd.requires_grad_(True), w.to(dev).requires_grad_(True), b.to(dev).requires_grad_(True)
    pkg.causal_conv1d_fn(xg, wg, bg, activation="silu").backward(doutd)
    assert_close(xg.grad, rdx, dtype, "dx")
    assert_close(wg.grad, rdw, what="dweight", tol=TOL_W)
    assert_close(bg.grad, rdb, what="dbias", tol=TOL_W)
