"""Tensors with more than 2^31 elements: element offsets no longer fit 32 bits (the reference's
parameter block keeps uint32 strides, csrc/causal_conv1d.h:19-33).  The oracle cannot run at
this size in reasonable time, so the far end of the big tensor is checked against the same
kernel run on a small copy of that region, which the other tests pin to the oracle; equality
is bit-exact because the arithmetic per element is identical."""
import pytest
import torch

from helpers import gen, make_wb

pytestmark = pytest.mark.gpu


def _wb(dev, dim, width=4):
    w, b = make_wb(dim, width, True, gen(5))
    return w.to(dev), b.to(dev)


def test_channel_last_forward_backward_past_2_31_elements(pkg, gpu_device):
    dev = gpu_device
    dim, seqlen, tail = 1024, 2_200_000, 4096          # 2.25e9 elements, 4.5 GB in bf16
    w, b = _wb(dev, dim)
    x = torch.empty(1, seqlen, dim, dtype=torch.bfloat16, device=dev).transpose(1, 2)
    x[:, :, -tail - 3:].normal_(generator=None)
    x[:, :, :-tail - 3] = 0.5
    x.requires_grad_()
    out = pkg.causal_conv1d_fn(x, w, b, activation="silu")
    dout = torch.zeros_like(out)
    dout[:, :, -tail:] = torch.randn(1, tail, dim, device=dev, dtype=torch.bfloat16).transpose(1, 2)
    out.backward(dout)

    xs = x.detach()[:, :, -tail:].transpose(1, 2).contiguous().transpose(1, 2).requires_grad_()
    init = x.detach()[:, :, -tail - 3:-tail].transpose(1, 2).contiguous().transpose(1, 2)
    ds = dout[:, :, -tail:].transpose(1, 2).contiguous().transpose(1, 2)
    out_s = pkg.causal_conv1d_fn(xs, w, b, initial_states=init, activation="silu")
    out_s.backward(ds)
    assert torch.equal(out.detach()[:, :, -tail:], out_s.detach())
    assert torch.equal(x.grad[:, :, -tail:], xs.grad)
    assert torch.count_nonzero(x.grad[:, :, :-tail - 3]) == 0


def test_channel_first_forward_past_2_31_elements(pkg, gpu_device):
    dev = gpu_device
    batch, dim, seqlen = 3, 1024, 1_048_576            # 3.2e9 elements, 6.4 GB in fp16
    w, b = _wb(dev, dim)
    x = torch.empty(batch, dim, seqlen, dtype=torch.float16, device=dev)
    x[:2] = 0.25
    x[2].normal_()
    out = pkg.causal_conv1d_fn(x, w, b, activation="silu")
    small = pkg.causal_conv1d_fn(x[2:3, -64:].contiguous(), w[-64:].contiguous(), b[-64:].contiguous(), activation="silu")
    assert torch.equal(out[2:3, -64:], small)
