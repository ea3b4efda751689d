"""Argument checks of the backward, update and varlen-states entry points, through the Python
API and the extension module: what the reference's host code refuses
(csrc/causal_conv1d.cpp:281-380 backward, :476-531 update; causal_conv1d_interface.py:191-192)
is refused here too, with a RuntimeError / NotImplementedError raised before anything is
launched, and the tensors involved stay as they were."""
import pytest
import torch

pytestmark = pytest.mark.gpu


def _ext():
    import causal_conv1d_cuda
    return causal_conv1d_cuda


def test_update_error_behaviour(pkg, gpu_device):
    d = gpu_device
    B, D, S, W = 2, 16, 4, 4
    x = torch.zeros(B, D, device=d, dtype=torch.bfloat16)
    state = torch.ones(B, D, S, device=d, dtype=torch.bfloat16)
    w = torch.zeros(D, W, device=d)
    with pytest.raises(NotImplementedError):
        pkg.causal_conv1d_update(x, state, w, activation="gelu")
    with pytest.raises(RuntimeError, match="dtype of x"):
        pkg.causal_conv1d_update(x, state.float(), w)
    with pytest.raises(RuntimeError, match="width - 1"):
        pkg.causal_conv1d_update(x, state[:, :, :2], w)
    with pytest.raises(RuntimeError, match="width between 2 and 4"):
        pkg.causal_conv1d_update(x, torch.ones(B, D, 8, device=d, dtype=torch.bfloat16), torch.zeros(D, 5, device=d))
    with pytest.raises(RuntimeError, match="shape"):
        pkg.causal_conv1d_update(x, state, torch.zeros(D + 8, W, device=d))
    with pytest.raises(RuntimeError, match="shape"):                      # state batch must match without indices
        pkg.causal_conv1d_update(x, torch.ones(B + 1, D, S, device=d, dtype=torch.bfloat16), w)
    with pytest.raises(RuntimeError, match="int32"):
        pkg.causal_conv1d_update(x, state, w, conv_state_indices=torch.zeros(B, dtype=torch.int64, device=d))
    with pytest.raises(RuntimeError, match="int32"):
        pkg.causal_conv1d_update(x, state, w, cache_seqlens=torch.zeros(B, dtype=torch.int64, device=d))
    with pytest.raises(RuntimeError, match="shape"):
        pkg.causal_conv1d_update(x, state, w, cache_seqlens=torch.zeros(B + 1, dtype=torch.int32, device=d))
    with pytest.raises(RuntimeError, match="dtype of weight"):
        pkg.causal_conv1d_update(x, state, w, torch.zeros(D, device=d, dtype=torch.bfloat16))
    with pytest.raises(RuntimeError, match="GPU"):
        pkg.causal_conv1d_update(x, state.cpu(), w)
    assert torch.equal(state, torch.ones_like(state))                      # nothing ran


def test_bwd_error_behaviour(pkg, gpu_device):
    d = gpu_device
    ext = _ext()
    B, D, L, W = 2, 16, 32, 4
    x = torch.zeros(B, L, D, device=d, dtype=torch.float16).transpose(1, 2)
    dout = torch.zeros_like(x)
    dx = torch.full_like(x, 3.0)
    w = torch.zeros(D, W, device=d)
    bias = torch.zeros(D, device=d)
    dw = torch.full((D, W), 7.0, device=d)
    db = torch.full((D,), 7.0, device=d)

    def call(**kw):
        a = dict(x=x, weight=w, bias=bias, dout=dout, seq_idx=None, initial_states=None, dfinal_states=None,
                 dx=dx, dweight=dw, dbias=db, dinitial_states=None, silu=True)
        a.update(kw)
        ext.causal_conv1d_bwd(a["x"], a["weight"], a["bias"], a["dout"], a["seq_idx"], a["initial_states"],
                              a["dfinal_states"], a["dx"], a["dweight"], a["dbias"], a["dinitial_states"], a["silu"])

    with pytest.raises(RuntimeError, match="together"):
        call(dbias=None)
    with pytest.raises(RuntimeError, match="dtype of x"):
        call(dout=dout.float())
    with pytest.raises(RuntimeError, match="dtype of x"):
        call(dx=dx.float())
    with pytest.raises(RuntimeError, match="float32"):
        call(dweight=dw.half())
    with pytest.raises(RuntimeError, match="float32"):
        call(dbias=db.half())
    with pytest.raises(RuntimeError, match="width between 2 and 4"):
        call(weight=torch.zeros(D, 5, device=d), dweight=torch.zeros(D, 5, device=d))
    with pytest.raises(RuntimeError, match="int32"):
        call(seq_idx=torch.zeros(B, L, dtype=torch.int64, device=d))
    with pytest.raises(RuntimeError, match="channel last"):
        xf = x.contiguous()
        call(x=xf, dout=dout.contiguous(), dx=torch.empty_like(xf), seq_idx=torch.zeros(B, L, dtype=torch.int32, device=d))
    with pytest.raises(RuntimeError, match="dtype of x"):
        call(initial_states=torch.zeros(B, W - 1, D, device=d).transpose(1, 2))
    with pytest.raises(RuntimeError, match="dtype of x"):
        call(dfinal_states=torch.zeros(B, W - 1, D, device=d).transpose(1, 2))
    with pytest.raises(RuntimeError, match="shape"):
        call(dout=dout[:, :, :-1])
    with pytest.raises(RuntimeError, match="GPU"):
        call(dout=dout.cpu())
    torch.cuda.synchronize()
    assert torch.equal(dx, torch.full_like(dx, 3.0))
    assert torch.equal(dw, torch.full_like(dw, 7.0)) and torch.equal(db, torch.full_like(db, 7.0))
    # the autograd path refuses what the reference's Python layer refuses
    xg = x.detach().clone().requires_grad_()
    with pytest.raises(NotImplementedError):
        pkg.causal_conv1d_fn(xg, w, bias, activation="tanh")


def test_varlen_states_error_behaviour(pkg, gpu_device):
    d = gpu_device
    ext = _ext()
    x = torch.zeros(40, 16, device=d, dtype=torch.bfloat16)
    cu = torch.tensor([0, 10, 40], dtype=torch.int32, device=d)
    states = torch.ones(2, 3, 16, device=d, dtype=torch.bfloat16).transpose(1, 2)
    with pytest.raises(RuntimeError, match="total_tokens, dim"):
        ext.causal_conv1d_varlen_states(x[None], cu, states, 3)
    with pytest.raises(RuntimeError, match="int32 or int64|int64"):
        ext.causal_conv1d_varlen_states(x, cu.to(torch.int16), states, 3)
    with pytest.raises(RuntimeError, match="dtype of x"):
        ext.causal_conv1d_varlen_states(x, cu, states.float(), 3)
    with pytest.raises(RuntimeError, match="contiguous"):
        ext.causal_conv1d_varlen_states(x, torch.zeros(6, dtype=torch.int32, device=d)[::2], states, 3)
    with pytest.raises(RuntimeError, match="GPU"):
        ext.causal_conv1d_varlen_states(x, cu.cpu(), states, 3)
    with pytest.raises(RuntimeError):
        ext.causal_conv1d_varlen_states(x, cu, states, 4)                  # states hold 3 columns
    torch.cuda.synchronize()
    assert torch.equal(states, torch.ones_like(states))
