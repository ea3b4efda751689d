"""User-facing operators: `causal_conv1d_fn` (autograd-enabled) and `causal_conv1d_update`,
with the signatures, defaults, assertions and return conventions of
causal_conv1d/causal_conv1d_interface.py:9-129,174-202 of the reference, plus the
pure-PyTorch formula helpers `causal_conv1d_ref` / `causal_conv1d_update_ref`
(:132-171, :205-242) that downstream test-suites import from here.  The helpers are
documentation-grade PyTorch and are never called by the GPU path.

One deliberate widening: `initial_states` and `return_final_states` also work for
channel-first x (the reference asserts channel-last, :39-42).
"""
import torch
import torch.nn.functional as F

from causal_conv1d.cpp_functions import (
    causal_conv1d_bwd_function,
    causal_conv1d_fwd_function,
    causal_conv1d_update_function,
)

_ACTIVATIONS = (None, "silu", "swish")


def _check_activation(activation):
    if activation not in _ACTIVATIONS:
        raise NotImplementedError("activation must be None, silu, or swish")
    return activation in ("silu", "swish")


def _dense_along_dim_or_seq(t):
    """The kernels need unit stride along seqlen (channel-first) or dim (channel-last)."""
    return t if (t.stride(2) == 1 or t.stride(1) == 1) else t.contiguous()


class CausalConv1dFn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, weight, bias=None, seq_idx=None, initial_states=None,
                return_final_states=False, final_states_out=None, activation=None):
        silu = _check_activation(activation)
        x = _dense_along_dim_or_seq(x)
        if bias is not None:
            bias = bias.contiguous()
        if seq_idx is not None:
            assert initial_states is None, "initial_states must be None if seq_idx is not None"
            assert not return_final_states, "If seq_idx is not None, we don't return final_states_out"
            seq_idx = seq_idx.contiguous()
        if initial_states is not None:
            initial_states = _dense_along_dim_or_seq(initial_states)
        if return_final_states:
            if final_states_out is not None:
                assert final_states_out.stride(2) == 1 or final_states_out.stride(1) == 1
            else:
                batch, dim, _ = x.shape
                width = weight.shape[1]
                final_states_out = torch.empty(
                    batch, width - 1, dim, device=x.device, dtype=x.dtype
                ).transpose(1, 2)
        else:
            final_states_out = None
        ctx.activation = silu
        out = causal_conv1d_fwd_function(
            x, weight, bias, seq_idx, initial_states, final_states_out, silu
        )
        ctx.save_for_backward(x, weight, bias, seq_idx, initial_states)
        ctx.return_final_states = return_final_states
        ctx.return_dinitial_states = initial_states is not None and initial_states.requires_grad
        return (out, final_states_out) if return_final_states else out

    @staticmethod
    def backward(ctx, dout, *args):
        x, weight, bias, seq_idx, initial_states = ctx.saved_tensors
        dfinal_states = args[0] if ctx.return_final_states else None
        dout = _dense_along_dim_or_seq(dout)
        dx, dweight, dbias, dinitial_states = causal_conv1d_bwd_function(
            x, weight, bias, dout, seq_idx, initial_states, dfinal_states, None,
            ctx.return_dinitial_states, ctx.activation,
        )
        return (
            dx,
            dweight,
            dbias if bias is not None else None,
            None,
            dinitial_states if initial_states is not None else None,
            None,
            None,
            None,
        )


def causal_conv1d_fn(x, weight, bias=None, seq_idx=None, initial_states=None,
                     return_final_states=False, final_states_out=None, activation=None):
    """
    x: (batch, dim, seqlen)
    weight: (dim, width)
    bias: (dim,)
    seq_idx: (batch, seqlen) int32; taps never cross a change of seq_idx, negative = padding
    initial_states: (batch, dim, width - 1)
    final_states_out: (batch, dim, width - 1), to be written to
    activation: either None or "silu" or "swish"

    out: (batch, dim, seqlen), or (out, final_states) if return_final_states
    """
    return CausalConv1dFn.apply(
        x, weight, bias, seq_idx, initial_states, return_final_states, final_states_out, activation
    )


def causal_conv1d_ref(x, weight, bias=None, initial_states=None, return_final_states=False,
                      final_states_out=None, activation=None):
    """Pure-PyTorch statement of the operator (any device).  Computes in weight.dtype and
    casts the result back to x.dtype.

    x: (batch, dim, seqlen); weight: (dim, width); bias: (dim,)
    initial_states / final_states_out: (batch, dim, width - 1)
    """
    silu = _check_activation(activation)
    in_dtype = x.dtype
    seqlen = x.shape[-1]
    dim, width = weight.shape
    xw = x.to(weight.dtype)
    if initial_states is None:
        y = F.conv1d(xw, weight.unsqueeze(1), bias, padding=width - 1, groups=dim)
    else:
        xw = torch.cat([initial_states, xw], dim=-1)
        y = F.conv1d(xw, weight.unsqueeze(1), bias, padding=0, groups=dim)
    y = y[..., :seqlen]
    if return_final_states:
        tail = F.pad(xw, (width - 1 - xw.shape[-1], 0)).to(in_dtype)  # (batch, dim, width - 1)
        if final_states_out is not None:
            final_states_out.copy_(tail)
        else:
            final_states_out = tail
    y = (F.silu(y) if silu else y).to(dtype=in_dtype)
    return (y, final_states_out) if return_final_states else y


def causal_conv1d_update(x, conv_state, weight, bias=None, activation=None, cache_seqlens=None,
                         conv_state_indices=None):
    """
    x: (batch, dim) or (batch, dim, seqlen)
    conv_state: (batch, dim, state_len), where state_len >= width - 1; updated in place
    weight: (dim, width)
    bias: (dim,)
    cache_seqlens: (batch,), dtype int32.
        If not None, the conv_state is treated as a circular buffer: x is copied into
        conv_state starting at index cache_seqlens % state_len.
    conv_state_indices: (batch,), dtype int32
        If not None, conv_state is a larger tensor along the batch dim and entry b uses
        row conv_state_indices[b] (negative = padding: zero output, state untouched).

    out: (batch, dim) or (batch, dim, seqlen)
    """
    silu = _check_activation(activation)
    squeeze = x.dim() == 2
    if squeeze:
        x = x.unsqueeze(-1)
    out = causal_conv1d_update_function(
        x, conv_state, weight, bias, silu, cache_seqlens, conv_state_indices
    )
    return out.squeeze(-1) if squeeze else out


def causal_conv1d_update_ref(x, conv_state, weight, bias=None, activation=None, cache_seqlens=None):
    """Pure-PyTorch statement of the decode step (any device); conv_state is updated in place.

    x: (batch, dim) or (batch, dim, seqlen); conv_state: (batch, dim, state_len)
    """
    silu = _check_activation(activation)
    in_dtype = x.dtype
    squeeze = x.dim() == 2
    if squeeze:
        x = x.unsqueeze(-1)
    batch, dim, seqlen = x.shape
    width = weight.shape[1]
    state_len = conv_state.shape[-1]
    assert conv_state.shape == (batch, dim, state_len)
    assert weight.shape == (dim, width)
    if cache_seqlens is None:
        window = torch.cat([conv_state, x], dim=-1).to(weight.dtype)
        conv_state.copy_(window[:, :, -state_len:])
    else:
        offs = torch.arange(-(width - 1), 0, dtype=torch.long, device=x.device)
        read_idx = torch.remainder(offs.unsqueeze(0) + cache_seqlens.unsqueeze(1), state_len)
        read_idx = read_idx.unsqueeze(1).expand(-1, dim, -1)
        window = torch.cat([conv_state.gather(2, read_idx), x], dim=-1).to(weight.dtype)
        steps = torch.arange(seqlen, dtype=torch.long, device=x.device)
        write_idx = torch.remainder(steps.unsqueeze(0) + cache_seqlens.unsqueeze(1), state_len)
        conv_state.scatter_(2, write_idx.unsqueeze(1).expand(-1, dim, -1), x)
    y = F.conv1d(window, weight.unsqueeze(1), bias, padding=0, groups=dim)[:, :, -seqlen:]
    if squeeze:
        y = y.squeeze(-1)
    return (F.silu(y) if silu else y).to(dtype=in_dtype)
