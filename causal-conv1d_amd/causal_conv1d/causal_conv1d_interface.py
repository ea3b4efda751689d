"""User-facing operators `causal_conv1d_fn` (differentiable) and `causal_conv1d_update`, with
the names, argument order, defaults, assertions and return conventions of
causal_conv1d/causal_conv1d_interface.py:9-129,174-202 of the reference, so that code written
against that package runs unchanged.

`causal_conv1d_ref` and `causal_conv1d_update_ref` (reference :132-171, :205-242) are kept
because downstream test-suites import them from here.  They state the operator as an explicit
sum of shifted, tap-weighted copies of the padded input in plain PyTorch; nothing on the GPU
path calls them.

One deliberate widening: `initial_states` and `return_final_states` also work for
channel-first x (the reference asserts channel-last, :39-42).
"""
import torch

from causal_conv1d.cpp_functions import (
    _causal_conv1d_update_out_cpp,
    _states_like,
    causal_conv1d_bwd_function,
    causal_conv1d_fwd_function,
    causal_conv1d_update_function,
)


def _wants_silu(activation):
    if activation is None:
        return False
    if activation in ("silu", "swish"):
        return True
    raise NotImplementedError("activation must be None, silu, or swish")


def _kernel_layout(t):
    """Unit stride along seqlen (channel-first) or along dim (channel-last); else a copy."""
    return t if 1 in (t.stride(1), t.stride(2)) else t.contiguous()


def _forward(x, weight, bias, seq_idx, initial_states, return_final_states, final_states_out, silu):
    """Checks, layouts and the device call of the forward; returns what backward needs too."""
    x = _kernel_layout(x)
    bias = None if bias is None else bias.contiguous()
    if seq_idx is not None:
        assert initial_states is None, "initial_states must be None if seq_idx is not None"
        assert not return_final_states, "If seq_idx is not None, we don't return final_states_out"
        seq_idx = seq_idx.contiguous()
    if initial_states is not None:
        initial_states = _kernel_layout(initial_states)
    if not return_final_states:
        final_states_out = None
    elif final_states_out is None:
        final_states_out = _states_like(x, weight.shape[1])
    else:
        assert 1 in (final_states_out.stride(1), final_states_out.stride(2))
    out = causal_conv1d_fwd_function(x, weight, bias, seq_idx, initial_states, final_states_out, silu)
    return out, final_states_out, (x, weight, bias, seq_idx, initial_states)


class CausalConv1dFn(torch.autograd.Function):
    """Forward and backward through the device ops; saves only the inputs (the pre-activation
    is recomputed in backward)."""

    @staticmethod
    def forward(ctx, x, weight, bias=None, seq_idx=None, initial_states=None,
                return_final_states=False, final_states_out=None, activation=None):
        silu = _wants_silu(activation)
        out, final_states_out, saved = _forward(x, weight, bias, seq_idx, initial_states, return_final_states,
                                                final_states_out, silu)
        ctx.save_for_backward(*saved)
        ctx.activation = silu
        ctx.return_final_states = return_final_states
        ctx.return_dinitial_states = saved[4] is not None and saved[4].requires_grad
        return (out, final_states_out) if return_final_states else out

    @staticmethod
    def backward(ctx, dout, *more):
        x, weight, bias, seq_idx, initial_states = ctx.saved_tensors
        dfinal_states = more[0] if ctx.return_final_states else None
        dx, dweight, dbias, dinitial_states = causal_conv1d_bwd_function(
            x, weight, bias, _kernel_layout(dout), seq_idx, initial_states, dfinal_states, None,
            ctx.return_dinitial_states, ctx.activation)
        # one gradient per forward argument: x, weight, bias, seq_idx, initial_states,
        # return_final_states, final_states_out, activation
        return dx, dweight, dbias, None, dinitial_states, None, None, None


def causal_conv1d_fn(x, weight, bias=None, seq_idx=None, initial_states=None,
                     return_final_states=False, final_states_out=None, activation=None):
    """out[b, c, t] = act(bias[c] + sum_w weight[c, w] * x[b, c, t - (width-1-w)]), zero (or
    initial_states) in front of the sequence.

    x (batch, dim, seqlen), channel-first or channel-last; weight (dim, width); bias (dim,).
    seq_idx (batch, seqlen) int32: taps never cross a change of id, negative ids are padding and
    produce zeros; excludes initial_states / return_final_states.
    initial_states (batch, dim, width-1); with return_final_states the result is
    (out, final_states), final_states (batch, dim, width-1) written to final_states_out if given.
    activation: None, "silu" or "swish".
    """
    wants_grad = torch.is_grad_enabled() and (
        x.requires_grad or weight.requires_grad or (bias is not None and bias.requires_grad)
        or (initial_states is not None and initial_states.requires_grad))
    if not wants_grad:
        # Inference: no graph to record, so no autograd.Function around the call (it costs 3.5 us
        # of host time, as much as the kernel at small shapes).
        out, final_states_out, _ = _forward(x, weight, bias, seq_idx, initial_states, return_final_states,
                                            final_states_out, _wants_silu(activation))
        return (out, final_states_out) if return_final_states else out
    return CausalConv1dFn.apply(x, weight, bias, seq_idx, initial_states, return_final_states,
                                final_states_out, activation)


def _tap_sum(window, weight, bias, n_out):
    """sum_w weight[:, w] * window[..., w : w + n_out] + bias, for a (batch, dim, n_out+width-1)
    window whose last column lines up with the last output."""
    width = weight.shape[1]
    acc = torch.zeros(window.shape[0], window.shape[1], n_out, dtype=weight.dtype, device=window.device)
    for w in range(width):
        acc = acc + window[..., w:w + n_out] * weight[:, w].reshape(1, -1, 1)
    return acc if bias is None else acc + bias.reshape(1, -1, 1)


def causal_conv1d_ref(x, weight, bias=None, initial_states=None, return_final_states=False,
                      final_states_out=None, activation=None):
    """The forward operator in plain PyTorch on any device: arithmetic in weight.dtype, result
    cast back to x.dtype.  Same arguments as causal_conv1d_fn minus seq_idx."""
    silu = _wants_silu(activation)
    width = weight.shape[1]
    seqlen = x.shape[-1]
    front = initial_states if initial_states is not None else x.new_zeros(x.shape[0], x.shape[1], width - 1)
    padded = torch.cat([front.to(weight.dtype), x.to(weight.dtype)], dim=-1)
    y = _tap_sum(padded, weight, bias, seqlen)
    if silu:
        y = y * torch.sigmoid(y)
    y = y.to(x.dtype)
    if not return_final_states:
        return y
    tail = padded[..., -(width - 1):].to(x.dtype)
    if final_states_out is None:
        final_states_out = tail
    else:
        final_states_out.copy_(tail)
    return y, final_states_out


def causal_conv1d_update(x, conv_state, weight, bias=None, activation=None, cache_seqlens=None,
                         conv_state_indices=None):
    """Decode step(s): the convolution over the last width-1 cached inputs followed by x, and
    the cache advanced in place.

    x (batch, dim) or (batch, dim, seqlen); conv_state (batch, dim, state_len), state_len >=
    width-1; weight (dim, width); bias (dim,).
    cache_seqlens (batch,) int32: conv_state is a ring buffer and x goes in at
    cache_seqlens % state_len; without it the cache is shifted left and x appended.
    conv_state_indices (batch,) int32: conv_state has its own, larger batch and entry b uses
    row conv_state_indices[b]; a negative index gives zeros and leaves the cache alone.
    Returns out shaped like x.
    """
    return _causal_conv1d_update_out_cpp(x, conv_state, weight, bias, _wants_silu(activation), cache_seqlens,
                                         conv_state_indices)


def causal_conv1d_update_ref(x, conv_state, weight, bias=None, activation=None, cache_seqlens=None):
    """The decode step in plain PyTorch on any device; conv_state is updated in place."""
    silu = _wants_silu(activation)
    single = x.dim() == 2
    xs = x.unsqueeze(-1) if single else x
    batch, dim, seqlen = xs.shape
    width = weight.shape[1]
    state_len = conv_state.shape[-1]
    assert conv_state.shape == (batch, dim, state_len) and weight.shape == (dim, width)
    if cache_seqlens is None:
        joined = torch.cat([conv_state, xs], dim=-1)
        recent = joined[..., -(width - 1 + seqlen):]
        conv_state.copy_(joined[..., -state_len:])
    else:
        pos = cache_seqlens.to(torch.long).reshape(batch, 1)
        back = torch.arange(-(width - 1), 0, device=xs.device).reshape(1, -1)
        ahead = torch.arange(seqlen, device=xs.device).reshape(1, -1)
        read = ((pos + back) % state_len).unsqueeze(1).expand(batch, dim, width - 1)
        write = ((pos + ahead) % state_len).unsqueeze(1).expand(batch, dim, seqlen)
        recent = torch.cat([conv_state.gather(2, read), xs], dim=-1)
        conv_state.scatter_(2, write, xs)
    y = _tap_sum(recent.to(weight.dtype), weight, bias, seqlen)
    if silu:
        y = y * torch.sigmoid(y)
    y = y.to(x.dtype)
    return y.squeeze(-1) if single else y
