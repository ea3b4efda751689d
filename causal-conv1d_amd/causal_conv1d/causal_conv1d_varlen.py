"""`causal_conv1d_varlen_states`: the last `state_len` tokens of every packed sequence, as the
conv_state a decode loop starts from.  Signature and output layout of
causal_conv1d/causal_conv1d_varlen.py:35-64 of the reference; the gather itself is a HIP kernel
of the extension (the reference launches a Triton kernel, :49-63).
`causal_conv1d_varlen_states_ref` (:67-86 there) states the same thing with slices.

`causal_conv1d_fwd_varlen_states` is an addition: the forward over a packed batch and this gather
in one call (one kernel launch), for the prefill -> decode hand-off where the reference's users
call `causal_conv1d_fn` and `causal_conv1d_varlen_states` one after the other."""
import torch
from torch import Tensor

import causal_conv1d_cuda as _ext


def _empty_states(x: Tensor, batch: int, state_len: int, zero: bool) -> Tensor:
    make = torch.zeros if zero else torch.empty
    return make(batch, state_len, x.shape[1], dtype=x.dtype, device=x.device).transpose(1, 2)


def causal_conv1d_varlen_states(x: Tensor, cu_seqlens: Tensor, state_len: int) -> Tensor:
    """x (total_tokens, dim): sequences packed back to back.  cu_seqlens (batch + 1,), int32 or
    int64, ascending from 0: sequence b is x[cu_seqlens[b] : cu_seqlens[b+1]].
    Returns states (batch, dim, state_len) (memory order batch, state_len, dim) holding each
    sequence's last state_len tokens right-aligned, zeros where the sequence is shorter.
    No backward."""
    batch = cu_seqlens.shape[0] - 1
    states = _empty_states(x, batch, state_len, zero=False)
    _ext.causal_conv1d_varlen_states(x, cu_seqlens.contiguous(), states, state_len)
    return states


def causal_conv1d_varlen_states_ref(x: Tensor, cu_seqlens: Tensor, state_len: int) -> Tensor:
    """The same gather in plain PyTorch on any device."""
    bounds = [int(v) for v in cu_seqlens]
    states = _empty_states(x, len(bounds) - 1, state_len, zero=True)
    for b, (lo, hi) in enumerate(zip(bounds[:-1], bounds[1:])):
        keep = min(state_len, hi - lo)
        if keep > 0:
            states[b, :, state_len - keep:] = x[hi - keep:hi].t()
    return states


def causal_conv1d_fwd_varlen_states(x: Tensor, weight: Tensor, bias, seq_idx, cu_seqlens: Tensor,
                                    state_len: int, activation=None):
    """Inference-only pair `causal_conv1d_fn(x, weight, bias, seq_idx=seq_idx, activation=...)`
    and `causal_conv1d_varlen_states(tokens_of(x), cu_seqlens, state_len)` as one call.

    x (batch, dim, seqlen) whose tokens lie back to back in memory (batch == 1, or
    x.stride(0) == seqlen * x.stride(2)); cu_seqlens counts tokens of that flattened
    (batch * seqlen, dim) view.  Channel-last x takes one kernel launch for both results.
    Returns (out, states): out like x, states (len(cu_seqlens) - 1, dim, state_len) with unit
    stride along dim.  No backward."""
    if activation not in (None, "silu", "swish"):
        raise NotImplementedError("activation must be None, silu, or swish")
    batch, dim, seqlen = x.shape
    if x.stride(1) != 1 and x.stride(2) != 1:
        x = x.contiguous()
    assert batch == 1 or x.stride(0) == seqlen * x.stride(2), "tokens of x must lie back to back"
    tokens = x.as_strided((batch * seqlen, dim), (x.stride(2), x.stride(1)), x.storage_offset())
    out = torch.empty_like(x)
    states = _empty_states(x, cu_seqlens.shape[0] - 1, state_len, zero=False)
    _ext.causal_conv1d_fwd_varlen_states(
        x.detach(), weight.detach(), None if bias is None else bias.detach().contiguous(),
        None if seq_idx is None else seq_idx.contiguous(), out, tokens.detach(), cu_seqlens.contiguous(),
        states, state_len, activation is not None)
    return out, states
