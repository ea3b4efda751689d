"""`causal_conv1d_varlen_states`: the last `state_len` tokens of every packed sequence, as the
conv_state a decode loop starts from.  Signature and output layout of
causal_conv1d/causal_conv1d_varlen.py:35-64 of the reference; the gather itself is a HIP kernel
of the extension (the reference launches a Triton kernel, :49-63).
`causal_conv1d_varlen_states_ref` (:67-86 there) states the same thing with slices."""
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
