"""Varlen final-state gather: `causal_conv1d_varlen_states` with the signature and output
layout of causal_conv1d/causal_conv1d_varlen.py:35-64 of the reference, served by a HIP
kernel of the extension instead of a Triton kernel (Triton is not imported anywhere), and
the pure-PyTorch formula helper `causal_conv1d_varlen_states_ref` (:67-86)."""
import torch
from torch import Tensor

import causal_conv1d_cuda


def causal_conv1d_varlen_states(x: Tensor, cu_seqlens: Tensor, state_len: int) -> Tensor:
    """
    Forward pass only, does not support backward pass.
    Parameters:
        x: (total_tokens, dim)
        cu_seqlens: (batch + 1), int32 or int64, must already be sorted. The cumulative sum
            of the sequence lengths, starting from 0.
        state_len: int. For each cu_seqlens, how many elements from x should be copied to
            the state. If some of those elements belong to a different sequence, the value
            of the states will be zero.
    Return:
        states: (batch, dim, state_len), stored as (batch, state_len, dim)
    """
    _, dim = x.shape
    batch = cu_seqlens.shape[0] - 1
    cu_seqlens = cu_seqlens.contiguous()
    states = torch.empty(batch, state_len, dim, dtype=x.dtype, device=x.device).transpose(1, 2)
    causal_conv1d_cuda.causal_conv1d_varlen_states(x, cu_seqlens, states, state_len)
    return states


def causal_conv1d_varlen_states_ref(x: Tensor, cu_seqlens: Tensor, state_len: int) -> Tensor:
    """Pure-PyTorch statement of the gather (any device), same arguments and result."""
    _, dim = x.shape
    batch = cu_seqlens.shape[0] - 1
    states = torch.zeros(batch, state_len, dim, dtype=x.dtype, device=x.device).transpose(1, 2)
    for b in range(batch):
        end = int(cu_seqlens[b + 1])
        start = max(int(cu_seqlens[b]), end - state_len)
        if end > start:
            states[b, :, state_len - (end - start):] = x[start:end].T
    return states
