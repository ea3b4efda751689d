"""The three device operators as torch.library ops, and the allocating wrappers the autograd
layer calls.

Op names, argument order and ownership follow causal_conv1d/cpp_functions.py:11-183 of the
reference, because downstream code reaches the kernels through exactly these names
(torch.ops.DaoAILab._causal_conv1d_{fwd,bwd,update}_cpp): Python owns every output tensor, the
extension only writes into what it is given.  There is no fallback: without the compiled
module `causal_conv1d_cuda` this file does not import.
"""
from typing import Optional, Tuple

import torch
from torch import Tensor

import causal_conv1d_cuda as _ext  # noqa: F401  (loading it registers the DaoAILab ops with the dispatcher)

LIBRARY_NAME = "DaoAILab"
_Opt = Optional[Tensor]

# The ops are defined in C++ inside the extension (schema with the written arguments marked,
# a no-op meta kernel for tracing), so a call costs a dispatcher hop and no Python trampoline.
_causal_conv1d_fwd_cpp = torch.ops.DaoAILab._causal_conv1d_fwd_cpp
_causal_conv1d_bwd_cpp = torch.ops.DaoAILab._causal_conv1d_bwd_cpp
_causal_conv1d_update_cpp = torch.ops.DaoAILab._causal_conv1d_update_cpp
# Not an op of the reference: the backward with dweight / dbias as plain outputs, so that the
# wrapper below does not have to zero-fill them first (two small launches per backward call).
_causal_conv1d_bwd_overwrite_cpp = torch.ops.DaoAILab._causal_conv1d_bwd_overwrite_cpp
# Not an op of the reference either: the forward with `out` allocated in C++ (in x's layout) and
# returned, which saves the wrapper's empty_like.
_causal_conv1d_fwd_out_cpp = torch.ops.DaoAILab._causal_conv1d_fwd_out_cpp
# Also not an op of the reference: the decode step for x (batch, dim) or (batch, dim, seqlen) with
# the result allocated in C++, so that causal_conv1d_update is a single dispatcher hop.
_causal_conv1d_update_out_cpp = torch.ops.DaoAILab._causal_conv1d_update_out_cpp


def _states_like(x: Tensor, width: int) -> Tensor:
    """A (batch, dim, width-1) tensor with unit stride along dim, the layout the kernels
    write states in fastest."""
    batch, dim = x.shape[0], x.shape[1]
    return torch.empty(batch, width - 1, dim, device=x.device, dtype=x.dtype).transpose(1, 2)


# The ops below are called positionally on purpose: torch.compile rejects a keyword argument
# named `out` that is not contiguous, which a channel-last output never is.

def causal_conv1d_fwd_function(x: Tensor, weight: Tensor, bias: _Opt, seq_idx: _Opt, initial_states: _Opt,
                               final_states_out: _Opt, silu_activation: bool) -> Tensor:
    """Returns `out`, allocated in x's layout; `final_states_out`, if given, is filled too."""
    return _causal_conv1d_fwd_out_cpp(x, weight, bias, seq_idx, initial_states, final_states_out, silu_activation)


def causal_conv1d_bwd_function(x: Tensor, weight: Tensor, bias: _Opt, dout: Tensor, seq_idx: _Opt,
                               initial_states: _Opt, dfinal_states: _Opt, dx: _Opt,
                               return_dinitial_states: bool, silu_activation: bool) -> Tuple[_Opt, ...]:
    """Returns (dx, dweight, dbias, dinitial_states).  dx may be supplied by the caller; dweight
    and dbias are summed in fp32 (one buffer for both) and come back in the parameters' dtype."""
    dx = torch.empty_like(x) if dx is None else dx
    dim, width = weight.shape
    sums = torch.empty(dim * (width + (0 if bias is None else 1)), dtype=torch.float32, device=x.device)
    dweight32 = sums[:dim * width].view(dim, width)
    dbias32 = None if bias is None else sums[dim * width:]
    dinitial_states = _states_like(x, width) if return_dinitial_states else None
    _causal_conv1d_bwd_overwrite_cpp(x, weight, bias, dout, seq_idx, initial_states, dfinal_states,
                                     dx, dweight32, dbias32, dinitial_states, silu_activation)
    dbias = None if dbias32 is None else dbias32.type_as(bias)
    return dx, dweight32.type_as(weight), dbias, dinitial_states


def causal_conv1d_update_function(x: Tensor, conv_state: Tensor, weight: Tensor, bias: _Opt,
                                  silu_activation: bool, cache_seqlens: _Opt, conv_state_indices: _Opt) -> Tensor:
    """Allocates `out` like x; conv_state is advanced in place."""
    out = torch.empty_like(x)
    _causal_conv1d_update_cpp(x, conv_state, weight, bias, out, silu_activation, cache_seqlens, conv_state_indices)
    return out
