"""torch.library registration of the three mutating device ops and the allocating
wrappers around them.  Same op names, argument order and ownership rules as
causal_conv1d/cpp_functions.py:11-183 of the reference: Python allocates every output,
the extension only writes into them.

The extension module `causal_conv1d_cuda` is required: importing this file without it
raises ImportError (there is no fallback path).
"""
from typing import Optional, Tuple

import torch

import causal_conv1d_cuda

LIBRARY_NAME = "DaoAILab"


@torch.library.custom_op(
    f"{LIBRARY_NAME}::_causal_conv1d_fwd_cpp", mutates_args={"out", "final_states_out"}
)
def _causal_conv1d_fwd_cpp(
    x: torch.Tensor,
    weight: torch.Tensor,
    bias: Optional[torch.Tensor],
    seq_idx: Optional[torch.Tensor],
    initial_states: Optional[torch.Tensor],
    out: torch.Tensor,
    final_states_out: Optional[torch.Tensor],
    silu_activation: bool,
) -> None:
    causal_conv1d_cuda.causal_conv1d_fwd(
        x, weight, bias, seq_idx, initial_states, out, final_states_out, silu_activation
    )


@torch.library.custom_op(
    f"{LIBRARY_NAME}::_causal_conv1d_bwd_cpp",
    mutates_args={"dfinal_states", "dx", "dweight", "dbias", "dinitial_states"},
)
def _causal_conv1d_bwd_cpp(
    x: torch.Tensor,
    weight: torch.Tensor,
    bias: Optional[torch.Tensor],
    dout: torch.Tensor,
    seq_idx: Optional[torch.Tensor],
    initial_states: Optional[torch.Tensor],
    dfinal_states: Optional[torch.Tensor],
    dx: torch.Tensor,
    dweight: torch.Tensor,
    dbias: Optional[torch.Tensor],
    dinitial_states: Optional[torch.Tensor],
    silu_activation: bool,
) -> None:
    causal_conv1d_cuda.causal_conv1d_bwd(
        x, weight, bias, dout, seq_idx, initial_states, dfinal_states,
        dx, dweight, dbias, dinitial_states, silu_activation,
    )


@torch.library.custom_op(
    f"{LIBRARY_NAME}::_causal_conv1d_update_cpp", mutates_args={"out", "conv_state"}
)
def _causal_conv1d_update_cpp(
    x: torch.Tensor,
    conv_state: torch.Tensor,
    weight: torch.Tensor,
    bias: Optional[torch.Tensor],
    out: torch.Tensor,
    silu_activation: bool,
    cache_seqlens: Optional[torch.Tensor],
    conv_state_indices: Optional[torch.Tensor],
) -> None:
    causal_conv1d_cuda.causal_conv1d_update(
        x, conv_state, weight, bias, out, silu_activation, cache_seqlens, conv_state_indices
    )


def causal_conv1d_fwd_function(
    x: torch.Tensor,
    weight: torch.Tensor,
    bias: Optional[torch.Tensor],
    seq_idx: Optional[torch.Tensor],
    initial_states: Optional[torch.Tensor],
    final_states_out: Optional[torch.Tensor],
    silu_activation: bool,
) -> torch.Tensor:
    """out = empty_like(x), filled by the forward kernel (cpp_functions.py:94-114)."""
    out = torch.empty_like(x)
    # Positional on purpose: torch.compile rejects a keyword argument named `out` that is
    # not contiguous, which a channel-last output never is.
    _causal_conv1d_fwd_cpp(x, weight, bias, seq_idx, initial_states, out, final_states_out, silu_activation)
    return out


def causal_conv1d_bwd_function(
    x: torch.Tensor,
    weight: torch.Tensor,
    bias: Optional[torch.Tensor],
    dout: torch.Tensor,
    seq_idx: Optional[torch.Tensor],
    initial_states: Optional[torch.Tensor],
    dfinal_states: Optional[torch.Tensor],
    dx: Optional[torch.Tensor],
    return_dinitial_states: bool,
    silu_activation: bool,
) -> Tuple[Optional[torch.Tensor], ...]:
    """Allocates dx (unless given), fp32 zeroed dweight/dbias and a channel-last
    dinitial_states, runs the backward kernels and casts dweight/dbias to the
    parameter dtype (cpp_functions.py:117-160)."""
    batch, dim = x.shape[:2]
    width = weight.shape[-1]
    if dx is None:
        dx = torch.empty_like(x)
    dweight = torch.zeros_like(weight, dtype=torch.float32)
    dbias = torch.zeros_like(bias, dtype=torch.float32) if bias is not None else None
    dinitial_states = None
    if return_dinitial_states:
        dinitial_states = torch.empty(
            batch, width - 1, dim, device=x.device, dtype=x.dtype
        ).transpose(1, 2)
    _causal_conv1d_bwd_cpp(x, weight, bias, dout, seq_idx, initial_states, dfinal_states,
                           dx, dweight, dbias, dinitial_states, silu_activation)
    dweight = dweight.type_as(weight)
    if dbias is not None:
        dbias = dbias.type_as(bias)
    return dx, dweight, dbias, dinitial_states


def causal_conv1d_update_function(
    x: torch.Tensor,
    conv_state: torch.Tensor,
    weight: torch.Tensor,
    bias: Optional[torch.Tensor],
    silu_activation: bool,
    cache_seqlens: Optional[torch.Tensor],
    conv_state_indices: Optional[torch.Tensor],
) -> torch.Tensor:
    """out = empty_like(x); conv_state is advanced in place (cpp_functions.py:163-183)."""
    out = torch.empty_like(x)
    _causal_conv1d_update_cpp(x, conv_state, weight, bias, out, silu_activation, cache_seqlens, conv_state_indices)
    return out
