"""Causal depthwise conv1d for AMD MI355X (gfx950): same Python surface as
Dao-AILab/causal-conv1d 1.6.1 (causal_conv1d/__init__.py:1-3 of the reference)."""
__version__ = "1.6.1"

from causal_conv1d.causal_conv1d_interface import causal_conv1d_fn, causal_conv1d_update
from causal_conv1d.causal_conv1d_varlen import causal_conv1d_fwd_varlen_states, causal_conv1d_varlen_states

__all__ = ["causal_conv1d_fn", "causal_conv1d_update", "causal_conv1d_varlen_states",
           "causal_conv1d_fwd_varlen_states"]
