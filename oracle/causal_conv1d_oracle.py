"""CPU oracle for the causal depthwise conv1d hot path.  TEST INFRASTRUCTURE ONLY.

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may import this
module; no product code does, and the product never falls back to it.

It restates, in plain PyTorch, what the reference defines as the correct result:

  * forward ............ causal_conv1d_ref, causal_conv1d/causal_conv1d_interface.py:132-171
                         (compute in weight.dtype, F.conv1d with padding=W-1 and groups=dim,
                         slice to seqlen, optional SiLU, cast back to x.dtype)
  * seq_idx ............ independent convolutions per contiguous sub-sequence, as the
                         reference tests define it (tests/test_causal_conv1d.py:441-454),
                         exact zeros at padding positions (seq_idx < 0, :545-553);
                         `fwd_masked_taps` states the kernel's own rule
                         (csrc/causal_conv1d_fwd.cu:304-331) tap by tap
  * backward ........... torch.autograd through the forward oracle, as the reference tests
                         do (tests/test_causal_conv1d.py:121-137)
  * update ............. causal_conv1d_update_ref, causal_conv1d_interface.py:205-242,
                         extended with conv_state_indices the way
                         tests/test_causal_conv1d.py:185-321 exercise it
  * varlen states ...... causal_conv1d_varlen_states_ref,
                         causal_conv1d/causal_conv1d_varlen.py:67-86

How each function is pinned (see tests/test_oracle_pins.py): against the committed
fixtures in tests/golden/, against the independent plain-C restatement in
oracle/cc1d_oracle.c (scalar loops in double precision, closed-form gradients), against
closed forms (delta and all-ones kernels, linearity, causality, finite differences) and
against the identities that tie the operators together (chunked == unchunked through
final/initial states, step-by-step update == full forward, circular == linear).
No function here is "parity unpinned".
"""
from typing import List, Optional, Tuple

import torch
import torch.nn.functional as F


def _act(y: torch.Tensor, activation: Optional[str]) -> torch.Tensor:
    if activation not in (None, "silu", "swish"):
        raise NotImplementedError("activation must be None, silu, or swish")
    return y if activation is None else F.silu(y)


def fwd(x, weight, bias=None, initial_states=None, return_final_states=False, activation=None):
    """Dense forward.  x (B, D, L); weight (D, W); bias (D,); initial_states (B, D, W-1).
    Follows causal_conv1d_interface.py:152-171."""
    in_dtype = x.dtype
    L = x.shape[-1]
    D, W = weight.shape
    xc = x.to(weight.dtype)
    if initial_states is None:
        y = F.conv1d(xc, weight.unsqueeze(1), bias, padding=W - 1, groups=D)
    else:
        xc = torch.cat([initial_states.to(weight.dtype), xc], dim=-1)
        y = F.conv1d(xc, weight.unsqueeze(1), bias, padding=0, groups=D)
    y = _act(y[..., :L], activation).to(in_dtype)
    if not return_final_states:
        return y
    final_states = F.pad(xc, (W - 1 - xc.shape[-1], 0)).to(in_dtype)
    return y, final_states


def runs_of(seq_row: torch.Tensor) -> List[Tuple[int, int, int]]:
    """Contiguous runs (start, end, id) of one row of seq_idx."""
    vals = seq_row.tolist()
    runs, s = [], 0
    for t in range(1, len(vals) + 1):
        if t == len(vals) or vals[t] != vals[s]:
            runs.append((s, t, vals[s]))
            s = t
    return runs


def fwd_seq_idx(x, weight, bias, seq_idx, activation=None):
    """Packed sub-sequences: each contiguous run of equal seq_idx is convolved on its own
    (tests/test_causal_conv1d.py:448-454); runs with a negative id are padding and give
    exact zeros (:545-553).  Differentiable, so autograd yields the backward oracle."""
    B = x.shape[0]
    rows = []
    for b in range(B):
        pieces = []
        for (s, e, sid) in runs_of(seq_idx[b]):
            xs = x[b:b + 1, :, s:e]
            pieces.append(torch.zeros_like(xs) if sid < 0 else fwd(xs, weight, bias, activation=activation))
        rows.append(torch.cat(pieces, dim=2))
    return torch.cat(rows, dim=0)


def fwd_masked_taps(x, weight, bias, seq_idx, activation=None):
    """The kernel's rule stated tap by tap (csrc/causal_conv1d_fwd.cu:304-331): tap at
    position s feeds output t iff seq_idx[s] == seq_idx[t] (positions before 0 count as
    -1), and outputs with seq_idx[t] < 0 are exactly 0."""
    in_dtype = x.dtype
    B, D, L = x.shape
    W = weight.shape[1]
    xc = F.pad(x.to(weight.dtype), (W - 1, 0))
    sq = F.pad(seq_idx, (W - 1, 0), value=-1)
    y = torch.zeros(B, D, L, dtype=weight.dtype) if bias is None else bias.view(1, D, 1).expand(B, D, L).clone()
    cur = sq[:, W - 1:]
    for w in range(W):
        same = (sq[:, w:w + L] == cur).unsqueeze(1)
        y = y + weight[:, w].view(1, D, 1) * xc[:, :, w:w + L] * same
    y = _act(y, activation)
    y = torch.where((cur < 0).unsqueeze(1), torch.zeros_like(y), y)
    return y.to(in_dtype)


def bwd(x, weight, bias, dout, seq_idx=None, initial_states=None, dfinal_states=None, activation=None):
    """Gradients by autograd through the forward oracle, in weight.dtype (fp32 in every
    reference test).  Returns (dx, dweight, dbias, dinitial_states); dx / dinitial_states in
    x.dtype, dweight / dbias in weight.dtype, None where the input is absent."""
    xr = x.detach().clone().requires_grad_()
    wr = weight.detach().clone().requires_grad_()
    br = bias.detach().clone().requires_grad_() if bias is not None else None
    ir = initial_states.detach().clone().requires_grad_() if initial_states is not None else None
    if seq_idx is not None:
        out = fwd_seq_idx(xr, wr, br, seq_idx, activation=activation)
        out.backward(dout)
    elif dfinal_states is not None:
        out, fin = fwd(xr, wr, br, initial_states=ir, return_final_states=True, activation=activation)
        torch.autograd.backward([out, fin], [dout, dfinal_states])
    else:
        out = fwd(xr, wr, br, initial_states=ir, activation=activation)
        out.backward(dout)
    return (xr.grad, wr.grad, br.grad if br is not None else None,
            ir.grad if ir is not None else None)


def update(x, conv_state, weight, bias=None, activation=None, cache_seqlens=None,
           conv_state_indices=None):
    """Decode step; conv_state is advanced in place.  Linear and circular variants follow
    causal_conv1d_interface.py:229-239.  With conv_state_indices, entry b works on row
    conv_state_indices[b] of conv_state; a negative index yields zero output and leaves
    every row untouched (csrc/causal_conv1d_update.cu:43-54)."""
    in_dtype = x.dtype
    squeeze = x.dim() == 2
    if squeeze:
        x = x.unsqueeze(-1)
    B, D, L = x.shape
    W = weight.shape[1]
    S = conv_state.shape[-1]
    if conv_state_indices is not None:
        out = torch.zeros_like(x)
        valid = (conv_state_indices >= 0).nonzero().flatten().tolist()
        for b in valid:
            row = int(conv_state_indices[b])
            st = conv_state[row:row + 1].clone()
            cs = cache_seqlens[b:b + 1] if cache_seqlens is not None else None
            out[b:b + 1] = update(x[b:b + 1], st, weight, bias, activation, cs)
            conv_state[row:row + 1] = st
        return out.squeeze(-1) if squeeze else out
    assert conv_state.shape == (B, D, S) and weight.shape == (D, W)
    if cache_seqlens is None:
        window = torch.cat([conv_state, x], dim=-1).to(weight.dtype)
        conv_state.copy_(window[:, :, -S:])
    else:
        offs = torch.arange(-(W - 1), 0, dtype=torch.long)
        ridx = torch.remainder(offs.unsqueeze(0) + cache_seqlens.long().unsqueeze(1), S)
        ridx = ridx.unsqueeze(1).expand(-1, D, -1)
        window = torch.cat([conv_state.gather(2, ridx), x], dim=-1).to(weight.dtype)
        steps = torch.arange(L, dtype=torch.long)
        widx = torch.remainder(steps.unsqueeze(0) + cache_seqlens.long().unsqueeze(1), S)
        conv_state.scatter_(2, widx.unsqueeze(1).expand(-1, D, -1), x)
    y = F.conv1d(window, weight.unsqueeze(1), bias, padding=0, groups=D)[:, :, -L:]
    y = _act(y, activation).to(in_dtype)
    return y.squeeze(-1) if squeeze else y


def varlen_states(x, cu_seqlens, state_len: int):
    """states (batch, D, state_len): the last min(state_len, len_b) tokens of each packed
    sequence, right-aligned, zeros in front (causal_conv1d_varlen.py:79-85)."""
    _, D = x.shape
    batch = cu_seqlens.shape[0] - 1
    states = torch.zeros(batch, state_len, D, dtype=x.dtype).transpose(1, 2)
    for b in range(batch):
        end = int(cu_seqlens[b + 1])
        start = max(int(cu_seqlens[b]), end - state_len)
        if end > start:
            states[b, :, state_len - (end - start):] = x[start:end].T
    return states
