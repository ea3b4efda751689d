"""ctypes front of oracle/cc1d_oracle.c (double-precision scalar loops).  TEST
INFRASTRUCTURE ONLY — imported by tests/ and nothing else.

Every function takes torch CPU tensors in the logical (batch, dim, seqlen) order, widens
them to dense float32 (exact for fp16/bf16) and returns float64 tensors.
"""
import ctypes
import os
import subprocess

import numpy as np
import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libcc1d_oracle.so")
_lib = None


def build(force: bool = False) -> str:
    if force or not os.path.exists(_LIB_PATH) or \
            os.path.getmtime(_LIB_PATH) < os.path.getmtime(os.path.join(_HERE, "cc1d_oracle.c")):
        subprocess.run(["make", "-C", _HERE, "-B", "libcc1d_oracle.so"], check=True,
                       stdout=subprocess.DEVNULL)
    return _LIB_PATH


def lib():
    global _lib
    if _lib is None:
        _lib = ctypes.CDLL(build())
    return _lib


def _f32(t):
    return None if t is None else np.ascontiguousarray(t.detach().to(torch.float32).numpy())


def _i32(t):
    return None if t is None else np.ascontiguousarray(t.detach().to(torch.int32).numpy())


def _ptr(a):
    return None if a is None else a.ctypes.data_as(ctypes.c_void_p)


def fwd(x, weight, bias=None, seq_idx=None, initial_states=None, silu=False, return_final_states=False):
    B, D, L = x.shape
    W = weight.shape[1]
    xa, wa, ba, sa, ia = _f32(x), _f32(weight), _f32(bias), _i32(seq_idx), _f32(initial_states)
    out = np.empty((B, D, L), dtype=np.float64)
    fin = np.empty((B, D, W - 1), dtype=np.float64) if return_final_states else None
    lib().cc1d_oracle_fwd(_ptr(xa), _ptr(wa), _ptr(ba), _ptr(sa), _ptr(ia), B, D, L, W, int(silu),
                          _ptr(out), _ptr(fin))
    out = torch.from_numpy(out)
    return (out, torch.from_numpy(fin)) if return_final_states else out


def bwd(x, weight, bias, dout, seq_idx=None, initial_states=None, dfinal_states=None, silu=False):
    B, D, L = x.shape
    W = weight.shape[1]
    xa, wa, ba, da = _f32(x), _f32(weight), _f32(bias), _f32(dout)
    sa, ia, fa = _i32(seq_idx), _f32(initial_states), _f32(dfinal_states)
    dx = np.empty((B, D, L), dtype=np.float64)
    dw = np.empty((D, W), dtype=np.float64)
    db = np.empty((D,), dtype=np.float64) if bias is not None else None
    di = np.empty((B, D, W - 1), dtype=np.float64) if initial_states is not None else None
    lib().cc1d_oracle_bwd(_ptr(xa), _ptr(wa), _ptr(ba), _ptr(da), _ptr(sa), _ptr(ia), _ptr(fa),
                          B, D, L, W, int(silu), _ptr(dx), _ptr(dw), _ptr(db), _ptr(di))
    return (torch.from_numpy(dx), torch.from_numpy(dw),
            None if db is None else torch.from_numpy(db),
            None if di is None else torch.from_numpy(di))


def update(x, conv_state, weight, bias=None, silu=False, cache_seqlens=None, conv_state_indices=None):
    """Returns (out float64 (B, D, L), new_state float32 (SB, D, S)); conv_state is not modified."""
    B, D, L = x.shape
    W = weight.shape[1]
    S = conv_state.shape[-1]
    xa, wa, ba = _f32(x), _f32(weight), _f32(bias)
    st = _f32(conv_state).copy()
    ca, ia = _i32(cache_seqlens), _i32(conv_state_indices)
    out = np.empty((B, D, L), dtype=np.float64)
    lib().cc1d_oracle_update(_ptr(xa), _ptr(st), _ptr(wa), _ptr(ba), _ptr(ca), _ptr(ia),
                             B, D, L, W, S, int(silu), _ptr(out))
    return torch.from_numpy(out), torch.from_numpy(st)


def varlen_states(x, cu_seqlens, state_len):
    T, D = x.shape
    batch = cu_seqlens.shape[0] - 1
    xa = _f32(x)
    cu = np.ascontiguousarray(cu_seqlens.detach().to(torch.int64).numpy())
    st = np.empty((batch, D, state_len), dtype=np.float32)
    lib().cc1d_oracle_varlen_states(_ptr(xa), _ptr(cu), batch, D, state_len, _ptr(st))
    return torch.from_numpy(st)
