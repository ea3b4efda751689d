"""Writes tests/golden/cc1d_golden.npz: small input/output vectors for every operator of
the hot path, produced by the PyTorch oracle (oracle/causal_conv1d_oracle.py) on CPU.

The reference repository stores no golden vectors (its tests regenerate inputs on the
GPU and compare in-process), so these fixtures are this repository's own: they freeze the
oracle's answers so that neither the oracle nor the kernels can drift unnoticed.  They are
cross-checked against the independent C restatement in tests/test_oracle_pins.py.

16-bit tensors are stored as their raw bit patterns (uint16) next to a "<name>__dtype" tag.

Usage:  python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)

from oracle import causal_conv1d_oracle as orc  # noqa: E402

OUT = os.path.join(HERE, "cc1d_golden.npz")


def put(store, name, t):
    if t.dtype in (torch.float16, torch.bfloat16):
        store[name] = t.contiguous().view(torch.int16).numpy().view(np.uint16)
        store[name + "__dtype"] = np.array(str(t.dtype).replace("torch.", ""))
    else:
        store[name] = t.contiguous().numpy()


def gen(seed):
    g = torch.Generator()
    g.manual_seed(seed)
    return g


def main():
    store = {}

    # fwd_c1: forward, fp32 (2, 64, 512), channel-first, width 4, bias, SiLU.
    g = gen(1)
    x = torch.randn(2, 64, 512, generator=g)
    w = torch.rand(64, 4, generator=g) - 0.5
    b = torch.rand(64, generator=g) - 0.5
    put(store, "fwd_c1/x", x); put(store, "fwd_c1/weight", w); put(store, "fwd_c1/bias", b)
    put(store, "fwd_c1/out", orc.fwd(x, w, b, activation="silu"))

    # fwd_states: bf16, width 3, initial_states in, final_states out, no activation.
    g = gen(2)
    x = torch.randn(2, 16, 37, generator=g).to(torch.bfloat16)
    w = torch.rand(16, 3, generator=g) - 0.5
    b = torch.rand(16, generator=g) - 0.5
    init = torch.randn(2, 16, 2, generator=g).to(torch.bfloat16)
    out, fin = orc.fwd(x, w, b, initial_states=init, return_final_states=True)
    put(store, "fwd_states/x", x); put(store, "fwd_states/weight", w); put(store, "fwd_states/bias", b)
    put(store, "fwd_states/initial_states", init)
    put(store, "fwd_states/out", out); put(store, "fwd_states/final_states", fin)

    # fwd_seq: fp16, width 4, SiLU, packed sub-sequences with trailing padding (-1).
    g = gen(3)
    x = torch.randn(2, 16, 40, generator=g).to(torch.float16)
    w = torch.rand(16, 4, generator=g) - 0.5
    b = torch.rand(16, generator=g) - 0.5
    seq = torch.tensor([[0] * 7 + [1] * 1 + [2] * 20 + [3] * 12,
                        [0] * 18 + [1] * 15 + [-1] * 7], dtype=torch.int32)
    put(store, "fwd_seq/x", x); put(store, "fwd_seq/weight", w); put(store, "fwd_seq/bias", b)
    put(store, "fwd_seq/seq_idx", seq)
    put(store, "fwd_seq/out", orc.fwd_seq_idx(x, w, b, seq, activation="silu"))

    # bwd: fp32, width 4, SiLU, initial_states + dfinal_states.
    g = gen(4)
    x = torch.randn(2, 8, 33, generator=g)
    w = torch.rand(8, 4, generator=g) - 0.5
    b = torch.rand(8, generator=g) - 0.5
    init = torch.randn(2, 8, 3, generator=g)
    dout = torch.randn(2, 8, 33, generator=g)
    dfin = torch.randn(2, 8, 3, generator=g)
    dx, dw, db, di = orc.bwd(x, w, b, dout, initial_states=init, dfinal_states=dfin, activation="silu")
    for k, v in dict(x=x, weight=w, bias=b, initial_states=init, dout=dout, dfinal_states=dfin,
                     dx=dx, dweight=dw, dbias=db, dinitial_states=di).items():
        put(store, "bwd/" + k, v)

    # update_linear / update_circular: bf16, width 4, state_len 6, 2 steps.
    for name, circ in (("update_linear", False), ("update_circular", True)):
        g = gen(5 if not circ else 6)
        x = torch.randn(3, 16, 2, generator=g).to(torch.bfloat16)
        st = torch.randn(3, 16, 6, generator=g).to(torch.bfloat16)
        w = torch.rand(16, 4, generator=g) - 0.5
        b = torch.rand(16, generator=g) - 0.5
        cs = torch.tensor([0, 5, 1003], dtype=torch.int32) if circ else None
        st_new = st.clone()
        out = orc.update(x, st_new, w, b, activation="silu", cache_seqlens=cs)
        put(store, name + "/x", x); put(store, name + "/conv_state", st)
        put(store, name + "/weight", w); put(store, name + "/bias", b)
        if circ:
            put(store, name + "/cache_seqlens", cs)
        put(store, name + "/out", out); put(store, name + "/conv_state_after", st_new)

    # varlen_states: bf16, lengths include one shorter than state_len.
    g = gen(7)
    lens = torch.tensor([5, 1, 9, 2, 3])
    cu = torch.nn.functional.pad(lens.cumsum(0), (1, 0)).to(torch.int32)
    x = torch.randn(int(lens.sum()), 16, generator=g).to(torch.bfloat16)
    put(store, "varlen/x", x); put(store, "varlen/cu_seqlens", cu)
    put(store, "varlen/states", orc.varlen_states(x, cu, 3))

    np.savez_compressed(OUT, **store)
    print("wrote", OUT, os.path.getsize(OUT), "bytes,", len(store), "arrays")


if __name__ == "__main__":
    main()
