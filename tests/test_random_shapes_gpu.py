"""Seeded random small problems — odd channel counts (multiples of 8 that do not fill a
wavefront), sequence lengths around the width, every dtype, layout, state and seq_idx
combination — forward and backward against the oracle.  Complements the fixed grids of
test_fwd_gpu.py / test_bwd_gpu.py, which follow the reference's own parameter lists."""
import random

import pytest
import torch

from helpers import DTYPES, TOL_W, assert_close, gen, make_states, make_wb, make_x, random_seq_idx, to_dev_like
from oracle import causal_conv1d_oracle as orc

pytestmark = pytest.mark.gpu


def _cases(n):
    rnd = random.Random(20241125)
    out = []
    for i in range(n):
        out.append(dict(
            seed=i,
            batch=rnd.choice([1, 2, 3, 5]),
            dim=8 * rnd.choice([1, 2, 3, 5, 7, 9, 16, 33, 40]),
            seqlen=rnd.choice([1, 2, 3, 4, 5, 7, 8, 9, 15, 16, 17, 31, 33, 47, 63, 64, 65, 97, 130, 257]),
            width=rnd.choice([2, 3, 4]),
            dtype=rnd.choice(DTYPES),
            channel_last=rnd.random() < 0.6,
            bias=rnd.random() < 0.7,
            silu=rnd.random() < 0.7,
            mode=rnd.choice(["plain", "states", "init", "final", "seq", "seq_pad"]),
            sliced=rnd.random() < 0.5,
        ))
    return out


@pytest.mark.parametrize("c", _cases(160), ids=lambda c: "s%d" % c["seed"])
def test_random_problem_matches_oracle(pkg, gpu_device, c):
    dev = gpu_device
    g = gen(1000 + c["seed"])
    seq_mode = c["mode"].startswith("seq")
    cl = c["channel_last"] or seq_mode                      # seq_idx needs channel-last
    B, D, L, W, dtype = c["batch"], c["dim"], c["seqlen"], c["width"], c["dtype"]
    x = make_x(B, D, L, dtype, cl, g, sliced=c["sliced"])
    dout = make_x(B, D, L, dtype, cl, g, sliced=False)
    w, b = make_wb(D, W, c["bias"], g)
    act = "silu" if c["silu"] else None
    init = make_states(B, D, W - 1, dtype, g) if c["mode"] in ("states", "init") else None
    dfin = make_states(B, D, W - 1, dtype, g) if c["mode"] in ("states", "final") else None
    pad = c["mode"] == "seq_pad" and L >= 3
    seq = random_seq_idx(B, L, g, pad=pad) if seq_mode else None

    xd = to_dev_like(x, dev).requires_grad_()
    wd = w.to(dev).requires_grad_()
    bd = b.to(dev).requires_grad_() if b is not None else None
    idev = init.to(dev).requires_grad_() if init is not None else None
    res = pkg.causal_conv1d_fn(xd, wd, bd, seq_idx=None if seq is None else seq.to(dev), initial_states=idev,
                               return_final_states=dfin is not None, activation=act)
    if dfin is not None:
        out, fin = res
        torch.autograd.backward([out, fin], [to_dev_like(dout, dev), dfin.to(dev)])
    else:
        out = res
        out.backward(to_dev_like(dout, dev))

    if seq is not None:
        ref_out = orc.fwd_seq_idx(x, w, b, seq, activation=act)
        ref = orc.bwd(x, w, b, dout, seq_idx=seq, activation=act)
    else:
        r = orc.fwd(x, w, b, initial_states=init, return_final_states=dfin is not None, activation=act)
        ref_out = r[0] if dfin is not None else r
        if dfin is not None:
            assert torch.equal(fin.detach().cpu(), r[1])
        ref = orc.bwd(x, w, b, dout, initial_states=init, dfinal_states=dfin, activation=act)
    assert_close(out.detach(), ref_out, dtype, "out")
    if not pad:                                               # padding gradients: see test_bwd_gpu
        assert_close(xd.grad, ref[0].to(dtype), dtype, "dx")
        assert_close(wd.grad, ref[1], what="dweight", tol=TOL_W)
        if b is not None:
            assert_close(bd.grad, ref[2], what="dbias", tol=TOL_W)
        if init is not None:
            assert_close(idev.grad, ref[3].to(dtype), dtype, "dinitial_states")
