"""Seeded random cases against the oracle: shapes, dtypes, layouts and options drawn together, so
that combinations no hand-written grid lists still get exercised (the reference's tests walk
fixed grids, tests/test_causal_conv1d.py:50-137, 225-262, 426-557).  Every case prints nothing and
names itself in the assertion message; the seeds are fixed, so a failure reproduces.

Tolerances: helpers.TOL per dtype for out / dx / dinitial_states, helpers.TOL_W for dweight / dbias;
final_states and conv_state are raw copies and must be equal bit for bit."""
import random

import pytest
import torch

from helpers import TOL_W, assert_close, gen, make_states, make_wb, make_x, random_seq_idx, to_dev_like
from oracle import causal_conv1d_oracle as orc

pytestmark = pytest.mark.gpu

DTYPES = [torch.float32, torch.float16, torch.bfloat16]


def _draw_conv_case(rng, big):
    cl = rng.random() < 0.6
    if big:
        dim = rng.choice([1024, 2048, 2560, 5376]) if cl else rng.choice([512, 1024, 2048])
        seqlen = rng.choice([512, 1000, 1024, 2047, 2048, 4096])
        batch = rng.choice([1, 2, 4, 8])
        while batch * dim * seqlen > (24 << 20) and batch > 1:
            batch //= 2
    else:
        dim = rng.choice([8, 64, 72, 128, 192, 256, 320, 520, 1024]) if cl else rng.choice([1, 3, 17, 64, 130])
        seqlen = rng.choice([2, 3, 5, 8, 15, 16, 17, 31, 33, 48, 64, 100, 127, 128, 129, 255, 256, 511, 513, 1000, 1024, 1500, 2049])
        batch = rng.choice([1, 2, 3, 5])
    use_seq = cl and rng.random() < 0.5
    return dict(cl=cl, dim=dim, seqlen=seqlen, batch=batch, dtype=rng.choice(DTYPES), width=rng.choice([2, 3, 4]),
                silu=rng.random() < 0.7, has_bias=rng.random() < 0.8, use_seq=use_seq, pad=rng.random() < 0.5,
                use_states=(not use_seq) and rng.random() < 0.5, sliced=rng.random() < 0.3,
                backward=rng.random() < 0.4, final_only=rng.random() < 0.3)


def _run_conv_case(pkg, dev, c, seed):
    g = gen(seed)
    desc = "seed %d %r" % (seed, c)
    dtype, W, B, D, L = c["dtype"], c["width"], c["batch"], c["dim"], c["seqlen"]
    x = make_x(B, D, L, dtype, c["cl"], g, sliced=c["sliced"])
    w, b = make_wb(D, W, c["has_bias"], g)
    seq = random_seq_idx(B, L, g, pad=c["pad"]) if c["use_seq"] else None
    init = make_states(B, D, W - 1, dtype, g) if c["use_states"] else None
    act = "silu" if c["silu"] else None
    xd, wd = to_dev_like(x, dev), w.to(dev)
    bd = b.to(dev) if b is not None else None
    seqd = seq.to(dev) if seq is not None else None
    initd = init.to(dev) if init is not None else None
    if not c["backward"]:
        ret_final = (c["use_states"] or c["final_only"]) and not c["use_seq"]
        ref = (orc.fwd_seq_idx(x, w, b, seq, activation=act) if c["use_seq"]
               else orc.fwd(x, w, b, initial_states=init, return_final_states=ret_final, activation=act))
        got = pkg.causal_conv1d_fn(xd, wd, bd, seq_idx=seqd, initial_states=initd, return_final_states=ret_final, activation=act)
        if ret_final:
            assert_close(got[0], ref[0], dtype, desc + " out")
            assert torch.equal(got[1].cpu(), ref[1]), desc + " final_states"
        else:
            assert_close(got, ref, dtype, desc + " out")
        return
    dout = make_x(B, D, L, dtype, c["cl"], g, sliced=False)
    dfin = make_states(B, D, W - 1, dtype, g) if c["use_states"] else None
    rdx, rdw, rdb, rdi = orc.bwd(x, w, b, dout, seq_idx=seq, initial_states=init, dfinal_states=dfin, activation=act)
    xg, wg = xd.detach().requires_grad_(True), wd.detach().requires_grad_(True)
    bg = bd.detach().requires_grad_(True) if bd is not None else None
    ig = initd.detach().requires_grad_(True) if initd is not None else None
    out = pkg.causal_conv1d_fn(xg, wg, bg, seq_idx=seqd, initial_states=ig, return_final_states=c["use_states"], activation=act)
    if c["use_states"]:
        torch.autograd.backward([out[0], out[1]], [dout.to(dev), dfin.to(dev)])
    else:
        out.backward(dout.to(dev))
    assert_close(xg.grad, rdx, dtype, desc + " dx")
    assert_close(wg.grad, rdw, what=desc + " dweight", tol=TOL_W)
    if bg is not None:
        assert_close(bg.grad, rdb, what=desc + " dbias", tol=TOL_W)
    if ig is not None:
        assert_close(ig.grad, rdi, dtype, desc + " dinitial_states")


@pytest.mark.parametrize("block", range(4))
def test_random_forward_and_backward_cases(pkg, gpu_device, block):
    rng = random.Random(1000 + block)
    for case in range(60):
        _run_conv_case(pkg, gpu_device, _draw_conv_case(rng, big=False), (1000 + block) * 1000 + case)


@pytest.mark.parametrize("block", range(2))
def test_random_cases_at_launch_sizes_that_fill_the_chip(pkg, gpu_device, block):
    """Large enough for the launch rules that depend on how often a launch fills the chip (rows
    per run, workgroup order, parts per channel) to take their large-launch branches."""
    rng = random.Random(2000 + block)
    for case in range(12):
        _run_conv_case(pkg, gpu_device, _draw_conv_case(rng, big=True), (2000 + block) * 1000 + case)


@pytest.mark.parametrize("block", range(3))
def test_random_update_cases(pkg, gpu_device, block):
    rng = random.Random(3000 + block)
    dev = gpu_device
    for case in range(80):
        seed = (3000 + block) * 1000 + case
        g = gen(seed)
        dtype = rng.choice(DTYPES)
        W, B = rng.choice([2, 3, 4]), rng.choice([1, 2, 7, 8, 9, 33, 64, 256])
        D = rng.choice([4, 8, 64, 100, 256, 264, 1000, 1024, 5376])
        S = W - 1 + rng.choice([0, 0, 1, 5, 13])
        L = rng.choice([1, 1, 1, 2, 3, 4, 8, 9, 12])
        circ = rng.random() < 0.4 and L <= S          # a ring buffer takes at most state_len tokens a call
        idx, silu, has_bias = rng.random() < 0.3, rng.random() < 0.7, rng.random() < 0.8
        unit_dim = rng.random() < 0.7
        two_d = L == 1 and rng.random() < 0.5
        SB = B + rng.choice([0, 3, 17]) if idx else B
        desc = "seed %d %s W%d B%d D%d S%d L%d circ%d idx%d silu%d bias%d unit%d 2d%d" % (
            seed, dtype, W, B, D, S, L, circ, idx, silu, has_bias, unit_dim, two_d)
        if unit_dim:
            x = torch.randn(B, L, D, generator=g).to(dtype).transpose(1, 2)
            st = torch.randn(SB, S, D, generator=g).to(dtype).transpose(1, 2)
        else:
            x = torch.randn(B, D, L, generator=g).to(dtype)
            st = torch.randn(SB, D, S, generator=g).to(dtype)
        if two_d:
            x = x[:, :, 0]
        w, b = make_wb(D, W, has_bias, g)
        cs = torch.randint(0, 1000, (B,), generator=g, dtype=torch.int32) if circ else None
        ci = None
        if idx:
            ci = torch.randperm(SB, generator=g)[:B].to(torch.int32)
            if B > 2:
                ci[rng.randrange(B)] = -1
        st_ref = st.clone()
        ref = orc.update(x, st_ref, w, b, activation="silu" if silu else None, cache_seqlens=cs, conv_state_indices=ci)
        xd, std = to_dev_like(x, dev), to_dev_like(st, dev)
        got = pkg.causal_conv1d_update(xd, std, w.to(dev), b.to(dev) if b is not None else None, "silu" if silu else None,
                                       cs.to(dev) if cs is not None else None, ci.to(dev) if ci is not None else None)
        assert_close(got, ref, dtype, desc + " out")
        assert torch.equal(std.cpu(), st_ref), desc + " conv_state"
