"""Pins the CPU oracle (oracle/causal_conv1d_oracle.py) without a GPU.

Each test fixes the oracle from a direction that does not reuse its own formula:
closed forms (delta / all-ones kernels, linearity, causality), brute-force scalar loops in
double precision (oracle/cc1d_oracle.c, whose gradients are closed-form sums, not
autograd), finite differences, the identities tying the operators together (chunking
through states, update == forward, circular == linear), and the committed fixtures.
A dropped tap, a flipped kernel, an off-by-one in the state handling or a wrong mask
fails at least one of them.
"""
import math

import pytest
import torch
import torch.nn.functional as F

from oracle import causal_conv1d_oracle as orc
from oracle import c_oracle
from golden_io import load_case


def rnd(*shape, seed=0, dtype=torch.float32):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(*shape, generator=g).to(dtype)


# ----------------------------------------------------------------------------- forward
@pytest.mark.parametrize("W", [2, 3, 4])
def test_fwd_delta_kernel_is_a_shift(W):
    x = rnd(2, 5, 19, seed=W)
    for k in range(W):
        w = torch.zeros(5, W)
        w[:, k] = 1.0
        shift = W - 1 - k
        expect = F.pad(x, (shift, 0))[..., :19]
        assert torch.equal(orc.fwd(x, w), expect), f"tap {k} must read x[t-{shift}]"


@pytest.mark.parametrize("W", [2, 3, 4])
def test_fwd_ones_kernel_is_a_running_sum(W):
    x = torch.arange(1, 13, dtype=torch.float32).view(1, 1, 12)
    out = orc.fwd(x, torch.ones(1, W))
    cs = F.pad(x.cumsum(-1), (W, 0))
    expect = cs[..., W:] - cs[..., :-W]
    assert torch.allclose(out, expect, atol=1e-5)
    bias = torch.tensor([0.25])
    assert torch.allclose(orc.fwd(x, torch.ones(1, W), bias), expect + 0.25, atol=1e-5)


def test_fwd_silu_known_values():
    x = torch.tensor([[[0.0, 1.0, -1.0, 20.0, -20.0]]])
    w = torch.tensor([[0.0, 1.0]])
    out = orc.fwd(x, w, activation="silu")[0, 0]
    expect = [v / (1.0 + math.exp(-v)) for v in [0.0, 1.0, -1.0, 20.0, -20.0]]
    assert torch.allclose(out, torch.tensor(expect), atol=1e-6)
    assert torch.equal(orc.fwd(x, w, activation="swish"), orc.fwd(x, w, activation="silu"))
    with pytest.raises(NotImplementedError):
        orc.fwd(x, w, activation="relu")


def test_fwd_linearity_and_causality():
    x, y = rnd(2, 6, 23, seed=1), rnd(2, 6, 23, seed=2)
    w = rnd(6, 4, seed=3)
    assert torch.allclose(orc.fwd(2 * x - 3 * y, w), 2 * orc.fwd(x, w) - 3 * orc.fwd(y, w), atol=1e-5)
    x2 = x.clone()
    x2[:, :, 11] += 5.0
    a, b = orc.fwd(x, w, activation="silu"), orc.fwd(x2, w, activation="silu")
    assert torch.equal(a[..., :11], b[..., :11])
    assert not torch.equal(a[..., 11:15], b[..., 11:15])
    assert torch.equal(a[..., 15:], b[..., 15:])      # support is exactly W positions


@pytest.mark.parametrize("W", [2, 3, 4])
@pytest.mark.parametrize("silu", [False, True])
@pytest.mark.parametrize("with_init", [False, True])
def test_fwd_matches_c_scalar_loops(W, silu, with_init):
    x, w, b = rnd(2, 7, 21, seed=10 + W), rnd(7, W, seed=20), rnd(7, seed=30)
    init = rnd(2, 7, W - 1, seed=40) if with_init else None
    out, fin = orc.fwd(x, w, b, initial_states=init, return_final_states=True,
                       activation="silu" if silu else None)
    cout, cfin = c_oracle.fwd(x, w, b, initial_states=init, silu=silu, return_final_states=True)
    assert torch.allclose(out.double(), cout, atol=2e-6, rtol=1e-6)
    assert torch.equal(fin.double(), cfin)


@pytest.mark.parametrize("L", [1, 2, 3, 9])
def test_final_states_and_chunking(L):
    W = 4
    x, w, b = rnd(2, 5, L + 11, seed=L), rnd(5, W, seed=1), rnd(5, seed=2)
    init = rnd(2, 5, W - 1, seed=3)
    # final_states is the tail of [initial_states | x], also when the sequence is shorter
    head, fin = orc.fwd(x[..., :L], w, b, initial_states=init, return_final_states=True, activation="silu")
    assert torch.equal(fin, torch.cat([init, x[..., :L]], -1)[..., -(W - 1):])
    _, fin0 = orc.fwd(x[..., :L], w, b, return_final_states=True)
    assert torch.equal(fin0, F.pad(x[..., :L], (W - 1, 0))[..., -(W - 1):])
    # feeding final_states of the head as initial_states of the tail equals the unchunked run
    tail = orc.fwd(x[..., L:], w, b, initial_states=fin, activation="silu")
    whole = orc.fwd(x, w, b, initial_states=init, activation="silu")
    assert torch.allclose(torch.cat([head, tail], -1), whole, atol=1e-6)


def test_fwd_low_precision_rounds_once():
    x = rnd(2, 8, 33, seed=5, dtype=torch.bfloat16)
    w, b = rnd(8, 4, seed=6), rnd(8, seed=7)
    out = orc.fwd(x, w, b, activation="silu")
    assert out.dtype == torch.bfloat16
    exact = c_oracle.fwd(x, w, b, silu=True)
    assert torch.equal(out, exact.to(torch.float32).to(torch.bfloat16)) or \
        (out.double() - exact).abs().max() < 2 ** -6   # one bf16 ulp at |v| < 4


# ----------------------------------------------------------------------------- seq_idx
def _seq_case():
    x = rnd(3, 6, 29, seed=11)
    w, b = rnd(6, 4, seed=12), rnd(6, seed=13)
    seq = torch.tensor([[0] * 29,
                        [0] * 3 + [1] * 1 + [2] * 2 + [3] * 23,
                        [4] * 10 + [5] * 12 + [-1] * 7], dtype=torch.int32)
    return x, w, b, seq


@pytest.mark.parametrize("silu", [False, True])
def test_seq_idx_three_statements_agree(silu):
    x, w, b, seq = _seq_case()
    act = "silu" if silu else None
    per_segment = orc.fwd_seq_idx(x, w, b, seq, activation=act)
    masked = orc.fwd_masked_taps(x, w, b, seq, activation=act)
    scalar = c_oracle.fwd(x, w, b, seq_idx=seq, silu=silu)
    assert torch.allclose(per_segment, masked, atol=1e-6)
    assert torch.allclose(per_segment.double(), scalar, atol=2e-6)
    assert torch.equal(per_segment[0], orc.fwd(x[:1], w, b, activation=act)[0])   # one segment == dense
    assert torch.all(per_segment[2, :, 22:] == 0)                                  # padding is exact zero
    assert torch.equal(per_segment[1, :, 3:4], orc.fwd(x[1:2, :, 3:4], w, b, activation=act)[0])


# ---------------------------------------------------------------------------- backward
@pytest.mark.parametrize("W", [2, 3, 4])
@pytest.mark.parametrize("silu", [False, True])
@pytest.mark.parametrize("L", [1, 2, 17])
def test_bwd_autograd_matches_closed_form(W, silu, L):
    x, w, b = rnd(2, 5, L, seed=W), rnd(5, W, seed=1), rnd(5, seed=2)
    init, dout, dfin = rnd(2, 5, W - 1, seed=3), rnd(2, 5, L, seed=4), rnd(2, 5, W - 1, seed=5)
    act = "silu" if silu else None
    got = orc.bwd(x, w, b, dout, initial_states=init, dfinal_states=dfin, activation=act)
    ref = c_oracle.bwd(x, w, b, dout, initial_states=init, dfinal_states=dfin, silu=silu)
    for name, g, r in zip(("dx", "dweight", "dbias", "dinitial_states"), got, ref):
        assert torch.allclose(g.double(), r, atol=1e-5, rtol=1e-5), name
    got = orc.bwd(x, w, None, dout, activation=act)
    ref = c_oracle.bwd(x, w, None, dout, silu=silu)
    assert got[2] is None and got[3] is None
    assert torch.allclose(got[0].double(), ref[0], atol=1e-5, rtol=1e-5)
    assert torch.allclose(got[1].double(), ref[1], atol=1e-5, rtol=1e-5)


@pytest.mark.parametrize("silu", [False, True])
def test_bwd_seq_idx_autograd_matches_closed_form(silu):
    x, w, b, seq = _seq_case()
    dout = rnd(3, 6, 29, seed=14)
    got = orc.bwd(x, w, b, dout, seq_idx=seq, activation="silu" if silu else None)
    ref = c_oracle.bwd(x, w, b, dout, seq_idx=seq, silu=silu)
    for name, g, r in zip(("dx", "dweight", "dbias"), got, ref):
        assert torch.allclose(g.double(), r, atol=1e-5, rtol=1e-5), name
    assert torch.all(got[0][2, :, 22:] == 0)          # no gradient reaches padding tokens


def test_bwd_finite_differences_fp64():
    x = rnd(1, 2, 6, seed=1).double()
    w, b = rnd(2, 3, seed=2).double(), rnd(2, seed=3).double()
    init, dout, dfin = rnd(1, 2, 2, seed=4).double(), rnd(1, 2, 6, seed=5).double(), rnd(1, 2, 2, seed=6).double()

    def loss(x_, w_, b_, i_):
        o, f = orc.fwd(x_, w_, b_, initial_states=i_, return_final_states=True, activation="silu")
        return (o * dout).sum() + (f * dfin).sum()

    grads = orc.bwd(x, w, b, dout, initial_states=init, dfinal_states=dfin, activation="silu")
    eps = 1e-6
    for which, (t, g) in enumerate(zip((x, w, b, init), grads)):
        flat = t.reshape(-1)
        for i in range(flat.numel()):
            args = [x.clone(), w.clone(), b.clone(), init.clone()]
            args[which].reshape(-1)[i] += eps
            up = loss(*args)
            args[which].reshape(-1)[i] -= 2 * eps
            dn = loss(*args)
            assert abs((up - dn).item() / (2 * eps) - g.reshape(-1)[i].item()) < 1e-6


# ------------------------------------------------------------------------------ update
@pytest.mark.parametrize("W", [2, 3, 4])
@pytest.mark.parametrize("S_extra", [0, 1, 5])
def test_update_step_by_step_equals_forward(W, S_extra):
    S = W - 1 + S_extra
    x, w, b = rnd(2, 4, 9, seed=W), rnd(4, W, seed=1), rnd(4, seed=2)
    whole = orc.fwd(x, w, b, activation="silu")
    state = torch.zeros(2, 4, S)
    steps = [orc.update(x[..., t], state, w, b, activation="silu") for t in range(9)]
    assert torch.allclose(torch.stack(steps, -1), whole, atol=1e-6)
    assert torch.equal(state, F.pad(x, (S, 0))[..., -S:])
    # several tokens per call
    state2 = torch.zeros(2, 4, S)
    a = orc.update(x[..., :4], state2, w, b, activation="silu")
    c = orc.update(x[..., 4:], state2, w, b, activation="silu")
    assert torch.allclose(torch.cat([a, c], -1), whole, atol=1e-6)
    assert torch.equal(state2, state)


@pytest.mark.parametrize("W", [2, 3, 4])
def test_update_circular_equals_linear(W):
    S = 6
    x, w, b = rnd(3, 4, 11, seed=W), rnd(4, W, seed=1), rnd(4, seed=2)
    lin, circ = torch.zeros(3, 4, S), torch.zeros(3, 4, S)
    start = torch.tensor([0, 4, 1000], dtype=torch.int32)
    for t in range(11):
        a = orc.update(x[..., t], lin, w, b)
        c = orc.update(x[..., t], circ, w, b, cache_seqlens=start + t)
        assert torch.allclose(a, c, atol=1e-6)
    for bi in range(3):                                # same content, rotated by the write head
        head = (int(start[bi]) + 11) % S
        assert torch.equal(torch.roll(circ[bi], -head, dims=-1), lin[bi])


@pytest.mark.parametrize("circular", [False, True])
@pytest.mark.parametrize("L", [1, 4, 5])
def test_update_matches_c_scalar_loops(circular, L):
    W, S = 4, 7
    x, st = rnd(4, 6, L, seed=L, dtype=torch.bfloat16), rnd(9, 6, S, seed=1, dtype=torch.bfloat16)
    w, b = rnd(6, W, seed=2), rnd(6, seed=3)
    idx = torch.tensor([7, -1, 0, 3], dtype=torch.int32)
    cs = torch.tensor([5, 6, 1023, 0], dtype=torch.int32) if circular else None
    st_t = st.clone()
    out = orc.update(x, st_t, w, b, activation="silu", cache_seqlens=cs, conv_state_indices=idx)
    cout, cst = c_oracle.update(x, st, w, b, silu=True, cache_seqlens=cs, conv_state_indices=idx)
    assert torch.equal(st_t.float(), cst)                              # state moves are exact copies
    assert torch.all(out[1] == 0) and torch.equal(st_t[[1, 2, 4, 5, 6, 8]], st[[1, 2, 4, 5, 6, 8]])
    assert (out.double() - cout).abs().max() < 2 ** -5


# ----------------------------------------------------------------------- varlen states
def test_varlen_states_brute_force():
    lens = [5, 1, 9, 2, 3, 20]
    cu = torch.tensor([0] + list(torch.tensor(lens).cumsum(0)), dtype=torch.int64)
    x = rnd(sum(lens), 6, seed=9)
    S = 4
    got = orc.varlen_states(x, cu, S)
    assert got.shape == (6, 6, S) and got.stride(1) == 1
    for b, n in enumerate(lens):
        seq = x[int(cu[b]):int(cu[b + 1])]
        for s in range(S):
            src = n - (S - s)
            expect = seq[src] if src >= 0 else torch.zeros(6)
            assert torch.equal(got[b, :, s], expect)
    assert torch.equal(got, c_oracle.varlen_states(x, cu, S))
    assert torch.equal(got, orc.varlen_states(x, cu.to(torch.int32), S))


# ------------------------------------------------------------------- committed fixtures
def test_oracle_reproduces_golden_fixtures():
    c = load_case("fwd_c1")
    assert torch.allclose(orc.fwd(c["x"], c["weight"], c["bias"], activation="silu"), c["out"], atol=1e-6)
    c = load_case("fwd_states")
    out, fin = orc.fwd(c["x"], c["weight"], c["bias"], initial_states=c["initial_states"], return_final_states=True)
    assert torch.equal(out, c["out"]) and torch.equal(fin, c["final_states"])
    c = load_case("fwd_seq")
    assert torch.equal(orc.fwd_seq_idx(c["x"], c["weight"], c["bias"], c["seq_idx"], activation="silu"), c["out"])
    c = load_case("bwd")
    got = orc.bwd(c["x"], c["weight"], c["bias"], c["dout"], initial_states=c["initial_states"],
                  dfinal_states=c["dfinal_states"], activation="silu")
    for name, g in zip(("dx", "dweight", "dbias", "dinitial_states"), got):
        assert torch.allclose(g, c[name], atol=1e-6), name
    for case in ("update_linear", "update_circular"):
        c = load_case(case)
        st = c["conv_state"].clone()
        out = orc.update(c["x"], st, c["weight"], c["bias"], activation="silu", cache_seqlens=c.get("cache_seqlens"))
        assert torch.equal(out, c["out"]) and torch.equal(st, c["conv_state_after"])
    c = load_case("varlen")
    assert torch.equal(orc.varlen_states(c["x"], c["cu_seqlens"], 3), c["states"])


def test_golden_fixtures_match_c_scalar_loops():
    """The fixtures themselves are checked against the independent C restatement."""
    c = load_case("fwd_c1")
    assert torch.allclose(c["out"].double(), c_oracle.fwd(c["x"], c["weight"], c["bias"], silu=True), atol=2e-6)
    c = load_case("fwd_seq")
    ref = c_oracle.fwd(c["x"], c["weight"], c["bias"], seq_idx=c["seq_idx"], silu=True)
    assert (c["out"].double() - ref).abs().max() < 2 ** -8
    c = load_case("bwd")
    ref = c_oracle.bwd(c["x"], c["weight"], c["bias"], c["dout"], initial_states=c["initial_states"],
                       dfinal_states=c["dfinal_states"], silu=True)
    for name, r in zip(("dx", "dweight", "dbias", "dinitial_states"), ref):
        assert torch.allclose(c[name].double(), r, atol=1e-5, rtol=1e-5), name
    c = load_case("update_circular")
    out, st = c_oracle.update(c["x"], c["conv_state"], c["weight"], c["bias"], silu=True, cache_seqlens=c["cache_seqlens"])
    assert torch.equal(c["conv_state_after"].float(), st)
    assert (c["out"].double() - out).abs().max() < 2 ** -5
    c = load_case("varlen")
    assert torch.equal(c["states"].float(), c_oracle.varlen_states(c["x"], c["cu_seqlens"], 3))
