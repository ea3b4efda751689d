"""The reference's full parameter cross-product at dim 64 (tests/test_causal_conv1d.py:50-137):
seqlen x width x bias x SiLU x dtype x layout x initial_states x return_final_states, every
combination, forward and backward in one pass per case as the reference does it.  Where the
reference adds sigmoid(final_states) to the loss so that dfinal_states is not zero (:117-119),
this test hands the same random dfinal_states to both sides: built through the loss it is a sum
of dout over the whole sequence, which torch rounds differently on the GPU and on the CPU
(one 16-bit ulp of a value near 30 is already outside the tolerance of dx).  6,048 cases; one pytest
item per (dtype, layout) walks its 1,008 combinations and reports every failing one.  States
are also enumerated for channel-first, which the reference skips.

dim 4128 keeps the rotated grid of test_fwd_gpu.py / test_bwd_gpu.py.

The decode-step grids (:140-321) and the packed-sequence grids at dim 64 (:401-557) are enumerated
in full as well, below.

Tolerances as in those files: out / dx / dinitial_states fp32 1e-5 absolute, fp16 3e-3 / 5e-3,
bf16 1e-2 / 5e-2; dweight / dbias 1e-3 / 1e-3; final_states bit-exact.
"""
import itertools

import pytest
import torch

from helpers import DTYPES, TOL, TOL_W, gen, make_states, make_wb, make_x, random_seq_idx, to_dev_like
from oracle import causal_conv1d_oracle as orc

pytestmark = pytest.mark.gpu

SEQLENS = [1, 2, 8, 16, 32, 64, 128, 129, 130, 151, 256, 372, 512, 784, 1024, 1134, 2048, 4096]


def _outside(got, ref, rtol, atol):
    g, r = got.detach().float().cpu(), ref.detach().float().cpu()
    if g.shape != r.shape or not torch.isfinite(g).all():
        return True
    return bool(((g - r).abs() > atol + rtol * r.abs()).any())


@pytest.mark.parametrize("channel_last", [False, True], ids=["cf", "cl"])
@pytest.mark.parametrize("dtype", DTYPES, ids=lambda d: str(d)[6:])
def test_every_combination_at_dim_64(pkg, gpu_device, dtype, channel_last):
    dev = gpu_device
    dim, batch = 64, 2
    rtol, atol = TOL[dtype]
    failures, n = [], 0
    for seqlen, width, has_bias, silu, has_init, want_final in itertools.product(
            SEQLENS, (2, 3, 4), (False, True), (False, True), (False, True), (False, True)):
        n += 1
        g = gen(n * 13 + seqlen)
        x = make_x(batch, dim, seqlen, dtype, channel_last, g)
        w, b = make_wb(dim, width, has_bias, g)
        init = make_states(batch, dim, width - 1, dtype, g) if has_init else None
        dout = torch.randn(batch, dim, seqlen, generator=g).to(dtype)
        dfin = make_states(batch, dim, width - 1, dtype, g) if want_final else None
        act = "silu" if silu else None

        def run(fn, x_, w_, b_, init_, dout_, dfin_):
            x_ = x_.requires_grad_()
            w_ = w_.requires_grad_()
            b_ = b_.requires_grad_() if b_ is not None else None
            init_ = init_.requires_grad_() if init_ is not None else None
            res = fn(x_, w_, b_, initial_states=init_, return_final_states=want_final, activation=act)
            out, fin = res if want_final else (res, None)
            if fin is None:
                out.backward(dout_.to(out.dtype))
            else:
                torch.autograd.backward([out, fin], [dout_.to(out.dtype), dfin_.to(fin.dtype)])
            return (out, fin, x_.grad, w_.grad, None if b_ is None else b_.grad, None if init_ is None else init_.grad)

        ref = run(orc.fwd, x.detach().clone(), w.clone(), None if b is None else b.clone(),
                  None if init is None else init.detach().clone(), dout, dfin)
        got = run(pkg.causal_conv1d_fn, to_dev_like(x, dev), w.to(dev), None if b is None else b.to(dev),
                  None if init is None else init.to(dev), dout.to(dev), None if dfin is None else dfin.to(dev))
        bad = []
        names = ("out", "final_states", "dx", "dweight", "dbias", "dinitial_states")
        for name, a, r in zip(names, got, ref):
            if (a is None) != (r is None):
                bad.append(name + " presence")
            elif a is None:
                continue
            elif name == "final_states":
                if not torch.equal(a.cpu(), r.to(dtype)):
                    bad.append(name)
            elif name in ("dweight", "dbias"):
                if _outside(a, r, *TOL_W):
                    bad.append(name)
            elif _outside(a, r.to(dtype), rtol, atol):
                bad.append(name)
        if bad:
            failures.append("L%d w%d bias%d silu%d init%d final%d: %s" % (
                seqlen, width, has_bias, silu, has_init, want_final, ", ".join(bad)))
    assert n == len(SEQLENS) * 3 * 16
    assert not failures, "%d of %d combinations failed:\n%s" % (len(failures), n, "\n".join(failures[:40]))


def _segments(row):
    """[(start, end, id)] of the runs of equal ids in one row of seq_idx."""
    row = row.tolist()
    out, lo = [], 0
    for i in range(1, len(row) + 1):
        if i == len(row) or row[i] != row[lo]:
            out.append((lo, i, row[lo]))
            lo = i
    return out


@pytest.mark.parametrize("dtype", DTYPES, ids=lambda d: str(d)[6:])
def test_every_update_combination(pkg, gpu_device, dtype):
    """The reference's three decode-step grids in full (tests/test_causal_conv1d.py:140-321):
    dim x width x seqlen x cache_seqlens x bias x SiLU, each combination plain, through
    conv_state_indices into a larger cache, and with half the requests padding
    (index -1; the reference runs that one without cache_seqlens, here both).  648 cases per
    dtype; conv_state bit-exact, untouched rows untouched, padded outputs exactly zero."""
    dev = gpu_device
    rtol, atol = TOL[dtype]
    failures, n = [], 0
    batch = 64
    for dim, width, seqlen, circular, has_bias, silu in itertools.product(
            (2048, 2048 + 16, 4096), (2, 3, 4), (1, 4, 5), (False, True), (False, True), (False, True)):
        for variant in ("plain", "gather", "padding"):
            n += 1
            g = gen(n * 7 + dim)
            x = torch.randn(batch, seqlen, dim, generator=g).to(dtype).transpose(-1, -2)
            state_len = int(torch.randint(width - 1, width + 10, (1,), generator=g))
            entries = batch if variant == "plain" else 3 * batch    # (ten times in the reference: test_update_gpu.py keeps that)
            st = torch.randn(entries, state_len, dim, generator=g).to(dtype).transpose(-1, -2)
            w, b = make_wb(dim, width, has_bias, g)
            cs = torch.randint(0, 1024, (batch,), generator=g, dtype=torch.int32) if circular else None
            idx = None
            if variant != "plain":
                idx = torch.randperm(entries, generator=g)[:batch].to(torch.int32)
                if variant == "padding":
                    idx[torch.randperm(batch, generator=g)[:batch // 2]] = -1
            act = "silu" if silu else None
            st_ref = st.clone()
            ref = orc.update(x, st_ref, w, b, activation=act, cache_seqlens=cs, conv_state_indices=idx)
            st_dev = st.to(dev)
            got = pkg.causal_conv1d_update(x.to(dev), st_dev, w.to(dev), None if b is None else b.to(dev), activation=act,
                                           cache_seqlens=None if cs is None else cs.to(dev),
                                           conv_state_indices=None if idx is None else idx.to(dev))
            bad = []
            if not torch.equal(st_dev.cpu(), st_ref):
                bad.append("conv_state")
            if _outside(got, ref.to(dtype), rtol, atol):
                bad.append("out")
            if variant == "padding" and not bool((got.cpu()[idx < 0] == 0).all()):
                bad.append("padded outputs not zero")
            if bad:
                failures.append("%s d%d w%d l%d circ%d bias%d silu%d state_len %d: %s" % (
                    variant, dim, width, seqlen, circular, has_bias, silu, state_len, ", ".join(bad)))
    assert n == 3 * 3 * 3 * 8 * 3
    assert not failures, "%d of %d combinations failed:\n%s" % (len(failures), n, "\n".join(failures[:40]))


@pytest.mark.parametrize("dtype", DTYPES, ids=lambda d: str(d)[6:])
def test_every_varlen_combination_at_dim_64(pkg, gpu_device, dtype):
    """The reference's two packed-sequence grids at dim 64 in full
    (tests/test_causal_conv1d.py:401-472 forward and backward, :474-557 with padding): seqlen x width
    x bias x SiLU, batch 3, 1-4 cuts per row, x a channel slice of a wider channel-last tensor.
    The expected values come from independent convolutions of every sub-sequence, as there;
    padded positions (id -1) must hold exact zeros."""
    dev = gpu_device
    rtol, atol = TOL[dtype]
    failures, n = [], 0
    dim, batch = 64, 3
    grids = [(L, False) for L in (8, 16, 32, 64, 128, 151, 256, 372, 512, 784, 1024, 1134, 2048, 4096)] + \
            [(L, True) for L in (128, 256, 512, 1024)]
    for (seqlen, pad), width, has_bias, silu in itertools.product(grids, (2, 3, 4), (False, True), (False, True)):
        n += 1
        g = gen(n * 11 + seqlen)
        x = make_x(batch, dim, seqlen, dtype, True, g)
        w, b = make_wb(dim, width, has_bias, g)
        seq = random_seq_idx(batch, seqlen, g, max_splits=4, pad=pad)
        dout = torch.randn(batch, dim, seqlen, generator=g).to(dtype)
        act = "silu" if silu else None
        # expected: every sub-sequence on its own
        xr, wr = x.detach().clone().requires_grad_(), w.clone().requires_grad_()
        br = b.clone().requires_grad_() if b is not None else None
        rows = []
        for bi in range(batch):
            parts = []
            for lo, hi, sid in _segments(seq[bi]):
                seg = orc.fwd(xr[bi:bi + 1, :, lo:hi], wr, br, activation=act)
                parts.append(seg if sid >= 0 else torch.zeros_like(seg))
            rows.append(torch.cat(parts, dim=2))
        ref = torch.cat(rows, dim=0)
        xg, wg = to_dev_like(x, dev).requires_grad_(), w.to(dev).requires_grad_()
        bg = b.to(dev).requires_grad_() if b is not None else None
        got = pkg.causal_conv1d_fn(xg, wg, bg, seq_idx=seq.to(dev), activation=act)
        bad = []
        if _outside(got, ref.to(dtype), rtol, atol):
            bad.append("out")
        if pad and not bool((got.detach().cpu()[(seq < 0).unsqueeze(1).expand(-1, dim, -1)] == 0).all()):
            bad.append("padded outputs not zero")
        if not pad:                                     # the reference checks the backward without padding only
            ref.backward(dout.to(ref.dtype))
            got.backward(dout.to(dev))
            if _outside(xg.grad, xr.grad.to(dtype), rtol, atol):
                bad.append("dx")
            if _outside(wg.grad, wr.grad, *TOL_W):
                bad.append("dweight")
            if b is not None and _outside(bg.grad, br.grad, *TOL_W):
                bad.append("dbias")
        if bad:
            failures.append("L%d pad%d w%d bias%d silu%d: %s" % (seqlen, pad, width, has_bias, silu, ", ".join(bad)))
    assert n == 18 * 3 * 4
    assert not failures, "%d of %d combinations failed:\n%s" % (len(failures), n, "\n".join(failures[:40]))
