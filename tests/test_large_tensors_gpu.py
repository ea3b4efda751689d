"""Tensors of more than 2^32 bytes (2^31 and more elements): every offset the kernels form from
batch, row and token strides must be a 64-bit one.  The reference carries 32-bit strides in its
argument block (csrc/causal_conv1d.h:9-50) and so has no test of this size; here the sizes and
strides of the C ABI are 64-bit and 288 GB of HBM make such tensors ordinary.

The big call is compared, bit for bit, with calls on views of its far end that are small enough
to sit below 2^31 elements from their own base pointer (such calls are what the other parity
tests check against the oracle), and one window of the far end is checked against the oracle
directly.  Inputs are drawn on the device: 5 GB of host random numbers would take minutes.
"""
import pytest
import torch

from helpers import TOL_W, assert_close, gen, make_wb
from oracle import causal_conv1d_oracle as orc

pytestmark = pytest.mark.gpu

GIB = 1 << 30


def _randn(shape, dtype, dev, seed):
    g = torch.Generator(device=dev)
    g.manual_seed(seed)
    return torch.randn(shape, generator=g, device=dev, dtype=dtype)


def _free():
    torch.cuda.synchronize()
    torch.cuda.empty_cache()


def test_fwd_channel_last_batch_offsets_past_4gib(pkg, gpu_device):
    dev, dt = gpu_device, torch.bfloat16
    B, L, D, W = 18, 32768, 4096, 4                      # 2^27 elements a batch: batch 16 starts at 2^32 bytes
    x = _randn((B, L, D), dt, dev, 1).transpose(1, 2)
    assert x.numel() * x.element_size() > 4 * GIB
    w, b = (t.to(dev) for t in make_wb(D, W, True, gen(2)))
    out = pkg.causal_conv1d_fn(x, w, b, activation="silu")
    for bb in (15, 16, 17):
        part = pkg.causal_conv1d_fn(x[bb:bb + 1], w, b, activation="silu")
        assert torch.equal(out[bb:bb + 1], part), "batch %d" % bb
    # the far corner against the oracle
    win = slice(L - 64, L)
    ref = orc.fwd(x[17:18, :, L - 64 - (W - 1):].cpu(), w.cpu(), b.cpu(), activation="silu")[:, :, W - 1:]
    assert_close(out[17:18, :, win], ref, dt, "far corner")
    del x, out, part
    _free()


def test_fwd_channel_last_row_offsets_past_4gib(pkg, gpu_device):
    dev, dt = gpu_device, torch.float16
    B, L, D, W = 1, 280000, 8192, 3                      # one batch row of 2.29e9 elements
    x = _randn((B, L, D), dt, dev, 3).transpose(1, 2)
    assert L * D > (1 << 31)
    w, b = (t.to(dev) for t in make_wb(D, W, True, gen(4)))
    seq = torch.zeros(B, L, dtype=torch.int32, device=dev)
    seq[:, 100000:] = 1
    seq[:, L - 1000:] = 2
    out = pkg.causal_conv1d_fn(x, w, b, seq_idx=seq, activation="silu")
    t1 = L - 4096                                        # a tail view: its first W-1 outputs see zeros instead
    part = pkg.causal_conv1d_fn(x[:, :, t1:], w, b, seq_idx=seq[:, t1:].contiguous(), activation="silu")
    assert torch.equal(out[:, :, t1 + W - 1:], part[:, :, W - 1:])
    ref = orc.fwd_seq_idx(x[:, :, L - 1100:].cpu(), w.cpu(), b.cpu(), seq[:, L - 1100:].cpu(), activation="silu")
    assert_close(out[:, :, L - 1090:], ref[:, :, 10:], dt, "tail with a boundary")
    del x, out, part, seq
    _free()


def test_fwd_bwd_channel_first_offsets_past_4gib(pkg, gpu_device):
    dev, dt = gpu_device, torch.bfloat16
    B, D, L, W = 3, 4096, 200000, 4                      # 8.2e8 elements a batch; batch 2 ends at 4.9e9 bytes
    x = _randn((B, D, L), dt, dev, 5)
    dout = _randn((B, D, L), dt, dev, 6)
    assert x.numel() > (1 << 31)
    w, b = (t.to(dev) for t in make_wb(D, W, True, gen(7)))

    def run(xs, ds):
        xs = xs.detach().requires_grad_()
        ws, bs = w.detach().requires_grad_(), b.detach().requires_grad_()
        out = pkg.causal_conv1d_fn(xs, ws, bs, activation="silu")
        out.backward(ds)
        return out.detach(), xs.grad, ws.grad, bs.grad

    out, dx, dw, db = run(x, dout)
    dw_parts, db_parts = torch.zeros_like(dw), torch.zeros_like(db)
    for bb in range(B):
        o1, dx1, dw1, db1 = run(x[bb:bb + 1], dout[bb:bb + 1])
        assert torch.equal(out[bb:bb + 1], o1), "out of batch %d" % bb
        assert torch.equal(dx[bb:bb + 1], dx1), "dx of batch %d" % bb
        dw_parts += dw1
        db_parts += db1
    # 6e5 terms per sum, in another order: relative to the size of the sums
    scale = dw_parts.abs().max().item()
    assert_close(dw / scale, dw_parts / scale, what="dweight", tol=TOL_W)
    assert_close(db / scale, db_parts / scale, what="dbias", tol=TOL_W)
    # last channels of the last batch row against the oracle
    xs, ds = x[2:3, D - 8:, L - 512:].cpu(), dout[2:3, D - 8:, L - 512:].cpu()
    r_dx = orc.bwd(xs, w[D - 8:].cpu(), b[D - 8:].cpu(), ds, activation="silu")[0]
    assert_close(dx[2:3, D - 8:, L - 500:], r_dx[:, :, 12:], dt, "dx far corner")
    del x, dout, out, dx
    _free()


def test_bwd_channel_last_offsets_past_4gib(pkg, gpu_device):
    dev, dt = gpu_device, torch.bfloat16
    B, L, D, W = 18, 32768, 4096, 4
    x = _randn((B, L, D), dt, dev, 8).transpose(1, 2)
    dout = _randn((B, L, D), dt, dev, 9).transpose(1, 2)
    w, b = (t.to(dev) for t in make_wb(D, W, True, gen(10)))
    seq = torch.zeros(B, L, dtype=torch.int32, device=dev)
    seq[:, 20000:] = 1

    def run(xs, ds, sq):
        xs = xs.detach().requires_grad_()
        ws, bs = w.detach().requires_grad_(), b.detach().requires_grad_()
        pkg.causal_conv1d_fn(xs, ws, bs, seq_idx=sq, activation="silu").backward(ds)
        return xs.grad, ws.grad, bs.grad

    dx, dw, db = run(x, dout, seq)
    for bb in (15, 16, 17):
        dx1, _, _ = run(x[bb:bb + 1], dout[bb:bb + 1], seq[bb:bb + 1])
        assert torch.equal(dx[bb:bb + 1], dx1), "dx of batch %d" % bb
    # dweight / dbias: every batch row counted once, none twice (a wrapped offset would repeat one)
    dw_parts, db_parts = torch.zeros_like(dw), torch.zeros_like(db)
    for lo in range(0, B, 6):
        _, dw1, db1 = run(x[lo:lo + 6], dout[lo:lo + 6], seq[lo:lo + 6])
        dw_parts += dw1
        db_parts += db1
    scale = dw_parts.abs().max().item()
    assert_close(dw / scale, dw_parts / scale, what="dweight", tol=TOL_W)
    assert_close(db / scale, db_parts / scale, what="dbias", tol=TOL_W)
    del x, dout, dx
    _free()


def test_update_state_rows_past_4gib(pkg, gpu_device):
    dev, dt = gpu_device, torch.bfloat16
    N, S, D, W, B = 40000, 16, 4096, 4, 8                # 2.6e9 elements of state
    state = _randn((N, S, D), dt, dev, 11).transpose(1, 2)
    assert state.numel() > (1 << 31)
    idx = torch.tensor([0, N - 1, 32768, 32767, -1, 39000, 16384, 1], dtype=torch.int32, device=dev)
    rows = idx.clamp(min=0).long()
    used = idx >= 0                                      # entry 4 is skipped by the kernel
    w, b = (t.to(dev) for t in make_wb(D, W, True, gen(12)))
    for circular in (False, True):
        x = _randn((B, D), dt, dev, 13 + circular)
        cache = torch.randint(0, 1000, (B,), dtype=torch.int32, device=dev) if circular else None
        small = state[rows].clone()                      # (B, D, S), contiguous: the kernel's other layout is
        small = small.transpose(1, 2).contiguous().transpose(1, 2)    # made the same as the big one's
        small_idx = torch.arange(B, dtype=torch.int32, device=dev)
        small_idx[4] = -1
        untouched = state[N // 2].clone()
        out = pkg.causal_conv1d_update(x, state, w, b, activation="silu", cache_seqlens=cache, conv_state_indices=idx)
        ref = pkg.causal_conv1d_update(x, small, w, b, activation="silu", cache_seqlens=cache,
                                       conv_state_indices=small_idx)
        assert torch.equal(out, ref)
        assert not out[4].any()
        assert torch.equal(state[rows][used], small[used])
        assert torch.equal(state[N // 2], untouched)
    del state
    _free()


def test_update_contiguous_state_past_4gib(pkg, gpu_device):
    """The (slots, dim, state_len) contiguous cache (unit stride along state_len) with slots whose
    byte offsets do not fit 32 bits, state_len 4 (16-byte accesses) and 3 (word accesses)."""
    dev, dt = gpu_device, torch.bfloat16
    D, W, B = 4096, 4, 8
    for S, N in ((4, 140000), (3, 180000)):              # 2.3e9 and 2.2e9 elements of state
        state = _randn((N, D, S), dt, dev, 21 + S)
        assert state.numel() > (1 << 31)
        idx = torch.tensor([0, N - 1, 131072, 131071, -1, 139000, 65536, 1], dtype=torch.int32, device=dev)
        rows = idx.clamp(min=0).long()
        used = idx >= 0
        w, b = (t.to(dev) for t in make_wb(D, W, True, gen(22)))
        x = _randn((B, D), dt, dev, 23)
        small = state[rows].clone()
        small_idx = torch.arange(B, dtype=torch.int32, device=dev)
        small_idx[4] = -1
        untouched = state[N // 2].clone()
        out = pkg.causal_conv1d_update(x, state, w, b, activation="silu", conv_state_indices=idx)
        ref = pkg.causal_conv1d_update(x, small, w, b, activation="silu", conv_state_indices=small_idx)
        assert torch.equal(out, ref)
        assert not out[4].any()
        assert torch.equal(state[rows][used], small[used])
        assert torch.equal(state[N // 2], untouched)
        # the small call against the oracle: the slots moved as the reference moves them
        st_cpu = _randn((4, D, S), dt, dev, 31).cpu()
        st_dev = st_cpu.to(dev)
        x4 = x[:4].cpu()
        ref4 = orc.update(x4, st_cpu, w.cpu(), b.cpu(), activation="silu")
        got4 = pkg.causal_conv1d_update(x4.to(dev), st_dev, w, b, activation="silu")
        assert torch.equal(st_dev.cpu(), st_cpu)
        assert_close(got4, ref4, dt, "out")
        del state
        _free()


def test_varlen_states_tokens_past_4gib(pkg, gpu_device):
    dev, dt = gpu_device, torch.bfloat16
    T, D, S = 1200000, 2048, 3                           # 2.46e9 elements
    x = _randn((T, D), dt, dev, 15)
    assert x.numel() > (1 << 31)
    ends = [5, 7, 600000, 1048576, 1048578, 1100000, T - 1, T]
    cu = torch.tensor([0] + ends, dtype=torch.int64, device=dev)
    got = pkg.causal_conv1d_varlen_states(x, cu, S)
    ref = torch.zeros(len(ends), D, S, dtype=dt, device=dev)
    start = 0
    for i, e in enumerate(ends):
        k = min(S, e - start)
        ref[i, :, S - k:] = x[e - k:e].T
        start = e
    assert torch.equal(got, ref)
    got32 = pkg.causal_conv1d_varlen_states(x, cu.to(torch.int32), S)
    assert torch.equal(got32, ref)
    del x
    _free()
