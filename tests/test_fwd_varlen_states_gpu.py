"""Forward over a packed batch plus the varlen final-state gather as one call
(cc1d_fwd_varlen_states / causal_conv1d_fwd_varlen_states): the results must be exactly those of
the two separate calls, which the other test files pin against the oracle, and the oracle's
directly.  The reference has no such call; its users issue causal_conv1d_fn
(causal_conv1d_interface.py:99-129) and causal_conv1d_varlen_states (causal_conv1d_varlen.py:35-64)
back to back on the same tokens."""
import ctypes

import pytest
import torch

import cabi
from helpers import DTYPES, assert_close, gen, make_wb
from oracle import causal_conv1d_oracle as orc

pytestmark = pytest.mark.gpu


def packed_batch(total, n_seqs, g, pad=0):
    """Lengths of n_seqs sequences summing to total - pad, their cu_seqlens and seq_idx (1, total)
    with the last `pad` tokens marked as padding."""
    cuts = torch.randperm(total - pad - 1, generator=g)[:n_seqs - 1].sort().values + 1
    cu = torch.cat([torch.zeros(1, dtype=torch.long), cuts, torch.tensor([total - pad])])
    seq = torch.full((1, total), -1, dtype=torch.int32)
    for i in range(n_seqs):
        seq[0, cu[i]:cu[i + 1]] = i
    return cu, seq


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("dim,total,n_seqs,state_len,width,pad", [
    (64, 200, 5, 3, 4, 0), (512, 1000, 9, 8, 3, 17), (4096 + 32, 777, 4, 20, 2, 0), (5376, 4096, 16, 3, 4, 100)])
@pytest.mark.parametrize("cu_dtype", [torch.int32, torch.int64])
def test_one_call_equals_two_calls_and_the_oracle(pkg, gpu_device, dtype, dim, total, n_seqs, state_len, width, pad,
                                                  cu_dtype):
    g = gen(dim + total)
    cu, seq = packed_batch(total, n_seqs, g, pad)
    x = torch.randn(1, total, dim, generator=g).to(dtype).transpose(1, 2)
    w, b = make_wb(dim, width, True, g)
    dx, dw, db = x.to(gpu_device), w.to(gpu_device), b.to(gpu_device)
    dseq, dcu = seq.to(gpu_device), cu.to(cu_dtype).to(gpu_device)

    out, states = pkg.causal_conv1d_fwd_varlen_states(dx, dw, db, dseq, dcu, state_len, activation="silu")
    out2 = pkg.causal_conv1d_fn(dx, dw, db, seq_idx=dseq, activation="silu")
    states2 = pkg.causal_conv1d_varlen_states(dx[0].t(), dcu, state_len)
    assert out.shape == x.shape and out.stride() == dx.stride()
    assert states.shape == (n_seqs, dim, state_len) and states.stride(1) == 1
    assert torch.equal(out, out2) and torch.equal(states, states2)
    assert torch.equal(states.cpu(), orc.varlen_states(x[0].t(), cu, state_len))
    assert_close(out, orc.fwd_seq_idx(x, w, b, seq, activation="silu"), dtype, "out")


def test_channel_first_x_takes_two_launches_with_the_same_results(pkg, gpu_device):
    g = gen(5)
    total, dim = 300, 48
    cu, _ = packed_batch(total, 3, g)
    x = torch.randn(1, dim, total, generator=g).to(torch.float16)
    w, b = make_wb(dim, 4, True, g)
    out, states = pkg.causal_conv1d_fwd_varlen_states(x.to(gpu_device), w.to(gpu_device), b.to(gpu_device), None,
                                                      cu.to(gpu_device), 4, activation=None)
    assert torch.equal(states.cpu(), orc.varlen_states(x[0].t(), cu, 4))
    assert_close(out, orc.fwd(x, w, b), torch.float16, "out")


def test_batched_rows_back_to_back(pkg, gpu_device):
    """batch > 1: cu_seqlens counts tokens of the flattened (batch * seqlen, dim) view."""
    g = gen(6)
    B, L, dim = 3, 128, 256
    x = torch.randn(B, L, dim, generator=g).to(torch.bfloat16).transpose(1, 2)
    w, b = make_wb(dim, 4, False, g)
    cu = torch.tensor([0, 100, 128, 256, 300, 384], dtype=torch.int32)
    seq = torch.zeros(B, L, dtype=torch.int32)
    seq[0, 100:] = 1
    seq[2, 44:] = 1
    out, states = pkg.causal_conv1d_fwd_varlen_states(x.to(gpu_device), w.to(gpu_device), None, seq.to(gpu_device),
                                                      cu.to(gpu_device), 3, activation="silu")
    flat = x.transpose(1, 2).reshape(B * L, dim)
    assert torch.equal(states.cpu(), orc.varlen_states(flat, cu, 3))
    assert_close(out, orc.fwd_seq_idx(x, w, None, seq, activation="silu"), torch.bfloat16, "out")


def test_c_abi_entry_point_and_errors(gpu_device, cc1d_lib):
    lib = cabi.declare(cc1d_lib)
    g = gen(7)
    total, dim = 512, 128
    cu, seq = packed_batch(total, 4, g)
    x = torch.randn(1, total, dim, generator=g).to(torch.bfloat16).transpose(1, 2).to(gpu_device)
    w, b = (t.to(gpu_device) for t in make_wb(dim, 4, True, g))
    dseq, dcu = seq.to(gpu_device), cu.to(torch.int32).to(gpu_device)
    out = torch.empty_like(x)
    states = torch.empty(4, 3, dim, dtype=x.dtype, device=gpu_device).transpose(1, 2)
    fp = cabi.fwd_params(x, w, b, out, True, seq_idx=dseq)
    vp = cabi.varlen_params(x[0].t(), dcu, states)
    stream = torch.cuda.current_stream().cuda_stream
    rc = lib.cc1d_fwd_varlen_states(ctypes.byref(fp), ctypes.byref(vp), stream)
    assert rc == 0, lib.cc1d_strerror(rc)
    torch.cuda.synchronize()
    assert torch.equal(states.cpu(), orc.varlen_states(x[0].t().cpu(), cu, 3))
    assert_close(out, orc.fwd_seq_idx(x.cpu(), w.cpu(), b.cpu(), seq, activation="silu"), torch.bfloat16, "out")
    # either half failing validation fails the call before anything is launched
    assert lib.cc1d_fwd_varlen_states(None, ctypes.byref(vp), stream) == -1
    assert lib.cc1d_fwd_varlen_states(ctypes.byref(fp), None, stream) == -1
    fp.width = 5
    assert lib.cc1d_fwd_varlen_states(ctypes.byref(fp), ctypes.byref(vp), stream) == -3
