"""GPU parity of the varlen final-state gather: bit-exact against the CPU oracle.  Restates
tests/test_causal_conv1d.py:324-339 of the reference and adds the full-size packed batch."""
import ctypes

import pytest
import torch

import cabi
from golden_io import load_case
from helpers import DTYPES, gen
from oracle import causal_conv1d_oracle as orc

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("dim", [2048, 2048 + 16, 4096])
@pytest.mark.parametrize("cu_dtype", [torch.int64, torch.int32])
def test_varlen_states_matches_oracle(pkg, gpu_device, dim, dtype, cu_dtype):
    g = gen(dim)
    lens = torch.randint(1, 32, (100,), generator=g)
    cu = torch.nn.functional.pad(lens.cumsum(0), (1, 0)).to(cu_dtype)
    x = torch.randn(int(lens.sum()), dim, generator=g).to(dtype)
    got = pkg.causal_conv1d_varlen_states(x.to(gpu_device), cu.to(gpu_device), 20)
    assert got.shape == (100, dim, 20) and got.stride(1) == 1
    assert torch.equal(got.cpu(), orc.varlen_states(x, cu, 20))


def test_varlen_states_strided_x_takes_the_element_kernel(pkg, gpu_device):
    g = gen(4)
    lens = torch.tensor([3, 1, 40, 7])
    cu = torch.nn.functional.pad(lens.cumsum(0), (1, 0)).to(torch.int32)
    wide = torch.randn(int(lens.sum()), 100, generator=g).to(torch.float16)
    x = wide[:, 3:80]                                            # odd dim, odd offset, row stride 100
    got = pkg.causal_conv1d_varlen_states(wide.to(gpu_device)[:, 3:80], cu.to(gpu_device), 5)
    assert torch.equal(got.cpu(), orc.varlen_states(x, cu, 5))


def test_varlen_states_golden_and_full_size(pkg, gpu_device, cc1d_lib):
    import bench
    c = load_case("varlen")
    got = pkg.causal_conv1d_varlen_states(c["x"].to(gpu_device), c["cu_seqlens"].to(gpu_device), 3)
    assert torch.equal(got.cpu(), c["states"])
    # 64 packed sequences, 65536 tokens, dim 5376 -> states (64, 5376, 3), through the C ABI
    lib = cabi.declare(cc1d_lib)
    cfg = bench.config_c5a()
    x, cu = cfg["x"].to(gpu_device), cfg["cu_seqlens"].to(gpu_device)
    states = torch.empty(64, 3, 5376, dtype=x.dtype, device=gpu_device).transpose(1, 2)
    p = cabi.varlen_params(x, cu, states)
    rc = lib.cc1d_varlen_states(ctypes.byref(p), torch.cuda.current_stream().cuda_stream)
    assert rc == 0, lib.cc1d_strerror(rc)
    torch.cuda.synchronize()
    assert torch.equal(states.cpu(), orc.varlen_states(cfg["x"], cfg["cu_seqlens"], 3))
    # feeding the gathered states to the decode step continues each sequence correctly
    w, b = cfg_w = bench.make_weights(5376, 4, 9)
    nxt = torch.randn(64, 5376, generator=gen(1)).to(torch.bfloat16)
    st = states.clone()
    out = pkg.causal_conv1d_update(nxt.to(gpu_device), st, w.to(gpu_device), b.to(gpu_device), activation="silu")
    ends = cfg["cu_seqlens"][1:].long()
    tail = torch.stack([cfg["x"][e - 3:e] for e in ends])        # (64, 3, 5376)
    ref = orc.fwd(torch.cat([tail.transpose(1, 2), nxt.unsqueeze(-1)], dim=-1), w, b, activation="silu")[..., -1]
    assert ((out.float().cpu() - ref.float()).abs() <= 5e-2 + 1e-2 * ref.float().abs()).all()
