"""GPU parity of the decode-step update against the CPU oracle.  Grids restate
tests/test_causal_conv1d.py:140-183 (plain), :185-233 (conv_state_indices) and :236-321
(negative indices = padding) of the reference.  conv_state must be bit-exact; out within
the forward tolerances."""
import ctypes

import pytest
import torch

import cabi
from golden_io import load_case
from helpers import DTYPES, assert_close, gen, make_wb
from oracle import causal_conv1d_oracle as orc

pytestmark = pytest.mark.gpu


def _grid():
    cases, n = [], 0
    for dim in (2048, 2048 + 16, 4096):
        for width in (2, 3, 4):
            for seqlen in (1, 4, 5):
                for circular in (False, True):
                    for dtype in DTYPES:
                        has_bias = n % 2 == 0
                        silu = (n // 2) % 2 == 0
                        cases.append(pytest.param(dim, width, seqlen, circular, dtype, has_bias, silu,
                                                  id=f"d{dim}-w{width}-l{seqlen}-c{int(circular)}-{str(dtype)[6:]}"
                                                     f"-b{int(has_bias)}-s{int(silu)}"))
                        n += 1
    return cases


def _inputs(dim, width, seqlen, dtype, has_bias, g, batch=64, entries=None, state_dim_last=True):
    x = torch.randn(batch, seqlen, dim, generator=g).to(dtype).transpose(-1, -2)
    state_len = int(torch.randint(width - 1, width + 10, (1,), generator=g))
    n = entries or batch
    if state_dim_last:
        st = torch.randn(n, state_len, dim, generator=g).to(dtype).transpose(-1, -2)
    else:
        st = torch.randn(n, dim, state_len, generator=g).to(dtype)
    w, b = make_wb(dim, width, has_bias, g)
    return x, st, w, b


@pytest.mark.parametrize("dim,width,seqlen,circular,dtype,has_bias,silu", _grid())
def test_update_matches_oracle(pkg, gpu_device, dim, width, seqlen, circular, dtype, has_bias, silu):
    g = gen(dim + width * 10 + seqlen)
    x, st, w, b = _inputs(dim, width, seqlen, dtype, has_bias, g)
    cs = torch.randint(0, 1024, (64,), generator=g, dtype=torch.int32) if circular else None
    act = "silu" if silu else None
    st_ref = st.clone()
    ref = orc.update(x, st_ref, w, b, activation=act, cache_seqlens=cs)
    d = gpu_device
    st_dev = st.to(d)
    got = pkg.causal_conv1d_update(x.to(d), st_dev, w.to(d), None if b is None else b.to(d), activation=act,
                                   cache_seqlens=None if cs is None else cs.to(d))
    assert torch.equal(st_dev.cpu(), st_ref), "conv_state must be bit-exact"
    assert_close(got, ref, dtype, "out")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("circular", [False, True])
@pytest.mark.parametrize("dim,width,seqlen", [(2048, 4, 1), (2064, 3, 4), (4096, 2, 5), (2048, 4, 5)])
def test_update_with_batch_gather_and_padding(pkg, gpu_device, dim, width, seqlen, circular, dtype):
    g = gen(dim + width + seqlen + 1)
    x, st, w, b = _inputs(dim, width, seqlen, dtype, True, g, entries=640)
    idx = torch.randperm(640, generator=g)[:64].to(torch.int32)
    idx[torch.randperm(64, generator=g)[:32]] = -1                   # half the requests are padding
    cs = torch.randint(0, 1024, (64,), generator=g, dtype=torch.int32) if circular else None
    st_ref = st.clone()
    ref = orc.update(x, st_ref, w, b, activation="silu", cache_seqlens=cs, conv_state_indices=idx)
    d = gpu_device
    st_dev = st.to(d)
    got = pkg.causal_conv1d_update(x.to(d), st_dev, w.to(d), b.to(d), activation="silu",
                                   cache_seqlens=None if cs is None else cs.to(d), conv_state_indices=idx.to(d))
    assert torch.equal(st_dev.cpu(), st_ref), "gathered rows exact, every other row untouched"
    assert torch.all(got.cpu()[idx < 0] == 0), "padding requests must output exact zeros"
    assert_close(got, ref, dtype, "out")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("circular", [False, True])
def test_update_other_layouts_take_the_element_kernel(pkg, gpu_device, dtype, circular):
    """State stored (batch, dim, state_len)-contiguous, x (batch, dim) 2-D, odd dim."""
    g = gen(31)
    dim, width = 2052, 4
    x = torch.randn(16, dim, generator=g).to(dtype)
    st = torch.randn(16, dim, 7, generator=g).to(dtype)
    w, b = make_wb(dim, width, True, g)
    cs = torch.randint(0, 1024, (16,), generator=g, dtype=torch.int32) if circular else None
    st_ref = st.clone()
    ref = orc.update(x, st_ref, w, b, activation="silu", cache_seqlens=cs)
    d = gpu_device
    st_dev = st.to(d)
    got = pkg.causal_conv1d_update(x.to(d), st_dev, w.to(d), b.to(d), activation="silu",
                                   cache_seqlens=None if cs is None else cs.to(d))
    assert got.shape == (16, dim)
    assert torch.equal(st_dev.cpu(), st_ref)
    assert_close(got, ref, dtype, "out")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("width,state_len", [(4, 4), (4, 8), (3, 4), (3, 2), (2, 2), (2, 4), (2, 1), (4, 3), (3, 8),
                                             (3, 3), (2, 3), (2, 8), (4, 5), (4, 16)])
@pytest.mark.parametrize("indices", [False, True])
def test_update_contiguous_state_rows(pkg, gpu_device, width, state_len, dtype, indices):
    """conv_state (batch, dim, state_len) contiguous (unit stride along state_len), as mamba_ssm's
    Mamba block allocates it with state_len = d_conv and paged servers with state_len = width - 1:
    state lengths 2, 3, 4, 8 take the row-state kernel when dim is a whole number of the lanes'
    channel groups and x is aligned to a lane's access, the rest (other lengths, an odd channel
    count, x starting one element off) the element kernel; x as (batch, dim) and as (batch, dim, 1)."""
    g = gen(width * 100 + state_len)
    dev = gpu_device
    for dim, batch, two_d, x_off in ((2048, 33, True, 0), (5120, 7, False, 0), (1026, 5, True, 0), (517, 3, False, 0),
                                     (1024, 6, True, 1), (768, 4, True, 2)):
        entries = batch + 9 if indices else batch
        x_full = torch.randn(batch, dim + 8, generator=g).to(dtype)
        on_dev = lambda: x_full.to(dev)[:, x_off:x_off + dim] if two_d else x_full.to(dev)[:, :dim].contiguous().unsqueeze(-1)
        x = x_full[:, x_off:x_off + dim] if two_d else x_full[:, :dim].contiguous().unsqueeze(-1)
        st = torch.randn(entries, dim, state_len, generator=g).to(dtype)
        w, b = make_wb(dim, width, True, g)
        idx = None
        if indices:
            idx = torch.randperm(entries, generator=g)[:batch].to(torch.int32)
            idx[1] = -1
        st_ref = st.clone()
        ref = orc.update(x, st_ref, w, b, activation="silu", conv_state_indices=idx)
        st_dev = st.to(dev)
        got = pkg.causal_conv1d_update(on_dev(), st_dev, w.to(dev), b.to(dev), activation="silu",
                                       conv_state_indices=None if idx is None else idx.to(dev))
        assert got.shape == x.shape
        assert torch.equal(st_dev.cpu(), st_ref), (dim, batch)
        assert_close(got, ref, dtype, "out dim %d" % dim)
        # taps in the tensors' own 16-bit type, as an inference checkpoint holds them
        if dtype != torch.float32:
            st_ref2, st_dev2 = st.clone(), st.to(dev)
            ref2 = orc.update(x, st_ref2, w.to(dtype).float(), b.to(dtype).float(), activation="silu", conv_state_indices=idx)
            got2 = pkg.causal_conv1d_update(on_dev(), st_dev2, w.to(dtype).to(dev), b.to(dtype).to(dev), activation="silu",
                                            conv_state_indices=None if idx is None else idx.to(dev))
            assert torch.equal(st_dev2.cpu(), st_ref2)
            assert_close(got2, ref2, dtype, "out, 16-bit taps, dim %d" % dim)
        # no activation, no bias
        st_ref3, st_dev3 = st.clone(), st.to(dev)
        ref3 = orc.update(x, st_ref3, w, None, activation=None, conv_state_indices=idx)
        got3 = pkg.causal_conv1d_update(on_dev(), st_dev3, w.to(dev), None, activation=None,
                                        conv_state_indices=None if idx is None else idx.to(dev))
        assert torch.equal(st_dev3.cpu(), st_ref3)
        assert_close(got3, ref3, dtype, "out, plain, dim %d" % dim)


def test_update_golden_and_decode_loop(pkg, gpu_device):
    d = gpu_device
    for case in ("update_linear", "update_circular"):
        c = load_case(case)
        lay = lambda t: t.transpose(1, 2).contiguous().transpose(1, 2)
        st = lay(c["conv_state"]).to(d)
        cs = c.get("cache_seqlens")
        got = pkg.causal_conv1d_update(lay(c["x"]).to(d), st, c["weight"].to(d), c["bias"].to(d), activation="silu",
                                       cache_seqlens=None if cs is None else cs.to(d))
        assert torch.equal(st.cpu(), c["conv_state_after"])
        assert_close(got, c["out"], torch.bfloat16, case)
    # token-by-token decoding reproduces the prefill forward (fp32, so nearly exact)
    g = gen(8)
    x = torch.randn(3, 40, 128, generator=g).transpose(1, 2)
    w, b = make_wb(128, 4, True, g)
    whole = pkg.causal_conv1d_fn(x.to(d), w.to(d), b.to(d), activation="silu")
    state = torch.zeros(3, 3, 128, device=d).transpose(1, 2)
    steps = [pkg.causal_conv1d_update(x[:, :, t].to(d), state, w.to(d), b.to(d), activation="silu") for t in range(40)]
    assert_close(torch.stack(steps, dim=-1), whole.cpu(), torch.float32, "decode loop")
    assert torch.equal(state.cpu(), x[:, :, -3:])


@pytest.mark.parametrize("circular", [False, True])
def test_update_full_decode_shape_through_the_c_abi(gpu_device, cc1d_lib, circular):
    """bf16 (256, 5376, 1) with state (256, 5376, 3) linear / (256, 5376, 8) circular, called
    through the C ABI; the whole result is compared with the oracle."""
    import bench
    lib = cabi.declare(cc1d_lib)
    cfg = bench.config_c3(circular)
    st_ref = cfg["conv_state"].clone()
    ref = orc.update(cfg["x"], st_ref, cfg["weight"], cfg["bias"], activation="silu",
                     cache_seqlens=cfg.get("cache_seqlens"))
    d = gpu_device
    x, st, w, b = (cfg[k].to(d) for k in ("x", "conv_state", "weight", "bias"))
    cs = cfg["cache_seqlens"].to(d) if circular else None
    out = torch.empty_like(x)
    p = cabi.update_params(x, st, w, b, out, True, cache_seqlens=cs)
    rc = lib.cc1d_update(ctypes.byref(p), torch.cuda.current_stream().cuda_stream)
    assert rc == 0, lib.cc1d_strerror(rc)
    torch.cuda.synchronize()
    assert torch.equal(st.cpu(), st_ref)
    assert_close(out, ref, torch.bfloat16, "out")
