"""GPU parity of the forward kernels against the CPU oracle, through the public Python API
(package -> torch extension -> C ABI -> HIP kernels) and, for one case, through the C ABI
directly.  The grids restate tests/test_causal_conv1d.py:50-137 (dense), :401-472 (seq_idx)
and :474-557 (seq_idx with padding) of the reference; initial/final states are also
exercised for channel-first, which the reference refuses.

Tolerances: fp32 |diff| <= 1e-5; fp16 rtol 3e-3 / atol 5e-3; bf16 rtol 1e-2 / atol 5e-2;
final_states, a pure copy, bit-exact.
"""
import ctypes

import pytest
import torch

import cabi
from golden_io import load_case
from helpers import (DTYPES, TOL, assert_close, gen, make_states, make_wb, make_x, random_seq_idx,
                     to_dev_like)
from oracle import causal_conv1d_oracle as orc

pytestmark = pytest.mark.gpu

SEQLENS = [1, 2, 8, 16, 32, 64, 128, 129, 130, 151, 256, 372, 512, 784, 1000, 1024, 1134, 1544, 2048, 2568, 4096]


def _grid():
    """Every (dim, seqlen, dtype, layout); width / bias / SiLU / states rotate through all
    their combinations across the grid."""
    cases, n = [], 0
    for dim in (64, 4096 + 32):
        for seqlen in SEQLENS:
            for dtype in DTYPES:
                for channel_last in (False, True):
                    width = 2 + n % 3
                    has_bias = (n // 3) % 2 == 0
                    silu = (n // 6) % 2 == 0
                    states = (n // 12 + n) % 4            # 0 none, 1 initial, 2 final, 3 both
                    cases.append(pytest.param(dim, seqlen, dtype, channel_last, width, has_bias, silu, states,
                                              id=f"d{dim}-l{seqlen}-{str(dtype)[6:]}-{'cl' if channel_last else 'cf'}"
                                                 f"-w{width}-b{int(has_bias)}-s{int(silu)}-st{states}"))
                    n += 1
    return cases


@pytest.mark.parametrize("dim,seqlen,dtype,channel_last,width,has_bias,silu,states", _grid())
def test_fwd_matches_oracle(pkg, gpu_device, dim, seqlen, dtype, channel_last, width, has_bias, silu, states):
    g = gen(seqlen * 7 + dim + width)
    x = make_x(2, dim, seqlen, dtype, channel_last, g)
    w, b = make_wb(dim, width, has_bias, g)
    init = make_states(2, dim, width - 1, dtype, g) if states & 1 else None
    want_final = bool(states & 2)
    act = "silu" if silu else None

    ref = orc.fwd(x, w, b, initial_states=init, return_final_states=want_final, activation=act)
    got = pkg.causal_conv1d_fn(to_dev_like(x, gpu_device), w.to(gpu_device),
                               None if b is None else b.to(gpu_device),
                               initial_states=None if init is None else init.to(gpu_device),
                               return_final_states=want_final, activation=act)
    if want_final:
        (got, got_fin), (ref, ref_fin) = got, ref
        assert got_fin.shape == ref_fin.shape and got_fin.stride(1) == 1
        assert torch.equal(got_fin.cpu(), ref_fin), "final_states must be an exact copy"
    assert got.dtype == dtype and got.shape == x.shape
    assert_close(got, ref, dtype, "out")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("seqlen", [4, 8, 24, 40, 72, 136, 248, 256, 264, 512])
def test_fwd_channel_first_short_rows(pkg, gpu_device, seqlen, dtype):
    """Channel-first rows of at most 64 whole 16-byte vectors share a wavefront (8, 4, 2 or 1 rows
    each): a row count that does not fill the last wavefront, every vector count class, states
    in and out, and against the same rows one element longer (which take the walking kernel)."""
    dev = gpu_device
    batch, dim, width = 3, 24, 2 + seqlen % 3
    g = gen(1000 + seqlen)
    x = torch.randn(batch, dim, seqlen + 1, generator=g).to(dtype)
    w, b = make_wb(dim, width, True, g)
    init = make_states(batch, dim, width - 1, dtype, g)
    xs = x[:, :, :seqlen].contiguous()
    ref, ref_fin = orc.fwd(xs, w, b, initial_states=init, return_final_states=True, activation="silu")
    got, got_fin = pkg.causal_conv1d_fn(xs.to(dev), w.to(dev), b.to(dev), initial_states=init.to(dev),
                                        return_final_states=True, activation="silu")
    assert_close(got, ref, dtype, "out")
    assert torch.equal(got_fin.cpu(), ref_fin)
    # causality: the first seqlen outputs of the longer rows are the same numbers, bit for bit
    longer = pkg.causal_conv1d_fn(x.to(dev), w.to(dev), b.to(dev), initial_states=init.to(dev), activation="silu")
    assert torch.equal(longer[:, :, :seqlen], got)
    plain = pkg.causal_conv1d_fn(xs.to(dev), w.to(dev), None)
    assert_close(plain, orc.fwd(xs, w, None), dtype, "no bias, no activation, no states")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("seqlen", [1, 2, 3, 5, 7, 9, 60, 100, 255, 500, 1030])
def test_fwd_channel_first_short_rows_of_any_length(pkg, gpu_device, seqlen, dtype):
    """Channel-first rows of at most 64 vectors that are not whole vectors (a contiguous tensor
    whose seqlen is no multiple of 16 bytes) share wavefronts too, down to one lane per row; rows
    shorter than width-1 take part of final_states from initial_states (or zeros).  Contiguous
    tensors with rows of at least one vector are walked as one flat array of whole vectors, a
    vector spanning two rows; slices of a wider tensor take element accesses."""
    dev = gpu_device
    batch, dim = 3, 41                                 # batch * dim * seqlen is no whole number of vectors either
    for width in (2, 3, 4):
        g = gen(3000 + seqlen * 4 + width)
        x = torch.randn(batch, dim, seqlen, generator=g).to(dtype)
        w, b = make_wb(dim, width, True, g)
        init = make_states(batch, dim, width - 1, dtype, g)
        ref, ref_fin = orc.fwd(x, w, b, initial_states=init, return_final_states=True, activation="silu")
        got, got_fin = pkg.causal_conv1d_fn(x.to(dev), w.to(dev), b.to(dev), initial_states=init.to(dev),
                                            return_final_states=True, activation="silu")
        assert_close(got, ref, dtype, "out")
        assert torch.equal(got_fin.cpu(), ref_fin)
        ref, ref_fin = orc.fwd(x, w, None, return_final_states=True)
        got, got_fin = pkg.causal_conv1d_fn(x.to(dev), w.to(dev), None, return_final_states=True)
        assert_close(got, ref, dtype, "no bias, no activation, no initial states")
        assert torch.equal(got_fin.cpu(), ref_fin)
        wide = torch.zeros(batch, dim, seqlen + 3, dtype=dtype)
        wide[:, :, 2:2 + seqlen] = x
        ref, ref_fin = orc.fwd(x, w, b, initial_states=init, return_final_states=True, activation="silu")
        sliced, sliced_fin = pkg.causal_conv1d_fn(wide.to(dev)[:, :, 2:2 + seqlen], w.to(dev), b.to(dev),
                                                  initial_states=init.to(dev), return_final_states=True,
                                                  activation="silu")
        assert_close(sliced, ref, dtype, "out of a slice")
        # one arithmetic, whichever kernel the layout takes
        assert torch.equal(sliced, pkg.causal_conv1d_fn(x.to(dev), w.to(dev), b.to(dev),
                                                        initial_states=init.to(dev), activation="silu"))
        assert torch.equal(sliced_fin.cpu(), ref_fin)


@pytest.mark.parametrize("pad", [False, True])
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("dim,seqlen,width,has_bias,silu", [
    (64, 8, 2, True, True), (64, 16, 3, False, True), (64, 151, 4, True, False), (64, 372, 4, True, True),
    (64, 1134, 3, True, True), (4128, 32, 4, True, True), (4128, 128, 2, False, False),
    (4128, 784, 4, True, True), (4128, 2048, 3, True, True), (4128, 4096, 4, True, True),
])
def test_fwd_seq_idx_matches_per_segment_oracle(pkg, gpu_device, dim, seqlen, width, has_bias, silu, dtype, pad):
    g = gen(seqlen + dim + width)
    x = make_x(3, dim, seqlen, dtype, True, g)
    w, b = make_wb(dim, width, has_bias, g)
    seq = random_seq_idx(3, seqlen, g, pad=pad)
    act = "silu" if silu else None
    ref = orc.fwd_seq_idx(x, w, b, seq, activation=act)
    got = pkg.causal_conv1d_fn(to_dev_like(x, gpu_device), w.to(gpu_device),
                               None if b is None else b.to(gpu_device),
                               seq_idx=seq.to(gpu_device), activation=act)
    assert_close(got, ref, dtype, "out")
    if pad:
        assert torch.all(got.cpu()[(seq < 0).unsqueeze(1).expand_as(got)] == 0), "padding must be exact zeros"


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("dim,seqlen,width,every", [(64, 333, 4, 1), (64, 1000, 3, 3), (264, 517, 4, 5), (264, 2048, 2, 2),
                                                    (4128, 300, 4, 4), (128, 4096, 4, 16)])
def test_fwd_seq_idx_with_sub_sequences_of_a_few_tokens(pkg, gpu_device, dim, seqlen, width, every, dtype):
    """Boundaries every few rows (and a padded tail): most groups of a run hold one, which takes
    the masked pass without the walk; boundaries every 16 rows mark about half of them."""
    g = gen(seqlen + dim + every)
    x = make_x(2, dim, seqlen, dtype, True, g)
    w, b = make_wb(dim, width, True, g)
    rows = []
    for _ in range(2):
        cuts = torch.zeros(seqlen, dtype=torch.int32)
        cuts[torch.randperm(seqlen - 1, generator=g)[:seqlen // every] + 1] = 1
        ids = torch.cumsum(cuts, 0).to(torch.int32)
        if every % 2 == 1:
            ids[seqlen - int(torch.randint(1, seqlen // 3, (1,), generator=g)):] = -1   # padded tail
        rows.append(ids)
    seq = torch.stack(rows)
    ref = orc.fwd_seq_idx(x, w, b, seq, activation="silu")
    got = pkg.causal_conv1d_fn(to_dev_like(x, gpu_device), w.to(gpu_device), b.to(gpu_device),
                               seq_idx=seq.to(gpu_device), activation="silu")
    assert_close(got, ref, dtype, "out")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("seqlen", [40, 517, 2048])
def test_seq_idx_keeps_non_finite_values_inside_their_sub_sequence(pkg, gpu_device, dtype, seqlen):
    """Packed sequences are independent requests: Inf or NaN in one of them, or in padding tokens
    (whose memory may hold anything), must not reach the outputs or gradients of the others.  The
    reference adds a tap only where the ids agree (csrc/causal_conv1d_fwd.cu:316-329), so nothing
    is multiplied by a masked input there either."""
    dev = gpu_device
    g = gen(4242 + seqlen)
    B, D, W = 3, 136, 4
    x = make_x(B, D, seqlen, dtype, True, g, sliced=False)
    dout = make_x(B, D, seqlen, dtype, True, g, sliced=False)
    w, b = make_wb(D, W, True, g)
    third = seqlen // 3
    seq = torch.zeros(B, seqlen, dtype=torch.int32)
    seq[:, third:2 * third] = 1
    seq[:, 2 * third:] = 2
    seq[:, seqlen - seqlen // 8:] = -1                  # padding tokens
    poison = torch.tensor([float("nan"), float("inf"), -float("inf")]).to(dtype)
    dirty_mid, dirty_pad = x.clone(), x.clone()
    dirty_mid[:, :, third:2 * third] = poison[torch.randint(0, 3, (B, D, 2 * third - third), generator=g)]
    dirty_pad[:, :, seqlen - seqlen // 8:] = poison[torch.randint(0, 3, (B, D, seqlen // 8), generator=g)]
    dout_pad = dout.clone()
    dout_pad[:, :, seqlen - seqlen // 8:] = float("nan")
    wd, bd, sd = w.to(dev), b.to(dev), seq.to(dev)

    clean = pkg.causal_conv1d_fn(x.to(dev), wd, bd, seq_idx=sd, activation="silu")
    mid = pkg.causal_conv1d_fn(dirty_mid.to(dev), wd, bd, seq_idx=sd, activation="silu")
    keep = torch.ones(seqlen, dtype=torch.bool)
    keep[third:2 * third] = False
    assert torch.equal(mid[:, :, keep], clean[:, :, keep]), "a poisoned sub-sequence reached its neighbours"
    assert torch.isfinite(clean).all()

    def fwd_bwd(x_, dout_):
        xg, wg, bg = x_.to(dev).requires_grad_(), wd.clone().requires_grad_(), bd.clone().requires_grad_()
        out = pkg.causal_conv1d_fn(xg, wg, bg, seq_idx=sd, activation="silu")
        out.backward(dout_.to(dev))
        return out.detach(), xg.grad, wg.grad, bg.grad

    ref = fwd_bwd(x, dout)
    got = fwd_bwd(dirty_pad, dout_pad)
    valid = (seq[0] >= 0)
    assert torch.equal(got[0], ref[0]), "padding tokens reached the outputs"
    assert bool((got[0][:, :, ~valid] == 0).all())
    assert torch.equal(got[1][:, :, valid], ref[1][:, :, valid]), "padding tokens reached dx"
    assert bool((got[1][:, :, ~valid] == 0).all()), "dx of padding tokens is zero"
    assert torch.equal(got[2], ref[2]) and torch.equal(got[3], ref[3]), "padding tokens reached dweight / dbias"


@pytest.mark.parametrize("w_dtype", DTYPES)
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("channel_last", [False, True])
def test_fwd_all_nine_dtype_pairs(pkg, gpu_device, dtype, w_dtype, channel_last):
    """x dtype x weight dtype (csrc/causal_conv1d_fwd.cu:383-401); the oracle computes in the
    weight dtype, the kernel in fp32, so 16-bit weights get the 16-bit tolerance."""
    g = gen(3)
    x = make_x(2, 72, 200, dtype, channel_last, g, sliced=False)
    w, b = make_wb(72, 4, True, g, w_dtype)
    ref = orc.fwd(x.float(), w.float(), b.float(), activation="silu").to(dtype)
    got = pkg.causal_conv1d_fn(x.to(gpu_device), w.to(gpu_device), b.to(gpu_device), activation="silu")
    assert_close(got, ref, dtype, "out")
    # non-contiguous weight (a transposed view) takes the strided tap loads
    wt = w.t().contiguous().t()
    got2 = pkg.causal_conv1d_fn(x.to(gpu_device), wt.to(gpu_device).t().contiguous().t(), b.to(gpu_device), activation="silu")
    assert torch.equal(got.cpu(), got2.cpu())


def test_fwd_golden_fixtures(pkg, gpu_device):
    d = gpu_device
    c = load_case("fwd_c1")
    got = pkg.causal_conv1d_fn(c["x"].to(d), c["weight"].to(d), c["bias"].to(d), activation="silu")
    assert_close(got, c["out"], torch.float32, "fwd_c1")
    c = load_case("fwd_states")
    for cl in (False, True):
        x = c["x"].transpose(1, 2).contiguous().transpose(1, 2) if cl else c["x"]
        got, fin = pkg.causal_conv1d_fn(x.to(d), c["weight"].to(d), c["bias"].to(d),
                                        initial_states=c["initial_states"].to(d), return_final_states=True)
        assert_close(got, c["out"], torch.bfloat16, "fwd_states")
        assert torch.equal(fin.cpu(), c["final_states"])
    c = load_case("fwd_seq")
    x = c["x"].transpose(1, 2).contiguous().transpose(1, 2)
    got = pkg.causal_conv1d_fn(x.to(d), c["weight"].to(d), c["bias"].to(d), seq_idx=c["seq_idx"].to(d), activation="silu")
    assert_close(got, c["out"], torch.float16, "fwd_seq")


def test_fwd_chunking_is_bit_exact_at_prefill_size(pkg, gpu_device):
    """Size-independent property at the full Mamba-2 2.7B prefill shape: running the
    sequence in two chunks, handing final_states over as initial_states, reproduces the
    unchunked output bit for bit; and a slice of rows agrees with the oracle."""
    import bench
    cfg = bench.config_c2()
    d = gpu_device
    x, w, b = cfg["x"].to(d), cfg["weight"].to(d), cfg["bias"].to(d)
    whole = pkg.causal_conv1d_fn(x, w, b, activation="silu")
    cut = 1000                                             # rows keep their 8-element alignment
    head, fin = pkg.causal_conv1d_fn(x[:, :, :cut], w, b, return_final_states=True, activation="silu")
    tail = pkg.causal_conv1d_fn(x[:, :, cut:], w, b, initial_states=fin, activation="silu")
    assert torch.equal(torch.cat([head, tail], dim=2), whole)
    ref = orc.fwd(cfg["x"][3:4], cfg["weight"], cfg["bias"], activation="silu")
    assert_close(whole[3:4], ref, torch.bfloat16, "row 3")
    seq = cfg["seq_idx"].to(d)
    got = pkg.causal_conv1d_fn(x, w, b, seq_idx=seq, activation="silu")
    ref = orc.fwd_seq_idx(cfg["x"][5:6], cfg["weight"], cfg["bias"], cfg["seq_idx"][5:6], activation="silu")
    assert_close(got[5:6], ref, torch.bfloat16, "row 5 with seq_idx")
    # a single sub-sequence id per row is the dense result
    assert torch.equal(pkg.causal_conv1d_fn(x, w, b, seq_idx=torch.zeros_like(seq), activation="silu"), whole)


@pytest.mark.parametrize("dtype", DTYPES)
def test_fwd_launch_geometry_does_not_change_results(pkg, gpu_device, cc1d_lib, dtype):
    """Every run length and both tap loaders (packed and general) of the channel-last walk give
    the same bits, with seq_idx, padding, initial and final states."""
    lib = cabi.declare(cc1d_lib)
    g = gen(11)
    x = make_x(2, 264, 333, dtype, True, g).to(gpu_device)
    w, b = (t.to(gpu_device) for t in make_wb(264, 4, True, g))
    seq = random_seq_idx(2, 333, g, pad=True).to(gpu_device)
    init = make_states(2, 264, 3, dtype, g).to(gpu_device)
    outs = []
    try:
        for half in (0, -1):
            for rows in (8, 16, 32, 64, 128, 1024):
                assert lib.cc1d_set_tunable(b"fwd_cl_rows", rows) == 0
                assert lib.cc1d_set_tunable(b"fwd_cl_half_vec", half) == 0
                o1 = pkg.causal_conv1d_fn(x, w, b, seq_idx=seq, activation="silu")
                o2, f2 = pkg.causal_conv1d_fn(x, w, b, initial_states=init, return_final_states=True, activation="silu")
                outs.append((o1.cpu(), o2.cpu(), f2.cpu()))
    finally:
        lib.cc1d_set_tunable(b"fwd_cl_rows", 0)
        lib.cc1d_set_tunable(b"fwd_cl_half_vec", 0)
    for o in outs[1:]:
        for a, r in zip(o, outs[0]):
            assert torch.equal(a, r)
    xc = x.cpu()
    assert_close(outs[0][0], orc.fwd_seq_idx(xc, w.cpu(), b.cpu(), seq.cpu(), activation="silu"), dtype, "seq_idx")
    ref, fin = orc.fwd(xc, w.cpu(), b.cpu(), initial_states=init.cpu(), return_final_states=True, activation="silu")
    assert_close(outs[0][1], ref, dtype, "states")
    assert torch.equal(outs[0][2], fin)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("seqlen", [1544, 1552, 2000, 2047, 3000, 4104, 9000])
def test_fwd_channel_first_rows_off_the_cache_lines(pkg, gpu_device, cc1d_lib, seqlen, dtype):
    """Channel-first rows longer than three steps whose ends do not fall on 128-byte lines: the walk
    starts its steps on lines of out, with a partly filled first step and, where rows are cut, with
    segments that start on lines too.  Every segment length gives the same bits; initial and final
    states; a view whose rows start anywhere on the 16-byte grid."""
    lib = cabi.declare(cc1d_lib)
    dev = gpu_device
    g = gen(1000 + seqlen)
    B, D, W = 2, 24, 4
    big = torch.randn(B, D, seqlen + 24, generator=g).to(dtype)
    w, b = make_wb(D, W, True, g)
    init = make_states(B, D, W - 1, dtype, g)
    for off in (0, 8, 16 // big.element_size(), 3):
        x = big[:, :, off:off + seqlen]
        ref, fin = orc.fwd(x, w, b, initial_states=init, return_final_states=True, activation="silu")
        xd = big.to(dev)[:, :, off:off + seqlen]
        outs = []
        try:
            for vecs in (0, 128, 256, 1024):
                assert lib.cc1d_set_tunable(b"fwd_cf_vecs", vecs) == 0
                o, f = pkg.causal_conv1d_fn(xd, w.to(dev), b.to(dev), initial_states=init.to(dev),
                                            return_final_states=True, activation="silu")
                outs.append((o.cpu(), f.cpu()))
        finally:
            lib.cc1d_set_tunable(b"fwd_cf_vecs", 0)
        for o, f in outs[1:]:
            assert torch.equal(o, outs[0][0]) and torch.equal(f, outs[0][1])
        assert_close(outs[0][0], ref, dtype, "out, offset %d" % off)
        assert torch.equal(outs[0][1], fin)


@pytest.mark.parametrize("dtype", DTYPES)
def test_fwd_workgroup_order_does_not_change_results(pkg, gpu_device, cc1d_lib, dtype):
    """The channel-last forward hands its workgroups to the XCDs in contiguous slices or in chunks
    of runs, by shape; every order covers every run exactly once: same bits, ragged last run and
    a launch that is no whole number of chunks included."""
    lib = cabi.declare(cc1d_lib)
    g = gen(12)
    x = make_x(3, 1160, 1237, dtype, True, g).to(gpu_device)
    w, b = (t.to(gpu_device) for t in make_wb(1160, 4, True, g))
    seq = random_seq_idx(3, 1237, g, pad=True).to(gpu_device)
    outs = []
    try:
        for chunk in (-1, 0, 4, 8, 16, 64, -3, -7):
            assert lib.cc1d_set_tunable(b"fwd_cl_chunk_runs", chunk) == 0
            o = pkg.causal_conv1d_fn(x, w, b, seq_idx=seq, activation="silu")
            _, f = pkg.causal_conv1d_fn(x, w, b, return_final_states=True, activation="silu")
            outs.append((o.cpu(), f.cpu()))
    finally:
        lib.cc1d_set_tunable(b"fwd_cl_chunk_runs", 0)
    for o in outs[1:]:
        assert torch.equal(o[0], outs[0][0]) and torch.equal(o[1], outs[0][1])
    assert_close(outs[0][0], orc.fwd_seq_idx(x.cpu(), w.cpu(), b.cpu(), seq.cpu(), activation="silu"), dtype, "out")


def test_fwd_through_the_c_abi_on_a_side_stream(gpu_device, cc1d_lib):
    """The C ABI alone: raw pointers, element strides and an explicit stream handle."""
    lib = cabi.declare(cc1d_lib)
    g = gen(5)
    x = make_x(2, 64, 300, torch.float32, False, g, sliced=False)
    w, b = make_wb(64, 4, True, g)
    init = make_states(2, 64, 3, torch.float32, g)
    ref, ref_fin = orc.fwd(x, w, b, initial_states=init, return_final_states=True, activation="silu")
    xd, wd, bd, idev = (t.to(gpu_device) for t in (x, w, b, init))
    out, fin = torch.empty_like(xd), torch.empty(2, 64, 3, device=gpu_device)
    stream = torch.cuda.Stream()
    stream.wait_stream(torch.cuda.current_stream())
    p = cabi.fwd_params(xd, wd, bd, out, True, initial_states=idev, final_states=fin)
    st = lib.cc1d_fwd(ctypes.byref(p), ctypes.c_void_p(stream.cuda_stream))
    assert st == 0, lib.cc1d_strerror(st)
    stream.synchronize()
    assert_close(out, ref, torch.float32, "out")
    assert torch.equal(fin.cpu(), ref_fin)


def test_fwd_error_behaviour(pkg, gpu_device):
    d = gpu_device
    x = torch.zeros(2, 16, 32, device=d)
    with pytest.raises(RuntimeError, match="width between 2 and 4"):
        pkg.causal_conv1d_fn(x, torch.zeros(16, 5, device=d))
    with pytest.raises(NotImplementedError):
        pkg.causal_conv1d_fn(x, torch.zeros(16, 4, device=d), activation="relu")
    xcl = torch.zeros(2, 32, 12, device=d).transpose(1, 2)
    with pytest.raises(RuntimeError, match="divisible by 8"):
        pkg.causal_conv1d_fn(xcl, torch.zeros(12, 4, device=d))
    with pytest.raises(RuntimeError, match="channel last"):
        pkg.causal_conv1d_fn(x, torch.zeros(16, 4, device=d), seq_idx=torch.zeros(2, 32, dtype=torch.int32, device=d))
    with pytest.raises(AssertionError):
        pkg.causal_conv1d_fn(xcl, torch.zeros(12, 4, device=d), seq_idx=torch.zeros(2, 32, dtype=torch.int32, device=d),
                             return_final_states=True)
    empty = pkg.causal_conv1d_fn(torch.zeros(0, 16, 32, device=d), torch.zeros(16, 4, device=d))
    assert empty.shape == (0, 16, 32)


@pytest.mark.parametrize("channel_last", [False, True], ids=["cf", "cl"])
@pytest.mark.parametrize("dtype", DTYPES)
def test_fwd_one_buffer_for_initial_and_final_states(pkg, gpu_device, dtype, channel_last):
    """A chunked prefill that keeps ONE state tensor: initial_states and final_states_out are the
    same buffer (allowed by the reference, csrc/causal_conv1d.h:44).  Chunks of many runs, of a few
    rows, of fewer than width-1 rows and of odd lengths must reproduce the unchunked result bit
    for bit, and leave the last width-1 inputs in the buffer."""
    dev = gpu_device
    g = gen(91)
    B, D, W = 3, 264, 4
    L = 1500 if channel_last else 1499
    x = make_x(B, D, L, dtype, channel_last, g, sliced=False).to(dev)
    w, b = (t.to(dev) for t in make_wb(D, W, True, g))
    init = make_states(B, D, W - 1, dtype, g).to(dev)
    whole, whole_fin = pkg.causal_conv1d_fn(x, w, b, initial_states=init, return_final_states=True, activation="silu")
    # chunks of 512, 8, 2, 1, 477 and about 500 positions; channel-first slices start off the
    # 16-byte grid
    cuts = [0, 512, 520, 522, 523, 1000, L]
    for layout in ("dim_fastest", "len_fastest"):
        state = (init.clone() if layout == "dim_fastest" else init.contiguous().clone())
        outs = []
        for lo, hi in zip(cuts[:-1], cuts[1:]):
            o, fin = pkg.causal_conv1d_fn(x[:, :, lo:hi], w, b, initial_states=state, return_final_states=True,
                                          final_states_out=state, activation="silu")
            assert fin.data_ptr() == state.data_ptr()
            outs.append(o)
        assert torch.equal(torch.cat(outs, dim=2), whole), layout
        assert torch.equal(state, whole_fin), layout
    ref, ref_fin = orc.fwd(x.cpu(), w.cpu(), b.cpu(), initial_states=init.cpu(), return_final_states=True, activation="silu")
    assert_close(whole, ref, dtype, "out")
    assert torch.equal(whole_fin.cpu(), ref_fin)


def test_fwd_on_a_side_stream_through_the_package(pkg, gpu_device):
    """The binding launches on torch's current stream, whichever it is."""
    dev = gpu_device
    g = gen(92)
    x = make_x(2, 128, 777, torch.bfloat16, True, g, sliced=False).to(dev)
    w, b = (t.to(dev) for t in make_wb(128, 4, True, g))
    ref = pkg.causal_conv1d_fn(x, w, b, activation="silu")
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        got = pkg.causal_conv1d_fn(x, w, b, activation="silu")
    side.synchronize()
    assert torch.equal(got, ref)
