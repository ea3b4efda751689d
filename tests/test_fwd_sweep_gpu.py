"""Forward parity at the width / dtype / layout sweep's own shape, (batch 4, dim 2048, seqlen 4096)
with widths 2, 3, 4 in fp32, fp16 and bf16, both layouts (the grid of
tests/test_causal_conv1d.py:50-137 of the reference at one full-size shape), and the fp32
activation over the whole range of pre-activations, not only those N(0,1) inputs produce.

Tolerances: fp32 |diff| <= 1e-5; fp16 rtol 3e-3 / atol 5e-3; bf16 rtol 1e-2 / atol 5e-2.
"""
import pytest
import torch

import bench
from helpers import DTYPES, assert_close
from oracle import c_oracle
from oracle import causal_conv1d_oracle as orc

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("channel_last", [False, True], ids=["cf", "cl"])
@pytest.mark.parametrize("dtype", DTYPES, ids=["fp32", "fp16", "bf16"])
@pytest.mark.parametrize("width", [2, 3, 4])
def test_fwd_sweep_shape_matches_oracle(pkg, gpu_device, width, dtype, channel_last):
    """Exactly the tensors bench.py times for this cell: every element against the oracle."""
    cfg = bench.config_c5b(width, dtype, channel_last)
    x, w, b = cfg["x"], cfg["weight"], cfg["bias"]
    assert x.shape == (4, 2048, 4096) and (x.stride(1) == 1) == channel_last
    with torch.no_grad():
        ref = orc.fwd(x, w, b, activation="silu")
    got = pkg.causal_conv1d_fn(x.to(gpu_device), w.to(gpu_device), b.to(gpu_device), activation="silu")
    assert got.dtype == dtype and got.stride() == x.stride()
    assert_close(got, ref, dtype, "sweep w%d" % width)


@pytest.mark.parametrize("channel_last", [False, True], ids=["cf", "cl"])
def test_fp32_silu_is_within_1e5_for_every_preactivation(pkg, gpu_device, channel_last):
    """The fp32 kernels evaluate SiLU with the hardware exp2 and reciprocal.  With taps (0, 1) and
    no bias the pre-activation IS x, bit for bit, so the output isolates the activation: a dense
    sweep of z over [-104, 104] (past the point where exp(-z) overflows fp32) plus powers of two
    and denormal-sized values must stay within 1e-5 of z / (1 + exp(-z)) evaluated in double
    precision.  The error of the two hardware transcendentals is relative to sigmoid(z), which is
    within an ulp of 1 where |z| is large and positive and tiny where it is large and negative,
    so it never grows with |z|."""
    dim, n = 8, 1 << 16
    z = torch.cat([torch.linspace(-104.0, 104.0, n - 64, dtype=torch.float64).float(),
                   torch.tensor([2.0 ** k for k in range(-30, -14)] + [-(2.0 ** k) for k in range(-30, -14)] +
                                [0.0, -0.0, 88.7, -88.7, 87.3, -87.3, 16.6, -16.6, 17.3, -17.3, 1e-38, -1e-38,
                                 1.2785, -1.2785] + [float(k) for k in range(1, 19)])])
    assert z.numel() == n
    x = z.repeat(dim, 1).unsqueeze(0)                           # (1, dim, n) channel-first
    if channel_last:
        x = x.transpose(1, 2).contiguous().transpose(1, 2)
    w = torch.zeros(dim, 2)
    w[:, 1] = 1.0
    got = pkg.causal_conv1d_fn(x.to(gpu_device), w.to(gpu_device), None, activation="silu").cpu()
    zd = z.double()
    ref = zd / (1.0 + torch.exp(-zd))
    err = (got[0].double() - ref).abs().max(dim=0).values
    worst = int(err.argmax())
    assert torch.isfinite(got).all()
    assert float(err.max()) <= 1e-5, "z = %r: |err| = %.3e" % (float(z[worst]), float(err[worst]))
    # and no worse than an ulp or two of the result where the result is large
    big = zd.abs() > 20
    assert float((err[big] / ref[big].abs().clamp_min(1.0)).max()) <= 2.0 ** -22


@pytest.mark.parametrize("channel_last", [False, True], ids=["cf", "cl"])
@pytest.mark.parametrize("scale", [10.0, 20.0])
def test_fp32_large_preactivations_against_double_precision(pkg, gpu_device, scale, channel_last):
    """x scaled so that pre-activations reach |z| of 50 and more: fp32 forward against the
    double-precision C oracle.  At that size an fp32 result has an ulp of 4e-6 to 8e-6, so the
    absolute bound carries two ulps of the result on top of the 1e-5 that holds for N(0,1) inputs."""
    g = torch.Generator().manual_seed(int(scale))
    B, D, L, W = 2, 64, 3000, 4
    x = torch.randn(B, D, L, generator=g) * scale
    w = torch.rand(D, W, generator=g) - 0.5
    b = torch.rand(D, generator=g) - 0.5
    ref = c_oracle.fwd(x, w, b, silu=True)
    xin = x.transpose(1, 2).contiguous().transpose(1, 2) if channel_last else x
    got = pkg.causal_conv1d_fn(xin.to(gpu_device), w.to(gpu_device), b.to(gpu_device), activation="silu").cpu().double()
    assert float(ref.abs().max()) > 2.5 * scale
    err = (got - ref).abs()
    bound = 1e-5 + 2.0 ** -22 * ref.abs()
    assert bool((err <= bound).all()), "max |err| %.3e at |ref| %.1f" % (float(err.max()), float(ref.flatten()[err.argmax()].abs()))
    small = ref.abs() <= 8.0                                    # where one ulp is below 1e-6
    assert float(err[small].max()) <= 1e-5
