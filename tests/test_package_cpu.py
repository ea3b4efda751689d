"""CPU-side checks of the drop-in Python package: it imports (which loads the extension),
exposes the reference's names and signatures, its PyTorch formula helpers agree with the
oracle, and the GPU ops refuse CPU tensors instead of silently computing on the host."""
import inspect

import pytest
import torch

from oracle import causal_conv1d_oracle as orc


def test_public_surface(pkg):
    import causal_conv1d_cuda
    from causal_conv1d import causal_conv1d_interface as ci
    from causal_conv1d import causal_conv1d_varlen as cv
    from causal_conv1d import cpp_functions as cf
    assert pkg.__version__ == "1.6.1"
    assert list(inspect.signature(ci.causal_conv1d_fn).parameters) == [
        "x", "weight", "bias", "seq_idx", "initial_states", "return_final_states", "final_states_out", "activation"]
    assert list(inspect.signature(ci.causal_conv1d_update).parameters) == [
        "x", "conv_state", "weight", "bias", "activation", "cache_seqlens", "conv_state_indices"]
    assert list(inspect.signature(cv.causal_conv1d_varlen_states).parameters) == ["x", "cu_seqlens", "state_len"]
    for name in ("causal_conv1d_fwd", "causal_conv1d_bwd", "causal_conv1d_update", "causal_conv1d_varlen_states"):
        assert hasattr(causal_conv1d_cuda, name)
    for name in ("causal_conv1d_fwd_function", "causal_conv1d_bwd_function", "causal_conv1d_update_function"):
        assert hasattr(cf, name)
    for op in ("_causal_conv1d_fwd_cpp", "_causal_conv1d_bwd_cpp", "_causal_conv1d_update_cpp"):
        assert hasattr(torch.ops.DaoAILab, op)
    src = open(cv.__file__).read() + open(ci.__file__).read() + open(cf.__file__).read()
    assert "import triton" not in src


def test_formula_helpers_agree_with_the_oracle(pkg):
    from causal_conv1d.causal_conv1d_interface import causal_conv1d_ref, causal_conv1d_update_ref
    from causal_conv1d.causal_conv1d_varlen import causal_conv1d_varlen_states_ref
    g = torch.Generator().manual_seed(0)
    x = torch.randn(2, 8, 19, generator=g).to(torch.bfloat16)
    w, b = torch.randn(8, 4, generator=g), torch.randn(8, generator=g)
    init = torch.randn(2, 8, 3, generator=g).to(torch.bfloat16)
    # The helpers sum shifted copies tap by tap, the oracle calls F.conv1d: two formulations,
    # equal up to the rounding of the output type.
    a = causal_conv1d_ref(x, w, b, initial_states=init, return_final_states=True, activation="silu")
    r = orc.fwd(x, w, b, initial_states=init, return_final_states=True, activation="silu")
    assert torch.allclose(a[0].float(), r[0].float(), rtol=1e-2, atol=1e-2) and torch.equal(a[1], r[1])
    a32 = causal_conv1d_ref(x.float(), w, b, initial_states=init.float(), activation="silu")
    r32 = orc.fwd(x.float(), w, b, initial_states=init.float(), activation="silu")
    assert torch.allclose(a32, r32, rtol=0, atol=1e-5)
    for cs in (None, torch.tensor([1, 9], dtype=torch.int32)):
        s1, s2 = torch.randn(2, 8, 6, generator=g), None
        s2 = s1.clone()
        o1 = causal_conv1d_update_ref(x[..., :2].float(), s1, w, b, activation="silu", cache_seqlens=cs)
        o2 = orc.update(x[..., :2].float(), s2, w, b, activation="silu", cache_seqlens=cs)
        assert torch.allclose(o1, o2, rtol=0, atol=1e-5) and torch.equal(s1, s2)
    cu = torch.tensor([0, 2, 9, 19])
    xt = x[0].t().contiguous()
    assert torch.equal(causal_conv1d_varlen_states_ref(xt, cu, 4), orc.varlen_states(xt, cu, 4))


def test_no_host_fallback(pkg):
    x, w = torch.zeros(1, 8, 4), torch.zeros(8, 4)
    with pytest.raises(RuntimeError, match="GPU"):
        pkg.causal_conv1d_fn(x, w)
    with pytest.raises(RuntimeError, match="GPU"):
        pkg.causal_conv1d_update(x[..., 0], torch.zeros(1, 8, 3), w)
    with pytest.raises(RuntimeError, match="GPU"):
        pkg.causal_conv1d_varlen_states(torch.zeros(4, 8), torch.tensor([0, 4]), 3)
