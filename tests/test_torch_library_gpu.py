"""The three device ops as torch.library custom ops: schema / fake-tensor / functionalisation
checks (torch.library.opcheck) and whole-graph capture by torch.compile.  These are the names
current Mamba code reaches the kernels through (DaoAILab::_causal_conv1d_{fwd,bwd,update}_cpp,
causal_conv1d/cpp_functions.py:11-91 of the reference).

torch.compile runs with the aot_eager backend: it traces, functionalises and partitions the
graph exactly as the default backend does but generates no device code of its own, so the
only kernels that run are this library's.
"""
import pytest
import torch

from helpers import gen, make_states, make_wb, make_x, to_dev_like

pytestmark = pytest.mark.gpu

OPCHECKS = ("test_schema", "test_autograd_registration", "test_faketensor", "test_aot_dispatch_dynamic")


def _inputs(dev, dtype=torch.bfloat16, batch=2, dim=256, seqlen=96, width=4):
    g = gen(31)
    x = to_dev_like(make_x(batch, dim, seqlen, dtype, True, g, sliced=False), dev)
    w, b = make_wb(dim, width, True, g)
    return x, w.to(dev), b.to(dev)


def test_opcheck_fwd(pkg, gpu_device):
    x, w, b = _inputs(gpu_device)
    init = make_states(2, 256, 3, torch.bfloat16, gen(1)).to(gpu_device)
    out = torch.empty_like(x)
    fin = torch.empty(2, 3, 256, dtype=x.dtype, device=gpu_device).transpose(1, 2)
    op = torch.ops.DaoAILab._causal_conv1d_fwd_cpp
    torch.library.opcheck(op, (x, w, b, None, init, out, fin, True), test_utils=OPCHECKS)
    seq = torch.zeros(2, 96, dtype=torch.int32, device=gpu_device)
    seq[:, 40:] = 1
    torch.library.opcheck(op, (x, w, None, seq, None, out, None, False), test_utils=OPCHECKS)
    # the variant the Python layer uses: out allocated by the op and returned
    op = torch.ops.DaoAILab._causal_conv1d_fwd_out_cpp
    torch.library.opcheck(op, (x, w, b, None, init, fin, True), test_utils=OPCHECKS)
    torch.library.opcheck(op, (x, w, None, seq, None, None, False), test_utils=OPCHECKS)


def test_opcheck_bwd(pkg, gpu_device):
    x, w, b = _inputs(gpu_device)
    dout = torch.randn_like(x)
    dx = torch.empty_like(x)
    dw = torch.zeros_like(w)
    db = torch.zeros_like(b)
    init = make_states(2, 256, 3, torch.bfloat16, gen(2)).to(gpu_device)
    dfin = make_states(2, 256, 3, torch.bfloat16, gen(3)).to(gpu_device)
    dinit = torch.empty(2, 3, 256, dtype=x.dtype, device=gpu_device).transpose(1, 2)
    op = torch.ops.DaoAILab._causal_conv1d_bwd_cpp
    torch.library.opcheck(op, (x, w, b, dout, None, init, dfin, dx, dw, db, dinit, True), test_utils=OPCHECKS)
    # the variant the autograd function uses: dweight / dbias stored, not added to
    op = torch.ops.DaoAILab._causal_conv1d_bwd_overwrite_cpp
    torch.library.opcheck(op, (x, w, b, dout, None, init, dfin, dx, torch.empty_like(dw), torch.empty_like(db),
                               dinit, True), test_utils=OPCHECKS)


def test_opcheck_update(pkg, gpu_device):
    g = gen(4)
    dev = gpu_device
    x = torch.randn(4, 1, 256, generator=g).to(torch.bfloat16).transpose(1, 2).to(dev)
    state = torch.randn(6, 8, 256, generator=g).to(torch.bfloat16).transpose(1, 2).to(dev)
    w, b = make_wb(256, 4, True, g)
    out = torch.empty_like(x)
    cache = torch.tensor([0, 5, 9, 1000], dtype=torch.int32, device=dev)
    idx = torch.tensor([3, 0, -1, 5], dtype=torch.int32, device=dev)
    op = torch.ops.DaoAILab._causal_conv1d_update_cpp
    torch.library.opcheck(op, (x, state, w.to(dev), b.to(dev), out, True, cache, idx), test_utils=OPCHECKS)
    # the variant causal_conv1d_update uses: result allocated by the op, x (batch, dim) allowed
    op = torch.ops.DaoAILab._causal_conv1d_update_out_cpp
    torch.library.opcheck(op, (x, state, w.to(dev), b.to(dev), True, cache, idx), test_utils=OPCHECKS)
    torch.library.opcheck(op, (x[:, :, 0], state, w.to(dev), b.to(dev), False, None, idx), test_utils=OPCHECKS)


def test_compile_fn_forward_backward_matches_eager(pkg, gpu_device):
    x, w, b = _inputs(gpu_device)
    init = make_states(2, 256, 3, torch.bfloat16, gen(5)).to(gpu_device)

    def f(x, w, b, init):
        out, fin = pkg.causal_conv1d_fn(x, w, b, initial_states=init, return_final_states=True, activation="silu")
        return out, fin

    def run(fn):
        xs = [t.detach().clone().requires_grad_() for t in (x, w, b, init)]
        out, fin = fn(*xs)
        (out.float().square().sum() + fin.float().sum()).backward()
        return [out, fin] + [t.grad for t in xs]

    eager = run(f)
    compiled = run(torch.compile(f, backend="aot_eager", fullgraph=True))
    for a, e in zip(compiled, eager):
        assert torch.equal(a, e)


def test_compile_update_matches_eager(pkg, gpu_device):
    g = gen(6)
    dev = gpu_device
    w, b = make_wb(256, 4, True, g)
    w, b = w.to(dev), b.to(dev)
    x = torch.randn(4, 256, generator=g).to(torch.bfloat16).to(dev)
    state0 = torch.randn(4, 3, 256, generator=g).to(torch.bfloat16).transpose(1, 2).to(dev)

    def step(x, state):
        return pkg.causal_conv1d_update(x, state, w, b, activation="silu")

    s_eager, s_comp = state0.clone(), state0.clone()
    out_eager = step(x, s_eager)
    out_comp = torch.compile(step, backend="aot_eager", fullgraph=True)(x, s_comp)
    assert torch.equal(out_comp, out_eager)
    assert torch.equal(s_comp, s_eager)          # the in-place state advance survives functionalisation
    assert not torch.equal(s_comp, state0)
