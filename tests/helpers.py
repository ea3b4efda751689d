"""Helpers shared by the GPU parity tests: tolerances, seeded inputs in the layouts the
reference's tests use (tests/test_causal_conv1d.py:84-95), and comparison with context."""
import torch

# north-star tolerances: fp32 atol 1e-5; 16-bit rtol 1e-2 / atol 5e-2.  fp16 is held to the
# reference's own tighter pair (tests/test_causal_conv1d.py:75), which implies the former.
TOL = {torch.float32: (0.0, 1e-5), torch.float16: (3e-3, 5e-3), torch.bfloat16: (1e-2, 5e-2)}
TOL_W = (1e-3, 1e-3)      # dweight / dbias (tests/test_causal_conv1d.py:78)

DTYPES = [torch.float32, torch.float16, torch.bfloat16]


def gen(seed):
    g = torch.Generator()
    g.manual_seed(int(seed))
    return g


def make_x(batch, dim, seqlen, dtype, channel_last, g, sliced=True):
    """N(0,1) input of logical shape (batch, dim, seqlen).  `sliced` carves it out of a wider
    tensor (channels 4096 .. 4096+dim of 4096+dim+64) so batch/row strides are not dense."""
    full = 4096 + dim + 64 if sliced else dim
    lo = 4096 if sliced else 0
    if channel_last:
        return torch.randn(batch, seqlen, full, generator=g).to(dtype)[:, :, lo:lo + dim].transpose(1, 2)
    return torch.randn(batch, full, seqlen, generator=g).to(dtype)[:, lo:lo + dim, :]


def make_states(batch, dim, k, dtype, g):
    """(batch, dim, k) with unit stride along dim, as the reference allocates states."""
    return torch.randn(batch, k, dim, generator=g).to(dtype).transpose(1, 2)


def make_wb(dim, width, has_bias, g, w_dtype=torch.float32):
    w = (torch.rand(dim, width, generator=g) - 0.5).to(w_dtype)
    b = (torch.rand(dim, generator=g) - 0.5).to(w_dtype) if has_bias else None
    return w, b


def to_dev_like(t, dev):
    """Copy to the GPU keeping the (possibly non-dense) strides of a sliced tensor."""
    if t is None:
        return None
    if t.is_contiguous():
        return t.to(dev)
    base = torch.empty(t.untyped_storage().nbytes() // t.element_size(), dtype=t.dtype, device=dev)
    host = torch.empty(0, dtype=t.dtype).set_(t.untyped_storage(), 0, (base.numel(),), (1,))
    base.copy_(host)
    return torch.as_strided(base, t.shape, t.stride(), t.storage_offset())


def assert_close(got, ref, dtype=None, what="", tol=None):
    rtol, atol = tol if tol is not None else TOL[dtype if dtype is not None else ref.dtype]
    g, r = got.detach().float().cpu(), ref.detach().float().cpu()
    assert g.shape == r.shape, f"{what}: shape {tuple(g.shape)} vs {tuple(r.shape)}"
    bad = (g - r).abs() > atol + rtol * r.abs()
    if bad.any() or not torch.isfinite(g).all():
        idx = bad.nonzero()[0].tolist() if bad.any() else None
        raise AssertionError(
            f"{what}: {int(bad.sum())} of {g.numel()} outside rtol={rtol} atol={atol}; "
            f"max|diff|={(g - r).abs().max().item():.3e} first bad index {idx}")


def random_seq_idx(batch, seqlen, g, max_splits=4, pad=False):
    """int32 (batch, seqlen): 1..max_splits+1 sub-sequences per row with random boundaries
    (tests/test_causal_conv1d.py:426-442); with pad, a random tail of each row is -1
    (tests/test_causal_conv1d.py:499-532)."""
    rows, next_id = [], 0
    for _ in range(batch):
        true_len = seqlen if not pad else int(torch.randint(max(1, seqlen // 2), seqlen, (1,), generator=g))
        n = min(int(torch.randint(1, max_splits + 1, (1,), generator=g)), max(0, true_len - 1))
        cuts = (torch.randperm(true_len - 1, generator=g)[:n].sort().values + 1).tolist() if true_len > 1 else []
        bounds = [0] + cuts + [true_len]
        row = []
        for i in range(len(bounds) - 1):
            row += [next_id] * (bounds[i + 1] - bounds[i])
            next_id += 1
        row += [-1] * (seqlen - true_len)
        rows.append(torch.tensor(row, dtype=torch.int32))
        if not pad:
            next_id = 0
    return torch.stack(rows)
