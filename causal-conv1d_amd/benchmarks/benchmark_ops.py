#!/usr/bin/env python
"""Times one operator of the package at a shape given on the command line and prints
microseconds per call, achieved GB/s against the bytes the operator must move, and peak
device memory.  The role of tests/benchmark_determinism_kernels.py in the reference, for
all four operators; there is no deterministic/non-deterministic pair to compare because the
backward here is always a fixed-order two-stage sum.

  python benchmark_ops.py --op fwd --batch 8 --dim 5376 --seqlen 2048 --channel-last --seq-idx
  python benchmark_ops.py --op bwd --batch 4 --dim 4096 --seqlen 8192 --dtype fp16 --states
  python benchmark_ops.py --op update --batch 256 --dim 5376 --state-len 8 --circular
  python benchmark_ops.py --op varlen --batch 64 --dim 5376 --seqlen 1024
  python benchmark_ops.py --op prefill --batch 16 --dim 5376 --seqlen 256

With --rocprof DIR the same measurement runs once more as a child process under
`rocprofv3 --kernel-trace --stats -d DIR -o benchmark_ops -- python3 benchmark_ops.py ...` and the
device-side duration of every kernel of this library in that run (average, median, minimum,
maximum over its dispatches, without the gaps between dispatches that event timing includes) is
printed below the table; the raw trace stays in DIR.
"""
import argparse
import gc
import glob
import os
import sqlite3
import statistics
import subprocess
import sys

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))

import torch

from causal_conv1d import (causal_conv1d_fn, causal_conv1d_fwd_varlen_states, causal_conv1d_update,
                           causal_conv1d_varlen_states)
from causal_conv1d.cpp_functions import causal_conv1d_bwd_function

HBM_PEAK_GBS = 8000.0


def timed(fn, warmup, rep, iters):
    """Median over `iters` groups of `rep` back-to-back calls, in microseconds per call."""
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    groups = []
    for _ in range(iters):
        start.record()
        for _ in range(rep):
            fn()
        end.record()
        torch.cuda.synchronize()
        groups.append(start.elapsed_time(end) * 1e3 / rep)
    return statistics.median(groups)


def peak_mb(fn):
    fn()
    torch.cuda.synchronize()
    gc.collect()
    torch.cuda.empty_cache()
    torch.cuda.reset_peak_memory_stats()
    base = torch.cuda.memory_allocated()
    fn()
    torch.cuda.synchronize()
    return (torch.cuda.max_memory_allocated() - base) / 2**20


def kernel_durations(trace_dir):
    """{kernel name: [durations in us]} of this library's kernels from the rocprofv3 result
    database(s) under trace_dir (the `kernels` view: name, start and end in nanoseconds)."""
    per_kernel = {}
    for db_path in sorted(glob.glob(os.path.join(trace_dir, "**", "*_results.db"), recursive=True)):
        db = sqlite3.connect(db_path)
        try:
            rows = db.execute("select name, start, end from kernels order by start").fetchall()
        finally:
            db.close()
        for name, start, end in rows:
            if "cc1d" in name:
                short = name.replace("void cc1d::(anonymous namespace)::", "").replace("cc1d::", "")
                short = short[:short.find("(")] if "(" in short else short
                per_kernel.setdefault(short, []).append((end - start) * 1e-3)
    return per_kernel


def run_under_rocprof(trace_dir, argv):
    """The same command line, minus --rocprof, as a child of rocprofv3; returns the lines of the
    kernel table.  Called before anything here has touched the GPU."""
    child_args, skip = [], False
    for arg in argv:
        if skip:
            skip = False
        elif arg == "--rocprof":
            skip = True
        elif not arg.startswith("--rocprof="):
            child_args.append(arg)
    os.makedirs(trace_dir, exist_ok=True)
    # The program after `--` is this interpreter's own binary: a `python3` found on PATH may be a
    # shim or a script that starts the real interpreter by exec, after rocprofv3's preloaded
    # library has already initialised the GPU in it.
    interpreter = os.path.realpath(sys.executable)
    with open(interpreter, "rb") as f:
        if f.read(4) != b"\x7fELF":
            sys.exit("--rocprof: %s is not an ELF binary; rocprofv3 must start the interpreter itself" % interpreter)
    cmd = ["rocprofv3", "--kernel-trace", "--stats", "-d", trace_dir, "-o", "benchmark_ops", "--",
           interpreter, os.path.abspath(__file__)] + child_args
    print("+ " + " ".join(cmd), flush=True)
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if res.returncode != 0:
        sys.exit("rocprofv3 run failed (%d):\n%s" % (res.returncode, res.stdout[-4000:]))
    per_kernel = kernel_durations(trace_dir)
    if not per_kernel:
        sys.exit("rocprofv3 run left no kernel records of this library under " + trace_dir)
    lines = ["device-side kernel durations (rocprofv3 --kernel-trace), microseconds",
             "%6s %9s %9s %9s %9s  %s" % ("calls", "avg", "median", "min", "max", "kernel")]
    for name, d in sorted(per_kernel.items(), key=lambda kv: -sum(kv[1])):
        lines.append("%6d %9.2f %9.2f %9.2f %9.2f  %s" % (len(d), sum(d) / len(d), statistics.median(d), min(d), max(d), name))
    return lines


def nbytes(*ts):
    return sum(t.numel() * t.element_size() for t in ts if t is not None)


def main():
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--op", choices=["fwd", "bwd", "update", "varlen", "prefill"], default="fwd",
                    help="prefill: forward over --batch packed sequences plus their varlen final states, as one "
                         "call and as the two separate calls")
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--dim", type=int, default=5376)
    ap.add_argument("--seqlen", type=int, default=2048, help="per-sequence length (varlen: mean length)")
    ap.add_argument("--width", type=int, default=4, choices=[2, 3, 4])
    ap.add_argument("--dtype", choices=["fp16", "bf16", "fp32"], default="bf16")
    ap.add_argument("--channel-last", action="store_true")
    ap.add_argument("--seq-idx", action="store_true", help="fwd/bwd: 4 packed sub-sequences per row")
    ap.add_argument("--states", action="store_true", help="fwd/bwd: initial_states and final states")
    ap.add_argument("--no-bias", action="store_true")
    ap.add_argument("--activation", choices=["none", "silu"], default="silu")
    ap.add_argument("--state-len", type=int, default=3, help="update/varlen: conv_state length")
    ap.add_argument("--circular", action="store_true", help="update: cache_seqlens ring buffer")
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--rep", type=int, default=50)
    ap.add_argument("--iters", type=int, default=20)
    ap.add_argument("--rocprof", metavar="DIR", default=None,
                    help="also run under rocprofv3 --kernel-trace into DIR and print device-side kernel durations")
    a = ap.parse_args()
    # The profiled run goes first, while this process has not touched the GPU yet.
    profile_lines = run_under_rocprof(a.rocprof, sys.argv[1:]) if a.rocprof else []

    dev = "cuda"
    dtype = {"fp16": torch.float16, "bf16": torch.bfloat16, "fp32": torch.float32}[a.dtype]
    act = None if a.activation == "none" else "silu"
    B, D, L, W = a.batch, a.dim, a.seqlen, a.width
    weight = torch.rand(D, W, device=dev) - 0.5
    bias = None if a.no_bias else torch.rand(D, device=dev) - 0.5

    def make(shape_bld):
        b, d, l = shape_bld
        if a.channel_last:
            return torch.randn(b, l, d, device=dev, dtype=dtype).transpose(1, 2)
        return torch.randn(b, d, l, device=dev, dtype=dtype)

    if a.op in ("fwd", "bwd"):
        x = make((B, D, L))
        seq = None
        if a.seq_idx:
            seq = (torch.arange(L, device=dev, dtype=torch.int32) * 4 // L).expand(B, L).contiguous()
        init = torch.randn(B, W - 1, D, device=dev, dtype=dtype).transpose(1, 2) if a.states else None
        if a.op == "fwd":
            fn = lambda: causal_conv1d_fn(x, weight, bias, seq_idx=seq, initial_states=init,
                                          return_final_states=a.states, activation=act)
            moved = 2 * nbytes(x) + nbytes(seq, weight, bias, init) + (nbytes(init) if a.states else 0)
        else:
            dout = torch.randn_like(x)
            dx = torch.empty_like(x)
            dfin = torch.randn(B, W - 1, D, device=dev, dtype=dtype).transpose(1, 2) if a.states else None
            fn = lambda: causal_conv1d_bwd_function(x, weight, bias, dout, seq, init, dfin, dx, a.states, act == "silu")
            moved = 3 * nbytes(x) + nbytes(seq, weight, bias, init, dfin) + (nbytes(init) if a.states else 0) + \
                (W + (0 if a.no_bias else 1)) * D * 4
    elif a.op == "update":
        S = a.state_len
        x = torch.randn(B, D, device=dev, dtype=dtype)
        state = torch.randn(B, S, D, device=dev, dtype=dtype).transpose(1, 2)
        cache = torch.randint(0, 1000, (B,), device=dev, dtype=torch.int32) if a.circular else None
        fn = lambda: causal_conv1d_update(x, state, weight, bias, activation=act, cache_seqlens=cache)
        per_chan = (1 + (W - 1) + 1 + 1) if a.circular else (1 + S + S + 1)   # x, state reads, state writes, out
        moved = per_chan * B * D * x.element_size() + nbytes(weight, bias, cache)
    elif a.op == "prefill":
        S = a.state_len
        x = torch.randn(1, B * L, D, device=dev, dtype=dtype).transpose(1, 2)
        cu = torch.arange(B + 1, device=dev, dtype=torch.int32) * L
        seq = (torch.arange(B * L, device=dev, dtype=torch.int32) // L).reshape(1, B * L)
        tokens = x[0].t()

        def two_calls():
            causal_conv1d_fn(x, weight, bias, seq_idx=seq, activation=act)
            causal_conv1d_varlen_states(tokens, cu, S)
        with torch.no_grad():
            print("two calls: %.2f us" % timed(two_calls, a.warmup, a.rep, a.iters))
        fn = lambda: causal_conv1d_fwd_varlen_states(x, weight, bias, seq, cu, S, activation=act)
        moved = 2 * nbytes(x) + nbytes(seq, weight, bias, cu) + 2 * B * D * S * x.element_size()
    else:
        S = a.state_len
        lens = torch.randint(max(1, L // 2), L + L // 2, (B,))
        cu = torch.zeros(B + 1, dtype=torch.int32)
        cu[1:] = lens.cumsum(0)
        x = torch.randn(int(cu[-1]), D, device=dev, dtype=dtype)
        cu = cu.to(dev)
        fn = lambda: causal_conv1d_varlen_states(x, cu, S)
        moved = 2 * B * D * S * x.element_size() + nbytes(cu)

    with torch.no_grad():
        us = timed(fn, a.warmup, a.rep, a.iters)
        mb = peak_mb(fn)
    gbs = moved / us / 1e3
    print("GPU: %s" % torch.cuda.get_device_name(0))
    print("op=%s batch=%d dim=%d seqlen=%d width=%d dtype=%s channel_last=%s seq_idx=%s states=%s bias=%s act=%s"
          % (a.op, B, D, L, W, a.dtype, a.channel_last, a.seq_idx, a.states, not a.no_bias, a.activation))
    print("%10s %12s %10s %12s %10s" % ("us/call", "bytes moved", "GB/s", "% of 8 TB/s", "peak MB"))
    print("%10.2f %12d %10.1f %12.1f %10.1f" % (us, moved, gbs, 100 * gbs / HBM_PEAK_GBS, mb), flush=True)
    if profile_lines:
        print("\n".join(profile_lines), flush=True)


if __name__ == "__main__":
    main()
