#!/usr/bin/env python3
"""Benchmark of the causal conv1d hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-others] [--no-cpu] [--no-rotated]
                    [--no-settle] [--only update|rotated] [--decode-calls N]

Prints ONE JSON line.  A "step" is one forward call at the Mamba-2 2.7B prefill shape
(bf16, batch 8, dim 5376, seqlen 2048, channel-last, width 4, bias, SiLU, seq_idx with
1-4 packed sub-sequences per row), inputs resident in HBM before the timed region.

  value / unit ..... algorithmic bytes moved per second by that forward (GB/s); the
                     algorithmic bytes count every input element read once and every
                     output element written once (x, out, seq_idx, weight, bias)
  roofline ......... the same bytes over the average kernel time measured with HIP events
                     around the timed launches, against the 8 TB/s HBM3E peak.  `frac` (and
                     `value`) is the sustained rate: the K timed steps follow 400 untimed
                     back-to-back launches of the same call, so the clock has settled where it
                     stays under load; `frac_burst` is the same K steps out of an idle device
                     (a few milliseconds of load at the highest clock); `frac_rotated` runs over
                     six rotating sets of x and out (2.1 GB), where no launch finds its tensors in
                     a cache, as the layers of a model do, behind the same 400 untimed launches
                     (none with --no-settle); config.us_per_call_rotated_12_sets is the same over
                     twelve sets (4.2 GB).  `decode` repeats
                     the three figures for the two decode-step updates.  `traffic` is imported
                     from the committed rocprofv3 summary, not measured in this run
  cpu_baseline ..... the PyTorch oracle (F.conv1d per packed sub-sequence) timed on this
                     host's cores on the same inputs
  others ........... µs per call and GB/s of the remaining shapes: decode-step update
                     (linear and circular state), backward, varlen state gather, and the
                     forward width/dtype sweep; "rotated" figures cycle through enough
                     distinct buffer sets to exceed the 256 MB Infinity Cache

The timed loops call the extension entry points directly with pre-allocated outputs, the
way the reference's own benchmark does (tests/benchmark_determinism_kernels.py:72).
"""
import argparse
import json
import math
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
PKG_DIR = os.path.join(ROOT, "causal-conv1d_amd")
for _p in (ROOT, PKG_DIR):
    if _p not in sys.path:
        sys.path.insert(0, _p)

HBM_PEAK_GBS = 8000.0
INFINITY_CACHE_BYTES = 256 * 1024 * 1024


# --------------------------------------------------------------------------- workloads
def _gen(seed):
    import torch
    g = torch.Generator()
    g.manual_seed(seed)
    return g


def make_weights(dim, width, seed, w_dtype=None):
    import torch
    g = _gen(1000 + seed)
    w = torch.rand(dim, width, generator=g) - 0.5
    b = torch.rand(dim, generator=g) - 0.5
    if w_dtype is not None:
        w, b = w.to(w_dtype), b.to(w_dtype)
    return w, b


def make_seq_idx(batch, seqlen, seed, max_segments=4):
    """Per row: 1..max_segments packed sub-sequences with random boundaries, ids 0..n-1."""
    import torch
    g = _gen(2000 + seed)
    rows = []
    for _ in range(batch):
        n = int(torch.randint(1, max_segments + 1, (1,), generator=g))
        n = min(n, seqlen)
        cuts = torch.randperm(seqlen - 1, generator=g)[: n - 1].sort().values + 1 if seqlen > 1 else torch.tensor([], dtype=torch.long)
        bounds = [0] + cuts.tolist() + [seqlen]
        rows.append(torch.cat([torch.full((bounds[i + 1] - bounds[i],), i, dtype=torch.int32)
                               for i in range(len(bounds) - 1)]))
    return torch.stack(rows)


def make_x(batch, dim, seqlen, dtype, channel_last, seed):
    """N(0,1) tensor of logical shape (batch, dim, seqlen) in the requested memory layout."""
    import torch
    g = _gen(seed)
    if channel_last:
        return torch.randn(batch, seqlen, dim, generator=g).to(dtype).transpose(1, 2)
    return torch.randn(batch, dim, seqlen, generator=g).to(dtype)


def config_c1():
    import torch
    w, b = make_weights(64, 4, 1)
    return dict(x=make_x(2, 64, 512, torch.float32, False, 1), weight=w, bias=b)


def config_c2(batch=8, dim=5376, seqlen=2048):
    import torch
    w, b = make_weights(dim, 4, 2)
    return dict(x=make_x(batch, dim, seqlen, torch.bfloat16, True, 2), weight=w, bias=b,
                seq_idx=make_seq_idx(batch, seqlen, 2))


def config_c3(circular, batch=256, dim=5376, seed=3):
    import torch
    w, b = make_weights(dim, 4, 3)
    state_len = 8 if circular else 3
    g = _gen(3000 + seed)
    cfg = dict(x=make_x(batch, dim, 1, torch.bfloat16, True, seed), weight=w, bias=b,
               conv_state=make_x(batch, dim, state_len, torch.bfloat16, True, seed + 50))
    if circular:
        cfg["cache_seqlens"] = torch.randint(0, 1000, (batch,), generator=g, dtype=torch.int32)
    return cfg


def config_c4(batch=4, dim=4096, seqlen=8192):
    import torch
    w, b = make_weights(dim, 4, 4)
    return dict(x=make_x(batch, dim, seqlen, torch.float16, False, 4), weight=w, bias=b,
                dout=make_x(batch, dim, seqlen, torch.float16, False, 41),
                initial_states=make_x(batch, dim, 3, torch.float16, True, 42),
                dfinal_states=make_x(batch, dim, 3, torch.float16, False, 43))


def config_c5a(total=65536, n_seq=64, dim=5376):
    import torch
    g = _gen(5)
    lens = torch.randint(16, 2048, (n_seq,), generator=g).double()
    lens = torch.clamp((lens / lens.sum() * total).floor().long(), min=3)
    lens[-1] += total - int(lens.sum())
    assert int(lens.sum()) == total and int(lens.min()) >= 3
    cu = torch.nn.functional.pad(lens.cumsum(0), (1, 0)).to(torch.int32)
    x = torch.randn(total, dim, generator=g).to(torch.bfloat16)
    return dict(x=x, cu_seqlens=cu, state_len=3)


def config_c5b(width, dtype, channel_last, batch=4, dim=2048, seqlen=4096):
    w, b = make_weights(dim, width, 50 + width)
    return dict(x=make_x(batch, dim, seqlen, dtype, channel_last, 50 + width), weight=w, bias=b)


def kernel_sources_sha16(names):
    """First 16 hex digits of the SHA-256 over the named kernel sources, in order."""
    import hashlib
    h = hashlib.sha256()
    for n in names:
        with open(os.path.join(PKG_DIR, "csrc", n), "rb") as f:
            h.update(f.read())
    return h.hexdigest()[:16]


def profile_figures(profile, sources):
    """`key: number` lines of a committed rocprofv3 summary under profiles/, or {} when the
    summary is missing or was made from other kernel sources than the ones in the tree (it
    names them by hash): a counter figure is only reported next to the code it was read on."""
    path = os.path.join(ROOT, "profiles", profile)
    if not os.path.exists(path):
        return {}
    figs = {}
    for ln in open(path):
        key, sep, val = ln.partition(":")
        if sep and key.strip().replace("_", "").isalnum() and " " not in key.strip():
            figs[key.strip()] = val.strip()
    if figs.get("kernel_sources_sha16") != kernel_sources_sha16(sources):
        return {}
    figs["profile"] = "profiles/" + profile
    return figs


FWD_CL_SOURCES = ("cc1d_fwd_channellast.hip", "cc1d_device.hpp", "cc1d_varlen_gather.hpp")
UPDATE_SOURCES = ("cc1d_update.hip", "cc1d_device.hpp")


def nbytes(*tensors):
    return sum(t.numel() * t.element_size() for t in tensors if t is not None)


# ------------------------------------------------------------------------------ timing
def time_gpu(fn, steps, warmup):
    """Average µs per call of fn(i) over `steps` calls after `warmup`, by HIP events on the
    current stream, with the device idle on both sides."""
    import torch
    for i in range(warmup):
        fn(i)
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    start.record()
    for i in range(steps):
        fn(i)
    stop.record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    return start.elapsed_time(stop) * 1e3 / steps, wall * 1e6 / steps


def to_dev(cfg, dev):
    import torch
    return {k: (v.to(dev) if isinstance(v, torch.Tensor) else v) for k, v in cfg.items()}


def clone_sets(cfg, bytes_per_set, max_sets=64):
    """Enough independent copies of the device tensors to exceed the Infinity Cache."""
    import torch
    n = min(max_sets, max(2, math.ceil(2 * INFINITY_CACHE_BYTES / max(1, bytes_per_set))))
    def cp(v):
        if not isinstance(v, torch.Tensor):
            return v
        if v.dim() == 3 and v.stride(1) == 1 and v.stride(2) > 1:      # keep channel-last
            return v.transpose(1, 2).clone().transpose(1, 2)
        return v.clone()
    return [{k: cp(v) for k, v in cfg.items()} for _ in range(n)]


def update_algorithmic_bytes(cfg, circular):
    """Decode step: x, out, taps and bias once; the state's W-1 window rows read and, linear, every
    state row written (S = W-1 here), or, circular, one row written plus cache_seqlens."""
    x, st = cfg["x"], cfg["conv_state"]
    n = nbytes(x, x, cfg["weight"], cfg["bias"])
    if circular:
        return n + 3 * nbytes(x) + nbytes(x) + nbytes(cfg["cache_seqlens"])
    return n + 2 * nbytes(st)


def gbs(n_bytes, us):
    return n_bytes / us * 1e-3 if us > 0 else 0.0


# ---------------------------------------------------------------------- the other shapes
def bench_others(ext, dev, steps, warmup, rotated=True, only_update=False, decode_calls=400):
    import torch
    res = {}

    def record(name, us, n_bytes, extra=None):
        res[name] = {"us": round(us, 3), "GBps": round(gbs(n_bytes, us), 1),
                     "frac_of_hbm_peak": round(gbs(n_bytes, us) / HBM_PEAK_GBS, 4),
                     "algorithmic_bytes": int(n_bytes)}
        if extra:
            res[name].update(extra)

    def settled(call, n_bytes):
        """The same call behind 400 untimed launches (40-60 ms of load), where the clock has
        settled: `us` above is a burst out of a nearly idle device."""
        us, _ = time_gpu(call, max(10, steps // 4), 400)
        return {"us_settled": round(us, 3), "frac_of_hbm_peak_settled": round(gbs(n_bytes, us) / HBM_PEAK_GBS, 4)}

    # C3: decode-step update, linear and circular.
    prof = profile_figures("update_step_decode_device_time.txt", UPDATE_SOURCES)
    for circular in (False, True):
        name = "update_circular_s8" if circular else "update_linear_s3"
        cfg = to_dev(config_c3(circular), dev)
        x, st = cfg["x"], cfg["conv_state"]
        n_bytes = update_algorithmic_bytes(cfg, circular)
        out = torch.empty_like(x)
        cs = cfg.get("cache_seqlens")
        # A launch of 4-7 us: a few hundred of them, so that the figure is the device's steady rate
        # and not the first launches of an empty queue, and no Python work per call beyond the call.
        n_calls, n_warm = max(steps, decode_calls), max(warmup, decode_calls // 10)
        update = ext.causal_conv1d_update
        args = (x, st, cfg["weight"], cfg["bias"], out, True, cs, None)
        us, wall = time_gpu(lambda i: update(*args), n_calls, n_warm)
        extra = {"us_wall_per_call": round(wall, 2), "calls_timed": n_calls}
        if rotated:
            sets = clone_sets(cfg, nbytes(x, st, x))
            rot_args = [(s["x"], s["conv_state"], s["weight"], s["bias"], torch.empty_like(s["x"]), True,
                         s.get("cache_seqlens"), None) for s in sets]
            n_sets = len(rot_args)
            us_rot, _ = time_gpu(lambda i: update(*rot_args[i % n_sets]), n_calls, n_warm)
            extra.update({"us_rotated": round(us_rot, 3), "GBps_rotated": round(gbs(n_bytes, us_rot), 1),
                          "frac_of_hbm_peak_rotated": round(gbs(n_bytes, us_rot) / HBM_PEAK_GBS, 4),
                          "rotated_sets": len(sets)})
            del sets, rot_args
        # Device duration of the warm launches by rocprofv3 (no dispatch gap in it), from the
        # committed summary of `bench.py --only update`, while the kernel is the one profiled.
        key = "circular_us_device_avg" if circular else "linear_us_device_avg"
        if key in prof:
            extra.update({"us_device_rocprof": float(prof[key]), "us_device_rocprof_source": prof["profile"]})
        record(name, us, n_bytes, extra)
    # The same step on the cache layout of mamba_ssm's Mamba block and transformers' MambaCache:
    # conv_state (batch, d_inner, d_conv) contiguous, unit stride along state_len.  Algorithmic
    # bytes: x, out, taps, bias, the W-1 window positions read and every state position written.
    cfg = to_dev(config_c3(False, dim=5120), dev)
    x = cfg["x"]
    st = torch.randn(x.shape[0], x.shape[1], 4, device=dev).to(x.dtype)
    out = torch.empty_like(x)
    n_bytes = nbytes(x, x, cfg["weight"], cfg["bias"]) + nbytes(st) * 7 // 4
    n_calls, n_warm = max(steps, decode_calls), max(warmup, decode_calls // 10)
    args = (x, st, cfg["weight"], cfg["bias"], out, True, None, None)
    us, wall = time_gpu(lambda i: ext.causal_conv1d_update(*args), n_calls, n_warm)
    extra = {"us_wall_per_call": round(wall, 2), "calls_timed": n_calls,
             "layout": "conv_state (256, 5120, 4) contiguous, bf16, width 4"}
    if rotated:
        n_sets = 40
        rot_args = [(torch.randn_like(x), torch.randn_like(st), cfg["weight"].clone(), cfg["bias"].clone(),
                     torch.empty_like(x), True, None, None) for _ in range(n_sets)]
        us_rot, _ = time_gpu(lambda i: ext.causal_conv1d_update(*rot_args[i % n_sets]), n_calls, n_warm)
        extra.update({"us_rotated": round(us_rot, 3), "GBps_rotated": round(gbs(n_bytes, us_rot), 1),
                      "frac_of_hbm_peak_rotated": round(gbs(n_bytes, us_rot) / HBM_PEAK_GBS, 4), "rotated_sets": n_sets})
        del rot_args
    if "contiguous_us_device_avg" in prof:
        extra.update({"us_device_rocprof": float(prof["contiguous_us_device_avg"]), "us_device_rocprof_source": prof["profile"]})
    record("update_linear_s4_state_contiguous", us, n_bytes, extra)

    if only_update:
        return res

    # What this box charges for any launch of the decode step's size, measured the same way:
    # a device-to-device copy moving as many bytes as the linear step (half read, half written)
    # and a one-element fill (a launch that moves nothing).
    half = res["update_linear_s3"]["algorithmic_bytes"] // 2
    src = torch.empty(half, dtype=torch.uint8, device=dev)
    dst = torch.empty_like(src)
    one = torch.empty(1, device=dev)
    us_copy, _ = time_gpu(lambda i: dst.copy_(src), n_calls, n_warm)
    us_fill, _ = time_gpu(lambda i: one.fill_(1.0), n_calls, n_warm)
    res["launch_floors"] = {"copy_of_update_linear_bytes_us": round(us_copy, 3),
                            "one_element_fill_us": round(us_fill, 3), "copy_bytes": 2 * half}
    del src, dst

    # C4: backward, fp16 channel-first with initial states and dfinal.
    cfg = to_dev(config_c4(), dev)
    x = cfg["x"]
    dx = torch.empty_like(x)
    dw = torch.zeros(x.shape[1], 4, device=dev, dtype=torch.float32)
    db = torch.zeros(x.shape[1], device=dev, dtype=torch.float32)
    dinit = torch.empty(x.shape[0], 3, x.shape[1], device=dev, dtype=x.dtype).transpose(1, 2)
    n_bytes = nbytes(x, cfg["dout"], dx, cfg["initial_states"], cfg["dfinal_states"], dinit,
                     cfg["weight"], cfg["bias"], dw, db)
    call = lambda i: ext.causal_conv1d_bwd(x, cfg["weight"], cfg["bias"], cfg["dout"], None,
                                           cfg["initial_states"], cfg["dfinal_states"], dx, dw, db, dinit, True)
    us, _ = time_gpu(call, max(10, steps // 4), max(3, warmup // 4))
    record("bwd_c4_fp16_channelfirst", us, n_bytes, settled(call, n_bytes))
    del cfg, x, dx

    # Backward, channel-last at the prefill shape (bf16, seq_idx).
    cfg = to_dev(config_c2(), dev)
    x = cfg["x"]
    dout = to_dev(dict(d=make_x(8, 5376, 2048, torch.bfloat16, True, 21)), dev)["d"]
    dx = torch.empty_like(x)
    dw = torch.zeros(x.shape[1], 4, device=dev, dtype=torch.float32)
    db = torch.zeros(x.shape[1], device=dev, dtype=torch.float32)
    n_bytes = nbytes(x, dout, dx, cfg["seq_idx"], cfg["weight"], cfg["bias"], dw, db)
    call = lambda i: ext.causal_conv1d_bwd(x, cfg["weight"], cfg["bias"], dout, cfg["seq_idx"],
                                           None, None, dx, dw, db, None, True)
    us, _ = time_gpu(call, max(10, steps // 4), max(3, warmup // 4))
    record("bwd_prefill_bf16_channellast_seqidx", us, n_bytes, settled(call, n_bytes))
    del cfg, x, dx, dout

    # C5a: varlen state gather.
    cfg = to_dev(config_c5a(), dev)
    states = torch.empty(64, 3, 5376, device=dev, dtype=torch.bfloat16).transpose(1, 2)
    n_bytes = 2 * nbytes(states) + nbytes(cfg["cu_seqlens"])
    us, _ = time_gpu(lambda i: ext.causal_conv1d_varlen_states(cfg["x"], cfg["cu_seqlens"], states, 3), steps, warmup)
    record("varlen_states_c5a", us, n_bytes, {"bound": "launch: 4 MB move in well under the ~2.5 us a dispatch costs"})
    del cfg

    # C5b: forward sweep over width x dtype x layout.
    for dtype, dn in ((torch.float32, "fp32"), (torch.float16, "fp16"), (torch.bfloat16, "bf16")):
        for layout in (False, True):
            for width in (2, 3, 4):
                cfg = to_dev(config_c5b(width, dtype, layout), dev)
                x = cfg["x"]
                out = torch.empty_like(x)
                n_bytes = nbytes(x, out, cfg["weight"], cfg["bias"])
                us, _ = time_gpu(lambda i: ext.causal_conv1d_fwd(x, cfg["weight"], cfg["bias"], None, None, out, None, True),
                                 max(20, steps // 2), max(5, warmup // 2))
                record("fwd_sweep_%s_%s_w%d" % (dn, "channellast" if layout else "channelfirst", width), us, n_bytes)
    return res


# ------------------------------------------------------------------------ CPU baseline
def cpu_baseline(cfg_cpu, n_bytes, gpu_out):
    """The PyTorch oracle on the host, same inputs, whole C2 workload per repetition.  Its
    result doubles as the check of what the GPU just produced (`gpu_out`, already on the
    host): this is the only place the benchmark touches the oracle."""
    import torch
    from oracle import causal_conv1d_oracle as orc
    cores = os.cpu_count() or 1
    cores = min(cores, int(os.environ.get("OMP_NUM_THREADS", cores)))
    torch.set_num_threads(cores)
    x, w, b, seq = cfg_cpu["x"], cfg_cpu["weight"], cfg_cpu["bias"], cfg_cpu["seq_idx"]
    with torch.no_grad():
        orc.fwd_seq_idx(x, w, b, seq, activation="silu")           # warm-up
        times = []
        t_end = time.perf_counter() + 20.0
        while len(times) < 5 and (len(times) < 2 or time.perf_counter() < t_end):
            t0 = time.perf_counter()
            ref = orc.fwd_seq_idx(x, w, b, seq, activation="silu")
            times.append(time.perf_counter() - t0)
    med = sorted(times)[len(times) // 2]
    err = (gpu_out.float() - ref.float()).abs_()
    parity_ok = bool(torch.all(err <= 5e-2 + 1e-2 * ref.float().abs()))      # bf16: rtol 1e-2, atol 5e-2
    model = "unknown"
    try:
        with open("/proc/cpuinfo") as f:
            model = next((ln.split(":", 1)[1].strip() for ln in f if ln.startswith("model name")), model)
    except OSError:
        pass
    return {"value": round(n_bytes / med * 1e-9, 3), "unit": "GB/s", "cores": torch.get_num_threads(),
            "kind": "port", "us_per_call": round(med * 1e6, 1), "cpu_model": model,
            "host_cpu_count": os.cpu_count(),
            "gpu_output_matches": parity_ok, "gpu_max_abs_err": float(err.max()),
            "sample": "the full prefill workload (8 x 5376 x 2048 bf16 + seq_idx), median of %d calls "
                      "of the PyTorch F.conv1d oracle after one warm-up" % len(times)}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=30)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--no-others", action="store_true", help="time only the headline forward")
    ap.add_argument("--no-cpu", action="store_true", help="skip the host CPU baseline")
    ap.add_argument("--no-rotated", action="store_true", help="skip the headline over rotating buffer sets")
    ap.add_argument("--no-settle", action="store_true",
                    help="time the K steps out of an idle device (the burst figure) instead of after 400 "
                         "untimed launches; `value` is then the burst")
    ap.add_argument("--decode-calls", type=int, default=400,
                    help="launches timed per decode-step figure (at least --steps); counter passes use few")
    ap.add_argument("--only", choices=["update", "rotated"], default=None,
                    help="update: time nothing but the warm decode-step launches (linear, then circular); "
                         "rotated: nothing but the headline forward over its six rotating buffer sets, then "
                         "torch.add over the same sets (K steps each behind --warmup untimed ones).  The "
                         "commands whose rocprofv3 kernel traces and counters give device durations and traffic")
    ap.add_argument("--copy-probe", action="store_true",
                    help="also run a plain device copy of x (a kernel of known size, to scale profiler counters)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on one GPU; --gpus %d is not supported "
                 "(the operator needs no cross-GPU communication; run one process per GPU on disjoint batches)" % args.gpus)

    import torch
    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible; the benchmark has no CPU fallback")
    import causal_conv1d_cuda as ext          # fails loudly if the extension was not built
    dev = torch.device("cuda:0")
    if args.only == "update":
        res = bench_others(ext, dev, args.steps, args.warmup, rotated=False, only_update=True,
                           decode_calls=args.decode_calls)
        print(json.dumps({"only": "update", "steps": args.steps, "warmup": args.warmup, "others": res}), flush=True)
        return

    cfg_cpu = config_c2()
    cfg = to_dev(cfg_cpu, dev)
    x, w, b, seq = cfg["x"], cfg["weight"], cfg["bias"], cfg["seq_idx"]
    out = torch.empty_like(x)
    n_bytes = nbytes(x, out, seq, w, b)

    def step(i):
        ext.causal_conv1d_fwd(x, w, b, seq, None, out, None, True)

    def rotated_sets():
        # Six sets of x and out (2.1 GB): a launch never finds its tensors in a cache.
        return [(x, out)] + [(torch.randn_like(x), torch.empty_like(x)) for _ in range(5)]

    if args.only == "rotated":
        sets = rotated_sets()
        rot_us, _ = time_gpu(lambda i: ext.causal_conv1d_fwd(sets[i % 6][0], w, b, seq, None, sets[i % 6][1], None, True),
                             args.steps, args.warmup)
        add_us, _ = time_gpu(lambda i: torch.add(sets[i % 6][0], 1.0, out=sets[i % 6][1]), args.steps, args.warmup)
        print(json.dumps({"only": "rotated", "steps": args.steps, "warmup": args.warmup, "rotated_sets": 6,
                          "us_per_call_rotated": round(rot_us, 3), "algorithmic_bytes": int(n_bytes),
                          "frac_rotated": round(gbs(n_bytes, rot_us) / HBM_PEAK_GBS, 4),
                          "us_torch_add_rotated": round(add_us, 3)}), flush=True)
        return

    # The burst: K steps out of an idle device.  Then the figure the line carries: the same K steps
    # right behind 400 untimed launches (about 22 ms of load), where the clock has settled.
    burst_us, burst_wall = time_gpu(step, args.steps, args.warmup)
    if args.no_settle:
        us, wall_us, settle = burst_us, burst_wall, 0
    else:
        settle = 400
        us, wall_us = time_gpu(step, args.steps, args.warmup + settle)
    if args.copy_probe:
        flat_src = torch.empty(x.numel(), dtype=x.dtype, device=dev).normal_()
        flat_dst = torch.empty_like(flat_src)
        copy_us, _ = time_gpu(lambda i: flat_dst.copy_(flat_src), args.steps, args.warmup)
        print("copy probe: %d bytes read + %d bytes written per launch, %.2f us" %
              (nbytes(flat_src), nbytes(flat_dst), copy_us), file=sys.stderr)
        del flat_src, flat_dst

    gpu_out_host = out.cpu()                # checked against the CPU baseline's result below

    # End-to-end through the public Python API (allocation + op dispatch included).
    from causal_conv1d import causal_conv1d_fn
    with torch.no_grad():
        _, api_wall = time_gpu(lambda i: causal_conv1d_fn(x, w, b, seq_idx=seq, activation="silu"),
                               max(20, args.steps // 4), max(5, args.warmup // 4))

    line = {
        "metric": "fwd/bwd/update µs per call + achieved HBM GB/s (% of MI355X peak)",
        "value": round(gbs(n_bytes, us), 1),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(us * 1e-3, 6),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": "Mamba-2 2.7B prefill forward: bf16 x (8, 5376, 2048) channel-last, width 4, "
                               "bias, SiLU, int32 seq_idx with 1-4 packed sub-sequences per row",
                   "algorithmic_bytes": int(n_bytes), "us_per_call": round(us, 3),
                   "timed": "K steps behind %d untimed back-to-back launches (sustained clock)" % settle
                            if settle else "K steps out of an idle device (burst)",
                   "us_per_call_burst": round(burst_us, 3),
                   "us_per_call_python_api_wall": round(api_wall, 2)},
        "roofline": {"bound": "hbm", "achieved": round(gbs(n_bytes, us), 1), "peak": HBM_PEAK_GBS,
                     "unit": "GB/s", "frac": round(gbs(n_bytes, us) / HBM_PEAK_GBS, 4), "traffic": None,
                     "frac_burst": round(gbs(n_bytes, burst_us) / HBM_PEAK_GBS, 4)},
    }
    # HBM bytes per launch by FETCH_SIZE / WRITE_SIZE: only rocprofv3 can read those, so the figure
    # is imported from the committed summary, and only while the kernel sources are the ones it was
    # read on (the summary names them by hash); otherwise null.
    prof = profile_figures("fwd_channellast_prefill_traffic.txt", FWD_CL_SOURCES)
    if "traffic_bytes_per_launch" in prof:
        line["roofline"]["traffic"] = int(float(prof["traffic_bytes_per_launch"]))
        line["roofline"]["traffic_source"] = {"profile": prof["profile"], "imported": True,
                                              "kernel_sources_sha16": prof["kernel_sources_sha16"]}
    if not args.no_others and not args.no_rotated:
        # The same call over six rotating sets of x and out (2.1 GB): no launch finds its tensors in a
        # cache, as the layers of a model do; next to it PyTorch's elementwise add over the same sets
        # (the same bytes in, the same bytes out).  Both behind the same untimed launches as `value`.
        sets = rotated_sets()
        rot_us, _ = time_gpu(lambda i: ext.causal_conv1d_fwd(sets[i % 6][0], w, b, seq, None, sets[i % 6][1], None, True),
                             args.steps, args.warmup + settle)
        add_us, _ = time_gpu(lambda i: torch.add(sets[i % 6][0], 1.0, out=sets[i % 6][1]), args.steps, args.warmup + settle)
        line["config"].update({"us_per_call_rotated": round(rot_us, 3), "rotated_sets": 6,
                               "GBps_rotated": round(gbs(n_bytes, rot_us), 1),
                               "us_torch_add_rotated": round(add_us, 3)})
        line["roofline"]["frac_rotated"] = round(gbs(n_bytes, rot_us) / HBM_PEAK_GBS, 4)
        # Twelve sets (4.2 GB): past the reach of the address-translation caches as well, which a
        # kernel that walks rows a row stride apart feels and a linear sweep does not.
        sets += [(torch.randn_like(x), torch.empty_like(x)) for _ in range(6)]
        rot12_us, _ = time_gpu(lambda i: ext.causal_conv1d_fwd(sets[i % 12][0], w, b, seq, None, sets[i % 12][1], None, True),
                               args.steps, args.warmup + settle)
        add12_us, _ = time_gpu(lambda i: torch.add(sets[i % 12][0], 1.0, out=sets[i % 12][1]), args.steps, args.warmup + settle)
        line["config"].update({"us_per_call_rotated_12_sets": round(rot12_us, 3),
                               "us_torch_add_rotated_12_sets": round(add12_us, 3)})
        del sets
    if not args.no_cpu:
        line["cpu_baseline"] = cpu_baseline(cfg_cpu, n_bytes, gpu_out_host)
    del cfg, x, out
    if not args.no_others:
        try:
            line["others"] = bench_others(ext, dev, args.steps, args.warmup, decode_calls=args.decode_calls)
        except Exception as e:                                      # keep the headline line intact
            line["others"] = {"error": repr(e)}
        # The decode step's fractions beside the headline's: events over 400 warm launches, the same
        # over 40 rotating buffer sets, and the device-side duration imported from the committed trace.
        dec = {}
        for key, name in (("update_linear_s3", "linear_s3"), ("update_circular_s8", "circular_s8")):
            r = line["others"].get(key)
            if isinstance(r, dict):
                dec[name] = {"frac": r["frac_of_hbm_peak"], "frac_rotated": r.get("frac_of_hbm_peak_rotated"),
                             "frac_device": round(gbs(r["algorithmic_bytes"], r["us_device_rocprof"]) / HBM_PEAK_GBS, 4)
                                            if "us_device_rocprof" in r else None,
                             "us": r["us"], "us_rotated": r.get("us_rotated")}
        if dec:
            line["roofline"]["decode"] = dec
    print(json.dumps(line), flush=True)


if __name__ == "__main__":
    main()
