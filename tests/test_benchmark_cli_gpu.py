"""The benchmark command line (the counterpart of tests/benchmark_determinism_kernels.py:42-91 of
the reference, for all operators) runs for every --op at a small shape and prints a table that
parses; with --rocprof it also reports device-side kernel durations from a rocprofv3 kernel trace
of the same command."""
import os
import subprocess
import sys

import pytest

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CLI = os.path.join(ROOT, "causal-conv1d_amd", "benchmarks", "benchmark_ops.py")
SMALL = ["--batch", "2", "--dim", "256", "--seqlen", "128", "--warmup", "2", "--rep", "3", "--iters", "3"]


def _table(stdout):
    lines = stdout.splitlines()
    head = next(i for i, l in enumerate(lines) if l.split()[:1] == ["us/call"])
    us, moved, gbs, pct, mb = lines[head + 1].split()
    return float(us), int(moved), float(gbs), float(pct), float(mb)


@pytest.mark.parametrize("op,extra", [
    ("fwd", ["--channel-last", "--seq-idx"]), ("fwd", ["--states", "--dtype", "fp32"]),
    ("bwd", ["--states", "--dtype", "fp16"]), ("bwd", ["--channel-last", "--seq-idx"]),
    ("update", ["--state-len", "8", "--circular"]), ("update", []),
    ("varlen", []), ("prefill", []),
])
def test_benchmark_cli_runs_and_prints_its_table(gpu_device, op, extra):
    res = subprocess.run([sys.executable, CLI, "--op", op] + SMALL + extra, capture_output=True, text=True, timeout=300)
    assert res.returncode == 0, res.stderr[-2000:]
    us, moved, gbs, pct, mb = _table(res.stdout)
    assert us > 0 and moved > 0 and gbs > 0 and 0 <= pct < 100 and mb >= 0
    assert abs(gbs - moved / us / 1e3) <= 0.06 + 0.02 * gbs           # the columns agree with each other
    assert ("op=%s " % op) in res.stdout


def test_benchmark_cli_rocprof_capture(gpu_device, tmp_path):
    res = subprocess.run([sys.executable, CLI, "--op", "fwd", "--channel-last", "--rocprof", str(tmp_path)] + SMALL,
                         capture_output=True, text=True, timeout=600)
    assert res.returncode == 0, (res.stdout[-2000:], res.stderr[-2000:])
    assert "rocprofv3 --kernel-trace --stats" in res.stdout
    rows = [l.split(None, 5) for l in res.stdout.split("device-side kernel durations")[1].splitlines()[2:] if l.strip()]
    fwd = [r for r in rows if r[5].startswith("fwd_channellast_kernel")]
    assert fwd, res.stdout[-2000:]
    calls, avg, med, lo, hi = int(fwd[0][0]), *map(float, fwd[0][1:5])
    assert calls >= 2 + 3 * 3 and 0 < lo <= med <= hi and lo <= avg <= hi
    # the event-timed figure includes the dispatch gap, the device-side one does not
    us = _table(res.stdout)[0]
    assert avg < us * 1.5 + 5.0
    assert any(f.endswith("_results.db") for _, _, fs in os.walk(tmp_path) for f in fs)
