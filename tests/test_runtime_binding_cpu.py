"""libcc1d.so must bind to the HIP runtime that is already in the process (PyTorch ships its own
libamdhip64.so under the soname the kernel library needs) and never map a second one: two
runtimes in one process means streams and device pointers of one are foreign to the other.
Each case runs in a fresh interpreter, because what a process has mapped cannot be undone."""
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LIB = os.path.join(ROOT, "causal-conv1d_amd", "libcc1d.so")

PROBE = r"""
import ctypes, os, sys
lib_path, order = sys.argv[1], sys.argv[2]
def runtimes():
    seen = set()
    for line in open("/proc/self/maps"):
        path = line.split()[-1]
        if os.path.basename(path).startswith("libamdhip64.so"):
            seen.add(os.path.realpath(path))
    return sorted(seen)
if order == "torch_first":
    import torch
    lib = ctypes.CDLL(lib_path)
elif order == "runtime_then_lib_then_torch":
    import importlib.util
    torch_lib = os.path.join(os.path.dirname(importlib.util.find_spec("torch").origin), "lib", "libamdhip64.so")
    ctypes.CDLL(torch_lib, mode=ctypes.RTLD_GLOBAL)
    lib = ctypes.CDLL(lib_path)
    import torch
else:
    raise SystemExit("unknown order")
buf = ctypes.create_string_buffer(4096)
assert lib.cc1d_hip_runtime_path(buf, ctypes.c_size_t(len(buf))) == 0
print("BOUND", os.path.realpath(buf.value.decode()))
for r in runtimes():
    print("MAPPED", r)
"""


def _run(order):
    res = subprocess.run([sys.executable, "-c", PROBE, LIB, order], capture_output=True, text=True, timeout=300)
    assert res.returncode == 0, res.stderr[-2000:]
    bound = [l.split(" ", 1)[1] for l in res.stdout.splitlines() if l.startswith("BOUND ")]
    mapped = [l.split(" ", 1)[1] for l in res.stdout.splitlines() if l.startswith("MAPPED ")]
    return bound, mapped


@pytest.mark.parametrize("order", ["torch_first", "runtime_then_lib_then_torch"])
def test_one_hip_runtime_in_the_process(cc1d_lib, order):
    bound, mapped = _run(order)
    assert len(mapped) == 1, "more than one HIP runtime mapped: %s" % mapped
    assert bound == mapped, "libcc1d.so launches through %s, the process uses %s" % (bound, mapped)
    import torch
    assert mapped[0].startswith(os.path.realpath(os.path.dirname(torch.__file__))), mapped


def test_no_runpath_in_the_kernel_library(cc1d_lib):
    out = subprocess.run(["readelf", "-d", LIB], capture_output=True, text=True, check=True).stdout
    assert "RUNPATH" not in out and "RPATH" not in out, out
    assert "libamdhip64.so.7" in out
