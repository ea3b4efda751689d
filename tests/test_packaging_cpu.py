"""The ROCm-only packaging (the counterpart of setup.py:134-251 of the reference: no nvcc branch, no
wheel download) builds and installs into a fresh directory, and the installed copy, imported
from outside the source tree, is the drop-in package: same version, the extension module with
its kernel library beside it, the three DaoAILab ops registered.  Needs no GPU and no network."""
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PKG_DIR = os.path.join(ROOT, "causal-conv1d_amd")

CHECK = r"""
import os, sys
site = sys.argv[1]
import torch
import causal_conv1d, causal_conv1d_cuda
assert os.path.realpath(causal_conv1d.__file__).startswith(os.path.realpath(site)), causal_conv1d.__file__
assert os.path.realpath(causal_conv1d_cuda.__file__).startswith(os.path.realpath(site)), causal_conv1d_cuda.__file__
assert causal_conv1d.__version__ == "1.6.1"
for op in ("_causal_conv1d_fwd_cpp", "_causal_conv1d_bwd_cpp", "_causal_conv1d_update_cpp"):
    assert hasattr(torch.ops.DaoAILab, op), op
for fn in ("causal_conv1d_fn", "causal_conv1d_update", "causal_conv1d_varlen_states"):
    assert callable(getattr(causal_conv1d, fn)), fn
# the binding found the kernel library that was installed beside it, not the one in the source tree
mapped = [l.split()[-1] for l in open("/proc/self/maps") if l.rstrip().endswith("libcc1d.so")]
assert mapped and all(os.path.realpath(m).startswith(os.path.realpath(site)) for m in mapped), mapped
print("installed copy ok")
"""


def test_build_step_compiles_device_code_and_binding(cc1d_lib, tmp_path):
    """The two tests below install what build.py has already built in the tree (up-to-date objects
    are not recompiled).  This one makes the build step compile: one kernel source into a fresh
    object, which must hold a gfx950 code object, and the torch binding into a fresh directory,
    which must import from there beside a copy of the kernel library."""
    import shutil
    import time
    sys.path.insert(0, PKG_DIR)
    import build as cc1d_build
    started = time.time()
    obj = cc1d_build.compile_source("cc1d_varlen_states.hip", str(tmp_path / "obj" / "cc1d_varlen_states.o"))
    assert os.path.getmtime(obj) >= started - 1.0
    blob = open(obj, "rb").read()
    assert blob[:4] == b"\x7fELF" and b"gfx950" in blob and b"varlen_states" in blob
    site = str(tmp_path / "site")
    os.makedirs(site)
    ext = cc1d_build.build_binding(force=True, out_dir=site)
    assert os.path.dirname(ext) == site and os.path.getmtime(ext) >= started - 1.0
    shutil.copy2(os.path.join(PKG_DIR, cc1d_build.LIB_NAME), site)
    shutil.copytree(os.path.join(PKG_DIR, "causal_conv1d"), os.path.join(site, "causal_conv1d"),
                    ignore=shutil.ignore_patterns("__pycache__"))
    _check_installed(site)


def _check_installed(site):
    env = {k: v for k, v in os.environ.items() if k != "PYTHONPATH"}
    env["PYTHONPATH"] = site
    res = subprocess.run([sys.executable, "-c", CHECK, site], cwd=site, env=env, capture_output=True, text=True, timeout=300)
    assert res.returncode == 0 and "installed copy ok" in res.stdout, res.stderr[-3000:]


def test_setup_py_build_into_a_fresh_directory(cc1d_lib, tmp_path):
    site, temp = str(tmp_path / "lib"), str(tmp_path / "temp")
    res = subprocess.run([sys.executable, "setup.py", "-q", "build", "--build-lib", site, "--build-temp", temp],
                         cwd=PKG_DIR, capture_output=True, text=True, timeout=1500)
    assert res.returncode == 0, res.stdout[-3000:] + res.stderr[-3000:]
    assert os.path.exists(os.path.join(site, "libcc1d.so"))
    _check_installed(site)


def test_pip_install_into_a_fresh_directory(cc1d_lib, tmp_path):
    site = str(tmp_path / "site")
    res = subprocess.run([sys.executable, "-m", "pip", "install", "-q", "--no-deps", "--no-build-isolation", "--no-index",
                          "--no-cache-dir", "--target", site, "."],
                         cwd=PKG_DIR, capture_output=True, text=True, timeout=1500)
    assert res.returncode == 0, res.stdout[-3000:] + res.stderr[-3000:]
    assert any(d.startswith("causal_conv1d-1.6.1") for d in os.listdir(site))
    _check_installed(site)
