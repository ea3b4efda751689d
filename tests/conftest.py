"""Shared test plumbing: path set-up, the `gpu` marker, and loading of the in-tree native
libraries (built on demand when nothing has been built yet)."""
import ctypes
import faulthandler
import glob
import os
import sys

import pytest

# A crash on the host (segmentation fault, abort) must leave its Python stack in the log.
faulthandler.enable(all_threads=True)

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PKG_DIR = os.path.join(ROOT, "causal-conv1d_amd")
for p in (ROOT, PKG_DIR):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


def _ensure_built():
    lib = os.path.join(PKG_DIR, "libcc1d.so")
    ext = glob.glob(os.path.join(PKG_DIR, "causal_conv1d_cuda*.so"))
    if not (os.path.exists(lib) and ext):
        sys.path.insert(0, PKG_DIR)
        import build as _build
        _build.build_kernels()
        _build.build_binding()
    return lib


@pytest.fixture(scope="session")
def cc1d_lib():
    """The C-ABI kernel library, loaded with ctypes."""
    lib = ctypes.CDLL(_ensure_built())
    lib.cc1d_strerror.restype = ctypes.c_char_p
    return lib


@pytest.fixture(scope="session")
def pkg():
    """The drop-in Python package (imports the torch extension)."""
    _ensure_built()
    import causal_conv1d
    return causal_conv1d


@pytest.fixture(scope="session")
def gpu_device():
    import torch
    if not torch.cuda.is_available():
        pytest.fail("a test marked `gpu` needs a GPU; run GPU tests on the MI355X box")
    return torch.device("cuda:0")
