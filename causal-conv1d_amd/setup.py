"""ROCm-only packaging: `pip install .` in this directory builds libcc1d.so (hipcc, gfx950)
and the host-only torch binding (g++) with build.py and installs them next to the
`causal_conv1d` package, so `import causal_conv1d` / `import causal_conv1d_cuda` work as with
the reference wheel.  Takes the place of the reference's setup.py:134-251; there is no nvcc
branch, no source translation and no prebuilt-wheel download (setup.py:265-344 there).
"""
import os
import shutil
import sys

from setuptools import Extension, find_packages, setup
from setuptools.command.build_ext import build_ext

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, HERE)
import build as cc1d_build  # noqa: E402  (build.py of this directory)


def read_version():
    for line in open(os.path.join(HERE, "causal_conv1d", "__init__.py")):
        if line.startswith("__version__"):
            return line.split("=")[1].strip().strip("\"'")
    raise RuntimeError("no __version__ in causal_conv1d/__init__.py")


class BuildNative(build_ext):
    """Runs build.py, then copies the two shared objects to where setuptools expects the
    extension (the binding finds libcc1d.so through its $ORIGIN rpath)."""

    def build_extension(self, ext):
        lib = cc1d_build.build_kernels(force=self.force)
        binding = cc1d_build.build_binding(force=self.force)
        target = self.get_ext_fullpath(ext.name)
        os.makedirs(os.path.dirname(target), exist_ok=True)
        shutil.copy2(binding, target)
        shutil.copy2(lib, os.path.join(os.path.dirname(target), cc1d_build.LIB_NAME))


setup(
    name="causal_conv1d",
    version=read_version(),
    description="Causal depthwise conv1d for AMD MI355X (gfx950), drop-in for Dao-AILab/causal-conv1d",
    packages=find_packages(include=["causal_conv1d", "causal_conv1d.*"]),
    ext_modules=[Extension("causal_conv1d_cuda", sources=[])],
    cmdclass={"build_ext": BuildNative},
    python_requires=">=3.9",
    install_requires=["torch"],
    zip_safe=False,
)
