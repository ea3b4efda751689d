"""Builds the two native libraries, in-tree, next to this file:

  libcc1d.so                      hand-written gfx950 HIP kernels + the C ABI of include/cc1d.h
                                  (hipcc, device code for gfx950 only)
  causal_conv1d_cuda.*.so         host-only PyTorch binding (g++), links libcc1d.so

Plays the part of the reference's setup.py build step (setup.py:134-251) for ROCm only:
no nvcc branch, no source translation, no wheel download.

Usage:  python build.py [--force] [--no-binding]
"""
import argparse
import os
import shlex
import subprocess
import sys
import sysconfig
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
INCLUDE = os.path.join(ROOT, "include")
OBJDIR = os.path.join(HERE, "build")

KERNEL_SOURCES = [
    "cc1d_api.cpp",
    "cc1d_fwd_channellast.hip",
    "cc1d_fwd_channelfirst.hip",
    "cc1d_fwd_channelfirst_tile.hip",
    "cc1d_bwd_channellast.hip",
    "cc1d_bwd_channellast_lanes4.hip",
    "cc1d_bwd_channellast_lanes8.hip",
    "cc1d_bwd_channelfirst.hip",
    "cc1d_bwd_channelfirst_tile.hip",
    "cc1d_bwd_noalloc.hip",
    "cc1d_update.hip",
    "cc1d_varlen_states.hip",
]
KERNEL_HEADERS = ["cc1d_device.hpp", "cc1d_internal.hpp", "cc1d_bwd_channellast_kernel.hpp"]

LIB_NAME = "libcc1d.so"
EXT_NAME = "causal_conv1d_cuda" + (sysconfig.get_config_var("EXT_SUFFIX") or ".so")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
ROCM = os.environ.get("ROCM_PATH", "/opt/rocm")

# Packed-FP32 VALU forms are switched off for all device code.
HIP_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
    "-I" + INCLUDE, "-I" + CSRC,
]


def _run(cmd):
    print("+", " ".join(shlex.quote(c) for c in cmd), flush=True)
    # A compile that does not finish in ten minutes is stuck in the compiler, not slow.
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=600)
    out = "\n".join(l for l in res.stdout.splitlines()
                    if "packed-fp32-ops" not in l and l.strip())
    if out:
        print(out, flush=True)
    if res.returncode != 0:
        raise RuntimeError("command failed (%d): %s" % (res.returncode, " ".join(cmd)))


def _newer(target, deps):
    if not os.path.exists(target):
        return False
    t = os.path.getmtime(target)
    return all(os.path.getmtime(d) <= t for d in deps)


def compile_command(src, obj, extra_flags=()):
    """The hipcc command line that turns one source of csrc/ into an object with gfx950 device code."""
    s = os.path.join(CSRC, src)
    lang = ["-x", "hip"] if src.endswith(".cpp") else []
    return [HIPCC] + HIP_FLAGS + list(extra_flags) + lang + ["-c", s, "-o", obj]


def compile_source(src, obj, extra_flags=()):
    """Compile one source of csrc/ (always: no up-to-date check)."""
    os.makedirs(os.path.dirname(obj), exist_ok=True)
    _run(compile_command(src, obj, extra_flags))
    return obj


def build_kernels(force=False, extra_flags=(), lib_path=None):
    """Compile every HIP source for gfx950 and link libcc1d.so."""
    os.makedirs(OBJDIR, exist_ok=True)
    lib_path = lib_path or os.path.join(HERE, LIB_NAME)
    headers = [os.path.join(CSRC, h) for h in KERNEL_HEADERS] + [os.path.join(INCLUDE, "cc1d.h")]
    tag = "" if not extra_flags else "_" + str(abs(hash(tuple(extra_flags))) % 10**8)
    jobs, objs = [], []
    for src in KERNEL_SOURCES:
        s = os.path.join(CSRC, src)
        o = os.path.join(OBJDIR, os.path.splitext(src)[0] + tag + ".o")
        objs.append(o)
        if force or not _newer(o, [s] + headers):
            jobs.append(compile_command(src, o, extra_flags))
    with ThreadPoolExecutor(max_workers=min(8, max(1, len(jobs)))) as ex:
        list(ex.map(_run, jobs))
    if force or jobs or not _newer(lib_path, objs):
        # Linked by the host compiler, not by hipcc: hipcc's link step writes the toolkit's own
        # lib directory into RUNPATH, and a process that has PyTorch loaded must bind to the HIP
        # runtime PyTorch ships (same soname, libamdhip64.so.7), never map a second one.  With
        # no RUNPATH the NEEDED entry resolves to the runtime already in the process, or to the
        # system's (ld.so.conf) when there is none.
        _run([os.environ.get("CXX", "g++"), "-shared", "-fPIC", "-o", lib_path] + objs +
             ["-L" + os.path.join(ROCM, "lib"), "-lamdhip64", "-ldl"])
    return lib_path


def build_binding(force=False, out_dir=None):
    """Compile the host-only torch binding with g++ and link it against libcc1d.so.  `out_dir`:
    where the extension module goes (default: next to this file, beside libcc1d.so, which the
    module looks for in its own directory)."""
    from torch.utils import cpp_extension as ce
    import torch

    src = os.path.join(CSRC, "causal_conv1d.cpp")
    out = os.path.join(out_dir or HERE, EXT_NAME)
    if not force and _newer(out, [src, os.path.join(INCLUDE, "cc1d.h")]):
        return out
    cmd = [os.environ.get("CXX", "g++"), "-O2", "-std=c++17", "-fPIC", "-shared",
           "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1",
           "-DTORCH_EXTENSION_NAME=causal_conv1d_cuda", "-DTORCH_API_INCLUDE_EXTENSION_H",
           "-D_GLIBCXX_USE_CXX11_ABI=%d" % int(torch._C._GLIBCXX_USE_CXX11_ABI),
           "-Wno-deprecated-declarations"]
    for inc in ce.include_paths():
        cmd += ["-isystem", inc]
    cmd += ["-isystem", os.path.join(ROCM, "include"),
            "-isystem", sysconfig.get_paths()["include"], "-I" + INCLUDE,
            src, "-o", out]
    for lp in ce.library_paths():
        cmd += ["-L" + lp, "-Wl,-rpath," + lp]
    cmd += ["-lc10", "-lc10_hip", "-ltorch_cpu", "-ltorch", "-ltorch_python",
            "-L" + HERE, "-l:" + LIB_NAME, "-Wl,-rpath,$ORIGIN"]
    _run(cmd)
    return out


def main():
    ap = argparse.ArgumentParser(description=__doc__)
    ap.add_argument("--force", action="store_true", help="recompile everything")
    ap.add_argument("--no-binding", action="store_true", help="kernel library only")
    args = ap.parse_args()
    print("built", build_kernels(force=args.force))
    if not args.no_binding:
        print("built", build_binding(force=args.force))


if __name__ == "__main__":
    sys.exit(main())
