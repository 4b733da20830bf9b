"""Compiles fsadam.hip (with the kernel headers next to it) into libfsadam.so next to this file (hipcc, gfx950 only), and the host-side
helper tensor_rows.cpp into a CPython extension module (g++, against the installed torch).

Usage: ``python -m fairscale_amd.csrc.build`` (``--membench``: the microbenchmark library instead), or ``build_library()`` /
``build_rows_module()``.  Both
files are kept in-tree so that a process which loads them shows them among its mapped files.
"""
from __future__ import annotations

import os
import shutil
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
REPO = os.path.dirname(os.path.dirname(HERE))
SOURCE = os.path.join(HERE, "fsadam.hip")
LIBRARY = os.path.join(HERE, "libfsadam.so")
INCLUDE = os.path.join(REPO, "include")

# -ffp-contract=off: multiplies and adds stay separate, as the update equations are written.
# No -ffast-math: division and square root stay correctly rounded, isfinite logic stays meaningful.
# packed fp32 arithmetic is switched off for the device code.
HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared", "-ffp-contract=off",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]


def hipcc_path() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise RuntimeError("hipcc not found (looked at $HIPCC, PATH and /opt/rocm/bin/hipcc)")


def build_library(verbose: bool = False) -> str:
    """Always recompiles; returns the path of the shared library."""
    target = LIBRARY
    cmd = [hipcc_path(), *HIPCC_FLAGS, "-I", INCLUDE, "-I", HERE, "-o", target + ".tmp", SOURCE]
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    noise = "is not a recognized feature for this target"  # the host pass does not know the device feature
    log = "\n".join(line for line in proc.stdout.splitlines() if noise not in line)
    if proc.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + " ".join(cmd) + "\n" + log)
    os.replace(target + ".tmp", target)
    if verbose and log.strip():
        print(log, file=sys.stderr)
    return target


MEMBENCH_SOURCE = os.path.join(HERE, "membench.hip")
MEMBENCH_LIBRARY = os.path.join(HERE, "libfsadam_membench.so")


def membench_is_current() -> bool:
    """The microbenchmark library is there and not older than its source."""
    return os.path.exists(MEMBENCH_LIBRARY) and os.path.getmtime(MEMBENCH_LIBRARY) >= os.path.getmtime(MEMBENCH_SOURCE)


def build_membench(verbose: bool = False) -> str:
    """The microbenchmark kernels of ``bench.py --micro`` and the copy kernel of ``bench.py --calib-copy-bytes`` (a library
    of their own: nothing in the product loads it, and it is built when one of those two asks for it)."""
    cmd = [hipcc_path(), *HIPCC_FLAGS, "-o", MEMBENCH_LIBRARY + ".tmp", MEMBENCH_SOURCE]
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    noise = "is not a recognized feature for this target"
    log = "\n".join(line for line in proc.stdout.splitlines() if noise not in line)
    if proc.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + " ".join(cmd) + "\n" + log)
    os.replace(MEMBENCH_LIBRARY + ".tmp", MEMBENCH_LIBRARY)
    if verbose and log.strip():
        print(log, file=sys.stderr)
    return MEMBENCH_LIBRARY


ROWS_SOURCE = os.path.join(HERE, "tensor_rows.cpp")


def rows_module_path() -> str:
    import sysconfig

    return os.path.join(HERE, "_tensor_rows" + sysconfig.get_config_var("EXT_SUFFIX"))


def build_rows_module(verbose: bool = False) -> str:
    """Always recompiles the list-gathering helper; returns the path of the extension module."""
    import sysconfig

    import pybind11
    import torch
    from torch.utils import cpp_extension

    cxx = os.environ.get("CXX") or shutil.which("g++") or shutil.which("c++")
    if not cxx:
        raise RuntimeError("no C++ compiler found for the host-side helper")
    out = rows_module_path()
    cmd = [cxx, "-O2", "-std=c++17", "-fPIC", "-shared", "-fvisibility=hidden",
           f"-D_GLIBCXX_USE_CXX11_ABI={int(torch._C._GLIBCXX_USE_CXX11_ABI)}"]
    for inc in [*cpp_extension.include_paths(), pybind11.get_include(), sysconfig.get_paths()["include"]]:
        cmd += ["-isystem", inc]
    for lib in cpp_extension.library_paths():
        cmd += ["-L", lib, f"-Wl,-rpath,{lib}"]
    cmd += ["-o", out + ".tmp", ROWS_SOURCE, "-ltorch_python", "-ltorch", "-ltorch_cpu", "-lc10"]
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if proc.returncode != 0:
        raise RuntimeError("compiling tensor_rows.cpp failed:\n" + " ".join(cmd) + "\n" + proc.stdout)
    os.replace(out + ".tmp", out)
    if verbose and proc.stdout.strip():
        print(proc.stdout, file=sys.stderr)
    return out


if __name__ == "__main__":
    if "--membench" in sys.argv[1:]:  # the microbenchmark kernels only (bench.py --micro builds them itself when they are missing)
        print(build_membench(verbose=True))
        sys.exit(0)
    print(build_library(verbose=True))
    print(build_rows_module(verbose=True))
