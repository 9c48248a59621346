"""Builds the native parts of the package in-tree.

  libcahel_hip.so   HIP kernels + C-ABI (include/cahel_hip.h), compiled with hipcc for gfx950
  libcahel_probe.so issue-rate micro-benchmarks for bench.py (include/cahel_probe.h), hipcc for gfx950
  pyCAHEL*.so       C++ host layer + pybind11 binding (g++), linked against libcahel_hip.so

Run as `python -m lancelot_amd.build`.  Nothing here needs a GPU: hipcc cross-compiles.
"""
from __future__ import annotations

import concurrent.futures
import glob
import os
import subprocess
import sys
import sysconfig

PKG = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(PKG)
CSRC = os.path.join(PKG, "csrc")
HOST = os.path.join(CSRC, "host")
OBJ = os.path.join(PKG, "build")
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
LIB = os.path.join(PKG, "libcahel_hip.so")
PROBE_LIB = os.path.join(PKG, "libcahel_probe.so")

HIP_FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-Wall", "-Wno-unused-function", "-ffp-contract=off",
             "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]


def _run(cmd):
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in proc.stdout.splitlines() if "packed-fp32-ops" not in l)
    if proc.returncode != 0:
        raise RuntimeError("command failed: %s\n%s" % (" ".join(cmd), out))
    return out


def build_hip(verbose: bool = False) -> str:
    os.makedirs(OBJ, exist_ok=True)
    sources = sorted(glob.glob(os.path.join(CSRC, "*.hip")))
    objs = [os.path.join(OBJ, os.path.basename(s)[:-4] + ".o") for s in sources]
    with concurrent.futures.ThreadPoolExecutor(max_workers=4) as pool:
        list(pool.map(lambda so: _run([HIPCC, *HIP_FLAGS, "-c", so[0], "-o", so[1]]), zip(sources, objs)))
    _run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB, *objs])
    if verbose:
        print("built", LIB)
    return LIB


def build_probe(verbose: bool = False) -> str:
    """The measurement library that bench.py loads beside the engine (not linked into it)."""
    sources = sorted(glob.glob(os.path.join(CSRC, "probe", "*.hip")))
    _run([HIPCC, *HIP_FLAGS, "-shared", "-o", PROBE_LIB, *sources])
    if verbose:
        print("built", PROBE_LIB)
    return PROBE_LIB


def module_path() -> str:
    return os.path.join(PKG, "pyCAHEL" + sysconfig.get_config_var("EXT_SUFFIX"))


def build_host(verbose: bool = False) -> str:
    import pybind11
    os.makedirs(OBJ, exist_ok=True)
    sources = sorted(glob.glob(os.path.join(HOST, "*.cpp")))
    if not sources:
        return ""
    objs = [os.path.join(OBJ, "host_" + os.path.basename(s)[:-4] + ".o") for s in sources]
    inc = ["-I", os.path.join(ROOT, "include"), "-I", HOST, "-I", pybind11.get_include(),
           "-I", sysconfig.get_paths()["include"]]
    flags = ["-O2", "-std=c++17", "-fPIC", "-Wall", "-fvisibility=hidden", "-fopenmp"]
    with concurrent.futures.ThreadPoolExecutor(max_workers=4) as pool:
        list(pool.map(lambda so: _run(["g++", *flags, *inc, "-c", so[0], "-o", so[1]]), zip(sources, objs)))
    out = module_path()
    _run(["g++", "-shared", "-fopenmp", "-o", out, *objs, "-L", PKG, "-lcahel_hip", "-Wl,-rpath,$ORIGIN"])
    if verbose:
        print("built", out)
    return out


def build_all(verbose: bool = False):
    build_hip(verbose)
    build_probe(verbose)
    build_host(verbose)


if __name__ == "__main__":
    if "--help" in sys.argv[1:] or "-h" in sys.argv[1:]:
        print(__doc__)
    else:
        build_all(verbose=True)
