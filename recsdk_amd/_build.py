"""Build recipe for the two shared libraries of the package.

``libhstu_hip.so``      the C-ABI + gfx950 kernels (hipcc, no torch dependency)
``libmxrec_hstu_ops.so`` the ``mxrec`` torch op registration (g++ against libtorch), linked to the former

Both are written next to this file under ``lib/`` so that they travel with the source tree.
"""
from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "lib")
OBJ = os.path.join(HERE, "lib", "obj")
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")

HIP_SOURCES = ["hstu_abi.hip", "hstu_generic.hip", "hstu_mfma.hip", "hstu_mfma_fp8.hip", "hstu_backward.hip", "hstu_mfma_bwd.hip", "hstu_kvcache.hip", "hstu_kvcache_fp8.hip", "hstu_bias.hip", "hstu_layer.hip", "hstu_linear.hip", "hstu_linear_bwd.hip"]
HIP_FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-fno-gpu-rdc",
             # packed fp32 VALU forms are kept out of every kernel in this library
             "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
             "-Wno-unused-command-line-argument"]


def _run(cmd):
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in r.stdout.splitlines() if "packed-fp32-ops" not in l)
    if r.returncode != 0:
        raise RuntimeError("command failed: %s\n%s" % (" ".join(cmd), out))
    return out


def hip_lib_path():
    return os.path.join(LIB, "libhstu_hip.so")


def ops_lib_path():
    return os.path.join(LIB, "libmxrec_hstu_ops.so")


def build_hip(verbose=False, extra_flags=()):
    os.makedirs(OBJ, exist_ok=True)
    objs = []

    def one(src):
        o = os.path.join(OBJ, src.replace(".hip", ".o"))
        out = _run([HIPCC, *HIP_FLAGS, *extra_flags, "-c", os.path.join(CSRC, src), "-o", o])
        if verbose and out.strip():
            print(out)
        return o

    with ThreadPoolExecutor(max_workers=4) as ex:
        objs = list(ex.map(one, HIP_SOURCES))
    _run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", hip_lib_path(), *objs])
    return hip_lib_path()


def timeline_lib_path():
    return os.path.join(LIB, "libhstu_hip_timeline.so")


def build_timeline(verbose=False):
    """Diagnostics flavour of the library: the same sources with the main forward kernel compiled under
    ``-DHSTU_ITEM_TIMING`` (every workgroup stamps its start, first tile, last K loop and end), as a library of its own next
    to the product's, which stays free of it.  ``bench.py --timeline`` loads it.  Needs the objects of ``build_hip``."""
    o = os.path.join(OBJ, "hstu_mfma_timeline.o")
    out = _run([HIPCC, *HIP_FLAGS, "-DHSTU_ITEM_TIMING", "-c", os.path.join(CSRC, "hstu_mfma.hip"), "-o", o])
    if verbose and out.strip():
        print(out)
    objs = [os.path.join(OBJ, s.replace(".hip", ".o")) for s in HIP_SOURCES if s != "hstu_mfma.hip"]
    _run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", timeline_lib_path(), o, *objs])
    return timeline_lib_path()


def build_ops(verbose=False):
    import torch
    from torch.utils import cpp_extension as ce

    inc = []
    for d in ce.include_paths("cuda"):
        inc += ["-isystem", d]
    tlib = os.path.join(os.path.dirname(torch.__file__), "lib")
    cmd = ["g++", "-O2", "-std=c++17", "-fPIC", "-shared", "-D_GLIBCXX_USE_CXX11_ABI=%d" % int(torch._C._GLIBCXX_USE_CXX11_ABI),
           "-DUSE_ROCM", "-D__HIP_PLATFORM_AMD__", *inc, "-I", os.path.join(HERE, "..", "include"),
           os.path.join(CSRC, "mxrec_hstu_ops.cpp"), "-o", ops_lib_path(),
           "-L", LIB, "-lhstu_hip", "-Wl,-rpath,$ORIGIN",
           "-L", tlib, "-ltorch", "-ltorch_cpu", "-lc10", "-ltorch_hip", "-lc10_hip", "-lamdhip64"]
    out = _run(cmd)
    if verbose and out.strip():
        print(out)
    return ops_lib_path()


def build_all(verbose=False):
    build_hip(verbose)
    build_timeline(verbose)
    build_ops(verbose)


if __name__ == "__main__":
    what = sys.argv[1] if len(sys.argv) > 1 else "all"
    {"hip": build_hip, "timeline": build_timeline, "ops": build_ops, "all": build_all}[what](verbose=True)
    print("built", what)
