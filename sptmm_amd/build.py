"""Builds the engine in-tree for gfx950: libsptmm.so (C ABI + HIP kernels) and
the `rcr` bench driver.  `python -m sptmm_amd.build` or build_all()."""
from __future__ import annotations

import os
import shutil
import subprocess
import sys

PKG = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(PKG, "csrc")
LIB = os.path.join(PKG, "libsptmm.so")
RCR = os.path.join(PKG, "bin", "rcr")

HIPCC = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
# packed-fp32 code generation stays off for every device compile
HIPFLAGS = ["-O3", "-std=c++17", "--offload-arch=gfx950", "-fPIC", "-Wall", "-Wno-unused-result",
            "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]


def _run(cmd):
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in r.stdout.splitlines() if "packed-fp32-ops" not in l)
    if r.returncode:
        raise RuntimeError("build failed: %s\n%s" % (" ".join(cmd), out))
    if out.strip():
        print(out, file=sys.stderr)


def build_lib() -> str:
    srcs = [os.path.join(CSRC, f) for f in ("formats.cpp", "kernels.hip", "capi.hip")]
    tmp = LIB + ".tmp"
    _run([HIPCC, *HIPFLAGS, "-shared", "-pthread", "-o", tmp, "-x", "hip", *srcs])
    os.replace(tmp, LIB)
    return LIB


def build_rcr() -> str:
    os.makedirs(os.path.dirname(RCR), exist_ok=True)
    src = os.path.join(CSRC, "rcr.cpp")
    if not os.path.exists(src):
        return ""
    _run(["g++", "-O2", "-std=c++17", "-Wall", "-o", RCR, src, "-L" + PKG, "-lsptmm",
          "-Wl,-rpath,$ORIGIN/..", "-pthread"])
    return RCR


def build_all():
    return build_lib(), build_rcr()


if __name__ == "__main__":
    print(build_all())
