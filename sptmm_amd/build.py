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


SOURCES = ("formats.cpp", "ragged.cpp", "wide.cpp", "lists_wide.hip", "capi.hip", "i2s.hip", "lists_u16_scaled.hip", "lists_u16_plain.hip",
           "lists_runs8.hip", "lists_runs16.hip", "lists_ragged_u16_scaled.hip", "lists_ragged_u16_plain.hip",
           "lists_ragged_runs8.hip", "lists_ragged_runs16.hip", "quantise.hip")


def build_lib() -> str:
    """One translation unit per stream flavour, compiled side by side, then linked."""
    from concurrent.futures import ThreadPoolExecutor

    objdir = os.path.join(PKG, "build")
    os.makedirs(objdir, exist_ok=True)

    def compile_one(f):
        obj = os.path.join(objdir, f + ".o")
        _run([HIPCC, *HIPFLAGS, "-c", "-o", obj, "-x", "hip", os.path.join(CSRC, f)])
        return obj

    with ThreadPoolExecutor(max_workers=min(8, os.cpu_count() or 1)) as ex:
        objs = list(ex.map(compile_one, SOURCES))
    tmp = LIB + ".tmp"
    _run([HIPCC, "--offload-arch=gfx950", "-shared", "-pthread", "-o", tmp, *objs])
    os.replace(tmp, LIB)
    return LIB


def build_rcr() -> str:
    os.makedirs(os.path.dirname(RCR), exist_ok=True)
    src = os.path.join(CSRC, "rcr.cpp")
    if not os.path.exists(src):
        return ""
    _run(["g++", "-O2", "-std=c++17", "-Wall", "-o", RCR, src, "-L" + PKG, "-lsptmm",
          "-Wl,-rpath,$ORIGIN/..", "-pthread", "-ldl"])
    return RCR


def build_all():
    return build_lib(), build_rcr()


if __name__ == "__main__":
    print(build_all())
