"""The library's host-side launch paths, run end to end without a GPU.

tests/hipstub/ holds a stand-in for the HIP runtime (launches are counted, nothing runs) and a driver that pushes
every stream kind (u16 lists, gap streams for single rows, i2s, ragged, wide) through every protocol of
sptmm_measure_gemv and sptmm_measure_sequence -- plain, synchronised, graph capture, batched, four streams, fork /
join -- at M = 1, 4, 8, 16, from one thread and from four at once.  Hundreds of thousands of launches have to go
through with status 0: shape checks, the launch-shape model, per-launch argument blocks and batching hold no state that
grows with the number of launches queued.
"""
import os
import re
import subprocess

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PKG = os.path.join(ROOT, "sptmm_amd")
STUB = os.path.join(ROOT, "tests", "hipstub")


def test_every_launch_path_runs_against_a_stub_runtime(tmp_path):
    import sptmm_amd

    sptmm_amd.lib()  # the built library (raises if missing)
    exe = str(tmp_path / "launch_stress")
    r = subprocess.run(["g++", "-O1", "-std=c++17", "-D__HIP_PLATFORM_AMD__", "-I/opt/rocm/include", "-rdynamic", "-pthread", "-o", exe,
                        os.path.join(STUB, "launch_stress.cpp"), os.path.join(STUB, "hipstub.cpp"), "-L" + PKG, "-lsptmm",
                        "-Wl,-rpath," + PKG], capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr[-3000:]
    r = subprocess.run([exe, "1000"], capture_output=True, text=True, timeout=600)
    assert r.returncode == 0, (r.stdout + r.stderr)[-3000:]
    one = re.search(r"single thread: (\d+) launches", r.stdout)
    four = re.search(r"four threads: (\d+) launches in all", r.stdout)
    assert one and four, r.stdout
    assert int(one.group(1)) > 100000 and int(four.group(1)) > int(one.group(1)) + 100000
