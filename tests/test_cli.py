"""The `rcr` bench driver keeps the reference's command line (main.cu:38-49), banner
(main.cu:813-832) and one bare ms-per-call float per method (main.cu:1459)."""
import os
import re
import signal
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
RCR = os.path.join(ROOT, "sptmm_amd", "bin", "rcr")


def rcr(*args, timeout=120):
    return subprocess.run([RCR, *args], capture_output=True, text=True, timeout=timeout)


@pytest.fixture(scope="module", autouse=True)
def built():
    if not os.path.exists(RCR):
        from sptmm_amd import build
        build.build_all()
    assert os.path.exists(RCR)


def test_unknown_flag_is_exit_1():
    r = rcr("-no_such_flag=3")
    assert r.returncode == 1 and "unknown command line flag 'no_such_flag'" in r.stderr


@pytest.mark.parametrize("args,msg", [
    (["-iter", "abc"], "illegal value 'abc'"),
    (["-M=-1"], "illegal value '-1'"),
    (["-K"], "missing its argument"),
    (["-i2s=maybe"], "illegal value 'maybe'"),
    (["stray"], "unexpected argument"),
])
def test_bad_values_are_exit_1(args, msg):
    r = rcr(*args)
    assert r.returncode == 1 and msg in r.stderr


@pytest.mark.parametrize("args,msg", [
    (["-row_split3_small", "32", "-M=1", "-K=6912", "-N=2560", "-S=4097"], "S mod 2"),          # main.cu:90
    (["-row_split3_small", "32", "-M=1", "-K=6900", "-N=2560", "-S=4096"], "K mod 16"),         # main.cu:87
    (["-row_split3_small", "32", "-M=1", "-K=6912", "-N=2570", "-S=4096"], "N mod 16"),         # main.cu:88
    (["-row_split3_small", "32", "-M=1", "-K=65536", "-N=2560", "-S=4096"], "16-bit"),          # main.cu:89
    (["-row_split3_small", "32", "-M=1", "-K=4096", "-N=2560", "-S=4096"], "bigger than S"),    # main.cu:91
    (["-row_split3_small", "12", "-M=1", "-K=6912", "-N=2560", "-S=4096"], "Wrong split size"),  # main.cu:1056
    (["-row_split_delta2", "128", "-M=1", "-K=6912", "-N=2560", "-S=4096"], "Wrong split size"),  # main.cu:1838
    (["-row_split3_small", "32", "-M=1", "-K=6912", "-N=2560", "-S=4160", "--row_split_delta2=64"], "Wrong split size"),
])
def test_invalid_shapes_abort_like_strict_assert(args, msg):
    # macro.cuh:66: message on stderr, then abort()
    r = rcr(*args)
    assert r.returncode == -signal.SIGABRT, (r.returncode, r.stderr)
    assert msg in r.stderr


def test_help_lists_reference_flags():
    r = rcr("--help")
    assert r.returncode == 0
    for flag in ("-row_split3_small", "-row_split_delta2", "-i2s", "-cu_blas", "-iter"):
        assert flag in r.stdout


CPU_LINE = re.compile(r"^# cpu: us/call threads=(\d+) median=([0-9.]+) min=([0-9.]+) reps=(\d+) \(([0-9.]+) GB/s\); "
                      r"threads=1 median=([0-9.]+) min=([0-9.]+) reps=(\d+) ")


def check_cpu_line(out):
    """`# cpu:` names the cores the process may use (its affinity mask) and gives median and minimum of at least 3 timed calls,
    for all of them and for one thread."""
    lines = [l for l in out.splitlines() if l.startswith("# cpu:")]
    assert len(lines) == 1, out
    m = CPU_LINE.match(lines[0])
    assert m, lines[0]
    assert int(m.group(1)) == len(os.sched_getaffinity(0))
    assert float(m.group(3)) <= float(m.group(2)) and float(m.group(7)) <= float(m.group(6))
    assert int(m.group(4)) >= 3 and int(m.group(8)) >= 3 and float(m.group(3)) > 0


@pytest.mark.parametrize("args", [
    ["-row_split3_small", "32", "-M=1", "-K=6912", "-N=2560", "-S=4096"],       # the headline shape, int8 rows
    ["-row_split_delta2", "16", "-M=3", "-K=512", "-N=48", "-S=96", "-act", "f16"],
    ["-i2s", "-M=2", "-K=256", "-N=32", "-S=128", "-act=f32"],
    ["-row_split3_small", "8"],                                                  # the reference's default shape (main.cu:43-47)
])
def test_cpu_only_needs_no_device_and_checks_the_lists_against_the_dense_product(args):
    """-cpu_only: the host gather-sum over the lists (main.cu:577-593 on the host) is timed and compared with the plain
    dense product of the same seeded matrix; nothing touches a device."""
    r = rcr(*args, "-cpu_only")
    assert r.returncode == 0, r.stderr
    lines = r.stdout.strip().splitlines()
    assert lines[0] == "make_X done" and lines[2].startswith("Start: M=")
    check_cpu_line(r.stdout)
    assert lines[-1] == "# check=PASS (host gather-sum == host dense product; no device used)"
    assert not [l for l in lines[3:] if not l.startswith("#")]  # no ms-per-call line: nothing ran on a device


def test_cpu_only_without_a_method_aborts():
    r = rcr("-cpu_only", "-M=1", "-K=64", "-N=16", "-S=32")
    assert r.returncode == -signal.SIGABRT and "needs a method" in r.stderr


FLOAT = re.compile(r"^[0-9]+(\.[0-9]+)?(e-?[0-9]+)?$")


def check_output(out, n_methods, M, K, N, S, iters):
    lines = out.strip().splitlines()
    assert lines[0] == "make_X done"
    assert lines[1].startswith("Compiled on ")
    sparsity = 100.0 - 100.0 * (S / K)
    assert lines[2].startswith("Start: M=%d K=%d N=%d ITER=%d S=%d (" % (M, K, N, iters, S))
    got = float(re.search(r"\(([0-9.]+)% Sparsity\)", lines[2]).group(1))
    assert abs(got - sparsity) < 1e-3
    assert lines[2].endswith("L=1 B=8 X_MAJOR=ROW W_MAJOR=COL C_MAJOR=ROW")
    bare = [l for l in lines[3:] if not l.startswith("#")]
    assert len(bare) == n_methods and all(FLOAT.match(b) for b in bare), bare
    assert all(0 < float(b) < 10 for b in bare)  # milliseconds per call
    checks = [l for l in lines if l.startswith("# check=")]
    assert len(checks) == 1 and checks[0].startswith("# check=PASS ("), out
    # every method that ran is compared with the host's own gather-sum, not with another device result
    assert checks[0].count("== host") == n_methods, checks[0]
    check_cpu_line(out)


@pytest.mark.gpu
@pytest.mark.parametrize("args,n", [
    (["-row_split3_small", "32", "-M=1", "-K=6912", "-N=2560", "-S=4096", "-iter=200"], 1),   # README.md:23
    (["-row_split3_small", "32", "-M=4", "-K=6912", "-N=2560", "-S=4096", "-iter=200"], 1),   # README.md:24
    (["-row_split_delta2", "32", "-M=1", "-K=6912", "-N=2560", "-S=4096", "-iter=200"], 1),   # README.md:25
    (["-i2s", "-M=1", "-K=6912", "-N=2560", "-S=4096", "-iter=200"], 1),                      # README.md:27
    (["--row_split3_small=32", "--row_split_delta2", "32", "-i2s", "-M", "1", "-K=6912", "-N=2560", "-S=4096",
      "-iter=100", "-cold=8"], 3),
])
def test_readme_command_lines(args, n):
    r = rcr(*args)
    assert r.returncode == 0, r.stderr
    M = int(re.search(r"-M[= ]?(\d+)", " ".join(args)).group(1))
    iters = int(re.search(r"-iter=(\d+)", " ".join(args)).group(1))
    check_output(r.stdout, n, M, 6912, 2560, 4096, iters)


@pytest.mark.gpu
def test_float_activations_and_cublas_refusal():
    r = rcr("-row_split3_small", "32", "-row_split_delta2", "32", "-M=1", "-K=6912", "-N=2560", "-S=4096",
            "-iter=50", "-act", "f16")
    assert r.returncode == 0 and "# check=PASS (sptmm ~ host; sptmm-delta ~ host; max rel diff" in r.stdout, r.stdout + r.stderr
    r = rcr("-row_split3_small", "32", "-M=2", "-K=512", "-N=64", "-S=128", "-iter=20", "-nocpu")
    assert r.returncode == 0 and "# cpu:" not in r.stdout and "# check=PASS (sptmm == host)" in r.stdout, r.stdout + r.stderr


@pytest.mark.gpu
@pytest.mark.parametrize("M", [1, 4, 16])
def test_cu_blas_runs_the_dense_product_of_the_same_matrix(M):
    """-cu_blas (main.cu:842-873): the dense int8 product through rocBLAS, first of the methods as in the reference, its
    int32 result compared with the host's gather-sum like every other method's."""
    r = rcr("-cu_blas", "-row_split3_small", "32", "-i2s", "-M=%d" % M, "-K=6912", "-N=2560", "-S=4096", "-iter=50", timeout=300)
    assert r.returncode == 0, r.stdout + r.stderr
    check_output(r.stdout, 3, M, 6912, 2560, 4096, 50)
    lines = r.stdout.splitlines()
    first_comment = [l for l in lines if l.startswith("# ") and "us/call sync_each" in l][0]
    assert first_comment.startswith("# cu_blas:") and "rocBLAS int8 x int8 -> int32" in first_comment
    assert "cu_blas == host" in [l for l in lines if l.startswith("# check=")][0]
    r = rcr("-cu_blas", "-M=1", "-K=6912", "-N=2560", "-S=4096", "-act", "f16")
    assert r.returncode == -signal.SIGABRT and "int8 activations" in r.stderr
